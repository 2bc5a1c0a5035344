"""Every mechanism the Galupel family added to the operators, alone, against the plain restatement in
tests/oracle_galupel.py: on the CPU the engine's plumbing operators, on the GPU (marked gpu) the HIP kernels of libhymix
and libseqmix in float32 and bfloat16.  Batches are built by hand: several sequences, portions that start in the middle
of a sequence, scattered cache blocks that hold stale data."""
import math
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "nano-vllm-hw3_amd"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import oracle_galupel as O  # noqa: E402
from test_hymix_ops import CASES, F64, batch, gen, near, rnd  # noqa: E402  (operator test helpers)

from nanovllm import hy_ops, seq_ops  # noqa: E402
from nanovllm.layers.feedforward import RoutedExperts  # noqa: E402
from nanovllm.layers.latent_attention import LatentAttention  # noqa: E402
from nanovllm.layers.rotary_attention import PagedRotaryAttention  # noqa: E402


# ------------------------------------------------------------------------------------------ residual side
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W,groups", [(40, 5), (7, 1), (264, 264), (96, 2)])
def test_group_norm_residual(device, dtype, W, groups):
    g = gen(W)
    T, eps = 9, 1e-4
    embed, w0, w1, w2 = rnd(g, 19, W, dtype=dtype), 1 + rnd(g, W, s=0.2, dtype=dtype), rnd(g, W, dtype=dtype), 1 + rnd(g, W, s=0.2, dtype=dtype)
    ids = torch.randint(0, 19, (T,), generator=g)
    x, h = hy_ops.group_norm_residual(None, embed.to(device), w0.to(device), groups, eps, dtype, ids=ids.to(device))
    ref = O.group_rms_norm(embed[ids].to(F64), w0.to(F64), groups, eps)
    near(x, ref, torch.float32, f32=3e-6)
    near(h, ref, dtype)
    assert x.dtype == torch.float32 and h.dtype == dtype
    y = rnd(g, T, W, s=3.0, dtype=dtype)
    x, h = hy_ops.group_norm_residual(x, y.to(device), w1.to(device), groups, eps, dtype)
    ref = ref + O.group_rms_norm(y.to(F64), w1.to(F64), groups, eps)
    near(x, ref, torch.float32, f32=3e-6)
    near(h, ref, dtype)
    y2 = rnd(g, T, W, dtype=dtype)
    x, h = hy_ops.group_norm_residual(x, y2.to(device), w1.to(device), groups, eps, dtype, next_w=w2.to(device))
    ref = ref + O.group_rms_norm(y2.to(F64), w1.to(F64), groups, eps)
    near(x, ref, torch.float32, f32=3e-6)
    near(h, O.group_rms_norm(ref, w2.to(F64), groups, eps), dtype)


@pytest.mark.parametrize("device,dtype", [c for c in CASES if "bfloat16" not in str(c)])
def test_scale_softcap(device, dtype):
    z = rnd(gen(1), 5, 33, s=20.0)
    near(hy_ops.scale_softcap_(z.clone().to(device), 1.5, 25.0), 25.0 * torch.tanh(z.to(F64) * 1.5 / 25.0), torch.float32)
    near(hy_ops.scale_softcap_(z.clone().to(device), 0.5, 0.0), z.to(F64) * 0.5, torch.float32)


# ------------------------------------------------------------------------------------------ pooled-window attention
def run_attention(device, dtype, H, G, D, V, window, pool, lengths, cuts, seed=0, sharp=None, reader=None, force_rows=False):
    """The layer module fed sequence by sequence in the given cuts (several sequences per step) against the oracle's mixer
    on every whole sequence.  ``sharp`` = (query position, key position): that query and key are made to point the same way
    and far longer than the rest, so that whether the key (or its block) is seen decides the row.  ``reader`` = (window, pool):
    a second layer that reads the first one's keys and values with a mask of its own."""
    g = gen(seed)
    W, eps, scale = 32, 1e-5, 0.35
    old = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        mods = [PagedRotaryAttention(W, H, G, D, V, scale, eps, 0, 1.0, window=window, pool=pool, head_norm=True, head_temp=True)]
        if reader:
            mods.append(PagedRotaryAttention(W, H, G, D, V, scale, eps, 0, 1.0, window=reader[0], pool=reader[1], head_norm=True,
                                             head_temp=True, kv_source=mods[0]))
    finally:
        torch.set_default_dtype(old)
    params, ms = [], []
    for mod in mods:
        p = {"mix.q": rnd(g, H * D, W, s=W ** -0.5, dtype=dtype), "mix.q.norm": 1.5 + rnd(g, D, s=0.3, dtype=dtype),
             "mix.temp": 1 + rnd(g, H, s=0.4, dtype=dtype), "mix.o": rnd(g, W, H * V, s=(H * V) ** -0.5, dtype=dtype)}
        if mod.kv_source is None:
            p.update({"mix.k": rnd(g, G * D, W, s=W ** -0.5, dtype=dtype), "mix.v": rnd(g, G * V, W, s=W ** -0.5, dtype=dtype),
                      "mix.k.norm": 1.5 + rnd(g, D, s=0.3, dtype=dtype)})
            mod.qkv_proj.data.copy_(torch.cat([p["mix.q"], p["mix.k"], p["mix.v"]]))
            mod.k_head_norm.data.copy_(p["mix.k.norm"])
        else:
            mod.qkv_proj.data.copy_(p["mix.q"])
        mod.q_head_norm.data.copy_(p["mix.q.norm"])
        mod.temp.data.copy_(p["mix.temp"].float())
        mod.o_proj.data.copy_(p["mix.o"])
        mod.to(device)
        params.append({k: v.to(F64) for k, v in p.items()})
        ms.append(dict(heads=H, kv_heads=G, dim=D, vdim=V, scale=scale, mask=dict(size=mod.window, pool=mod.pool)))
    hs = [rnd(g, n, W, dtype=dtype) for n in lengths]
    if sharp:
        qi, kj = sharp
        hs[0][qi] = hs[0][kj] = (hs[0][kj].float() * 6).to(dtype)      # equal inputs: with k = q's first group they align
        for p, mod in zip(params, mods):
            if mod.kv_source is None:
                p["mix.k"][:] = p["mix.q"][:G * D]
                p["mix.k.norm"][:] = p["mix.q.norm"]
                mod.qkv_proj.data[H * D:H * D + G * D].copy_(mod.qkv_proj.data[:G * D])
                mod.k_head_norm.data.copy_(mod.q_head_norm.data)
    refs = []
    for h in hs:
        y0, kv = O.attention_mixer(h.to(F64), params[0], ms[0], eps, rounding=(lambda t: t.to(dtype).to(F64)))
        refs.append([y0] + ([O.attention_mixer(h.to(F64), params[1], ms[1], eps, kv=kv)[0]] if reader else []))
    # pages: scattered, and full of stale numbers
    n_steps = max(len(c) for c in cuts)
    done = [0] * len(lengths)
    ctx0, blocks = batch([(0, n) for n in lengths], device=device, seed=seed)
    for mod in mods:
        mod.allocate(blocks, 64, dtype, device)
    for c in (mods[0].k_cache, mods[0].v_cache, mods[0].kp_cache, mods[0].vp_cache, mods[-1].kp_cache, mods[-1].vp_cache):
        if c is not None:
            c.copy_(torch.randn(c.shape, generator=g).to(dtype).to(device) * 30)
    tables = ctx0.block_tables
    outs = [[[] for _ in lengths] for _ in mods]
    for s in range(n_steps):
        portions = [(done[b], cuts[b][s]) for b in range(len(lengths)) if s < len(cuts[b])]
        who = [b for b in range(len(lengths)) if s < len(cuts[b])]
        ctx, _ = batch(portions, device=device, seed=seed)
        ctx.block_tables = tables[who][:, :max(1, max((p + n + 63) // 64 for p, n in portions))].contiguous()
        bt = ctx.block_tables.cpu()
        sm = [int(bt[i, pos // 64]) * 64 + pos % 64 for i, (p, n) in enumerate(portions) for pos in range(p, p + n)]
        ctx.slot_mapping = torch.tensor(sm, dtype=torch.int32, device=device)
        seq_ops.set_step(ctx)
        x = torch.cat([hs[b][done[b]:done[b] + cuts[b][s]] for b in who]).to(device)
        try:
            old_tiles = hy_ops.USE_TILES
            hy_ops.USE_TILES = not force_rows
            ys = [mod(x)[0] for mod in mods]
        finally:
            hy_ops.USE_TILES = old_tiles
            seq_ops.set_step(None)
        row = 0
        for b in who:
            for k, y in enumerate(ys):
                outs[k][b].append(y[row:row + cuts[b][s]])
            row += cuts[b][s]
            done[b] += cuts[b][s]
    for k in range(len(mods)):
        for b in range(len(lengths)):
            near(torch.cat(outs[k][b]), refs[b][k], dtype, f32=5e-5, bf16=3e-2)


ATTN_SHAPES = [(4, 2, 16, 8), (2, 1, 64, 64), (6, 6, 8, 24), (3, 1, 72, 40)]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,G,D,V", ATTN_SHAPES)
@pytest.mark.parametrize("window,pool", [(9, 4), (1, 1), (64, 3), (70, 64), (40, 70), (300, 2)])
def test_pooled_window_attention_whole_and_cut(device, dtype, H, G, D, V, window, pool):
    """Whole prompts, portions behind a context, single tokens; windows and pooled blocks of 1, of a cache block, of more;
    a window longer than every prompt (no block is ever seen)."""
    lengths = [150, 70, 9]
    cuts = [[61, 3, 1, 64, 1, 1, 19], [70], [2, 1, 1, 5]]
    run_attention(device, dtype, H, G, D, V, window, pool, lengths, cuts, seed=window + pool)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("forced", [False, True])
def test_pooled_window_attention_edges_show(device, dtype, forced):
    """One query whose score for one key stands far above the rest, with the key placed: far back (seen only through its
    block), at a cache-block border, just inside and just outside the window, and in the newest seen and the oldest unseen
    block; as a prompt's row and decoded alone; on the matrix-core kernels and on the portable one."""
    window, pool, n = 10, 3, 140
    for key in (2, 63, 64, n - 1 - 9, n - 1 - 10, n - 1 - 12, n - 1 - 13, n - 1 - 15):
        for cuts in ([[n]], [[n - 1, 1]], [[100, n - 101, 1]]):
            run_attention(device, dtype, 4, 2, 16, 16, window, pool, [n], cuts, seed=key, sharp=(n - 1, key), force_rows=forced)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("reader", [(9, 4), (5, 4), (20, 7), (3, 1)])
def test_shared_keys_and_values(device, dtype, reader):
    """A layer that reads another layer's keys and values: with the source's block size it reads the source's pooled
    blocks, with another it keeps pooled blocks of its own, made from the source's cache."""
    run_attention(device, dtype, 4, 2, 16, 8, 9, 4, [131, 40], [[50, 14, 1, 66], [1, 39]], seed=reader[0], reader=reader)


# ------------------------------------------------------------------------------------------ latent attention, rotated part
def run_latent(device, dtype, H, D, Rd, V, R, window, dims, lengths, cuts, seed=0, sharp=None, force_rows=False):
    g = gen(seed)
    W, eps, scale, base = 32, 1e-5, 0.3, 50.0
    old = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        mod = LatentAttention(W, H, D, V, R, scale, eps, rot_dim=Rd, rot_dims=dims, rot_base=base, window=window)
    finally:
        torch.set_default_dtype(old)
    p = {"mix.q": rnd(g, H * (D + Rd), W, s=2 * W ** -0.5, dtype=dtype), "mix.dkv": rnd(g, R + Rd, W, s=2 * W ** -0.5, dtype=dtype),
         "mix.dkv.norm": 1 + rnd(g, R, s=0.2, dtype=dtype), "mix.uk": rnd(g, H * D, R, s=R ** -0.5, dtype=dtype),
         "mix.uv": rnd(g, H * V, R, s=R ** -0.5, dtype=dtype), "mix.o": rnd(g, W, H * V, s=(H * V) ** -0.5, dtype=dtype)}
    mod.qc_proj.data.copy_(torch.cat([p["mix.q"], p["mix.dkv"]]))
    mod.latent_norm.data.copy_(p["mix.dkv.norm"])
    mod.uk.data.copy_(p["mix.uk"].view(H, D, R))
    mod.uv.data.copy_(p["mix.uv"].view(H, V, R))
    mod.o_proj.data.copy_(p["mix.o"])
    mod.to(device)
    m = dict(heads=H, dim=D, rot_dim=Rd, vdim=V, kv_rank=R, scale=scale, rot=dict(dims=dims, base=base), mask=dict(size=window))
    hs = [rnd(g, n, W, dtype=dtype) for n in lengths]
    if sharp:                      # a far token equal to the query's token, scaled up: their unrotated parts align
        qi, kj = sharp
        hs[0][qi] = hs[0][kj] = (hs[0][kj].float() * 4).to(dtype)
    refs = [O.latent_attention_mixer(h.to(F64), {k: v.to(F64) for k, v in p.items()}, m, eps) for h in hs]
    ctx0, blocks = batch([(0, n) for n in lengths], device=device, seed=seed)
    mod.allocate(0, blocks, 64, dtype, device)
    mod.cache[0].copy_(torch.randn(mod.cache[0].shape, generator=g).to(dtype).to(device) * 30)
    tables = ctx0.block_tables
    done = [0] * len(lengths)
    outs = [[] for _ in lengths]
    for s in range(max(len(c) for c in cuts)):
        who = [b for b in range(len(lengths)) if s < len(cuts[b])]
        portions = [(done[b], cuts[b][s]) for b in who]
        ctx, _ = batch(portions, device=device, seed=seed)
        ctx.block_tables = tables[who][:, :max(1, max((q + n + 63) // 64 for q, n in portions))].contiguous()
        bt = ctx.block_tables.cpu()
        sm = [int(bt[i, pos // 64]) * 64 + pos % 64 for i, (q, n) in enumerate(portions) for pos in range(q, q + n)]
        ctx.slot_mapping = torch.tensor(sm, dtype=torch.int32, device=device)
        seq_ops.set_step(ctx)
        x = torch.cat([hs[b][done[b]:done[b] + cuts[b][s]] for b in who]).to(device)
        try:
            old_tiles = seq_ops.USE_TILES
            seq_ops.USE_TILES = not force_rows
            y = mod(x)
        finally:
            seq_ops.USE_TILES = old_tiles
            seq_ops.set_step(None)
        row = 0
        for b in who:
            outs[b].append(y[row:row + cuts[b][s]])
            row += cuts[b][s]
            done[b] += cuts[b][s]
    for b in range(len(lengths)):
        near(torch.cat(outs[b]), refs[b], dtype, f32=5e-5, bf16=5e-2)      # (five bf16 products in a row)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,D,Rd,V,R,dims", [(3, 8, 8, 16, 24, 8), (1, 4, 2, 4, 8, 2), (2, 16, 32, 8, 96, 32), (5, 24, 16, 40, 136, 12),
                                             (40, 8, 8, 8, 64, 8), (2, 8, 64, 8, 192, 64)])
@pytest.mark.parametrize("window", [1, 21, 64, 65, 400])
def test_latent_attention_rotated_and_windowed(device, dtype, H, D, Rd, V, R, dims, window):
    lengths = [150, 70, 9]
    cuts = [[61, 3, 1, 64, 1, 1, 19], [70], [2, 1, 1, 5]]
    run_latent(device, dtype, H, D, Rd, V, R, window, dims, lengths, cuts, seed=window)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("forced", [False, True])
def test_latent_window_edges_show(device, dtype, forced):
    """A key that stands out just inside and just outside the window, at a cache-block border and at the window's first
    tile, as a prompt's row and decoded alone."""
    window, n = 30, 140
    for key in (n - 1 - 29, n - 1 - 30, 127, 128, n - 2):
        for cuts in ([[n]], [[n - 1, 1]], [[100, n - 101, 1]]):
            run_latent(device, dtype, 2, 16, 8, 8, 40, window, 8, [n], cuts, seed=key, sharp=(n - 1, key), force_rows=forced)


# ------------------------------------------------------------------------------------------ router and experts
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("E,top,groups,keep", [(8, 3, 4, 2), (10, 3, 5, 2), (5, 1, 1, 1), (6, 6, 2, 2), (16, 4, 8, 3), (9, 2, 9, 4)])
def test_sigmoid_router_with_correction(device, dtype, E, top, groups, keep):
    """The chosen experts and their weights.  Corrections are large and of both signs, so that the choice differs from the
    order of the scores and choice scores are negative (a dropped group must count as minus infinity, not as zero)."""
    g = gen(E + top)
    T, W = 37, 24
    h = rnd(g, T, W, dtype=dtype)
    rw = rnd(g, E, W, s=3 * W ** -0.5, dtype=torch.bfloat16).float()
    corr = (rnd(g, E, s=1.0) - 1.2).to(torch.bfloat16).float()
    idx, wts = seq_ops.moe_route(h.to(device), rw.to(device), top, groups, keep, seq_ops.ROUTE_SIGMOID, corr.to(device), 2, False)
    ridx, rwts = O.route(h.to(F64), rw.to(F64), corr.to(F64), top, groups, keep)
    # rows whose choice is clear beyond rounding must agree exactly; the chosen sets are compared, then the weights
    s = torch.sigmoid(h.to(F64) @ rw.to(F64).T) + corr.to(F64)
    got = torch.zeros(T, E, dtype=F64)
    got.scatter_(1, idx.cpu().long(), wts.cpu().to(F64))
    ref = torch.zeros(T, E, dtype=F64).scatter_(1, ridx, rwts)
    srt = s.sort(-1).values
    clear = (srt[:, 1:] - srt[:, :-1]).min(-1).values > 1e-3
    assert clear.float().mean() > 0.5
    assert torch.equal(got[clear] != 0, ref[clear] != 0)
    assert (got[clear] - ref[clear]).abs().max() < 1e-5
    assert (idx >= 0).all() and (idx < E).all()


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("form", [None, "pairs", "grouped", "tiles128"])
@pytest.mark.parametrize("E,top,W,F,T", [(6, 2, 32, 24, 19), (4, 4, 72, 8, 150), (3, 1, 40, 136, 5), (2, 2, 16, 7608, 3)])
def test_gelu_experts(device, dtype, form, E, top, W, F, T):
    if form in ("grouped", "tiles128") and (device == "cpu" or dtype != torch.bfloat16):
        pytest.skip("the matrix-core forms are bfloat16 kernels")
    g = gen(E * T)
    old = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        mod = RoutedExperts(W, E, top, F, groups=1, keep=1, score="sigmoid", correction=True, group_top=2, renorm=False, act="gelu")
    finally:
        torch.set_default_dtype(old)
    p = {"mlp.router": rnd(g, E, W, s=3 * W ** -0.5, dtype=torch.bfloat16).float(), "mlp.correction": rnd(g, E, s=0.5, dtype=torch.bfloat16).float()}
    for e in range(E):
        p[f"mlp.e{e}.up"], p[f"mlp.e{e}.down"] = rnd(g, F, W, s=2 * W ** -0.5, dtype=dtype), rnd(g, W, F, s=F ** -0.5, dtype=dtype)
    mod.router.data.copy_(p["mlp.router"])
    mod.correction.data.copy_(p["mlp.correction"])
    mod.w_gu.data.copy_(torch.stack([p[f"mlp.e{e}.up"] for e in range(E)]))
    mod.w_down.data.copy_(torch.stack([p[f"mlp.e{e}.down"] for e in range(E)]))
    mod.to(device)
    h = rnd(g, T, W, dtype=dtype)
    idx, wts = O.route(h.to(F64), p["mlp.router"].to(F64), p["mlp.correction"].to(F64), top, 1, 1)
    ref = torch.zeros(T, W, dtype=F64)
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            ref[t] += wts[t, j] * (O.gelu_erf(h[t].to(F64) @ p[f"mlp.e{e}.up"].to(F64).T) @ p[f"mlp.e{e}.down"].to(F64).T)
    y = seq_ops.moe_experts(h.to(device), idx.int().to(device), wts.float().to(device), mod.w_gu, mod.w_down, 0.0, form=form,
                            act_kind=seq_ops.ACT_GELU)
    near(y, ref, dtype, f32=2e-5, bf16=3e-2)
    assert math.isfinite(float(y.float().abs().sum()))
