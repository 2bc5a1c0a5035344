"""Every mechanism the Lilevik family added to the operators, alone, against the plain restatement in
tests/oracle_lilevik.py: on the CPU the engine's plumbing operators, on the GPU (marked gpu) the HIP kernels of libhymix
and libseqmix in float32 and bfloat16.  Batches are built by hand: several sequences, portions that start in the middle
of a sequence, scattered cache blocks and state slots that hold stale data."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "nano-vllm-hw3_amd"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import oracle_lilevik as O  # noqa: E402
from test_hymix_ops import CASES, F64, batch, gen, near, rnd  # noqa: E402  (operator test helpers)

from nanovllm import hy_ops, seq_ops  # noqa: E402
from nanovllm.layers.feedforward import RoutedExperts  # noqa: E402
from nanovllm.layers.latent_attention import LatentAttention  # noqa: E402
from nanovllm.layers.lightning import LightningAttention  # noqa: E402
from nanovllm.layers.rotary_attention import PagedRotaryAttention  # noqa: E402


def module(dtype, make):
    old = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        return make()
    finally:
        torch.set_default_dtype(old)


def run_cut(mod, hs, cuts, device, dtype, seed, caches, forward=None):
    """A layer module fed sequence by sequence in the given cuts (several sequences per step) over scattered pages and
    slots; returns every sequence's outputs joined.  ``caches``: called with the number of pages and slots to allocate
    the module's caches (the test fills them with stale numbers)."""
    lengths = [h.shape[0] for h in hs]
    ctx0, blocks = batch([(0, n) for n in lengths], device=device, seed=seed)
    caches(blocks, len(lengths) + 2)
    tables, slots = ctx0.block_tables, ctx0.seq_slot.tolist()
    done = [0] * len(lengths)
    outs = [[] for _ in lengths]
    for s in range(max(len(c) for c in cuts)):
        who = [b for b in range(len(lengths)) if s < len(cuts[b])]
        portions = [(done[b], cuts[b][s]) for b in who]
        ctx, _ = batch(portions, device=device, seed=seed, slots=[slots[b] for b in who])
        ctx.block_tables = tables[who][:, :max(1, max((p + n + 63) // 64 for p, n in portions))].contiguous()
        bt = ctx.block_tables.cpu()
        sm = [int(bt[i, pos // 64]) * 64 + pos % 64 for i, (p, n) in enumerate(portions) for pos in range(p, p + n)]
        ctx.slot_mapping = torch.tensor(sm, dtype=torch.int32, device=device)
        seq_ops.set_step(ctx)
        x = torch.cat([hs[b][done[b]:done[b] + cuts[b][s]] for b in who]).to(device)
        try:
            y = (forward or mod)(x)
        finally:
            seq_ops.set_step(None)
        y = y[0] if isinstance(y, tuple) else y
        row = 0
        for b in who:
            outs[b].append(y[row:row + cuts[b][s]])
            row += cuts[b][s]
            done[b] += cuts[b][s]
    return [torch.cat(o) for o in outs]


def stale(t, g, s=30.0):
    t.copy_((torch.randn(t.shape, generator=g) * s).to(t.dtype).to(t.device))


# ------------------------------------------------------------------------------------------ residual side
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W", [40, 7, 264])
def test_dyt_residual(device, dtype, W):
    g = gen(W)
    T = 9
    embed = rnd(g, 19, W, dtype=dtype)
    ids = torch.randint(0, 19, (T,), generator=g)

    def norm():
        return (1 + rnd(g, W, s=0.2, dtype=dtype)), rnd(g, W, s=0.3, dtype=dtype), (0.7 + rnd(g, 1, s=0.2)).abs()
    n0, n1, n2 = norm(), norm(), norm()
    dev = lambda n: tuple(t.to(device) for t in n)  # noqa: E731
    ref_of = lambda z, n: O.dyn_tanh(z, n[0].to(F64), n[1].to(F64), n[2].to(F64))  # noqa: E731
    x, h = hy_ops.dyt_residual(None, embed.to(device), None, dev(n0), dtype, ids=ids.to(device))
    ref = embed[ids].to(F64)                                    # the embedding enters as it is
    near(x, ref, torch.float32, f32=1e-6)
    near(h, ref_of(ref, n0), dtype)
    assert x.dtype == torch.float32 and h.dtype == dtype
    y = rnd(g, T, W, s=3.0, dtype=dtype)
    x, h = hy_ops.dyt_residual(x, y.to(device), dev(n1), dev(n2), dtype)
    ref = ref + ref_of(y.to(F64), n1)
    near(x, ref, torch.float32, f32=3e-6)
    near(h, ref_of(ref, n2), dtype)
    y2 = rnd(g, T, W, dtype=dtype)
    x, h = hy_ops.dyt_residual(x, y2.to(device), dev(n2), None, dtype)
    ref = ref + ref_of(y2.to(F64), n2)
    near(x, ref, torch.float32, f32=3e-6)
    near(h, ref, dtype)


def test_rotary_table_against_the_oracle():
    for rot in (dict(dims=32, base=10000.0), dict(dims=8, base=100.0, scaling=dict(factor=4.0, original=64, fast=8.0, slow=1.0)),
                dict(dims=64, base=500000.0, scaling=dict(factor=32.0, original=4096, fast=32.0, slow=1.0)),
                dict(dims=2, base=10.0, scaling=dict(factor=2.0, original=16, fast=4.0, slow=0.5)),
                dict(dims=16, base=10000.0, scaling=dict(factor=8.0, original=8, fast=64.0, slow=32.0))):
        f, mag = hy_ops.rotary_table(rot["dims"], rot["base"], "cpu", rot.get("scaling"))
        rf, rmag = O.rotary_table(rot)
        assert torch.allclose(f.double(), rf, rtol=1e-6, atol=0) and abs(mag - rmag) < 1e-12
    # a table that is stretched in part: its fast pairs are kept, its slow pairs divided by the factor
    f, _ = hy_ops.rotary_table(48, 10000.0, "cpu", dict(factor=8.0, original=512, fast=16.0, slow=1.0))
    plain, _ = hy_ops.rotary_table(48, 10000.0, "cpu")
    lo, hi = 4, 12                             # floor and ceil of 48 ln(512 / (2 pi t)) / (2 ln 10000) at t = 16 and t = 1
    assert torch.equal(f[:lo + 1], plain[:lo + 1]) and torch.allclose(f[hi:] * 8, plain[hi:], rtol=1e-6)
    assert all(0.125 < float(f[i] / plain[i]) < 1.0 for i in range(lo + 1, hi))


# ------------------------------------------------------------------------------------------ chunked sigmoid attention
def run_attention(device, dtype, H, G, D, V, chunk, lengths, cuts, seed=0, dims=None, scaling=(4.0, 64, 8.0, 1.0), sharp=None,
                  force_rows=False, pb=-1.0):
    g = gen(seed)
    W, eps, scale = 32, 1e-5, 0.35
    dims = D // 2 // 2 * 2 if dims is None else dims
    rot = dict(dims=dims, base=100.0)
    if scaling:
        rot["scaling"] = dict(factor=scaling[0], original=scaling[1], fast=scaling[2], slow=scaling[3])
    mod = module(dtype, lambda: PagedRotaryAttention(W, H, G, D, V, scale, eps, dims, 100.0, proj_norm=True, interleaved=True,
                                                     rot_scaling=rot.get("scaling"), v_unit_norm=True, chunk=chunk, weights="sigmoid"))
    p = {"mix.q": rnd(g, H * D, W, s=W ** -0.5, dtype=dtype), "mix.k": rnd(g, G * D, W, s=W ** -0.5, dtype=dtype),
         "mix.v": rnd(g, G * V, W, s=W ** -0.5, dtype=dtype), "mix.q.norm": 1.5 + rnd(g, H * D, s=0.3, dtype=dtype),
         "mix.k.norm": 1.5 + rnd(g, G * D, s=0.3, dtype=dtype), "mix.pb": pb + rnd(g, H, s=0.5),
         "mix.o": rnd(g, W, H * V, s=(H * V) ** -0.5, dtype=dtype)}
    hs = [rnd(g, n, W, dtype=dtype) for n in lengths]
    if sharp:                                  # the query's and the key's inputs agree, and k = q's first heads
        qi, kj = sharp
        hs[0][qi] = hs[0][kj]
        p["mix.k"] = p["mix.q"][:G * D].clone()
        p["mix.k.norm"] = p["mix.q.norm"][:G * D].clone()
    mod.qkv_proj.data.copy_(torch.cat([p["mix.q"], p["mix.k"], p["mix.v"]]))
    mod.q_norm.data.copy_(p["mix.q.norm"])
    mod.k_norm.data.copy_(p["mix.k.norm"])
    mod.head_bias.data.copy_(p["mix.pb"])
    mod.o_proj.data.copy_(p["mix.o"])
    mod.to(device)
    m = dict(heads=H, kv_heads=G, dim=D, vdim=V, scale=scale, rot=rot, mask=dict(size=chunk))
    p64 = {k: v.to(F64) for k, v in p.items()}
    refs = [O.attention_mixer(h.to(F64), p64, m, eps, rounding=(lambda t: t.to(dtype).to(F64))) for h in hs]

    def caches(blocks, slots):
        mod.allocate(blocks, 64, dtype, device)
        stale(mod.k_cache, g)
        stale(mod.v_cache, g)
    old = hy_ops.USE_TILES
    hy_ops.USE_TILES = not force_rows
    try:
        outs = run_cut(mod, hs, cuts, device, dtype, seed, caches)
    finally:
        hy_ops.USE_TILES = old
    for o, r in zip(outs, refs):
        near(o, r, dtype, f32=5e-5, bf16=3e-2)


ATTN_SHAPES = [(4, 2, 16, 8), (2, 1, 64, 64), (6, 6, 8, 24), (3, 1, 72, 40), (8, 2, 120, 88)]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,G,D,V", ATTN_SHAPES)
@pytest.mark.parametrize("chunk", [9, 1, 64, 70, 300, 0])
def test_chunked_sigmoid_attention_whole_and_cut(device, dtype, H, G, D, V, chunk):
    """Whole prompts, portions behind a context, single tokens; chunks of 1, of a cache block, of more, longer than every
    prompt, and no chunking; whole-projection norms, interleaved rotation on a stretched table, unit-RMS values."""
    lengths = [150, 70, 9]
    cuts = [[61, 3, 1, 64, 1, 1, 19], [70], [2, 1, 1, 5]]
    run_attention(device, dtype, H, G, D, V, chunk, lengths, cuts, seed=chunk + H)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("forced", [False, True])
def test_chunk_edges_show(device, dtype, forced):
    """One query whose score for one key stands far above the rest (the bias keeps every other weight near zero), with the
    key placed: at the first position of the query's chunk, one before it, at a cache-block border inside and outside the
    chunk, far back, and the query as the first token of its chunk; as a prompt's row, decoded alone, and behind a portion
    that starts inside the chunk; on the matrix-core kernels and on the portable one."""
    chunk, n = 40, 140                         # the last query (139) lives in chunk [120, 160)
    for key in (120, 119, 121, 64, 63, 2, 138):
        for cuts in ([[n]], [[n - 1, 1]], [[100, 25, n - 126, 1]]):
            run_attention(device, dtype, 4, 2, 16, 16, chunk, [n], cuts, seed=key, sharp=(n - 1, key), force_rows=forced, pb=-6.0,
                          dims=4, scaling=None)
    for cuts in ([[121]], [[120, 1]], [[64, 56, 1]]):        # the query is the first token of its chunk: it sees itself alone
        run_attention(device, dtype, 4, 2, 16, 16, chunk, [121], cuts, seed=1, sharp=(120, 119), force_rows=forced, pb=-6.0,
                      dims=4, scaling=None)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,V", ATTN_SHAPES)
@pytest.mark.parametrize("chunk", [0, 1, 50, 64, 200])
def test_matrix_core_attention_equals_portable(H, G, D, V, chunk):
    """bf16: the tile kernel (portions) and the split-key kernel (single tokens) against the portable kernel on the same
    cache, chunked mask and sigmoid weights."""
    g = gen(chunk + D)
    dev, dt = "cuda", torch.bfloat16
    portions = [(0, 200), (130, 70), (64, 1), (300, 33)]
    for pp in (portions, [(199, 1), (63, 1), (64, 1), (332, 1)]):
        ctx, blocks = batch(pp, device=dev, seed=chunk)
        kc = (torch.randn(blocks, 64, G, D, generator=g) * 0.7).to(dt).to(dev)
        vc = (torch.randn(blocks, 64, G, V, generator=g) * 0.7).to(dt).to(dev)
        q = (torch.randn(ctx.num_tokens, H, D, generator=g) * 0.7).to(dt).to(dev)
        hb = (torch.randn(H, generator=g) - 1.0).to(dev)
        a = hy_ops.paged_attention(q, kc, vc, ctx, 0.2, chunk=chunk, sigmoid=True, head_bias=hb)
        b = hy_ops.paged_attention(q, kc, vc, ctx, 0.2, chunk=chunk, sigmoid=True, head_bias=hb, force_rows=True)
        near(a, b.double().cpu(), dt, bf16=2e-2)


# ------------------------------------------------------------------------------------------ latent attention with a query latent
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,D,Rd,V,R,Q", [(3, 8, 8, 16, 24, 20), (1, 4, 2, 4, 8, 4), (2, 40, 24, 72, 136, 56), (4, 24, 8, 40, 112, 64),
                                          (5, 16, 0, 8, 40, 12)])
def test_latent_attention_with_query_latent(device, dtype, H, D, Rd, V, R, Q):
    g = gen(H + R)
    W, eps, scale = 32, 1e-5, 0.3
    mod = module(dtype, lambda: LatentAttention(W, H, D, V, R, scale, eps, rot_dim=Rd, rot_dims=Rd, rot_base=50.0, q_rank=Q))
    p = {"mix.dq": rnd(g, Q, W, s=2 * W ** -0.5, dtype=dtype), "mix.dq.norm": 1 + rnd(g, Q, s=0.2, dtype=dtype),
         "mix.uq": rnd(g, H * (D + Rd), Q, s=2 * Q ** -0.5, dtype=dtype), "mix.dkv": rnd(g, R + Rd, W, s=2 * W ** -0.5, dtype=dtype),
         "mix.dkv.norm": 1 + rnd(g, R, s=0.2, dtype=dtype), "mix.uk": rnd(g, H * D, R, s=R ** -0.5, dtype=dtype),
         "mix.uv": rnd(g, H * V, R, s=R ** -0.5, dtype=dtype), "mix.o": rnd(g, W, H * V, s=(H * V) ** -0.5, dtype=dtype)}
    mod.qc_proj.data.copy_(torch.cat([p["mix.dq"], p["mix.dkv"]]))
    mod.q_latent_norm.data.copy_(p["mix.dq.norm"])
    mod.uq.data.copy_(p["mix.uq"])
    mod.latent_norm.data.copy_(p["mix.dkv.norm"])
    mod.uk.data.copy_(p["mix.uk"].view(H, D, R))
    mod.uv.data.copy_(p["mix.uv"].view(H, V, R))
    mod.o_proj.data.copy_(p["mix.o"])
    mod.to(device)
    m = dict(heads=H, dim=D, rot_dim=Rd, vdim=V, kv_rank=R, q_rank=Q, scale=scale, rot=dict(dims=Rd, base=50.0))
    hs = [rnd(g, n, W, dtype=dtype) for n in (150, 70, 9)]
    p64 = {k: v.to(F64) for k, v in p.items()}
    refs = [O.latent_attention_mixer(h.to(F64), p64, m, eps, rounding=(lambda t: t.to(dtype).to(F64))) for h in hs]

    def caches(blocks, slots):
        mod.allocate(0, blocks, 64, dtype, device)
        stale(mod.cache[0], g)
    outs = run_cut(mod, hs, [[61, 3, 1, 64, 1, 1, 19], [70], [2, 1, 1, 5]], device, dtype, H, caches)
    for o, r in zip(outs, refs):
        near(o, r, dtype, f32=5e-5, bf16=4e-2)


# ------------------------------------------------------------------------------------------ lightning recurrence
def lightning_case(device, dtype, H, D, V, decay, lengths, cuts, seed):
    g = gen(seed)
    W, eps = 32, 1e-5
    mod = module(dtype, lambda: LightningAttention(W, H, D, V, decay, eps))
    p = {"mix.q": rnd(g, H * D, W, s=2 * W ** -0.5, dtype=dtype), "mix.k": rnd(g, H * D, W, s=2 * W ** -0.5, dtype=dtype),
         "mix.v": rnd(g, H * V, W, s=2 * W ** -0.5, dtype=dtype), "mix.g": rnd(g, H * V, W, s=2 * W ** -0.5, dtype=dtype),
         "mix.norm": 1 + rnd(g, H * V, s=0.2, dtype=dtype), "mix.o": rnd(g, W, H * V, s=(H * V) ** -0.5, dtype=dtype)}
    mod.in_proj.data.copy_(torch.cat([p["mix.q"], p["mix.k"], p["mix.v"], p["mix.g"]]))
    mod.out_norm.data.copy_(p["mix.norm"])
    mod.o_proj.data.copy_(p["mix.o"])
    mod.to(device)
    m = dict(heads=H, dim=D, vdim=V, decay=list(decay))
    hs = [rnd(g, n, W, dtype=dtype) for n in lengths]
    p64 = {k: v.to(F64) for k, v in p.items()}
    refs = [O.lightning_mixer(h.to(F64), p64, m, eps) for h in hs]

    def caches(blocks, slots):
        mod.allocate(slots, device)
        stale(mod.state, g)                    # a slot is never cleared: a portion at position 0 starts from zero by position
    outs = run_cut(mod, hs, cuts, device, dtype, seed, caches)
    for o, r in zip(outs, refs):
        near(o, r, dtype, f32=5e-5, bf16=4e-2)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,D,V,decay", [(3, 8, 16, (0.5, 0.9, 0.995)), (1, 4, 12, (1.0,)), (5, 12, 4, (0.1, 0.5, 0.9, 0.99, 0.999)),
                                         (2, 72, 40, (0.9, 0.99)), (2, 128, 128, (0.97, 0.6)), (1, 200, 36, (0.95,))])
def test_lightning_whole_and_cut(device, dtype, H, D, V, decay):
    """Whole prompts, portions behind a context, single tokens, three sequences per step over stale slots; key and value
    sizes on and off the register tiles and unequal both ways; decays from fast to none."""
    lightning_case(device, dtype, H, D, V, decay, [150, 70, 9], [[61, 3, 1, 64, 1, 1, 19], [70], [2, 1, 1, 5]], seed=H + D)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("sizes", [[1], [7], [600]])
def test_lightning_long_recurrence(device, dtype, sizes):
    """600 tokens in portions of 1, of 7 and at once: the state travels through the slot between steps."""
    n = 600
    cuts = [[sizes[0]] * (n // sizes[0]) + ([n % sizes[0]] if n % sizes[0] else [])]
    lightning_case(device, dtype, 2, 16, 16, (0.999, 0.9), [n], cuts, seed=sizes[0])


# ------------------------------------------------------------------------------------------ router and experts
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W,E,top,bias_s", [(32, 8, 3, 0.5), (48, 16, 4, 3.0), (20, 5, 1, 1.0), (64, 4, 4, 0.2), (136, 12, 5, 8.0), (24, 1, 1, 1.0)])
def test_router_with_bias(device, dtype, W, E, top, bias_s):
    """Logits W h + b in float32, the largest chosen, weights = the softmax over the chosen logits; biases large enough to
    overrule the products."""
    g = gen(W + E)
    T = 37
    h = rnd(g, T, W, dtype=dtype)
    rw, rb = rnd(g, E, W, s=2 * W ** -0.5, dtype=torch.bfloat16).float(), rnd(g, E, s=bias_s, dtype=torch.bfloat16).float()
    idx, wts = seq_ops.moe_route(h.to(device), rw.to(device), top, bias=rb.to(device))
    ridx, rwts = O.route(h.to(F64), rw.to(F64), rb.to(F64), top)
    order = idx.cpu().long().sort(-1)
    rorder = ridx.sort(-1)
    assert torch.equal(order.values, rorder.values)
    near(wts.cpu().gather(1, order.indices), rwts.gather(1, rorder.indices), torch.float32, f32=2e-5)
    near(wts.sum(-1), torch.ones(T, dtype=F64), torch.float32, f32=1e-5)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W,E,top,ff,T", [(32, 8, 3, 24, 19), (48, 6, 2, 16, 1), (64, 4, 4, 40, 300), (40, 5, 1, 8, 64)])
def test_silu_gated_experts(device, dtype, W, E, top, ff, T):
    """The whole feed-forward (router + experts) against the oracle; on the GPU in bfloat16 in all three forms."""
    g = gen(W + T)
    mod = module(dtype, lambda: RoutedExperts(W, E, top, ff, score="softmax", renorm=True, act="silu_glu", bias=True))
    p = {"mlp.router": rnd(g, E, W, s=3 * W ** -0.5, dtype=torch.bfloat16), "mlp.router.b": rnd(g, E, s=0.5, dtype=torch.bfloat16)}
    for e in range(E):
        p.update({f"mlp.e{e}.gate": rnd(g, ff, W, s=2 * W ** -0.5, dtype=dtype), f"mlp.e{e}.up": rnd(g, ff, W, s=2 * W ** -0.5, dtype=dtype),
                  f"mlp.e{e}.down": rnd(g, W, ff, s=ff ** -0.5, dtype=dtype)})
        mod.w_gu.data[e].copy_(torch.cat([p[f"mlp.e{e}.gate"], p[f"mlp.e{e}.up"]]))
        mod.w_down.data[e].copy_(p[f"mlp.e{e}.down"])
    mod.router.data.copy_(p["mlp.router"].float())
    mod.bias.data.copy_(p["mlp.router.b"].float())
    mod.to(device)
    h = rnd(g, T, W, dtype=dtype)
    ref = O.experts(h.to(F64), {k: v.to(F64) for k, v in p.items()}, dict(router=dict(experts=E, top=top), expert=dict(ff=ff)))
    near(mod(h.to(device)), ref, dtype, f32=3e-5, bf16=4e-2)
    if device == "cuda" and dtype == torch.bfloat16:
        idx, wts = seq_ops.moe_route(h.to(device), mod.router, top, bias=mod.bias)
        for form in ("pairs", "grouped", "tiles128"):
            y = seq_ops.moe_experts(h.to(device), idx, wts, mod.w_gu, mod.w_down, mod.limit, mod.alpha, form=form,
                                    act_kind=seq_ops.ACT_SILU_GLU)
            near(y, ref, dtype, bf16=4e-2)
