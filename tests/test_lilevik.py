"""The Lilevik model family in the engine against the plain restatement in tests/oracle_lilevik.py.

Every test makes its own small configuration and random checkpoint.  ``device`` = "cpu" drives the engine's plumbing
operators (scheduler, block and slot pools, portion batching are the same code as on the GPU); "cuda" (marked gpu) drives
the HIP kernels of libhymix and libseqmix, in float32 against tight bounds and in bfloat16 against the rounding of that
format."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "nano-vllm-hw3_amd"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import oracle_lilevik as O  # noqa: E402
from test_pasizen import DEVICES, cut, dtypes_for, replay, tokens, write_model  # noqa: E402  (engine test helpers)


def attn(heads=4, kv_heads=2, dim=16, vdim=8, scale=0.3, chunk=9, dims=8, base=100.0, scaling=(4.0, 64, 8.0, 1.0)):
    rot = dict(dims=dims, base=base)
    if scaling:
        rot["scaling"] = dict(factor=scaling[0], original=scaling[1], fast=scaling[2], slow=scaling[3])
    return "attention", dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, rot=rot, mask=dict(size=chunk))


def latent(heads=3, dim=8, rot_dim=8, vdim=16, kv_rank=24, q_rank=20, scale=0.3, base=50.0):
    return "latent_attention", dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale,
                                    rot=dict(dims=rot_dim, base=base))


def lightning(heads=3, dim=8, vdim=16, decay=(0.5, 0.9, 0.995)):
    return "lightning", dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)[:heads])


def moe(experts=8, top=3, ff=24):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))


def config(layers, width=48, vocab=61, eps=1e-5):
    return dict(architecture="Lilevik", vocab=vocab, width=width, norm=dict(eps=eps),
                layers=[dict(type=kind, mixer=m, mlp=mlp) for (kind, m), mlp in layers])


DEFAULT = [(lightning(), moe()), (latent(), moe(experts=6, top=2, ff=16)), (attn(), None),
           (attn(heads=2, kv_heads=1, dim=24, vdim=24, chunk=70, dims=24, scaling=None), moe(experts=4, top=1)),
           (lightning(heads=2, dim=16, vdim=8, decay=(0.97, 0.7)), None), (latent(heads=2, dim=16, rot_dim=4, vdim=8, kv_rank=40, q_rank=8), None)]


def weights(cfg, seed=0, pb=-1.0):
    """A random checkpoint under the design's tensor names, bf16-representable values."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)
    t = {"embed": rnd(cfg["vocab"], W, s=0.7)}

    def norm(name):
        t.update({name: 1 + rnd(W, s=0.1), name + ".b": rnd(W, s=0.1), name + ".alpha": 0.8 + rnd((), s=0.1)})
    norm("final.norm")
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, D, V = m["heads"], m["dim"], m["vdim"]
        norm(p + "norm1")
        norm(p + "norm1b")
        if L["type"] == "attention":
            G = m["kv_heads"]
            t.update({p + "mix.q": rnd(H * D, W, s=W ** -0.5), p + "mix.k": rnd(G * D, W, s=W ** -0.5),
                      p + "mix.v": rnd(G * V, W, s=W ** -0.5), p + "mix.q.norm": 1.5 + rnd(H * D, s=0.3),
                      p + "mix.k.norm": 1.5 + rnd(G * D, s=0.3), p + "mix.pb": pb + rnd(H, s=0.5),
                      p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
        elif L["type"] == "latent_attention":
            R, Rd, Q = m["kv_rank"], m["rot_dim"], m["q_rank"]
            t.update({p + "mix.dq": rnd(Q, W, s=2 * W ** -0.5), p + "mix.dq.norm": 1 + rnd(Q, s=0.2),
                      p + "mix.uq": rnd(H * (D + Rd), Q, s=2 * Q ** -0.5), p + "mix.dkv": rnd(R + Rd, W, s=2 * W ** -0.5),
                      p + "mix.dkv.norm": 1 + rnd(R, s=0.2), p + "mix.uk": rnd(H * D, R, s=R ** -0.5),
                      p + "mix.uv": rnd(H * V, R, s=R ** -0.5), p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
        else:
            t.update({p + "mix.q": rnd(H * D, W, s=2 * W ** -0.5), p + "mix.k": rnd(H * D, W, s=2 * W ** -0.5),
                      p + "mix.v": rnd(H * V, W, s=2 * W ** -0.5), p + "mix.g": rnd(H * V, W, s=2 * W ** -0.5),
                      p + "mix.norm": 1 + rnd(H * V, s=0.2), p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
        if L["mlp"] is not None:
            E, ff = L["mlp"]["router"]["experts"], L["mlp"]["expert"]["ff"]
            norm(p + "norm2")
            norm(p + "norm2b")
            t.update({p + "mlp.router": rnd(E, W, s=3 * W ** -0.5), p + "mlp.router.b": rnd(E, s=0.5)})
            for e in range(E):
                t.update({f"{p}mlp.e{e}.gate": rnd(ff, W, s=2 * W ** -0.5), f"{p}mlp.e{e}.up": rnd(ff, W, s=2 * W ** -0.5),
                          f"{p}mlp.e{e}.down": rnd(W, ff, s=ff ** -0.5)})
    return {k: v.to(torch.bfloat16).contiguous() for k, v in t.items()}


def close(got, ref, dtype, frac=0.0):
    """Logit rows against the oracle's (difference with its mean removed, relative to the spread of the logits): float32
    to accumulation order, bfloat16 to that format's rounding through the layers.  ``frac``: the share of rows that may
    lie outside (bfloat16 only: a router's near-tie may turn under rounding and swap an expert for that token)."""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape and np.isfinite(got).all()
    d = got - ref
    d = d - d.mean(-1, keepdims=True)
    err = np.sqrt((d ** 2).mean(-1)) / ref.std()
    bound = 2e-4 if dtype == torch.float32 else 6e-2
    bad = (err >= bound).mean()
    allowed = frac if dtype == torch.bfloat16 else 0.0
    assert bad <= allowed, f"{bad:.3f} of the rows beyond {bound}; relative error {err.max():.3g} at row {int(err.argmax())}"


# share of rows a turned near-tie of these small random routers may move in bfloat16: a token whose expert changed also
# stays in the lightning layers' state, so the rows behind it move with it until the decay has worn it off
BF16_TIES = 0.2


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = config(DEFAULT)
    w = weights(cfg, seed=1)
    return write_model(tmp_path_factory.mktemp("lilevik_default"), cfg, w), cfg, w


def forward(cfg, w, toks, **kw):
    return O.forward(cfg, w, toks, **kw)[0].numpy()


# ------------------------------------------------------------------------------------------ whole model, schedules
@pytest.mark.parametrize("device", DEVICES)
def test_whole_prompt_and_layer_trace(model, tmp_path, device):
    """One step per prompt: every position's logits; and the residual after every layer, through the runner itself."""
    path, cfg, w = model
    toks = tokens(90, cfg["vocab"], 3)
    ref, layers = O.forward(cfg, w, toks)
    for dtype in dtypes_for(device):
        got = replay(path, [([("a", toks, list(range(90)))], ["a"])], tmp_path, device, dtype)
        close(got[0], ref.numpy(), dtype, BF16_TIES)
    from nanovllm.engine.llm_engine import LLMEngine
    from nanovllm.engine.sequence import ACTIVE, Sequence
    eng = LLMEngine(path, device=device, dtype=torch.float32, max_num_seqs=2, num_kvcache_blocks=4, max_num_batched_tokens=4096)
    seq = Sequence(toks)
    seq.state = ACTIVE
    assert eng.scheduler.reserve_portion(seq, 90)
    trace = []
    eng.model_runner.run_portions([(seq, 90)], trace=trace)
    assert len(trace) == len(layers) == 6
    for got_l, ref_l in zip(trace, layers):
        assert torch.allclose(got_l.cpu().double(), ref_l, atol=3e-4, rtol=3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_equals_token_by_token(model, tmp_path, device):
    """A prompt fed one token per step (caches and recurrent state built from the very first token) gives the logits of
    the whole prompt in one step; 150 tokens cross two cache-block borders and every chunk's edge."""
    path, cfg, w = model
    toks = tokens(150, cfg["vocab"], 4)
    ref = forward(cfg, w, toks)
    steps = [([("a", [t], [0])], ["a"] if i == 149 else []) for i, t in enumerate(toks)]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=192)
        close(np.concatenate([got[i] for i in range(150)]), ref, dtype, BF16_TIES)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7, 2, 64, 1, 5], [63, 2, 1, 64], [65, 1, 1, 1, 2], [9, 1, 8, 10]])
def test_portions(model, tmp_path, device, sizes):
    """Prompts cut into portions of several sizes (down to two tokens, across cache-block borders and chunk edges, single
    tokens between): a chunk is counted from position 0 of the sequence wherever a portion starts, and the recurrent
    state travels from portion to portion."""
    path, cfg, w = model
    toks = tokens(133, cfg["vocab"], 5)
    ref = forward(cfg, w, toks)
    parts = cut(133, sizes)
    steps = [([("r", toks[a:b], list(range(b - a)))], ["r"] if b == 133 else []) for a, b in parts]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=192)
        close(np.concatenate([got[i] for i in range(len(parts))]), ref, dtype, BF16_TIES)


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_reused_pages_and_slots(model, tmp_path, device):
    """Unequal requests share steps (prompt portions beside single tokens), more requests than state slots and more tokens
    than cache blocks over the run: blocks and slots are freed and taken again, also by a request whose first tokens land
    in a slot that still holds another request's recurrent state.  Each request equals itself alone."""
    path, cfg, w = model
    V = cfg["vocab"]
    reqs = {f"q{i}": tokens(n, V, 10 + i) for i, n in enumerate([97, 5, 130, 66, 1, 71, 64])}
    ref = {k: forward(cfg, w, v) for k, v in reqs.items()}
    plan = {"q0": cut(97, [40, 1, 1, 30, 1]), "q1": cut(5, [2, 1]), "q2": cut(130, [64, 3, 1]), "q3": cut(66, [66]),
            "q4": cut(1, [1]), "q5": cut(71, [7, 1]), "q6": cut(64, [62, 2])}
    live, waiting, steps, rows = [], list(reqs), [], []
    cursor = {k: 0 for k in reqs}
    while live or waiting:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, end = [], []
        for k in list(live):
            a, b = plan[k][cursor[k]]
            cursor[k] += 1
            entries.append((k, reqs[k][a:b], list(range(b - a))))
            rows.append((len(steps), k, a, b))
            if b == len(reqs[k]):
                end.append(k)
                live.remove(k)
        steps.append((entries, end))
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=7 * 64, max_live=3)
        at, all_got, all_ref = {}, [], []
        for s, k, a, b in rows:
            o = at.get(s, 0)
            all_got.append(got[s][o:o + b - a])
            all_ref.append(ref[k][a:b])
            at[s] = o + b - a
        close(np.concatenate(all_got), np.concatenate(all_ref), dtype, BF16_TIES)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(model, tmp_path, device):
    """A short prompt and 200 single-token steps: three block borders and every chunk's edge pass over decoded tokens,
    and the slowly decaying heads carry the prompt through all of them."""
    path, cfg, w = model
    toks = tokens(215, cfg["vocab"], 6)
    ref = forward(cfg, w, toks)
    steps = [([("a", toks[:15], [14])], [])] + [([("a", [t], [0])], []) for t in toks[15:]]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=256)
        close(np.concatenate([got[i] for i in range(len(steps))]), ref[14:], dtype, BF16_TIES)


VARIANTS = {
    # sizes that the default makes equal are unequal here and the other way round; values of 1
    "attention_only_one_head_chunk_1": config([(attn(heads=1, kv_heads=1, dim=8, vdim=8, chunk=1, dims=2, scaling=(2.0, 16, 4.0, 1.0)), None)]),
    "latent_only_top_1": config([(latent(heads=1, dim=4, rot_dim=2, vdim=4, kv_rank=8, q_rank=4), moe(experts=5, top=1))], width=16),
    "lightning_only_all_experts": config([(lightning(heads=1, dim=4, vdim=12, decay=(1.0,)), moe(experts=4, top=4)),
                                          (lightning(heads=5, dim=12, vdim=4, decay=(0.1, 0.5, 0.9, 0.99, 0.999)), None)], width=24),
    "chunk_of_a_page_and_more": config([(attn(chunk=64, dims=16, scaling=(8.0, 32, 16.0, 0.5)), None), (attn(chunk=65, dims=4), moe(top=2)),
                                        (attn(chunk=500, scaling=None), None)], width=24),
    "big_heads": config([(attn(heads=2, kv_heads=2, dim=72, vdim=40, chunk=33, dims=36), None),
                         (latent(heads=2, dim=40, rot_dim=24, vdim=72, kv_rank=136, q_rank=56), None),
                         (lightning(heads=2, dim=72, vdim=40, decay=(0.9, 0.99)), None)]),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_shapes(tmp_path, device, name):
    """Other sizes, orders and constants: each mixer alone, one head, chunks of one token / of a cache block / one more /
    longer than the prompt, rotation of two channels and of the whole head, frequency tables stretched over all, some and
    none of their pairs, a decay of exactly one, key and value sizes that differ both ways, top 1 and all experts, sizes
    off the matrix-core tiles.  Portions and a batch."""
    cfg = VARIANTS[name]
    w = weights(cfg, seed=7)
    path = write_model(tmp_path / "m", cfg, w)
    a, b = tokens(150, cfg["vocab"], 8), tokens(9, cfg["vocab"], 9)
    ra, rb = forward(cfg, w, a), forward(cfg, w, b)
    steps = [([("a", a[:31], list(range(31)))], []),
             ([("a", a[31:131], list(range(100))), ("b", b[:2], [0, 1])], []),
             ([("b", b[2:], list(range(7))), ("a", a[131:132], [0])], ["b"])] + \
            [([("a", [t], [0])], []) for t in a[132:]]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=256)
        allg = np.concatenate([got[i] for i in range(len(steps))])
        allr = np.concatenate([ra[:31], ra[31:131], rb[:2], rb[2:], ra[131:132], ra[132:]])
        close(allg, allr, dtype, BF16_TIES)


def random_config(seed):
    """A configuration drawn from the design's whole space: width, 1-6 layers of any mixer in any order, head counts and
    sizes on and off the matrix-core tiles, chunks around and beyond a cache block, stretched and plain frequency tables,
    decays from fast to none, layers without a feed-forward, routers of 1-12 experts."""
    import random
    r = random.Random(seed)
    width = r.choice([32, 48, 64, 96, 136])
    layers = []
    for _ in range(r.randint(1, 6)):
        mlp = None
        if r.random() < 0.7:
            experts = r.randint(1, 12)
            mlp = moe(experts=experts, top=r.randint(1, min(experts, 5)), ff=r.choice([8, 16, 24, 40]))
        kind = r.choice(["attention", "latent_attention", "lightning"])
        if kind == "attention":
            kvh, rep = r.choice([1, 2, 4]), r.choice([1, 2, 4])
            dim = r.choice([8, 16, 32, 64, 20])
            dims = r.choice([d for d in (2, 4, 8, 16, 20, 32, 64) if d <= dim])
            scaling = (r.choice([2.0, 4.0, 16.0]), r.choice([16, 64, 256]), r.choice([4.0, 32.0]), r.choice([0.5, 1.0])) if r.random() < 0.7 else None
            layers.append((attn(heads=kvh * rep, kv_heads=kvh, dim=dim, vdim=r.choice([8, 16, 32, 64, 12]), scale=dim ** -0.5 * r.choice([1.0, 2.0]),
                                chunk=r.choice([1, 2, 7, 16, 40, 64, 100, 130, 1000]), dims=dims, base=r.choice([100.0, 10000.0]), scaling=scaling), mlp))
        elif kind == "latent_attention":
            layers.append((latent(heads=r.choice([1, 2, 3, 4, 8]), dim=r.choice([4, 8, 16, 32]), rot_dim=r.choice([2, 4, 8, 16, 32]),
                                  vdim=r.choice([4, 8, 16, 32]), kv_rank=r.choice([8, 16, 24, 64, 96, 36]), q_rank=r.choice([4, 12, 32, 50]),
                                  scale=0.2, base=r.choice([50.0, 10000.0])), mlp))
        else:
            heads = r.choice([1, 2, 3, 4, 8])
            layers.append((lightning(heads=heads, dim=r.choice([4, 8, 16, 32, 40]), vdim=r.choice([4, 8, 16, 32, 36]),
                                     decay=[r.choice([0.3, 0.8, 0.95, 0.999, 1.0]) for _ in range(heads)]), mlp))
    return config(layers, width=width, vocab=r.choice([37, 64, 200]))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("seed", range(6))
def test_random_configurations(tmp_path, device, seed):
    """Configurations drawn at random, in float32 (the sharp comparison; bfloat16 is bounded per mechanism and on the
    fixed configurations): a prompt in two portions, a second request beside it, then single tokens."""
    cfg = random_config(seed)
    w = weights(cfg, seed=seed)
    path = write_model(tmp_path / "m", cfg, w)
    n = 150
    a, b = tokens(n, cfg["vocab"], seed), tokens(40, cfg["vocab"], seed + 100)
    ra, rb = forward(cfg, w, a), forward(cfg, w, b)
    c1 = 1 + (seed * 37) % (n - 40)
    steps = [([("a", a[:c1], list(range(c1)))], []),
             ([("a", a[c1:n - 20], list(range(n - 20 - c1))), ("b", b[:7], list(range(7)))], []),
             ([("b", b[7:], list(range(33))), ("a", a[n - 20:n - 19], [0])], ["b"])] + [([("a", [t], [0])], []) for t in a[n - 19:]]
    got = replay(path, steps, tmp_path, device, torch.float32, max_tokens=256)
    close(np.concatenate([got[i] for i in range(len(steps))]),
          np.concatenate([ra[:c1], ra[c1:n - 20], rb[:7], rb[7:], ra[n - 20:n - 19], ra[n - 19:]]), torch.float32)


@pytest.mark.parametrize("device", DEVICES)
def test_chunk_edges_show(tmp_path, device):
    """Weights made so that faults show: a token's key is its first head's query, positions do not turn the heads
    (rot.dims = 0), the scores are steep and the bias is far below zero, so a query gives weight to equal tokens only.  A
    token repeated at the first position of the query's chunk counts, one position earlier it must not; the first
    token of a chunk sees itself alone.  A chunk edge one token off, or chunks counted from a portion's start instead of the
    sequence's, moves these rows by much more than the bound."""
    kind, m = attn(heads=2, kv_heads=1, dim=16, vdim=16, scale=6.0, chunk=20, dims=0, scaling=None)
    cfg = config([((kind, m), None)], width=32)
    w = weights(cfg, seed=3, pb=-12.0)
    w["l0.mix.k"] = w["l0.mix.q"][:16].clone()
    w["l0.mix.k.norm"] = w["l0.mix.q.norm"][:16].clone()
    path = write_model(tmp_path / "m", cfg, w)
    toks = tokens(300, cfg["vocab"], 12)
    # the query at `at` meets its own token at: the first position of its chunk (seen), the last of the chunk before
    # (unseen), inside the chunk across a cache-block border, and far back in an earlier chunk (unseen)
    for back, at in ((280, 290), (279, 291), (260, 270), (259, 271), (62, 291), (240, 259), (5, 295)):
        toks[back] = toks[at]
    ref = forward(cfg, w, toks)
    for size in (19, 21):
        wrong = O.forward(dict(cfg, layers=[dict(cfg["layers"][0], mixer=dict(m, mask=dict(size=size)))]), w, toks)[0].numpy()
        assert np.abs(ref[255:298] - wrong[255:298]).max() > 0.05 * ref.std()      # the edges matter in this model
    steps = [([("a", toks[:250], [249])], []), ([("a", toks[250:273], list(range(23)))], [])] + [([("a", [t], [0])], []) for t in toks[273:]]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=320)
        close(np.concatenate([got[i] for i in range(len(steps))]), ref[249:], dtype)
        whole = replay(path, [([("a", toks, list(range(240, 300)))], ["a"])], tmp_path, device, dtype, max_tokens=320)
        close(whole[0], ref[240:], dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_far_tokens_show(tmp_path, device):
    """A model whose far tokens decide: latent attention with steep scores whose keys follow the queries (equal tokens
    attract, wherever they are), and a lightning head that forgets nothing.  The repeated token lies far back, at a
    cache-block border and among the sequence's first tokens; the queries are decoded alone and as a prompt's rows."""
    cfg = config([(latent(heads=2, dim=16, rot_dim=4, vdim=16, kv_rank=16, q_rank=16, scale=4.0), None),
                  (lightning(heads=2, dim=8, vdim=8, decay=(1.0, 0.999)), None)], width=32)
    w = weights(cfg, seed=5)
    # k_h = c (the up-projection copies the latent) and q_h = the query's own latent: tokens whose latents agree score high
    w["l0.mix.uk"] = torch.eye(16).repeat(2, 1).to(torch.bfloat16)
    w["l0.mix.dq"] = w["l0.mix.dkv"][:16].clone()
    w["l0.mix.dq.norm"] = w["l0.mix.dkv.norm"].clone()
    uq = torch.zeros(2, 20, 16)
    uq[:, :16] = torch.eye(16)
    w["l0.mix.uq"] = uq.reshape(40, 16).to(torch.bfloat16)
    path = write_model(tmp_path / "m", cfg, w)
    toks = tokens(420, cfg["vocab"], 13)
    for back, at in ((0, 400), (1, 401), (63, 402), (64, 403), (127, 404), (250, 405), (399, 406)):
        toks[back] = toks[at]
    ref = forward(cfg, w, toks)
    cut_off = forward(cfg, w, toks[130:])          # without the far tokens the rows differ much
    assert np.abs(ref[400:406] - cut_off[270:276]).max() > 0.05 * ref.std()
    steps = [([("a", toks[:398], [397])], [])] + [([("a", [t], [0])], []) for t in toks[398:]]
    for dtype in dtypes_for(device):
        got = replay(path, steps, tmp_path, device, dtype, max_tokens=448)
        close(np.concatenate([got[i] for i in range(len(steps))]), ref[397:], dtype)
        whole = replay(path, [([("a", toks[:200], []), ], []), ([("a", toks[200:], list(range(190, 220)))], ["a"])], tmp_path, device, dtype,
                       max_tokens=448)
        close(whole[1], ref[390:], dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(model, device):
    """LLM.generate (the scheduler's own portions: a 16-token step budget cuts prompts, decoded tokens share steps with
    prompt pieces, five requests over three slots) continues every prompt as the oracle's greedy loop does."""
    from nanovllm import LLM, SamplingParams
    path, cfg, w = model
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (37, 3, 18, 1, 70)]

    def greedy(p, n):
        p = list(p)
        for _ in range(n):
            p.append(int(forward(cfg, w, p)[-1].argmax()))
        return p[-n:]
    llm = LLM(path, device=device, dtype=torch.float32, max_num_seqs=3, max_num_batched_tokens=16, num_kvcache_blocks=5)
    out = llm.generate(prompts, SamplingParams(max_tokens=6, ignore_eos=True))
    assert [o["token_ids"] for o in out] == [greedy(p, 6) for p in prompts]
    assert len(llm.scheduler.block_manager.free) == 5 and len(llm.scheduler.slots.free) == 3


def test_scheduler_preempts_when_blocks_run_out(model):
    """Two requests that cannot both grow in a three-block pool: the later one is put back, runs again afterwards from
    its first token (its pages and slot hold another request's rows and state by then), and both produce what they
    produce alone."""
    from nanovllm import LLM, SamplingParams
    path, cfg, w = model
    prompts = [tokens(60, cfg["vocab"], 31), tokens(62, cfg["vocab"], 32)]
    sp = SamplingParams(max_tokens=10, ignore_eos=True)
    alone = [LLM(path, device="cpu", dtype=torch.float32, max_num_seqs=2, num_kvcache_blocks=4).generate([p], sp)[0]["token_ids"]
             for p in prompts]
    llm = LLM(path, device="cpu", dtype=torch.float32, max_num_seqs=2, num_kvcache_blocks=3)
    out = llm.generate(prompts, sp)
    assert [o["token_ids"] for o in out] == alone


def test_registry_config_and_dummy_weights(tmp_path):
    from nanovllm.models import registry
    assert registry.architecture_of({"architecture": "Lilevik"}) == "Lilevik"
    from nanovllm import LLM, SamplingParams
    bad = config([(("latent_attention", dict(latent()[1], rot=dict(dims=8, base=50.0, scaling=dict(factor=2.0, original=8, fast=4.0, slow=1.0)))), None)])
    with pytest.raises(ValueError):
        LLM(write_model(tmp_path / "bad", bad, {}), device="cpu", load_format="dummy")
    with pytest.raises(ValueError):
        LLM(write_model(tmp_path / "bad2", config([(("conv", {}), None)]), {}), device="cpu", load_format="dummy")
    # a model without a checkpoint: random tensors under the checkpoint's names go through the same placement
    path = write_model(tmp_path / "dummy", config(DEFAULT), {})
    llm = LLM(path, device="cpu", dtype=torch.float32, load_format="dummy", max_num_seqs=2, num_kvcache_blocks=4)
    out = llm.generate([tokens(20, 61, 1)], SamplingParams(max_tokens=3, ignore_eos=True))
    assert len(out[0]["token_ids"]) == 3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_decode_steps_equal_eager_steps(model, dtype):
    """Decode-only steps replay a hipGraph per batch-size bucket.  Three requests decode for 70 steps (a block border and
    chunk edges are crossed, recurrent states advance inside replays, the batch shrinks from 3 to 2 to 1: three buckets,
    padding rows in the bucket of 4) with an eager prefill of a fourth request between replays; every step's logits equal
    those of an engine that runs everything eagerly."""
    from nanovllm.engine.llm_engine import LLMEngine
    from nanovllm.engine.sequence import ACTIVE, Sequence
    path, cfg, w = model
    engines = [LLMEngine(path, dtype=dtype, enforce_eager=eager, max_num_seqs=4, num_kvcache_blocks=12, max_model_len=256,
                         max_num_batched_tokens=4096) for eager in (True, False)]
    assert not engines[0].model_runner.portion_graphs and sorted(engines[1].model_runner.portion_graphs) == [1, 2, 4]
    prompts = [tokens(n, cfg["vocab"], 40 + n) for n in (50, 3, 61)]
    cont = [tokens(70, cfg["vocab"], 50 + i) for i in range(3)]
    outs = []
    for eng in engines:
        seqs, got = [], []
        for p in prompts:
            s = Sequence(p)
            s.state = ACTIVE
            assert eng.scheduler.reserve_portion(s, len(p))
            seqs.append(s)
        got.append(eng.forward_portions([(s, len(s)) for s in seqs]))
        for s in seqs:
            s.num_computed = s.num_tokens
        for step in range(70):
            live = [(i, s) for i, s in enumerate(seqs) if not (i == 1 and step >= 20) and not (i == 2 and step >= 45)]
            for i, s in live:
                s.extend([cont[i][step]])
                assert eng.scheduler.reserve_portion(s, 1)
            got.append(eng.forward_portions([(s, 1) for _, s in live]))
            for _, s in live:
                s.num_computed += 1
            if step == 30:                      # eager work between replays: another request's prompt
                extra = Sequence(tokens(40, cfg["vocab"], 99))
                extra.state = ACTIVE
                assert eng.scheduler.reserve_portion(extra, 40)
                got.append(eng.forward_portions([(extra, 40)]))
                eng.scheduler.release(extra)
        outs.append([g.float().cpu() for g in got])
    assert [a.shape for a in outs[0]] == [b.shape for b in outs[1]]
    # (float32 is the sharp comparison; in bfloat16 the split count of decode attention differs between the graph's fixed
    # table width and the eager step's, and that rounding may turn a router's near-tie)
    close(torch.cat(outs[1]).numpy(), torch.cat(outs[0]).numpy(), dtype, BF16_TIES)
