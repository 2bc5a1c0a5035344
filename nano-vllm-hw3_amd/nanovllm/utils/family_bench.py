"""Throughput of the Pasizen or the Lipelix family beside the Qwen3 decoder at equal size (random weights, bf16, one
GPU), and the time of every libseqmix / libhymix kernel beside the like kernel of the Qwen3 path with both against their
rooflines; for the Galupel family the comparison is with Pasizen, the closest of the three (latent attention and routed
experts), and its kernels stand beside the forms of the same kernels that Pasizen and Lipelix run; for the Lilevik
family with Galupel (latent attention, masked attention, routed experts) and Lipelix (a recurrent mixer).  Used by
``bench.py --families [--family NAME]``; prints one JSON object."""
import json
import os
import tempfile
import time

import torch

HBM_GBPS, MFMA_TFLOPS = 8000.0, 2500.0        # MI355X: HBM3E peak, dense bf16 matrix peak
VALU_F32_TFLOPS = 157.3                        # float32 vector peak: the bound of arithmetic that must stay float32

SIZES = {                                      # name -> (width, heads, ff, layers, latent rank)
    "w1024": (1024, 16, 3072, 4, 128),
    "w2048": (2048, 16, 6144, 4, 256),
    "w4096": (4096, 32, 12288, 2, 256),
}
VOCAB = 32768


def qwen3_config(width, heads, ff, layers):
    return dict(architectures=["Qwen3ForCausalLM"], hidden_size=width, num_hidden_layers=layers, num_attention_heads=heads,
                num_key_value_heads=max(1, heads // 2), head_dim=128, intermediate_size=ff, vocab_size=VOCAB, rms_norm_eps=1e-6,
                rope_theta=1e6, max_position_embeddings=8192, tie_word_embeddings=False, attention_bias=False,
                hidden_act="silu", torch_dtype="bfloat16")


def pasizen_config(width, heads, ff, layers, rank):
    """Dense (PolyNorm) and routed layers alternate; 16 experts of ff/4 with 4 chosen + one shared: the active
    feed-forward width of a routed layer is that of the dense one."""
    mixer = dict(heads=heads, dim=128, vdim=128, kv_rank=rank, scale=128 ** -0.5)
    moe = dict(kind="moe", expert=dict(ff=ff // 4, limit=7.0),
               router=dict(experts=16, top=4, groups=dict(count=4, keep=2)), shared=dict(ff=ff // 4, limit=7.0))
    return dict(architecture="Pasizen", vocab=VOCAB, width=width, max_positions=8192, norm=dict(eps=1e-5), streams=4,
                canon=dict(taps=4),
                layers=[dict(type="latent_attention", mixer=mixer, mlp=dict(kind="dense", ff=ff) if i % 2 == 0 else moe)
                        for i in range(layers)])


def lipelix_config(width, heads, ff, layers):
    """Full attention, windowed attention, delta rule, full attention, and so on; grouped heads as the Qwen3 model of the
    size has them (heads / 2 key/value heads of 128), half of every head rotated, 512-token windows that keep 4 tokens,
    delta-rule heads of 64 over the model's width."""
    full = dict(heads=heads, kv_heads=max(1, heads // 2), dim=128, vdim=128, rot=dict(dims=64, base=10000.0), scale=128 ** -0.5,
                v_mix=True)
    kinds = [("attention", full), ("attention_2", dict(full, mask=dict(size=512, keep_first=4))),
             ("general_delta", dict(heads=width // 64, dim=64, decay_rank=64)), ("attention", full)]
    return dict(architecture="Lipelix", vocab=VOCAB, width=width, norm=dict(eps=1e-5), residual_mult=0.5, embedding=dict(scale=1.0),
                max_positions=8192,
                layers=[dict(type=kinds[i % 4][0], mixer=kinds[i % 4][1], mlp=dict(kind="dense", ff=ff)) for i in range(layers)])


def galupel_config(width, heads, ff, layers, rank):
    """Latent attention (a 64-channel rotated part beside the latent, so that a cache row is as wide as Pasizen's at the
    size; 512-token window) and grouped-head attention (heads / 2 key/value heads of 128, 512-token window, pooled blocks
    of 64 tokens) alternate; every second attention layer reads the keys and values of the one before it; every layer has
    16 GELU experts of ff/4 with 4 chosen (best 2 of 4 groups): the active feed-forward width is ff."""
    lat = dict(heads=heads, dim=128, rot_dim=64, vdim=128, kv_rank=rank - 64, scale=192 ** -0.5, rot=dict(dims=64, base=10000.0),
               mask=dict(size=512))
    att = dict(heads=heads, kv_heads=max(1, heads // 2), dim=128, vdim=128, scale=128 ** -0.5, mask=dict(size=512, pool=64))
    moe = dict(kind="moe", expert=dict(ff=ff // 4), router=dict(experts=16, top=4, groups=dict(count=4, keep=2)))
    specs = []
    for i in range(layers):
        if i % 2 == 0:
            specs.append(dict(type="latent_attention", mixer=lat, mlp=moe))
        else:
            specs.append(dict(type="attention", mixer=dict(att, kv_from=i - 2) if i % 4 == 3 else att, mlp=moe))
    return dict(architecture="Galupel", vocab=VOCAB, width=width, norm=dict(eps=1e-5, groups=4), logit_scale=1.0, logit_softcap=30.0,
                max_positions=8192, layers=specs)


def lilevik_config(width, heads, ff, layers, rank):
    """Lightning attention (heads of 128 x 128 over the model's width), latent attention (queries through a latent of
    3 x rank, a 64-channel rotated part beside the key/value latent: a cache row as wide as Galupel's at the size), and two
    grouped-head attention layers (heads / 2 key/value heads of 128, chunks of 512 positions, sigmoid weights, half of
    every head rotated on a table stretched 4x); every layer has 16 SiLU-gated experts of ff/4 with 4 chosen."""
    lh = max(1, width // 128)
    light = dict(heads=lh, dim=128, vdim=128, decay=[1.0 - 2.0 ** -(3 + 6 * i / max(1, lh - 1)) for i in range(lh)])
    lat = dict(heads=heads, dim=128, rot_dim=64, vdim=128, kv_rank=rank - 64, q_rank=3 * rank, scale=192 ** -0.5,
               rot=dict(dims=64, base=10000.0))
    att = dict(heads=heads, kv_heads=max(1, heads // 2), dim=128, vdim=128, scale=128 ** -0.5, mask=dict(size=512),
               rot=dict(dims=64, base=10000.0, scaling=dict(factor=4.0, original=2048, fast=32.0, slow=1.0)))
    moe = dict(kind="moe", expert=dict(ff=ff // 4), router=dict(experts=16, top=4))
    kinds = [("lightning", light), ("latent_attention", lat), ("attention", att), ("attention", att)]
    return dict(architecture="Lilevik", vocab=VOCAB, width=width, norm=dict(eps=1e-5), max_positions=8192,
                layers=[dict(type=kinds[i % 4][0], mixer=kinds[i % 4][1], mlp=moe) for i in range(layers)])


def _model_dir(cfg):
    d = tempfile.mkdtemp(prefix="family_bench_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    return d


def _timed(fn, reps):
    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps


def engine_throughput(family, size, prefill_seqs=8, prefill_len=1024, decode_seqs=64, decode_ctx=1024, reps=5):
    """tokens/s of one prefill step (prefill_seqs x prefill_len tokens) and of one decode step (decode_seqs sequences
    with decode_ctx cached tokens) through the engine's own step function."""
    from nanovllm import LLM
    from nanovllm.engine.sequence import ACTIVE, Sequence
    width, heads, ff, layers, rank = SIZES[size]
    cfg = (pasizen_config(width, heads, ff, layers, rank) if family == "pasizen" else
           lipelix_config(width, heads, ff, layers) if family == "lipelix" else
           galupel_config(width, heads, ff, layers, rank) if family == "galupel" else
           lilevik_config(width, heads, ff, layers, rank) if family == "lilevik" else qwen3_config(width, heads, ff, layers))
    llm = LLM(_model_dir(cfg), load_format="dummy", enforce_eager=False, max_model_len=2048,
              max_num_seqs=decode_seqs, max_num_batched_tokens=prefill_seqs * prefill_len, gpu_memory_utilization=0.5)
    g = torch.Generator().manual_seed(0)
    runner, sch = llm.model_runner, llm.scheduler

    def seqs_of(n, length):
        out = []
        for _ in range(n):
            s = Sequence(torch.randint(0, VOCAB, (length,), generator=g).tolist())
            s.state = ACTIVE
            out.append(s)
        return out
    res = {}
    if family != "qwen3":
        pre = seqs_of(prefill_seqs, prefill_len)
        for s in pre:
            assert sch.reserve_portion(s, prefill_len)
        res["prefill_s"] = _timed(lambda: runner.run_portions([(s, prefill_len) for s in pre]), reps)
        for s in pre:
            sch.release(s)
        dec = seqs_of(decode_seqs, decode_ctx + 1)
        for s in dec:
            assert sch.reserve_portion(s, decode_ctx)
        for i in range(0, decode_seqs, 8):
            runner.run_portions([(s, decode_ctx) for s in dec[i:i + 8]])
        for s in dec:
            s.num_computed = decode_ctx
            assert sch.reserve_portion(s, 1)
        res["decode_s"] = _timed(lambda: runner.run_portions([(s, 1) for s in dec]), reps * 4)       # hipGraph replay
        graphs, runner.portion_graphs = runner.portion_graphs, {}
        res["decode_eager_s"] = _timed(lambda: runner.run_portions([(s, 1) for s in dec]), reps * 4)
        runner.portion_graphs = graphs
    else:
        pre = seqs_of(prefill_seqs, prefill_len)
        for s in pre:
            sch.block_manager.allocate(s)
        res["prefill_s"] = _timed(lambda: runner.run(pre, True), reps)
        for s in pre:
            sch.block_manager.deallocate(s)
        dec = seqs_of(decode_seqs, decode_ctx + 1)
        for s in dec:
            sch.block_manager.allocate(s)
        res["decode_s"] = _timed(lambda: runner.run(dec, False), reps * 4)            # hipGraph replay
        runner.enforce_eager = True
        res["decode_eager_s"] = _timed(lambda: runner.run(dec, False), reps * 4)
    out = dict(family=family, size=size, layers=layers, prefill_tokens=prefill_seqs * prefill_len,
               prefill_tok_per_s=round(prefill_seqs * prefill_len / res["prefill_s"]), decode_batch=decode_seqs,
               decode_ctx=decode_ctx, decode_tok_per_s=round(decode_seqs / res["decode_s"]),
               decode_ms_per_step=round(res["decode_s"] * 1e3, 3))
    if "decode_eager_s" in res:
        out["decode_eager_tok_per_s"] = round(decode_seqs / res["decode_eager_s"])
    del llm
    torch.cuda.empty_cache()
    return out


def _event_time(fn, reps=20):
    fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e-3 / reps


def kernel_table(width=2048, heads=16, rank=256, ff=6144, T=8192, seq=1024, B=64, ctx=1024, streams=4, taps=4):
    """Seconds per launch of every libseqmix kernel at a layer's size, the bound it works against (bytes / HBM peak or
    flops / matrix peak) and the fraction of that bound it reaches; beside each the like kernel of the Qwen3 path."""
    from nanovllm import ops, seq_ops
    dev, bf = "cuda", torch.bfloat16
    rows = []

    def add(name, like, sec, bytes_=0, flops=0):
        bound = max(bytes_ / (HBM_GBPS * 1e9), flops / (MFMA_TFLOPS * 1e12))
        rows.append(dict(kernel=name, like=like, us=round(sec * 1e6, 1), bound_us=round(bound * 1e6, 1),
                         of_roofline=round(bound / sec, 3), bound="flops" if flops / (MFMA_TFLOPS * 1e12) > bytes_ / (HBM_GBPS * 1e9) else "bytes"))
    r = lambda *s: torch.randn(*s, device=dev).to(bf)  # noqa: E731
    nseq = T // seq
    # ---- step contexts: a prefill of nseq sequences, a decode of B sequences
    bs = 64

    def context(portions):
        tables, nxt = [], 0
        for p0, n in portions:
            nb = (p0 + n + bs - 1) // bs
            tables.append(list(range(nxt, nxt + nb)))
            nxt += nb
        import numpy as np
        tok_seq = np.concatenate([np.full(n, b) for b, (_, n) in enumerate(portions)])
        tok_pos = np.concatenate([np.arange(p0, p0 + n) for p0, n in portions])
        slot = np.concatenate([np.asarray(tables[b])[np.arange(p0, p0 + n) // bs] * bs + np.arange(p0, p0 + n) % bs
                               for b, (p0, n) in enumerate(portions)])
        mb = max(len(t) for t in tables)
        bt = np.zeros((len(portions), mb), dtype=np.int32)
        for b, t in enumerate(tables):
            bt[b, :len(t)] = t
        qs = np.concatenate([[0], np.cumsum([n for _, n in portions])])
        i32 = lambda v: torch.tensor(np.asarray(v), dtype=torch.int32, device=dev)  # noqa: E731
        return seq_ops.StepContext(tok_seq=i32(tok_seq), tok_pos=i32(tok_pos), qstart=i32(qs), seq_pos0=i32([p for p, _ in portions]),
                                   ctx_lens=i32([p + n for p, n in portions]), seq_slot=i32(list(range(len(portions)))),
                                   slot_mapping=i32(slot), block_tables=i32(bt), num_seqs=len(portions), num_tokens=int(qs[-1]),
                                   max_q=max(n for _, n in portions), block_size=bs), nxt
    pre, nblk_p = context([(0, seq)] * nseq)
    dec, nblk_d = context([(ctx - 1, 1)] * B)
    # ---- residual streams + norm  |  Qwen3: residual add + RMS norm
    X, y, nw = torch.randn(T, streams, width, device=dev), r(T, width), r(width)
    mix, out, w_in = torch.randn(streams, streams, device=dev), torch.randn(streams, device=dev), torch.randn(streams, device=dev)
    add("sm_stream_step (T=%d)" % T, "ql_add_rmsnorm", _event_time(lambda: seq_ops.stream_step(X, y, mix, out, w_in, nw, 1e-5, bf)),
        bytes_=T * width * (8 * streams + 4))
    x2, res = r(T, width), r(T, width)
    add("ql_add_rmsnorm (T=%d)" % T, "-", _event_time(lambda: ops.add_rmsnorm(x2, res, nw, 1e-6)), bytes_=T * width * 8)
    # ---- short convolution | Qwen3 has none: its elementwise launch (SiLU * mul) is the like kernel
    h, cw = r(T, width), r(width, taps)
    state = torch.zeros(nseq, 1, taps - 1, width, device=dev, dtype=bf)
    add("sm_canon_conv+update (T=%d)" % T, "ql_silu_mul", _event_time(lambda: seq_ops.canon_conv(h, cw, state, 0, pre)), bytes_=T * width * 4)
    gu = r(T, 2 * ff)
    add("ql_silu_mul (T=%d)" % T, "-", _event_time(lambda: ops.silu_mul(gu)), bytes_=T * ff * 6)
    # ---- activations
    z, coef = r(T, ff), torch.tensor([0.6, 0.3, 0.1, 0.0], device=dev)
    add("sm_poly_norm (T=%d)" % T, "ql_silu_mul", _event_time(lambda: seq_ops.poly_norm(z, coef, 1e-5)), bytes_=T * ff * 4)
    add("sm_clamped_glu (T=%d)" % T, "ql_silu_mul", _event_time(lambda: seq_ops.clamped_glu(gu, 7.0)), bytes_=T * ff * 6)
    # ---- attention, prefill: absorbed queries over the latent | Qwen3: flash attention over K/V of head_dim 128
    cache = r(max(nblk_p, nblk_d), bs, rank)
    qa = r(T, heads, rank)
    pairs = nseq * seq * (seq + 1) / 2 * heads
    add("sm_latent_attn_tiles (%dx%d, H=%d, R=%d)" % (nseq, seq, heads, rank), "ql_attn_prefill",
        _event_time(lambda: seq_ops.latent_attention(qa, cache, pre, 0.09), 5), flops=pairs * 4 * rank)
    q, k, v = r(T, heads, 128), r(T, heads // 2, 128), r(T, heads // 2, 128)
    cu = torch.arange(0, T + 1, seq, dtype=torch.int32, device=dev)
    add("ql_attn_prefill (%dx%d, H=%d, D=128)" % (nseq, seq, heads), "-", _event_time(lambda: ops.attn_prefill(q, k, v, cu, seq, 0.09), 5),
        flops=pairs * 4 * 128)
    # ---- attention, decode
    qd = r(B, heads, rank)
    add("sm_latent_attn_decode (B=%d, ctx=%d, R=%d)" % (B, ctx, rank), "ql_paged_attn_decode",
        _event_time(lambda: seq_ops.latent_attention(qd, cache, dec, 0.09)), bytes_=B * ctx * rank * 2)
    kc, vc = r(B * ((ctx + 255) // 256), 256, heads // 2, 128), r(B * ((ctx + 255) // 256), 256, heads // 2, 128)
    nb = (ctx + 255) // 256
    tables = torch.arange(B * nb, dtype=torch.int32, device=dev).view(B, nb)
    lens = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    ops.reserve_attn_workspace(B, heads, heads // 2, 256, nb, dev)
    qq = r(B, heads, 128)
    add("ql_paged_attn_decode (B=%d, ctx=%d, Hkv=%d)" % (B, ctx, heads // 2), "-",
        _event_time(lambda: ops.paged_attn_decode(qq, kc, vc, tables, lens, 0.09)), bytes_=B * ctx * (heads // 2) * 128 * 4)
    # ---- latent norm + store | Qwen3: q/k norm + RoPE + K/V store
    qc = r(T, heads * 128 + rank)
    add("sm_latent_norm_store (T=%d)" % T, "ql_qknorm_rope_store",
        _event_time(lambda: seq_ops.latent_norm_store(qc[:, heads * 128:], nw[:rank].contiguous(), 1e-5, cache, pre.slot_mapping)), bytes_=T * rank * 4)
    # ---- routed experts: many tokens (grouped, matrix cores) and few (pair by pair, weight reads)
    E, top, F = 16, 4, ff // 4
    rw = torch.randn(E, width, device=dev)
    w_gu, w_down = r(E, 2 * F, width), r(E, width, F)
    add("sm_moe_route (T=%d, E=%d)" % (T, E), "-", _event_time(lambda: seq_ops.moe_route(h, rw, top, 4, 2)), bytes_=T * width * 2)
    idx, wts = seq_ops.moe_route(h, rw, top, 4, 2)
    tiled = (seq_ops.tile_expert_weights(w_gu, 2), seq_ops.tile_expert_weights(w_down))
    wgu_d, wd_d = r(2 * ff, width), r(width, ff)
    add("sm_moe_grouped (T=%d, top %d of %d, F=%d)" % (T, top, E, F), "bf16 GEMM of the dense MLP (hipBLASLt)",
        _event_time(lambda: seq_ops.moe_experts(h, idx, wts, w_gu, w_down, 7.0, form="grouped", tiled=tiled), 5), flops=T * top * 6 * width * F)
    add("sm_moe_tiles128 (T=%d, top %d of %d, F=%d)" % (T, top, E, F), "bf16 GEMM of the dense MLP (hipBLASLt)",
        _event_time(lambda: seq_ops.moe_experts(h, idx, wts, w_gu, w_down, 7.0, form="tiles128", tiled=tiled), 5), flops=T * top * 6 * width * F)
    hm = h[:512].contiguous()
    idx_m, wts_m = seq_ops.moe_route(hm, rw, top, 4, 2)
    add("sm_moe_grouped (T=512)", "bf16 GEMM of the dense MLP (hipBLASLt)",
        _event_time(lambda: seq_ops.moe_experts(hm, idx_m, wts_m, w_gu, w_down, 7.0, form="grouped", tiled=tiled), 5), flops=512 * top * 6 * width * F,
        bytes_=E * 3 * F * width * 2)
    add("dense MLP GEMMs, hipBLASLt (T=512)", "-",
        _event_time(lambda: torch.nn.functional.linear(torch.nn.functional.linear(hm, wgu_d)[:, :ff], wd_d), 5), flops=512 * 6 * width * ff,
        bytes_=3 * ff * width * 2)
    add("dense MLP GEMMs, hipBLASLt (T=%d, ff=%d)" % (T, ff), "-",
        _event_time(lambda: torch.nn.functional.linear(torch.nn.functional.linear(h, wgu_d)[:, :ff], wd_d), 5), flops=T * 6 * width * ff)
    hd = h[:B].contiguous()
    idx_d, wts_d = seq_ops.moe_route(hd, rw, top, 4, 2)
    touched = len(torch.unique(idx_d))
    add("sm_moe_grouped (T=%d: decode)" % B, "bf16 GEMM of the dense MLP (hipBLASLt)",
        _event_time(lambda: seq_ops.moe_experts(hd, idx_d, wts_d, w_gu, w_down, 7.0, form="grouped", tiled=tiled)), bytes_=touched * 3 * F * width * 2)
    add("dense MLP GEMMs, hipBLASLt (T=%d: decode)" % B, "-",
        _event_time(lambda: torch.nn.functional.linear(torch.nn.functional.linear(hd, wgu_d)[:, :ff], wd_d)), bytes_=3 * ff * width * 2)
    return rows


def hymix_kernel_table(width=2048, heads=16, ff=6144, T=8192, seq=1024, B=64, ctx=1024, window=512, keep=4):
    """Seconds per launch of every libhymix kernel at a layer's size, its bound and the fraction of it reached; beside each
    the like kernel of the Qwen3 path."""
    from nanovllm import hy_ops, ops, seq_ops
    dev, bf = "cuda", torch.bfloat16
    rows = []

    def add(name, like, sec, bytes_=0, flops=0):
        bound = max(bytes_ / (HBM_GBPS * 1e9), flops / (MFMA_TFLOPS * 1e12))
        rows.append(dict(kernel=name, like=like, us=round(sec * 1e6, 1), bound_us=round(bound * 1e6, 1),
                         of_roofline=round(bound / sec, 3), bound="flops" if flops / (MFMA_TFLOPS * 1e12) > bytes_ / (HBM_GBPS * 1e9) else "bytes"))
    r = lambda *s: torch.randn(*s, device=dev).to(bf)  # noqa: E731
    nseq, bs, G, D = T // seq, 64, heads // 2, 128
    import numpy as np

    def context(portions):
        tables, nxt = [], 0
        for p0, n in portions:
            nb = (p0 + n + bs - 1) // bs
            tables.append(list(range(nxt, nxt + nb)))
            nxt += nb
        tok_seq = np.concatenate([np.full(n, b) for b, (_, n) in enumerate(portions)])
        tok_pos = np.concatenate([np.arange(p0, p0 + n) for p0, n in portions])
        slot = np.concatenate([np.asarray(tables[b])[np.arange(p0, p0 + n) // bs] * bs + np.arange(p0, p0 + n) % bs
                               for b, (p0, n) in enumerate(portions)])
        mb = max(len(t) for t in tables)
        bt = np.zeros((len(portions), mb), dtype=np.int32)
        for b, t in enumerate(tables):
            bt[b, :len(t)] = t
        qs = np.concatenate([[0], np.cumsum([n for _, n in portions])])
        i32 = lambda v: torch.tensor(np.asarray(v), dtype=torch.int32, device=dev)  # noqa: E731
        return seq_ops.StepContext(tok_seq=i32(tok_seq), tok_pos=i32(tok_pos), qstart=i32(qs), seq_pos0=i32([p for p, _ in portions]),
                                   ctx_lens=i32([p + n for p, n in portions]), seq_slot=i32(list(range(len(portions)))),
                                   slot_mapping=i32(slot), block_tables=i32(bt), num_seqs=len(portions), num_tokens=int(qs[-1]),
                                   max_q=max(n for _, n in portions), block_size=bs, qstart_host=qs.tolist()), nxt
    pre, nblk_p = context([(0, seq)] * nseq)
    dec, nblk_d = context([(ctx - 1, 1)] * B)
    nblk = max(nblk_p, nblk_d)
    # ---- sublayer boundary | Qwen3: residual add + RMS norm
    x, y, gate, gb, pw, nw = torch.randn(T, width, device=dev), r(T, width), r(T, width), r(width), r(width), r(width)
    src, state = r(T, width), torch.zeros(nseq + 1, 1, width, device=dev, dtype=bf)
    add("hm_sublayer_close (T=%d)" % T, "ql_add_rmsnorm",
        _event_time(lambda: hy_ops.sublayer_close(x, y, gate, gb, pw, 0.5, nw, 1e-5, bf, carry=(src, state, 0, pre))),
        bytes_=T * width * (8 + 2 + 2 + 2))
    x2, res = r(T, width), r(T, width)
    add("ql_add_rmsnorm (T=%d)" % T, "-", _event_time(lambda: ops.add_rmsnorm(x2, res, nw, 1e-6)), bytes_=T * width * 8)
    # ---- elementwise launches | Qwen3: SiLU * mul
    h, mu = r(T, width), r(width)
    add("hm_token_shift (T=%d)" % T, "ql_silu_mul", _event_time(lambda: hy_ops.token_shift(h, mu, state, 0, pre)), bytes_=T * width * 4)
    z = r(T, ff + width)
    add("hm_relu_squared (T=%d, ff=%d)" % (T, ff), "ql_silu_mul", _event_time(lambda: hy_ops.relu_squared(z[:, :ff])), bytes_=T * ff * 4)
    gu = r(T, 2 * ff)
    add("ql_silu_mul (T=%d)" % T, "-", _event_time(lambda: ops.silu_mul(gu)), bytes_=T * ff * 6)
    # ---- q/k/v preparation | Qwen3: per-head q/k norm + RoPE + K/V store
    kc, vc = r(nblk, bs, G, D), r(nblk, bs, G, D)
    qkv = r(T, (heads + 2 * G) * D)
    qw, kw = r(heads * D), r(G * D)
    inv_freq = hy_ops.rotary_inv_freq(64, 1e4, dev)
    vf, lam = r(T, G * D), torch.tensor([0.3], device=dev)
    add("hm_qkv_prepare (T=%d, proj norm, v mix)" % T, "ql_qknorm_rope_store",
        _event_time(lambda: hy_ops.qkv_prepare(qkv, heads, G, D, D, qw, kw, 1e-5, inv_freq, False, pre, kc, vc, vf, lam)),
        bytes_=T * ((heads + 2 * G) * D * 4 + G * D * 2))
    add("hm_qkv_prepare (T=%d, unit norm)" % T, "ql_qknorm_rope_store",
        _event_time(lambda: hy_ops.qkv_prepare(qkv, heads, G, D, D, None, None, 1e-5, inv_freq, True, pre, kc, vc, None, None)),
        bytes_=T * (heads + 2 * G) * D * 4)
    cos_sin = torch.randn(T, D, device=dev)
    kq, vq = r(nblk * bs // 256 + 1, 256, G, D), r(nblk * bs // 256 + 1, 256, G, D)
    add("ql_qknorm_rope_store (T=%d)" % T, "-",
        _event_time(lambda: ops.qknorm_rope_store(qkv, None, cos_sin, qw[:D].contiguous(), kw[:D].contiguous(), 1e-6, heads, G, D, kq, vq,
                                                  pre.slot_mapping, want_kv=False)), bytes_=T * (heads + 2 * G) * D * 4)
    # ---- attention, prefill
    q = r(T, heads, D)
    sink = torch.randn(heads, device=dev)
    pairs = nseq * seq * (seq + 1) / 2 * heads
    add("hm_attn_tiles full (%dx%d, H=%d/%d, D=128)" % (nseq, seq, heads, G), "ql_attn_prefill",
        _event_time(lambda: hy_ops.paged_attention(q, kc, vc, pre, 0.09, sink), 5), flops=pairs * 4 * D)
    wpairs = nseq * heads * sum(min(i + 1, window) + min(keep, max(0, i + 1 - window)) for i in range(seq))
    add("hm_attn_tiles window %d+%d (%dx%d)" % (window, keep, nseq, seq), "ql_attn_prefill",
        _event_time(lambda: hy_ops.paged_attention(q, kc, vc, pre, 0.09, sink, window, keep), 5), flops=wpairs * 4 * D)
    k, v = r(T, G, D), r(T, G, D)
    cu = torch.arange(0, T + 1, seq, dtype=torch.int32, device=dev)
    add("ql_attn_prefill (%dx%d, H=%d/%d, D=128)" % (nseq, seq, heads, G), "-", _event_time(lambda: ops.attn_prefill(q, k, v, cu, seq, 0.09), 5),
        flops=pairs * 4 * D)
    # ---- attention, decode
    qd = r(B, heads, D)
    add("hm_attn_decode full (B=%d, ctx=%d, G=%d)" % (B, ctx, G), "ql_paged_attn_decode",
        _event_time(lambda: hy_ops.paged_attention(qd, kc, vc, dec, 0.09, sink)), bytes_=B * ctx * G * D * 4)
    add("hm_attn_decode window %d+%d (B=%d, ctx=%d)" % (window, keep, B, ctx), "ql_paged_attn_decode",
        _event_time(lambda: hy_ops.paged_attention(qd, kc, vc, dec, 0.09, sink, window, keep)), bytes_=B * (window + keep) * G * D * 4)
    nb = (ctx + 255) // 256
    kc2, vc2 = r(B * nb, 256, G, D), r(B * nb, 256, G, D)
    tables = torch.arange(B * nb, dtype=torch.int32, device=dev).view(B, nb)
    lens = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    ops.reserve_attn_workspace(B, heads, G, 256, nb, dev)
    add("ql_paged_attn_decode (B=%d, ctx=%d, G=%d)" % (B, ctx, G), "-",
        _event_time(lambda: ops.paged_attn_decode(qd, kc2, vc2, tables, lens, 0.09)), bytes_=B * ctx * G * D * 4)
    # ---- delta rule: heads of 64 over the width
    Hd, Dd, rank = width // 64, 64, 64
    hd = Hd * Dd
    proj = r(T, 5 * hd + rank)
    w2, w0, ab, onw = r(hd, rank), r(hd), r(hd), r(hd)
    cols = ((0, hd), (hd, hd), (4 * hd, hd), (5 * hd, rank))
    add("hm_delta_prepare (T=%d, H=%d, D=%d)" % (T, Hd, Dd), "ql_qknorm_rope_store",
        _event_time(lambda: hy_ops.delta_prepare(proj, cols, w2, w0, ab, Hd, Dd, 0.6)), bytes_=T * (hd * 6 + hd * 20))
    prep = hy_ops.delta_prepare(proj, cols, w2, w0, ab, Hd, Dd, 0.6)
    st = torch.zeros(max(nseq, B), Hd, Dd, Dd, device=dev)
    vv = proj[:, 2 * hd:3 * hd]
    add("hm_delta_recurrence prefill (%dx%d)" % (nseq, seq), "ql_attn_prefill", _event_time(lambda: hy_ops.delta_recurrence(prep, vv, st, pre), 5),
        bytes_=T * hd * 26, flops=0)
    prep_d = prep[:B].contiguous()
    add("hm_delta_recurrence decode (B=%d)" % B, "ql_paged_attn_decode", _event_time(lambda: hy_ops.delta_recurrence(prep_d, vv[:B], st, dec)),
        bytes_=B * Hd * Dd * Dd * 8)
    o = torch.randn(T, Hd, Dd, device=dev)
    add("hm_delta_gate_norm (T=%d)" % T, "ql_silu_mul", _event_time(lambda: hy_ops.delta_gate_norm(o, proj[:, 3 * hd:4 * hd], onw, 1e-5, bf)),
        bytes_=T * hd * 8)
    return rows


def galupel_kernel_table(width=2048, heads=16, rank=256, ff=6144, T=8192, seq=1024, B=64, ctx=1024, window=512, pool=64):
    """Seconds per launch of every kernel form the Galupel family runs at a layer's size, its bound and the fraction of it
    reached; beside each the form of the same kernel that the closest existing family runs (`like`)."""
    from nanovllm import hy_ops, seq_ops
    dev, bf = "cuda", torch.bfloat16
    rows = []

    def add(name, like, sec, bytes_=0, flops=0):
        bound = max(bytes_ / (HBM_GBPS * 1e9), flops / (MFMA_TFLOPS * 1e12))
        rows.append(dict(kernel=name, like=like, us=round(sec * 1e6, 1), bound_us=round(bound * 1e6, 1),
                         of_roofline=round(bound / sec, 3), bound="flops" if flops / (MFMA_TFLOPS * 1e12) > bytes_ / (HBM_GBPS * 1e9) else "bytes"))
    r = lambda *s: torch.randn(*s, device=dev).to(bf)  # noqa: E731
    nseq, bs, G, D, Rd = T // seq, 64, heads // 2, 128, 64
    R = rank - Rd
    import numpy as np

    def context(portions):
        tables, nxt = [], 0
        for p0, n in portions:
            nb = (p0 + n + bs - 1) // bs
            tables.append(list(range(nxt, nxt + nb)))
            nxt += nb
        tok_seq = np.concatenate([np.full(n, b) for b, (_, n) in enumerate(portions)])
        tok_pos = np.concatenate([np.arange(p0, p0 + n) for p0, n in portions])
        slot = np.concatenate([np.asarray(tables[b])[np.arange(p0, p0 + n) // bs] * bs + np.arange(p0, p0 + n) % bs
                               for b, (p0, n) in enumerate(portions)])
        mb = max(len(t) for t in tables)
        bt = np.zeros((len(portions), mb), dtype=np.int32)
        for b, t in enumerate(tables):
            bt[b, :len(t)] = t
        qs = np.concatenate([[0], np.cumsum([n for _, n in portions])])
        i32 = lambda v: torch.tensor(np.asarray(v), dtype=torch.int32, device=dev)  # noqa: E731
        return seq_ops.StepContext(tok_seq=i32(tok_seq), tok_pos=i32(tok_pos), qstart=i32(qs), seq_pos0=i32([p for p, _ in portions]),
                                   ctx_lens=i32([p + n for p, n in portions]), seq_slot=i32(list(range(len(portions)))),
                                   slot_mapping=i32(slot), block_tables=i32(bt), num_seqs=len(portions), num_tokens=int(qs[-1]),
                                   max_q=max(n for _, n in portions), block_size=bs, qstart_host=qs.tolist()), nxt
    pre, nblk_p = context([(0, seq)] * nseq)
    dec, nblk_d = context([(ctx - 1, 1)] * B)
    nblk = max(nblk_p, nblk_d)
    # ---- residual boundary: grouped norm of the result + add + the reader's copy | Pasizen: stream step, Lipelix: gated close
    x, y, pw, nw = torch.randn(T, width, device=dev), r(T, width), r(width), r(width)
    add("hm_group_norm_residual (T=%d)" % T, "hm_sublayer_close", _event_time(lambda: hy_ops.group_norm_residual(x, y, pw, 4, 1e-5, bf)),
        bytes_=T * width * (8 + 2 + 2))
    gate, gb = r(T, width), r(width)
    add("hm_sublayer_close (T=%d)" % T, "-", _event_time(lambda: hy_ops.sublayer_close(x, y, gate, gb, pw, 0.5, nw, 1e-5, bf)),
        bytes_=T * width * (8 + 2 + 2 + 2))
    # ---- q/k/v preparation: per-head norm with a shared weight row, per-head temperature | Lipelix: unit-norm heads + rotation
    kc, vc = r(nblk, bs, G, D), r(nblk, bs, G, D)
    qkv = r(T, (heads + 2 * G) * D)
    hw, temp = r(D), torch.rand(heads, device=dev) + 0.5
    add("hm_qkv_prepare (T=%d, head norm + temperature)" % T, "hm_qkv_prepare (unit norm)",
        _event_time(lambda: hy_ops.qkv_prepare(qkv, heads, G, D, D, None, None, 1e-5, None, False, pre, kc, vc, None, None, hw, hw, temp)),
        bytes_=T * (heads + 2 * G) * D * 4)
    inv_freq = hy_ops.rotary_inv_freq(64, 1e4, dev)
    add("hm_qkv_prepare (T=%d, unit norm)" % T, "-",
        _event_time(lambda: hy_ops.qkv_prepare(qkv, heads, G, D, D, None, None, 1e-5, inv_freq, True, pre, kc, vc, None, None)),
        bytes_=T * (heads + 2 * G) * D * 4)
    pr = hy_ops.pool_rows_per_page(bs, pool)
    kp, vp = r(nblk, pr, G, D), r(nblk, pr, G, D)
    add("hm_pool_blocks (T=%d, pool %d)" % (T, pool), "-", _event_time(lambda: hy_ops.pool_blocks(kc, vc, kp, vp, pool, pre)),
        bytes_=T * G * D * 4 + T // pool * G * D * 4)
    # ---- attention, prefill: window + pooled blocks | Lipelix: window + kept first tokens
    q = r(T, heads, D)
    wpairs = nseq * heads * sum(min(i + 1, window) + max(0, (i + 1 - window) // pool) for i in range(seq))
    add("hm_attn_tiles window %d + pooled %d (%dx%d)" % (window, pool, nseq, seq), "hm_attn_tiles window",
        _event_time(lambda: hy_ops.paged_attention(q, kc, vc, pre, 0.09, None, window, 0, pooled=(kp, vp, pool)), 5), flops=wpairs * 4 * D)
    sink = torch.randn(heads, device=dev)
    kpairs = nseq * heads * sum(min(i + 1, window) + min(4, max(0, i + 1 - window)) for i in range(seq))
    add("hm_attn_tiles window %d+4 kept (%dx%d)" % (window, nseq, seq), "-",
        _event_time(lambda: hy_ops.paged_attention(q, kc, vc, pre, 0.09, sink, window, 4), 5), flops=kpairs * 4 * D)
    # ---- attention, decode
    qd = r(B, heads, D)
    seen = max(0, (ctx - window) // pool)
    add("hm_attn_decode window %d + pooled %d (B=%d, ctx=%d)" % (window, pool, B, ctx), "hm_attn_decode window",
        _event_time(lambda: hy_ops.paged_attention(qd, kc, vc, dec, 0.09, None, window, 0, pooled=(kp, vp, pool))),
        bytes_=B * (window + seen) * G * D * 4)
    add("hm_attn_decode window %d+4 kept (B=%d, ctx=%d)" % (window, B, ctx), "-",
        _event_time(lambda: hy_ops.paged_attention(qd, kc, vc, dec, 0.09, sink, window, 4)), bytes_=B * (window + 4) * G * D * 4)
    # ---- latent side: norm + rotation + store | Pasizen: norm + store
    cache = r(nblk, bs, rank)
    qc = r(T, heads * (D + Rd) + rank)
    qa = r(T, heads, rank)
    lw = r(R)
    nq = heads * (D + Rd)
    add("sm_latent_rope_store (T=%d, H=%d)" % (T, heads), "sm_latent_norm_store",
        _event_time(lambda: seq_ops.latent_rope_store(qc[:, nq:], lw, 1e-5, qc[:, :nq], qa, inv_freq, Rd, heads, D, R, Rd, cache, pre)),
        bytes_=T * (rank * 4 + heads * Rd * 4))
    add("sm_latent_norm_store (T=%d)" % T, "-",
        _event_time(lambda: seq_ops.latent_norm_store(qc[:, nq:], nw[:rank].contiguous(), 1e-5, cache, pre.slot_mapping)), bytes_=T * rank * 4)
    lpairs = nseq * heads * sum(min(i + 1, window) for i in range(seq))
    add("sm_latent_attn_tiles window %d, row %d+%d (%dx%d, H=%d)" % (window, R, Rd, nseq, seq, heads), "sm_latent_attn_tiles",
        _event_time(lambda: seq_ops.latent_attention(qa, cache, pre, 0.09, value_cols=R, window=window), 5), flops=lpairs * 2 * (rank + R))
    pairs = nseq * seq * (seq + 1) / 2 * heads
    add("sm_latent_attn_tiles full, row %d (%dx%d, H=%d)" % (rank, nseq, seq, heads), "-",
        _event_time(lambda: seq_ops.latent_attention(qa, cache, pre, 0.09), 5), flops=pairs * 4 * rank)
    qad = r(B, heads, rank)
    add("sm_latent_attn_decode window %d, row %d+%d (B=%d, ctx=%d)" % (window, R, Rd, B, ctx), "sm_latent_attn_decode",
        _event_time(lambda: seq_ops.latent_attention(qad, cache, dec, 0.09, value_cols=R, window=window)), bytes_=B * window * rank * 2)
    add("sm_latent_attn_decode full, row %d (B=%d, ctx=%d)" % (rank, B, ctx), "-",
        _event_time(lambda: seq_ops.latent_attention(qad, cache, dec, 0.09)), bytes_=B * ctx * rank * 2)
    # ---- router and experts: sigmoid + correction + no renormalisation, GELU experts | Pasizen: softmax, clamped GLU
    E, top, F = 16, 4, ff // 4
    h = r(T, width)
    rw, corr = torch.randn(E, width, device=dev), torch.randn(E, device=dev) * 0.1
    add("sm_moe_route sigmoid + correction (T=%d, E=%d)" % (T, E), "sm_moe_route softmax",
        _event_time(lambda: seq_ops.moe_route(h, rw, top, 4, 2, seq_ops.ROUTE_SIGMOID, corr, 2, False)), bytes_=T * width * 2)
    add("sm_moe_route softmax (T=%d, E=%d)" % (T, E), "-", _event_time(lambda: seq_ops.moe_route(h, rw, top, 4, 2)), bytes_=T * width * 2)
    idx, wts = seq_ops.moe_route(h, rw, top, 4, 2, seq_ops.ROUTE_SIGMOID, corr, 2, False)
    w_up, w_gu, w_down = r(E, F, width), r(E, 2 * F, width), r(E, width, F)
    t_gelu = (seq_ops.tile_expert_weights(w_up, 1), seq_ops.tile_expert_weights(w_down))
    t_glu = (seq_ops.tile_expert_weights(w_gu, 2), t_gelu[1])
    add("sm_moe_tiles128 GELU experts (T=%d, top %d of %d, F=%d)" % (T, top, E, F), "sm_moe_tiles128 clamped GLU",
        _event_time(lambda: seq_ops.moe_experts(h, idx, wts, w_up, w_down, 0.0, form="tiles128", tiled=t_gelu, act_kind=seq_ops.ACT_GELU), 5),
        flops=T * top * 4 * width * F)
    add("sm_moe_tiles128 clamped GLU (T=%d)" % T, "-",
        _event_time(lambda: seq_ops.moe_experts(h, idx, wts, w_gu, w_down, 7.0, form="tiles128", tiled=t_glu), 5), flops=T * top * 6 * width * F)
    hd = h[:B].contiguous()
    idx_d, wts_d = seq_ops.moe_route(hd, rw, top, 4, 2, seq_ops.ROUTE_SIGMOID, corr, 2, False)
    touched = len(torch.unique(idx_d))
    add("sm_moe_grouped GELU experts (T=%d: decode)" % B, "sm_moe_grouped clamped GLU",
        _event_time(lambda: seq_ops.moe_experts(hd, idx_d, wts_d, w_up, w_down, 0.0, form="grouped", tiled=t_gelu, act_kind=seq_ops.ACT_GELU)),
        bytes_=touched * 2 * F * width * 2)
    add("sm_moe_grouped clamped GLU (T=%d: decode)" % B, "-",
        _event_time(lambda: seq_ops.moe_experts(hd, idx_d, wts_d, w_gu, w_down, 7.0, form="grouped", tiled=t_glu)),
        bytes_=touched * 3 * F * width * 2)
    lg = torch.randn(B, VOCAB, device=dev)
    add("hm_scale_softcap (B=%d, vocab %d)" % (B, VOCAB), "-", _event_time(lambda: hy_ops.scale_softcap_(lg, 1.0, 30.0)), bytes_=B * VOCAB * 8)
    return rows


def lilevik_kernel_table(width=2048, heads=16, rank=256, ff=6144, T=8192, seq=1024, B=64, ctx=1024, chunk=512):
    """Seconds per launch of every kernel form the Lilevik family runs at a layer's size, its bound and the fraction of it
    reached; beside each the form of the like kernel that the closest existing family runs (`like`): Galupel's for the
    residual boundary, attention, latent side, router and experts, Lipelix's for the recurrence."""
    from nanovllm import hy_ops, seq_ops
    dev, bf = "cuda", torch.bfloat16
    rows = []

    def add(name, like, sec, bytes_=0, flops=0, peak=MFMA_TFLOPS):
        bound = max(bytes_ / (HBM_GBPS * 1e9), flops / (peak * 1e12))
        rows.append(dict(kernel=name, like=like, us=round(sec * 1e6, 1), bound_us=round(bound * 1e6, 1),
                         of_roofline=round(bound / sec, 3), bound="flops" if flops / (peak * 1e12) > bytes_ / (HBM_GBPS * 1e9) else "bytes"))
    r = lambda *s: torch.randn(*s, device=dev).to(bf)  # noqa: E731
    nseq, bs, G, D, Rd = T // seq, 64, heads // 2, 128, 64
    R = rank - Rd
    import numpy as np

    def context(portions):
        tables, nxt = [], 0
        for p0, n in portions:
            nb = (p0 + n + bs - 1) // bs
            tables.append(list(range(nxt, nxt + nb)))
            nxt += nb
        tok_seq = np.concatenate([np.full(n, b) for b, (_, n) in enumerate(portions)])
        tok_pos = np.concatenate([np.arange(p0, p0 + n) for p0, n in portions])
        slot = np.concatenate([np.asarray(tables[b])[np.arange(p0, p0 + n) // bs] * bs + np.arange(p0, p0 + n) % bs
                               for b, (p0, n) in enumerate(portions)])
        mb = max(len(t) for t in tables)
        bt = np.zeros((len(portions), mb), dtype=np.int32)
        for b, t in enumerate(tables):
            bt[b, :len(t)] = t
        qs = np.concatenate([[0], np.cumsum([n for _, n in portions])])
        i32 = lambda v: torch.tensor(np.asarray(v), dtype=torch.int32, device=dev)  # noqa: E731
        return seq_ops.StepContext(tok_seq=i32(tok_seq), tok_pos=i32(tok_pos), qstart=i32(qs), seq_pos0=i32([p for p, _ in portions]),
                                   ctx_lens=i32([p + n for p, n in portions]), seq_slot=i32(list(range(len(portions)))),
                                   slot_mapping=i32(slot), block_tables=i32(bt), num_seqs=len(portions), num_tokens=int(qs[-1]),
                                   max_q=max(n for _, n in portions), block_size=bs, qstart_host=qs.tolist()), nxt
    pre, nblk_p = context([(0, seq)] * nseq)
    dec, nblk_d = context([(ctx - 1, 1)] * B)
    nblk = max(nblk_p, nblk_d)
    # ---- residual boundary: tanh norm of the result + add + the next tanh norm | Galupel: grouped RMS norms
    x, y = torch.randn(T, width, device=dev), r(T, width)
    n1, n2 = (r(width), r(width), torch.rand(1, device=dev)), (r(width), r(width), torch.rand(1, device=dev))
    add("hm_dyt_residual (T=%d)" % T, "hm_group_norm_residual", _event_time(lambda: hy_ops.dyt_residual(x, y, n1, n2, bf)),
        bytes_=T * width * (8 + 2 + 2))
    pw, nw = r(width), r(width)
    add("hm_group_norm_residual (T=%d)" % T, "-", _event_time(lambda: hy_ops.group_norm_residual(x, y, pw, 4, 1e-5, bf, next_w=nw)),
        bytes_=T * width * (8 + 2 + 2))
    # ---- q/k/v preparation: whole-projection norms, interleaved rotation, unit-RMS values | Galupel: per-head norm + temperature
    kc, vc = r(nblk, bs, G, D), r(nblk, bs, G, D)
    qkv = r(T, (heads + 2 * G) * D)
    qn, kn = r(heads * D), r(G * D)
    inv_freq, mag = hy_ops.rotary_table(64, 1e4, dev, dict(factor=4.0, original=2048, fast=32.0, slow=1.0))
    add("hm_qkv_prepare (T=%d, projection norm + interleaved rotation + unit values)" % T, "hm_qkv_prepare (head norm + temperature)",
        _event_time(lambda: hy_ops.qkv_prepare(qkv, heads, G, D, D, qn, kn, 1e-5, inv_freq, False, pre, kc, vc, interleaved=True,
                                               rot_mag=mag, v_unit_norm=True)), bytes_=T * (heads + 2 * G) * D * 4)
    hw, temp = r(D), torch.rand(heads, device=dev) + 0.5
    add("hm_qkv_prepare (T=%d, head norm + temperature)" % T, "-",
        _event_time(lambda: hy_ops.qkv_prepare(qkv, heads, G, D, D, None, None, 1e-5, None, False, pre, kc, vc, None, None, hw, hw, temp)),
        bytes_=T * (heads + 2 * G) * D * 4)
    # ---- attention, prefill: chunked mask + sigmoid weights | Galupel: window + pooled blocks in a softmax
    q = r(T, heads, D)
    hb = torch.randn(heads, device=dev) - 2.0
    cpairs = nseq * heads * sum(i % chunk + 1 for i in range(seq))
    add("hm_attn_tiles chunk %d, sigmoid (%dx%d)" % (chunk, nseq, seq), "hm_attn_tiles window + pooled",
        _event_time(lambda: hy_ops.paged_attention(q, kc, vc, pre, 0.09, chunk=chunk, sigmoid=True, head_bias=hb), 5), flops=cpairs * 4 * D)
    pool = 64
    pr = hy_ops.pool_rows_per_page(bs, pool)
    kp, vp = r(nblk, pr, G, D), r(nblk, pr, G, D)
    wpairs = nseq * heads * sum(min(i + 1, chunk) + max(0, (i + 1 - chunk) // pool) for i in range(seq))
    add("hm_attn_tiles window %d + pooled %d (%dx%d)" % (chunk, pool, nseq, seq), "-",
        _event_time(lambda: hy_ops.paged_attention(q, kc, vc, pre, 0.09, None, chunk, 0, pooled=(kp, vp, pool)), 5), flops=wpairs * 4 * D)
    # ---- attention, decode
    qd = r(B, heads, D)
    in_chunk = (ctx - 1) % chunk + 1
    add("hm_attn_decode chunk %d, sigmoid (B=%d, ctx=%d: %d keys)" % (chunk, B, ctx, in_chunk), "hm_attn_decode window + pooled",
        _event_time(lambda: hy_ops.paged_attention(qd, kc, vc, dec, 0.09, chunk=chunk, sigmoid=True, head_bias=hb)),
        bytes_=B * in_chunk * G * D * 4)
    seen = max(0, (ctx - chunk) // pool)
    add("hm_attn_decode window %d + pooled %d (B=%d, ctx=%d)" % (chunk, pool, B, ctx), "-",
        _event_time(lambda: hy_ops.paged_attention(qd, kc, vc, dec, 0.09, None, chunk, 0, pooled=(kp, vp, pool))),
        bytes_=B * (chunk + seen) * G * D * 4)
    # ---- lightning recurrence | Lipelix: delta rule (heads of 64 over the width).  Both states are float32 by design, so the
    # arithmetic of a step (4 D V flops per token and head here, 10 D^2 there) is priced at the float32 vector peak
    LH = width // 128
    proj = r(T, 4 * LH * 128)
    decay = torch.rand(LH, device=dev) * 0.1 + 0.9
    state = torch.zeros(max(nseq, B), LH, 128, 128, device=dev)
    add("hm_lightning_recurrence prefill (%dx%d, %d heads of 128x128)" % (nseq, seq, LH), "hm_delta_recurrence prefill",
        _event_time(lambda: hy_ops.lightning_recurrence(proj, 0, LH * 128, 2 * LH * 128, LH, 128, 128, decay, state, pre), 5),
        bytes_=T * LH * 128 * (3 * 2 + 4) + nseq * LH * 128 * 128 * 8, flops=T * LH * 4 * 128 * 128, peak=VALU_F32_TFLOPS)
    projd = proj[:B].contiguous()
    add("hm_lightning_recurrence decode (B=%d)" % B, "hm_delta_recurrence decode",
        _event_time(lambda: hy_ops.lightning_recurrence(projd, 0, LH * 128, 2 * LH * 128, LH, 128, 128, decay, state, dec)),
        bytes_=B * LH * 128 * 128 * 8)
    DH = width // 64
    prep, vd = torch.rand(T, DH, 5, 64, device=dev), r(T, DH * 64)
    dstate = torch.zeros(max(nseq, B), DH, 64, 64, device=dev)
    add("hm_delta_recurrence prefill (%dx%d, %d heads of 64)" % (nseq, seq, DH), "-",
        _event_time(lambda: hy_ops.delta_recurrence(prep, vd, dstate, pre), 3), bytes_=T * DH * 64 * (5 * 4 + 2 + 4) + nseq * DH * 64 * 64 * 8,
        flops=T * DH * 10 * 64 * 64, peak=VALU_F32_TFLOPS)
    prepd, vdd = prep[:B].contiguous(), vd[:B].contiguous()
    add("hm_delta_recurrence decode (B=%d)" % B, "-", _event_time(lambda: hy_ops.delta_recurrence(prepd, vdd, dstate, dec)),
        bytes_=B * DH * 64 * 64 * 8)
    o, gcol, ow = torch.randn(T, LH, 128, device=dev), r(T, LH * 128), r(LH * 128)
    add("hm_delta_gate_norm over all heads (T=%d)" % T, "hm_delta_gate_norm per head",
        _event_time(lambda: hy_ops.delta_gate_norm(o.view(T, 1, LH * 128), gcol, ow, 1e-5, bf)), bytes_=T * LH * 128 * (4 + 2 + 2))
    add("hm_delta_gate_norm per head (T=%d)" % T, "-", _event_time(lambda: hy_ops.delta_gate_norm(o, gcol, ow, 1e-5, bf)),
        bytes_=T * LH * 128 * (4 + 2 + 2))
    # ---- latent side: the query latent's norm; norm + rotation + store; attention without a window | Galupel: window 512
    Q = 3 * rank
    cache = r(nblk, bs, rank)
    first = r(T, Q + rank)
    qw = r(Q)
    add("sm_rms_norm_rows query latent (T=%d, %d)" % (T, Q), "sm_latent_norm_store",
        _event_time(lambda: seq_ops.rms_norm_rows(first[:, :Q], qw, 1e-5)), bytes_=T * Q * 4)
    lw, cache_r = r(R), r(nblk, bs, R)
    add("sm_latent_norm_store (T=%d)" % T, "-",
        _event_time(lambda: seq_ops.latent_norm_store(first[:, Q:Q + R], lw, 1e-5, cache_r, pre.slot_mapping)), bytes_=T * R * 4)
    q2, qa = r(T, heads * (D + Rd)), r(T, heads, rank)
    rf = hy_ops.rotary_inv_freq(64, 1e4, dev)
    add("sm_latent_rope_store (T=%d, H=%d)" % (T, heads), "(the same form as Galupel's)",
        _event_time(lambda: seq_ops.latent_rope_store(first[:, Q:], lw, 1e-5, q2, qa, rf, Rd, heads, D, R, Rd, cache, pre)),
        bytes_=T * (rank * 4 + heads * Rd * 4))
    pairs = nseq * seq * (seq + 1) / 2 * heads
    add("sm_latent_attn_tiles full, row %d+%d (%dx%d, H=%d)" % (R, Rd, nseq, seq, heads), "sm_latent_attn_tiles window",
        _event_time(lambda: seq_ops.latent_attention(qa, cache, pre, 0.09, value_cols=R), 5), flops=pairs * 2 * (rank + R))
    lpairs = nseq * heads * sum(min(i + 1, chunk) for i in range(seq))
    add("sm_latent_attn_tiles window %d, row %d+%d" % (chunk, R, Rd), "-",
        _event_time(lambda: seq_ops.latent_attention(qa, cache, pre, 0.09, value_cols=R, window=chunk), 5), flops=lpairs * 2 * (rank + R))
    qad = r(B, heads, rank)
    add("sm_latent_attn_decode full, row %d+%d (B=%d, ctx=%d)" % (R, Rd, B, ctx), "sm_latent_attn_decode window",
        _event_time(lambda: seq_ops.latent_attention(qad, cache, dec, 0.09, value_cols=R)), bytes_=B * ctx * rank * 2)
    add("sm_latent_attn_decode window %d, row %d+%d" % (chunk, R, Rd), "-",
        _event_time(lambda: seq_ops.latent_attention(qad, cache, dec, 0.09, value_cols=R, window=chunk)), bytes_=B * chunk * rank * 2)
    # ---- router and experts: biased logits, softmax over the chosen, SiLU-gated experts | Galupel: sigmoid + correction, GELU
    E, top, F = 16, 4, ff // 4
    h = r(T, width)
    rw, rb = torch.randn(E, width, device=dev), torch.randn(E, device=dev) * 0.1
    add("sm_moe_route softmax + bias (T=%d, E=%d)" % (T, E), "sm_moe_route sigmoid + correction",
        _event_time(lambda: seq_ops.moe_route(h, rw, top, bias=rb)), bytes_=T * width * 2)
    add("sm_moe_route sigmoid + correction (T=%d, E=%d)" % (T, E), "-",
        _event_time(lambda: seq_ops.moe_route(h, rw, top, 4, 2, seq_ops.ROUTE_SIGMOID, rb, 2, False)), bytes_=T * width * 2)
    idx, wts = seq_ops.moe_route(h, rw, top, bias=rb)
    w_up, w_gu, w_down = r(E, F, width), r(E, 2 * F, width), r(E, width, F)
    t_gelu = (seq_ops.tile_expert_weights(w_up, 1), seq_ops.tile_expert_weights(w_down))
    t_glu = (seq_ops.tile_expert_weights(w_gu, 2), t_gelu[1])
    inf = float("inf")
    add("sm_moe_tiles128 SiLU-gated experts (T=%d, top %d of %d, F=%d)" % (T, top, E, F), "sm_moe_tiles128 GELU experts",
        _event_time(lambda: seq_ops.moe_experts(h, idx, wts, w_gu, w_down, inf, 1.0, form="tiles128", tiled=t_glu, act_kind=seq_ops.ACT_SILU_GLU), 5),
        flops=T * top * 6 * width * F)
    add("sm_moe_tiles128 GELU experts (T=%d)" % T, "-",
        _event_time(lambda: seq_ops.moe_experts(h, idx, wts, w_up, w_down, 0.0, form="tiles128", tiled=t_gelu, act_kind=seq_ops.ACT_GELU), 5),
        flops=T * top * 4 * width * F)
    hd = h[:B].contiguous()
    idx_d, wts_d = seq_ops.moe_route(hd, rw, top, bias=rb)
    touched = len(torch.unique(idx_d))
    add("sm_moe_grouped SiLU-gated experts (T=%d: decode)" % B, "sm_moe_grouped GELU experts",
        _event_time(lambda: seq_ops.moe_experts(hd, idx_d, wts_d, w_gu, w_down, inf, 1.0, form="grouped", tiled=t_glu, act_kind=seq_ops.ACT_SILU_GLU)),
        bytes_=touched * 3 * F * width * 2)
    add("sm_moe_grouped GELU experts (T=%d: decode)" % B, "-",
        _event_time(lambda: seq_ops.moe_experts(hd, idx_d, wts_d, w_up, w_down, 0.0, form="grouped", tiled=t_gelu, act_kind=seq_ops.ACT_GELU)),
        bytes_=touched * 2 * F * width * 2)
    return rows


def main(sizes=("w1024", "w2048"), kernels=True, family="pasizen"):
    out = dict(metric="family comparison", dtype="bf16", data="synthetic (random weights)", throughput=[], kernels=[])
    beside = {"galupel": ("pasizen", "qwen3"), "lilevik": ("galupel", "lipelix", "qwen3")}.get(family, ("qwen3",))
    for size in sizes:
        for fam in (family,) + beside:
            out["throughput"].append(engine_throughput(fam, size))
    if kernels:
        out["kernels"] = {"pasizen": kernel_table, "galupel": galupel_kernel_table, "lilevik": lilevik_kernel_table}.get(
            family, hymix_kernel_table)()
    return out
