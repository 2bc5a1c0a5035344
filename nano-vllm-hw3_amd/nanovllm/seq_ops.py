"""Operators of libseqmix behind torch tensors: the mechanisms between the matrix products of a decoder whose layers
use multi-stream residuals, short convolutions, latent attention, PolyNorm / clamped-GLU feed-forwards and routed
experts.  One kernel launch each on the current stream.  CPU tensors go to plain-torch counterparts
(nanovllm/cpu_ops.py): engine plumbing on a host without a GPU, never a fallback for a GPU tensor."""
from dataclasses import dataclass
from typing import Optional

import torch

from nanovllm import _seqmix as SM
from nanovllm import cpu_ops


@dataclass
class StepContext:
    """What one engine step's kernels need to know about its batch: B sequences contribute portions of consecutive
    tokens (a single token when decoding), T tokens in all, packed sequence after sequence."""
    tok_seq: torch.Tensor          # int32 [T]  index of the token's sequence in this step
    tok_pos: torch.Tensor          # int32 [T]  position of the token in its sequence
    qstart: torch.Tensor           # int32 [B+1] first row of every sequence's portion
    seq_pos0: torch.Tensor         # int32 [B]  position of the portion's first token (= tokens already cached)
    ctx_lens: torch.Tensor         # int32 [B]  tokens cached after this step
    seq_slot: torch.Tensor         # int32 [B]  state slot of the sequence
    slot_mapping: torch.Tensor     # int32 [T]  cache row (block * block_size + offset) every token is stored at
    block_tables: torch.Tensor     # int32 [B, max_blocks]
    num_seqs: int = 0
    num_tokens: int = 0
    max_q: int = 0                 # longest portion
    block_size: int = 64
    qstart_host: Optional[list] = None


_STEP: Optional[StepContext] = None


def set_step(ctx):
    global _STEP
    _STEP = ctx


def get_step() -> StepContext:
    return _STEP


def _dev(t):
    return SM.stream_ptr(t.device)


def embed_streams(ids, positions, embed, pos_table, streams):
    """X f32 [T, S, W]: every stream starts as embed[id] + pos_table[position]."""
    T, W = ids.numel(), embed.shape[1]
    if not embed.is_cuda:
        return cpu_ops.embed_streams(ids, positions, embed, pos_table, streams)
    X = torch.empty((T, streams, W), dtype=torch.float32, device=embed.device)
    SM.check(SM.load().sm_embed_streams(SM.dtype_code(embed.dtype), ids.data_ptr(), positions.data_ptr(), embed.data_ptr(),
                                        SM.ptr(pos_table), X.data_ptr(), T, streams, W, _dev(embed)))
    return X


def stream_step(X, y, mix, out, w_in, norm_w, eps, dtype):
    """Write phase (y given): X <- mix^T X + out * y in place.  Read phase (w_in given): returns
    rms_norm(sum_s w_in[s] X[:, s]) * norm_w in ``dtype``."""
    T, S, W = X.shape
    if not X.is_cuda:
        return cpu_ops.stream_step(X, y, mix, out, w_in, norm_w, eps, dtype)
    h = torch.empty((T, W), dtype=dtype, device=X.device) if w_in is not None else None
    if y is not None:
        SM.require_cuda(y, dtype, "y")
    SM.check(SM.load().sm_stream_step(SM.dtype_code(dtype), X.data_ptr(), SM.ptr(y), SM.ptr(mix), SM.ptr(out), SM.ptr(w_in),
                                      SM.ptr(norm_w), eps, SM.ptr(h), T, S, W, _dev(X)))
    return h


def canon_conv(h, w, state, run, ctx: StepContext):
    """h + causal_conv(h) per channel with the sequence's carried inputs; then the state takes this step's last inputs.
    h [T, W], w [W, taps], state [slots, runs, taps-1, W]."""
    T, W = h.shape
    taps = w.shape[1]
    if not h.is_cuda:
        return cpu_ops.canon_conv(h, w, state, run, ctx)
    SM.require_cuda(h, w.dtype, "h")
    out = torch.empty_like(h)
    lib, code, runs = SM.load(), SM.dtype_code(h.dtype), state.shape[1]
    SM.check(lib.sm_canon_conv(code, h.data_ptr(), w.data_ptr(), state.data_ptr(), run, runs, ctx.tok_seq.data_ptr(),
                               ctx.tok_pos.data_ptr(), ctx.qstart.data_ptr(), ctx.seq_slot.data_ptr(), out.data_ptr(), T, W,
                               taps, _dev(h)))
    SM.check(lib.sm_canon_update(code, h.data_ptr(), state.data_ptr(), run, runs, ctx.qstart.data_ptr(),
                                 ctx.seq_slot.data_ptr(), ctx.num_seqs, W, taps, _dev(h)))
    return out


def latent_norm_store(x, w, eps, cache, slot_mapping):
    """x [T, R] (rows may be strided: a column slice of a wider product) -> rms_norm(x) * w stored at the rows of
    ``cache`` [blocks, block_size, R] named by slot_mapping."""
    T, R = x.shape
    if not x.is_cuda:
        return cpu_ops.latent_norm_store(x, w, eps, cache, slot_mapping)
    assert x.stride(1) == 1 and x.dtype == cache.dtype == w.dtype
    SM.check(SM.load().sm_latent_norm_store(SM.dtype_code(x.dtype), x.data_ptr(), x.stride(0), w.data_ptr(), eps,
                                            cache.data_ptr(), slot_mapping.data_ptr(), T, R, _dev(x)))


def rms_norm_rows(x, w, eps):
    """x [T, R] (rows may be a column slice of a wider product) -> x / sqrt(mean(x^2) + eps) * w, dense [T, R]."""
    if not x.is_cuda:
        return cpu_ops.rms_norm_rows(x, w, eps)
    assert x.stride(1) == 1 and x.dtype == w.dtype
    T, R = x.shape
    out = torch.empty((T, R), dtype=x.dtype, device=x.device)
    SM.check(SM.load().sm_rms_norm_rows(SM.dtype_code(x.dtype), x.data_ptr(), x.stride(0), w.data_ptr(), eps, out.data_ptr(), T, R,
                                        _dev(x)))
    return out


def latent_rope_store(x, w, eps, q, qa, inv_freq, rot_dims, H, D, R, Rd, cache, ctx: StepContext):
    """A latent with a rotated key part.  x [T, R + Rd] (rows may be a column slice): rms_norm(x[:, :R]) * w and x[:, R:]
    with its first rot_dims channels turned by position * inv_freq (channel 2i pairs with 2i + 1) are stored as the
    tokens' rows of ``cache`` [blocks, block_size, R + Rd].  q [T, H * (D + Rd)] (rows may be a slice): every head's last
    Rd channels, turned the same way, go to qa[:, :, R:] (qa [T, H, R + Rd]; its first R columns are the caller's)."""
    if not x.is_cuda:
        return cpu_ops.latent_rope_store(x, w, eps, q, qa, inv_freq, rot_dims, H, D, R, Rd, cache, ctx)
    T = x.shape[0]
    assert x.stride(1) == 1 and q.stride(1) == 1 and qa.is_contiguous() and x.dtype == cache.dtype == w.dtype == q.dtype == qa.dtype
    assert x.shape[1] == R + Rd and q.shape[1] == H * (D + Rd) and qa.shape == (T, H, R + Rd) and cache.shape[2] == R + Rd
    SM.check(SM.load().sm_latent_rope_store(SM.dtype_code(x.dtype), x.data_ptr(), x.stride(0), w.data_ptr(), eps, q.data_ptr(),
                                            q.stride(0), qa.data_ptr(), SM.ptr(inv_freq), rot_dims, ctx.tok_pos.data_ptr(),
                                            cache.data_ptr(), ctx.slot_mapping.data_ptr(), T, H, D, R, Rd, _dev(x)))


USE_TILES = True       # bf16 latent attention on the matrix cores where the shape allows (tests compare both forms)


def latent_attention(q, cache, ctx: StepContext, scale, force_rows=False, value_cols=0, window=0):
    """Absorbed queries q [T, H, R] over the paged latent cache [blocks, block_size, R], causal inside each sequence.
    A cache row is the key; its first ``value_cols`` columns are the value (0 = all of it) -> [T, H, value_cols or R].
    ``window`` > 0: the token at position i sees only the keys j with i - j < window."""
    T, H, R = q.shape
    RV = value_cols or R
    if not q.is_cuda:
        return cpu_ops.latent_attention(q, cache, ctx, scale, RV, window)
    SM.require_cuda(q, cache.dtype, "q")
    o = torch.empty((T, H, RV), dtype=q.dtype, device=q.device)
    lib = SM.load()
    bs, mb = cache.shape[1], ctx.block_tables.shape[1]
    tiles_ok = (USE_TILES and not force_rows and q.dtype == torch.bfloat16 and R % 8 == 0 and RV % 4 == 0 and R <= 256 and
                bs % 64 == 0)
    if tiles_ok and ctx.max_q == 1 and H <= 128:
        splits = decode_splits(ctx.num_seqs, min(mb * bs, window + 64) if window > 0 else mb * bs)
        ws, n = SM.decode_workspace.get(q.device, lib.sm_latent_decode_workspace_bytes(T, H, R, splits))
        SM.check(lib.sm_latent_attn_decode(q.data_ptr(), cache.data_ptr(), ctx.block_tables.data_ptr(), ctx.ctx_lens.data_ptr(),
                                           o.data_ptr(), scale, T, H, R, bs, mb, splits, ws, n, RV, int(window), _dev(q)))
    elif tiles_ok:
        SM.check(lib.sm_latent_attn_tiles(q.data_ptr(), cache.data_ptr(), ctx.block_tables.data_ptr(), ctx.qstart.data_ptr(),
                                          ctx.seq_pos0.data_ptr(), o.data_ptr(), scale, ctx.num_seqs, ctx.max_q, H, R, bs, mb,
                                          RV, int(window), _dev(q)))
    else:
        SM.check(lib.sm_latent_attn_rows(SM.dtype_code(q.dtype), q.data_ptr(), cache.data_ptr(), ctx.block_tables.data_ptr(),
                                         ctx.tok_seq.data_ptr(), ctx.tok_pos.data_ptr(), o.data_ptr(), scale, T, H, R, bs, mb,
                                         RV, int(window), _dev(q)))
    return o


def decode_splits(num_seqs, max_keys):
    """Key splits of decode attention: about four workgroups per CU, at least two 64-key tiles per split.  Depends only on
    the batch size and the cache geometry, never on the sequences' lengths, so a result does not move with them."""
    want = max(1, 1024 // max(1, num_seqs))
    return int(max(1, min(want, (max_keys + 127) // 128, 64)))


def poly_norm(z, coef, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e per row; coef = f32 [4] = a, b, c, e."""
    if not z.is_cuda:
        return cpu_ops.poly_norm(z, coef, eps)
    SM.require_cuda(z, None, "z")
    out = torch.empty_like(z)
    SM.check(SM.load().sm_poly_norm(SM.dtype_code(z.dtype), z.data_ptr(), coef.data_ptr(), eps, out.data_ptr(),
                                    z.shape[0], z.shape[1], _dev(z)))
    return out


def clamped_glu(gu, limit, alpha=1.702):
    """gu [T, 2F] = gate | up -> min(g, limit) * sigmoid(alpha * min(g, limit)) * (clamp(u, +-limit) + 1)."""
    if not gu.is_cuda:
        return cpu_ops.clamped_glu(gu, limit, alpha)
    SM.require_cuda(gu, None, "gu")
    T, F2 = gu.shape
    out = torch.empty((T, F2 // 2), dtype=gu.dtype, device=gu.device)
    SM.check(SM.load().sm_clamped_glu(SM.dtype_code(gu.dtype), gu.data_ptr(), limit, alpha, out.data_ptr(), T, F2 // 2, _dev(gu)))
    return out


ROUTE_SOFTMAX, ROUTE_SIGMOID = 0, 1
ACT_CLAMPED_GLU, ACT_GELU, ACT_GELU_TANH, ACT_SILU_GLU = 0, 1, 2, 3
GATED_ACTS = (ACT_CLAMPED_GLU, ACT_SILU_GLU)      # experts with gate and up rows


def moe_route(h, router_w, top, groups=1, keep=1, score=ROUTE_SOFTMAX, correction=None, group_top=1, renorm=True, bias=None):
    """Router with group-limited top-k: (idx int32 [T, top], weights f32 [T, top]); router_w f32 [E, W].  Scores are the
    softmax or the sigmoid of the float32 logits; ``correction`` f32 [E] is added for the CHOICE only (groups and
    experts), the weights stay the scores; a group scores the sum of its ``group_top`` largest choice scores (1 = its
    maximum); ``renorm``: the chosen weights are divided by their sum.  ``bias`` f32 [E] is added to the logits (softmax
    scores with ``renorm`` are then the softmax over the chosen experts' logits)."""
    if not h.is_cuda:
        return cpu_ops.moe_route(h, router_w, top, groups, keep, score, correction, group_top, renorm, bias)
    if bias is not None:
        SM.require_cuda(bias, torch.float32, "bias")
    if correction is not None:
        SM.require_cuda(correction, torch.float32, "correction")
    SM.require_cuda(h, None, "h")
    SM.require_cuda(router_w, torch.float32, "router_w")
    T, W = h.shape
    E = router_w.shape[0]
    idx = torch.empty((T, top), dtype=torch.int32, device=h.device)
    wts = torch.empty((T, top), dtype=torch.float32, device=h.device)
    SM.check(SM.load().sm_moe_route(SM.dtype_code(h.dtype), h.data_ptr(), router_w.data_ptr(), idx.data_ptr(), wts.data_ptr(),
                                    T, W, E, top, groups, keep, int(score), SM.ptr(correction), int(group_top), int(bool(renorm)),
                                    SM.ptr(bias), _dev(h)))
    return idx, wts


TILES128_MIN_ROWS_PER_EXPERT = 64


def tile_expert_weights(w, parts=1):
    """Expert weights [E, parts * N, K] (K contiguous) -> the layout the matrix-core expert kernels stream: blocks of
    32 rows x 64 k (4 KB) in the order (expert, part, row block, k step), inside a block chunk s (8 k) of lane L =
    32 hi + row at 16 (64 s + L) bytes with k = 64 step + 32 hi + 8 s: every load of a wave is one contiguous KB, where
    the row-major matrix would be touched in 32 pieces a row apart.  Rows and k are zero-padded to whole blocks."""
    E, PN, K = w.shape
    N = PN // parts
    NB, KS = (N + 31) // 32, (K + 63) // 64
    x = torch.nn.functional.pad(w.view(E, parts, N, K), (0, KS * 64 - K, 0, NB * 32 - N))
    x = x.view(E, parts, NB, 32, KS, 2, 4, 8).permute(0, 1, 2, 4, 6, 5, 3, 7)      # [E, parts, NB, KS, s, hi, row, 8]
    return x.contiguous()


def moe_experts(h, idx, wts, w_gu, w_down, limit, alpha=1.702, shared=None, form=None, tiled=None, act_kind=ACT_CLAMPED_GLU):
    """y[t] = sum_k wts[t, k] * expert_{idx[t, k]}(h[t]) (+ shared[t]); w_gu [E, 2F, W] (gate rows then up rows),
    w_down [E, W, F]; an expert is a clamped GLU between its two products.  ``form``: "pairs" | "grouped" | "tiles128"
    forces one; by default float32 runs pair by pair and bf16 grouped by expert on the matrix cores, in tiles of 32 rows
    for small groups (decode) and of 128 rows for large ones (prefill).  ``tiled`` = (tile_expert_weights(w_gu, 2),
    tile_expert_weights(w_down)), what the grouped forms read (made here when the caller does not keep them).
    ``act_kind`` = ACT_GELU / ACT_GELU_TANH: an expert is down(gelu(up h)) instead, w_gu is [E, F, W] (tiled in one part);
    ACT_SILU_GLU: the gated form g sigmoid(alpha g) u without the one and, with limit = inf and alpha = 1, silu(gate) * up."""
    if not h.is_cuda:
        return cpu_ops.moe_experts(h, idx, wts, w_gu, w_down, limit, alpha, shared, act_kind)
    parts = 2 if act_kind in GATED_ACTS else 1
    assert w_gu.shape[1] == parts * w_down.shape[2]
    SM.require_cuda(h, w_gu.dtype, "h")
    T, W = h.shape
    top, F = idx.shape[1], w_down.shape[2]
    E = w_gu.shape[0]
    lib, code = SM.load(), SM.dtype_code(h.dtype)
    can_group = h.dtype == torch.bfloat16 and W % 8 == 0 and F % 8 == 0
    if form is None:
        # groups of 64 rows and more on average fill 128-row tiles well enough to pay for their padding
        form = "pairs" if not can_group else ("tiles128" if T * top >= TILES128_MIN_ROWS_PER_EXPERT * E else "grouped")
    if form in ("grouped", "tiles128"):
        assert can_group
        rows = 32 if form == "grouped" else 128
        n = lib.sm_moe_grouped_tiles(T, top, E) if form == "grouped" else lib.sm_moe_tiles128_count(T, top, E)
        ints = torch.empty(rows * n + n + T * top, dtype=torch.int32, device=h.device)
        row_pair, tile_expert, pair_row = ints[:rows * n], ints[rows * n:rows * n + n], ints[rows * n + n:]
        y = torch.empty_like(h)
        prod = torch.empty((rows * n, W), dtype=h.dtype, device=h.device)
        act = torch.empty((rows * n, F), dtype=h.dtype, device=h.device)
        fn = lib.sm_moe_grouped if form == "grouped" else lib.sm_moe_tiles128
        t_gu, t_down = tiled if tiled is not None else (tile_expert_weights(w_gu, parts), tile_expert_weights(w_down))
        SM.check(fn(h.data_ptr(), idx.data_ptr(), wts.data_ptr(), t_gu.data_ptr(), t_down.data_ptr(), SM.ptr(shared), limit, alpha,
                    int(act_kind), y.data_ptr(), T, top, E, W, F, row_pair.data_ptr(), tile_expert.data_ptr(), pair_row.data_ptr(),
                    act.data_ptr(), prod.data_ptr(), _dev(h)))
        return y
    assert form == "pairs", form
    act = torch.empty((T * top, F), dtype=h.dtype, device=h.device)
    y = torch.empty_like(h)
    SM.check(lib.sm_moe_pairs_gate_up(code, h.data_ptr(), idx.data_ptr(), w_gu.data_ptr(), limit, alpha, int(act_kind),
                                      act.data_ptr(), T, top, W, F, _dev(h)))
    SM.check(lib.sm_moe_pairs_down(code, act.data_ptr(), idx.data_ptr(), wts.data_ptr(), w_down.data_ptr(), SM.ptr(shared),
                                   y.data_ptr(), T, top, W, F, _dev(h)))
    return y
