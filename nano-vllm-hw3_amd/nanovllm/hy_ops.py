"""Operators of libhymix behind torch tensors: what sits between the matrix products of a decoder that mixes rotary
attention layers (sinks, sliding windows with kept first tokens, value mixing between layers) with delta-rule recurrent
layers, on a float32 residual whose sublayers are normalised on both sides, gated, and read a token-shifted input.
One kernel launch each on the current stream; the step's batch is a nanovllm.seq_ops.StepContext.  CPU tensors go to
plain-torch counterparts (nanovllm/cpu_ops.py): engine plumbing on a host without a GPU, never a fallback for a GPU tensor."""
import torch

from nanovllm import _hymix as HM
from nanovllm import cpu_ops
from nanovllm.seq_ops import StepContext


def _dev(t):
    return HM.stream_ptr(t.device)


def _rows(t, name):
    """A matrix whose rows may be a column slice of a wider product: unit stride inside a row."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise HM.QLinearError(f"{name} must be a matrix with contiguous rows")
    return t


def embed_scaled(ids, embed, scale):
    """x f32 [T, W] = embed[id] * scale."""
    if not embed.is_cuda:
        return cpu_ops.embed_scaled(ids, embed, scale)
    T, W = ids.numel(), embed.shape[1]
    x = torch.empty((T, W), dtype=torch.float32, device=embed.device)
    HM.check(HM.load().hm_embed_scaled(HM.dtype_code(embed.dtype), ids.data_ptr(), embed.data_ptr(), float(scale), x.data_ptr(),
                                       T, W, _dev(embed)))
    return x


def sublayer_close(x, y, gate, gate_bias, post_w, mult, next_w, eps, dtype, carry=None):
    """The boundary between two sublayers on a float32 residual x [T, W], per token in one launch:
      y given:      x <- x + mult * rms_norm(y * sigmoid(gate + gate_bias)) * post_w      (gate: pre-activation, rows may
                    be a column slice of a wider product)
      next_w given: returns rms_norm(x) * next_w in ``dtype`` (the next sublayer's input)
      carry = (src [T, W], state [slots, layers, W], layer, ctx): state[slot of the sequence, layer] <- src[last token of
                    the sequence's portion] (what a token shift of that layer reads at the next step)."""
    if not x.is_cuda:
        return cpu_ops.sublayer_close(x, y, gate, gate_bias, post_w, mult, next_w, eps, dtype, carry)
    T, W = x.shape
    h = torch.empty((T, W), dtype=dtype, device=x.device) if next_w is not None else None
    if y is not None:
        HM.require_cuda(y, dtype, "y")
        _rows(gate, "gate")
    src = state = None
    tok_seq = qstart = seq_slot = None
    slot_stride = 0
    if carry is not None:
        src, st, layer, ctx = carry
        HM.require_cuda(src, dtype, "carry source")
        assert st.dtype == dtype and st.is_contiguous() and st.shape[2] == W
        state, slot_stride = st[:, layer], st.stride(0)
        tok_seq, qstart, seq_slot = ctx.tok_seq, ctx.qstart, ctx.seq_slot
    HM.check(HM.load().hm_sublayer_close(HM.dtype_code(dtype), x.data_ptr(), HM.ptr(y), HM.ptr(gate),
                                         gate.stride(0) if gate is not None else 0, HM.ptr(gate_bias), HM.ptr(post_w), float(mult),
                                         HM.ptr(next_w), float(eps), HM.ptr(h), HM.ptr(src), HM.ptr(state), slot_stride,
                                         HM.ptr(tok_seq), HM.ptr(qstart), HM.ptr(seq_slot), T, W, _dev(x)))
    return h


def token_shift(h, mu, state, layer, ctx: StepContext):
    """h [T, W] -> h + (h_prev - h) * mu, h_prev = the previous token's h: the row above inside a portion, the sequence's
    carried row state[slot, layer] at a portion's start, zero at position 0 (a slot is never cleared)."""
    if not h.is_cuda:
        return cpu_ops.token_shift(h, mu, state, layer, ctx)
    HM.require_cuda(h, mu.dtype, "h")
    T, W = h.shape
    out = torch.empty_like(h)
    st = state[:, layer]
    HM.check(HM.load().hm_token_shift(HM.dtype_code(h.dtype), h.data_ptr(), mu.data_ptr(), st.data_ptr(), state.stride(0),
                                      ctx.tok_seq.data_ptr(), ctx.tok_pos.data_ptr(), ctx.qstart.data_ptr(),
                                      ctx.seq_slot.data_ptr(), out.data_ptr(), T, W, _dev(h)))
    return out


def rotary_inv_freq(dims, base, device):
    """f_i = base^(-2i/dims), i < dims/2, evaluated in float64 and kept in float32."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / dims)).to(torch.float32).to(device)


def rotary_table(dims, base, device, scaling=None):
    """(frequencies f32 [dims/2], factor on every cosine and sine).  Without ``scaling``: f_i = base^(-2i/dims) and 1.
    ``scaling`` = {factor, original, fast, slow} stretches the table for contexts longer than ``original`` positions: a
    pair that makes fewer than ``slow`` turns over ``original`` positions has its frequency divided by ``factor``, one that
    makes more than ``fast`` turns keeps it, and between them a linear ramp over the pair index blends the two (the ramp
    runs from pair lo = floor(d(fast)) to hi = ceil(d(slow)), d(t) = dims ln(original / (2 pi t)) / (2 ln base), clamped
    to the table); cosines and sines grow by 0.1 ln(factor) + 1.  Evaluated in float64, kept in float32."""
    import math
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    mag = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])

        def pair_of(turns):
            return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(float(base)))
        lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32).to(device), mag


def qkv_prepare(qkv, H, G, D, V, q_norm_w, k_norm_w, eps, inv_freq, unit_norm, ctx: StepContext, k_cache, v_cache,
                v_first=None, lam=None, q_head_w=None, k_head_w=None, q_head_scale=None, interleaved=False, rot_mag=1.0,
                v_unit_norm=False):
    """From the merged product qkv [T, H*D + G*D + G*V] of a step's tokens, in one launch per token:
      q_norm_w / k_norm_w given: RMS norm over the WHOLE q (k) projection with that weight;
      rotation of the first 2 * len(inv_freq) channels of every q and k head by position * inv_freq (channel i paired
      with channel i + len(inv_freq)), angles in float32;
      unit_norm: every rotated head of q and k divided by its RMS;
      v_first given: v <- (1 - lam) v + lam v_first (lam: float32 scalar on the device);
      k and v are stored at the tokens' cache rows; returns q [T, H, D].
    q_head_w / k_head_w [D]: before the rotation every q (k) head is divided by its own RMS and multiplied by that row,
    shared by the heads; q_head_scale f32 [H]: query head h times its number after that.  inv_freq None: no rotation.
    k_cache None: qkv holds q only [T, H*D] (the layer reads another layer's keys and values); nothing is stored.
    interleaved: channel 2i pairs with 2i + 1 instead; rot_mag multiplies every cosine and sine; v_unit_norm: every value
    head is divided by its RMS (no weight) before it is stored."""
    if not qkv.is_cuda:
        return cpu_ops.qkv_prepare(qkv, H, G, D, V, q_norm_w, k_norm_w, eps, inv_freq, unit_norm, ctx, k_cache, v_cache,
                                   v_first, lam, q_head_w, k_head_w, q_head_scale, interleaved, rot_mag, v_unit_norm)
    _rows(qkv, "qkv")
    T = qkv.shape[0]
    if k_cache is None:
        assert qkv.shape[1] == H * D and v_cache is None
    else:
        assert qkv.shape[1] == H * D + G * D + G * V and k_cache.dtype == v_cache.dtype == qkv.dtype
        assert k_cache.shape[2:] == (G, D) and v_cache.shape[2:] == (G, V)
    assert inv_freq is None or inv_freq.dtype == torch.float32
    assert q_head_scale is None or q_head_scale.dtype == torch.float32
    if v_first is not None:
        _rows(v_first, "v_first")
        assert v_first.shape == (T, G * V) and lam.dtype == torch.float32
    q = torch.empty((T, H, D), dtype=qkv.dtype, device=qkv.device)
    HM.check(HM.load().hm_qkv_prepare(HM.dtype_code(qkv.dtype), qkv.data_ptr(), qkv.stride(0), H, G, D, V, HM.ptr(q_norm_w),
                                      HM.ptr(k_norm_w), float(eps), HM.ptr(inv_freq), inv_freq.numel() if inv_freq is not None else 0,
                                      int(bool(unit_norm)), ctx.tok_pos.data_ptr(), ctx.slot_mapping.data_ptr(), HM.ptr(k_cache),
                                      HM.ptr(v_cache), HM.ptr(v_first), v_first.stride(0) if v_first is not None else 0, HM.ptr(lam),
                                      q.data_ptr(), T, HM.ptr(q_head_w), HM.ptr(k_head_w), HM.ptr(q_head_scale),
                                      int(bool(interleaved)), float(rot_mag), int(bool(v_unit_norm)), _dev(qkv)))
    return q


def pool_rows_per_page(block_size, pool):
    """Rows of a pooled cache page: block e of a sequence (the mean of its tokens e*pool .. e*pool + pool - 1) is row
    e % rows of the page block_table[e // rows]; rows * pool >= block_size, so that page is the sequence's by the time
    the block is complete."""
    return (block_size + pool - 1) // pool


def pool_blocks(k_cache, v_cache, kp_cache, vp_cache, pool, ctx: StepContext):
    """For every block of ``pool`` tokens that the step completes: the block's mean key and mean value, as the caches hold
    them, into the pooled caches [blocks, pool_rows_per_page, G, D | V].  Call it after the step's keys
    and values are stored."""
    if not k_cache.is_cuda:
        return cpu_ops.pool_blocks(k_cache, v_cache, kp_cache, vp_cache, pool, ctx)
    bs, G, D, V = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3], v_cache.shape[3]
    assert kp_cache.shape[1] == vp_cache.shape[1] == pool_rows_per_page(bs, pool) and kp_cache.dtype == k_cache.dtype
    HM.check(HM.load().hm_pool_blocks(HM.dtype_code(k_cache.dtype), k_cache.data_ptr(), v_cache.data_ptr(), kp_cache.data_ptr(),
                                      vp_cache.data_ptr(), ctx.block_tables.data_ptr(), ctx.seq_pos0.data_ptr(),
                                      ctx.ctx_lens.data_ptr(), ctx.num_seqs, int(ctx.max_q), G, D, V, bs, ctx.block_tables.shape[1],
                                      int(pool), kp_cache.shape[1], _dev(k_cache)))


USE_TILES = True       # bf16 attention on the matrix cores where the shape allows (tests compare both forms)


def paged_attention(q, k_cache, v_cache, ctx: StepContext, scale, sink=None, window=0, keep_first=0, force_rows=False,
                    pooled=None, chunk=0, sigmoid=False, head_bias=None):
    """q [T, H, D] over the paged caches k [blocks, block_size, G, D], v [blocks, block_size, G, V]; query head h reads
    key/value head h // (H/G).  The token at position i sees key j <= i, and with window > 0 only if i - j < window or
    j < keep_first.  ``sink`` f32 [H]: one more term exp(sink[h]) in the softmax denominator, without a value (zeros
    = a sink of score 0).  Scores and weights are float32.  Returns [T, H * V].
    ``pooled`` = (kp_cache, vp_cache, pool) with window > 0: beside its window the token also sees one key and value for
    every block of ``pool`` tokens whose last token lies at or before i - window (the block means pool_blocks keeps), in the
    same softmax.
    ``chunk`` > 0: the token at position i sees key j <= i only if i // chunk == j // chunk (chunks of positions counted from
    the sequence's start).  ``sigmoid``: the weight of a visible key is sigmoid(score + head_bias[h]) (f32 [H], None = 0),
    not normalised over the keys."""
    if not q.is_cuda:
        return cpu_ops.paged_attention(q, k_cache, v_cache, ctx, scale, sink, window, keep_first, pooled, chunk, sigmoid,
                                       head_bias)
    kp, vp, pool = pooled if pooled is not None else (None, None, 0)
    pr = kp.shape[1] if kp is not None else 0
    ptail = (HM.ptr(kp), HM.ptr(vp), int(pool), int(pr), int(chunk), HM.ptr(head_bias), int(bool(sigmoid)))
    assert head_bias is None or head_bias.dtype == torch.float32
    HM.require_cuda(q, k_cache.dtype, "q")
    T, H, D = q.shape
    bs, G, V = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    mb = ctx.block_tables.shape[1]
    o = torch.empty((T, H * V), dtype=q.dtype, device=q.device)
    lib = HM.load()
    tiles_ok = (USE_TILES and not force_rows and q.dtype == torch.bfloat16 and D % 8 == 0 and V % 8 == 0 and D <= 128 and
                V <= 128 and bs % 64 == 0)
    if tiles_ok and ctx.max_q == 1 and H // G <= 32:
        keys = min(mb * bs, window + keep_first + 128) if window > 0 else mb * bs
        if chunk > 0:
            keys = min(keys, chunk + 64)
        if pool:
            keys = min(mb * bs, keys + mb * bs // pool + 64)
        splits = decode_splits(ctx.num_seqs * G, keys)
        ws, n = HM.decode_workspace.get(q.device, lib.hm_attn_decode_workspace_bytes(T, H, V, splits))
        HM.check(lib.hm_attn_decode(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), ctx.block_tables.data_ptr(),
                                    ctx.ctx_lens.data_ptr(), HM.ptr(sink), int(window), int(keep_first), float(scale), o.data_ptr(),
                                    T, H, G, D, V, bs, mb, splits, ws, n, *ptail, _dev(q)))
        return o
    if tiles_ok:
        HM.check(lib.hm_attn_tiles(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), ctx.block_tables.data_ptr(),
                                   ctx.qstart.data_ptr(), ctx.seq_pos0.data_ptr(), HM.ptr(sink), int(window), int(keep_first),
                                   float(scale), o.data_ptr(), ctx.num_seqs, ctx.max_q, H, G, D, V, bs, mb, *ptail, _dev(q)))
        return o
    HM.check(lib.hm_attn_rows(HM.dtype_code(q.dtype), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                              ctx.block_tables.data_ptr(), ctx.tok_seq.data_ptr(), ctx.tok_pos.data_ptr(), HM.ptr(sink),
                              int(window), int(keep_first), float(scale), o.data_ptr(), T, H, G, D, V, bs, mb, *ptail, _dev(q)))
    return o


def group_norm_residual(x, y, post_w, groups, eps, dtype, next_w=None, ids=None, want_h=True):
    """The boundary between two sublayers of a float32 residual x [T, W] that is normalised on the sublayers' OUTPUT, the
    RMS norm taken over ``groups`` equal consecutive parts of the vector; per token in one launch:
      y given:        x <- x + group_norm(y) * post_w   (ids given: x <- group_norm(y[ids]) * post_w, y an embedding table;
                      x may then be None and is made here)
      want_h:         returns group_norm(x) * next_w if next_w is given, else x itself, in ``dtype`` (what the next
                      sublayer, or the vocabulary product, reads); for float32 without next_w that is x, no copy.
    Returns (x, h)."""
    on_cpu = not (y if y is not None else x).is_cuda
    if on_cpu:
        return cpu_ops.group_norm_residual(x, y, post_w, groups, eps, dtype, next_w, ids, want_h)
    T = ids.numel() if ids is not None else (y if y is not None else x).shape[0]
    W = (y if y is not None else x).shape[1]
    if x is None:
        x = torch.empty((T, W), dtype=torch.float32, device=y.device)
    if y is not None:
        HM.require_cuda(y, dtype, "y")
    h = None
    if want_h and (next_w is not None or dtype != torch.float32):
        h = torch.empty((T, W), dtype=dtype, device=x.device)
    HM.check(HM.load().hm_group_norm_residual(HM.dtype_code(dtype), x.data_ptr(), HM.ptr(y), HM.ptr(ids), HM.ptr(post_w),
                                              HM.ptr(next_w), int(groups), float(eps), HM.ptr(h), T, W, _dev(x)))
    return x, (h if h is not None or not want_h else x)


def scale_softcap_(logits, scale, cap):
    """logits f32, in place: cap * tanh(logits * scale / cap) (cap <= 0 or None: logits * scale)."""
    if not logits.is_cuda:
        return cpu_ops.scale_softcap_(logits, scale, cap)
    assert logits.dtype == torch.float32 and logits.is_contiguous()
    HM.check(HM.load().hm_scale_softcap(logits.data_ptr(), logits.numel(), float(scale), float(cap or 0.0), _dev(logits)))
    return logits


def decode_splits(num_groups, max_keys):
    """Splits of the key tiles in decode attention: about four workgroups per CU, at least two 64-key tiles per split.
    Depends only on the batch size and the cache geometry, never on the sequences' lengths."""
    want = max(1, 1024 // max(1, num_groups))
    return int(max(1, min(want, (max_keys + 127) // 128, 64)))


def delta_prepare(proj, cols, w2, w0, a_bias, H, D, decay_scale, unit_eps=1e-6):
    """The float32 inputs of a delta-rule recurrence from the mixer's merged product.  cols = ((offset, size) of r, k, the
    removal gate's pre-activation, and the decay's inner activation z) in proj's columns.  Per token, head and channel:
      decay = exp(-decay_scale * sigmoid(w2 tanh(z) + w0)),  a = sigmoid(a_pre + a_bias),  u = k / sqrt(sum k^2 + unit_eps)
    Returns f32 [T, H, 5, D] = decay, a * u, u, k, r."""
    if not proj.is_cuda:
        return cpu_ops.delta_prepare(proj, cols, w2, w0, a_bias, H, D, decay_scale)
    _rows(proj, "proj")
    T = proj.shape[0]
    (r_off, _), (k_off, _), (a_off, _), (z_off, rank) = cols
    assert w2.shape == (H * D, rank) and w2.is_contiguous() and w2.dtype == proj.dtype
    prep = torch.empty((T, H, 5, D), dtype=torch.float32, device=proj.device)
    HM.check(HM.load().hm_delta_prepare(HM.dtype_code(proj.dtype), proj.data_ptr(), proj.stride(0), r_off, k_off, a_off, z_off,
                                        w2.data_ptr(), w0.data_ptr(), a_bias.data_ptr(), rank, float(decay_scale), float(unit_eps),
                                        prep.data_ptr(), T, H, D, _dev(proj)))
    return prep


def delta_recurrence(prep, v, state, ctx: StepContext):
    """Generalized delta rule over every sequence's portion, token after token, per head with a float32 state S [D, D]:
      S <- diag(decay) S - (a u)(u^T S) + k v^T  (both terms read the old S),  o = S^T r.
    state f32 [slots, H, D, D] is read at a portion's start (zero at position 0) and left at its end.  v [T, H*D] may be a
    column slice.  Returns o f32 [T, H, D]."""
    if not prep.is_cuda:
        return cpu_ops.delta_recurrence(prep, v, state, ctx)
    _rows(v, "v")
    T, H, _, D = prep.shape
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, D)
    o = torch.empty((T, H, D), dtype=torch.float32, device=prep.device)
    HM.check(HM.load().hm_delta_recurrence(HM.dtype_code(v.dtype), prep.data_ptr(), v.data_ptr(), v.stride(0), state.data_ptr(),
                                           ctx.qstart.data_ptr(), ctx.seq_pos0.data_ptr(), ctx.seq_slot.data_ptr(), o.data_ptr(),
                                           ctx.num_seqs, H, D, max(int(ctx.max_q), 1), _dev(prep)))
    return o


def delta_gate_norm(o, g, norm_w, eps, dtype):
    """o f32 [T, H, D] -> every head divided by its RMS, times norm_w [H*D], times sigmoid(g) (g [T, H*D], rows may be a
    column slice), in ``dtype``."""
    if not o.is_cuda:
        return cpu_ops.delta_gate_norm(o, g, norm_w, eps, dtype)
    _rows(g, "g")
    T, H, D = o.shape
    out = torch.empty((T, H * D), dtype=dtype, device=o.device)
    HM.check(HM.load().hm_delta_gate_norm(HM.dtype_code(dtype), o.data_ptr(), g.data_ptr(), g.stride(0), norm_w.data_ptr(),
                                          float(eps), out.data_ptr(), T, H, D, _dev(o)))
    return out


def relu_squared(z):
    """max(z, 0)^2; z [T, F] may be a column slice of a wider product."""
    if not z.is_cuda:
        return cpu_ops.relu_squared(z)
    _rows(z, "z")
    T, Fw = z.shape
    out = torch.empty((T, Fw), dtype=z.dtype, device=z.device)
    HM.check(HM.load().hm_relu_squared(HM.dtype_code(z.dtype), z.data_ptr(), z.stride(0), out.data_ptr(), T, Fw, _dev(z)))
    return out


def dyt_residual(x, y, post, nxt, dtype, ids=None, want_h=True):
    """The boundary between two sublayers of a float32 residual x [T, W] whose sublayers sit between two Dynamic-Tanh
    norms, dyt(z) = tanh(alpha z) * w + b with a norm given as (w [W], b [W], alpha f32 [1]); one elementwise launch:
      y given:   x <- x + dyt_post(y)     (ids given: x <- y[ids], y an embedding table, no norm; x may be None)
      want_h:    returns dyt_nxt(x), or x itself without ``nxt``, in ``dtype``.
    Returns (x, h)."""
    src = y if y is not None else x
    if not src.is_cuda:
        return cpu_ops.dyt_residual(x, y, post, nxt, dtype, ids, want_h)
    T = ids.numel() if ids is not None else src.shape[0]
    W = src.shape[1]
    if x is None:
        x = torch.empty((T, W), dtype=torch.float32, device=src.device)
    if y is not None:
        HM.require_cuda(y, dtype, "y")
    pw, pb, pa = post if post is not None else (None, None, None)
    nw, nb, na = nxt if nxt is not None else (None, None, None)
    for a in (pa, na):
        assert a is None or a.dtype == torch.float32
    h = None
    if want_h and (nxt is not None or dtype != torch.float32):
        h = torch.empty((T, W), dtype=dtype, device=x.device)
    HM.check(HM.load().hm_dyt_residual(HM.dtype_code(dtype), x.data_ptr(), HM.ptr(y), HM.ptr(ids), HM.ptr(pw), HM.ptr(pb), HM.ptr(pa),
                                       HM.ptr(nw), HM.ptr(nb), HM.ptr(na), HM.ptr(h), T, W, _dev(x)))
    return x, (h if h is not None or not want_h else x)


def lightning_recurrence(proj, q_off, k_off, v_off, H, D, V, decay, state, ctx: StepContext):
    """Linear attention with a constant decay per head over every sequence's portion, token after token, with a float32
    state S [D, V] per head:  S <- decay[h] S + k v^T,  o = S^T q,  where q, k [T, H*D] and v [T, H*V] are silu of the
    columns q_off, k_off, v_off of proj.  state f32 [slots, H, D, V] is read at a portion's start (zero at position 0) and
    left at its end.  decay f32 [H].  Returns o f32 [T, H, V]."""
    if not proj.is_cuda:
        return cpu_ops.lightning_recurrence(proj, q_off, k_off, v_off, H, D, V, decay, state, ctx)
    _rows(proj, "proj")
    T = proj.shape[0]
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, V)
    assert decay.dtype == torch.float32 and decay.numel() == H
    o = torch.empty((T, H, V), dtype=torch.float32, device=proj.device)
    HM.check(HM.load().hm_lightning_recurrence(HM.dtype_code(proj.dtype), proj.data_ptr(), proj.stride(0), q_off, k_off, v_off,
                                               decay.data_ptr(), state.data_ptr(), ctx.qstart.data_ptr(), ctx.seq_pos0.data_ptr(),
                                               ctx.seq_slot.data_ptr(), o.data_ptr(), ctx.num_seqs, H, D, V,
                                               max(int(ctx.max_q), 1), _dev(proj)))
    return o
