"""Plain-torch counterparts of nanovllm/ops.py for tensors that live on the CPU.  PLUMBING ONLY: they let the
unquantized model run through the engine on a host without a GPU (Config(device="cpu")), following the formulas
of the reference's layers (layernorm.py:16-40, rotary_embedding.py:7-48, activation.py:11-14, attention.py:43-75,
sampler.py:10-12).  Nothing quantized goes through here and no HIP kernel falls back to this file: ops.py
dispatches on the device of its input and refuses CPU tensors for every quantized operator."""
import torch
import torch.nn.functional as F


def add_rmsnorm(x, residual, weight, eps):
    s = x.float() if residual is None else x.float() + residual.float()
    new_res = x if residual is None else s.to(x.dtype)
    out = (s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * weight
    return out, new_res


def silu_mul(x):
    a, b = x.chunk(2, -1)
    return F.silu(a) * b


def _rope(x, positions, cos_sin):
    cs = cos_sin[positions] if positions is not None else cos_sin      # [T, D] f32: cos | sin
    half = cs.shape[-1] // 2
    cos, sin = cs[:, None, :half], cs[:, None, half:]
    x1, x2 = x.float()[..., :half], x.float()[..., half:]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), -1).to(x.dtype)


def _head_norm(x, w, eps):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * w


def qknorm_rope_store(qkv, positions, cos_sin, q_norm_w, k_norm_w, eps, num_heads, num_kv_heads, head_dim,
                      k_cache=None, v_cache=None, slot_mapping=None, want_kv=True):
    T = qkv.shape[0]
    q, k, v = qkv.split([num_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * head_dim], -1)
    q, k, v = q.view(T, num_heads, head_dim), k.view(T, num_kv_heads, head_dim), v.view(T, num_kv_heads, head_dim)
    if q_norm_w is not None:
        q, k = _head_norm(q, q_norm_w, eps), _head_norm(k, k_norm_w, eps)
    q, k = _rope(q, positions, cos_sin), _rope(k, positions, cos_sin)
    if slot_mapping is not None and k_cache is not None and k_cache.numel() > 0:
        slots = slot_mapping.long()
        keep = slots >= 0
        kc, vc = k_cache.view(-1, num_kv_heads, head_dim), v_cache.view(-1, num_kv_heads, head_dim)
        kc[slots[keep]] = k[keep]
        vc[slots[keep]] = v[keep]
    return q.contiguous(), (k.contiguous() if want_kv else None), (v.contiguous() if want_kv else None)


def _sdpa(q, k, v, scale, causal):
    # q [Tq, Hq, D], k/v [Tk, Hkv, D] -> [Tq, Hq, D]
    o = F.scaled_dot_product_attention(q.transpose(0, 1)[None].float(), k.transpose(0, 1)[None].float(),
                                       v.transpose(0, 1)[None].float(), is_causal=causal, scale=scale, enable_gqa=True)
    return o[0].transpose(0, 1).to(q.dtype)


def attn_prefill(q, k, v, cu_seqlens, max_seqlen, scale):
    cu = cu_seqlens.tolist()
    out = torch.empty_like(q)
    for a, b in zip(cu[:-1], cu[1:]):
        out[a:b] = _sdpa(q[a:b], k[a:b], v[a:b], scale, True)
    return out


def paged_attn_decode(q, k_cache, v_cache, block_tables, context_lens, scale):
    B = q.shape[0]
    block_size = k_cache.shape[1]
    out = torch.zeros_like(q)
    for b in range(B):
        n = int(context_lens[b])
        if n == 0:
            continue
        t = torch.arange(n)
        rows = block_tables[b, t // block_size].long() * block_size + t % block_size
        kk = k_cache.view(-1, *k_cache.shape[2:])[rows]
        vv = v_cache.view(-1, *v_cache.shape[2:])[rows]
        out[b:b + 1] = _sdpa(q[b:b + 1], kk, vv, scale, False)
    return out


def argmax_rows(logits):
    return logits.float().argmax(-1)


# ---- plumbing counterparts of nanovllm/seq_ops.py -------------------------------------------------------------------
def embed_streams(ids, positions, embed, pos_table, streams):
    x = embed[ids].float()
    if pos_table is not None:
        x = x + pos_table[positions.long()].float()
    return x[:, None, :].repeat(1, streams, 1).contiguous()


def stream_step(X, y, mix, out, w_in, norm_w, eps, dtype):
    if y is not None:
        X.copy_(torch.einsum("sr,tsw->trw", mix, X) + out[None, :, None] * y.float()[:, None, :])
    if w_in is None:
        return None
    u = torch.einsum("s,tsw->tw", w_in, X)
    return (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()).to(dtype)


def canon_conv(h, w, state, run, ctx):
    taps = w.shape[1]
    out = torch.empty_like(h)
    qs = ctx.qstart.tolist()
    for b in range(ctx.num_seqs):
        a, e = qs[b], qs[b + 1]
        if e <= a:
            continue
        slot, pos0 = int(ctx.seq_slot[b]), int(ctx.seq_pos0[b])
        prev = state[slot, run][:taps - 1].float().clone()                     # [taps-1, W]: inputs at pos0-(taps-1) .. pos0-1
        for k in range(taps - 1):
            if pos0 - (taps - 1) + k < 0:
                prev[k] = 0
        hist = torch.cat([prev, h[a:e].float()], 0)
        acc = h[a:e].float().clone()
        for j in range(taps):
            acc += w[:, j].float() * hist[j:j + e - a]
        out[a:e] = acc.to(h.dtype)
        if taps > 1:
            state[slot, run] = hist[-(taps - 1):].to(state.dtype)
    return out


def latent_norm_store(x, w, eps, cache, slot_mapping):
    xf = x.float()
    c = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(cache.dtype)
    keep = slot_mapping >= 0
    cache.view(-1, cache.shape[-1])[slot_mapping[keep].long()] = c[keep]


def rotate_pairs(x, pos, inv_freq, rot_dims):
    """Channels (2i, 2i + 1), i < rot_dims / 2, of the last dimension turned by pos * inv_freq[i]; x [T, ..., C] f32."""
    if not rot_dims:
        return x
    ang = pos.float()[:, None] * inv_freq.float()[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [rot_dims // 2]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
    out = x.clone()
    out[..., 0:rot_dims:2] = u * c - v * s
    out[..., 1:rot_dims:2] = v * c + u * s
    return out


def rms_norm_rows(x, w, eps):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(x.dtype)


def latent_rope_store(x, w, eps, q, qa, inv_freq, rot_dims, H, D, R, Rd, cache, ctx):
    T = x.shape[0]
    xf = x.float()
    c = xf[:, :R] * torch.rsqrt(xf[:, :R].pow(2).mean(-1, keepdim=True) + eps) * w.float()
    kr = rotate_pairs(xf[:, R:], ctx.tok_pos, inv_freq, rot_dims)
    rows = ctx.slot_mapping
    keep = rows >= 0
    cache.view(-1, R + Rd)[rows[keep].long()] = torch.cat([c, kr], -1).to(cache.dtype)[keep]
    qr = rotate_pairs(q.float().view(T, H, D + Rd)[..., D:], ctx.tok_pos, inv_freq, rot_dims)
    qa[..., R:] = qr.to(qa.dtype)


def latent_attention(q, cache, ctx, scale, RV=0, window=0):
    RV = RV or q.shape[-1]
    o = torch.empty(q.shape[:-1] + (RV,), dtype=q.dtype)
    bs = cache.shape[1]
    rows = cache.view(-1, cache.shape[-1])
    qs = ctx.qstart.tolist()
    for b in range(ctx.num_seqs):
        a, e = qs[b], qs[b + 1]
        if e <= a:
            continue
        n = int(ctx.ctx_lens[b])
        t = torch.arange(n)
        c = rows[ctx.block_tables[b, t // bs].long() * bs + t % bs].float()          # [n, R]
        s = torch.einsum("thr,nr->thn", q[a:e].float(), c) * scale
        pos = ctx.tok_pos[a:e].long()
        hidden = t[None, None, :] > pos[:, None, None]
        if window > 0:
            hidden = hidden | (pos[:, None, None] - t[None, None, :] >= window)
        s = s.masked_fill(hidden, float("-inf"))
        o[a:e] = torch.einsum("thn,nr->thr", torch.softmax(s, -1), c[:, :RV]).to(q.dtype)
    return o


def poly_norm(z, coef, eps):
    zf = z.float()

    def unit(v):
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    a, b, c, e = coef.tolist()
    return (a * unit(zf) + b * unit(zf * zf) + c * unit(zf * zf * zf) + e).to(z.dtype)


def clamped_glu(gu, limit, alpha):
    g, u = gu.float().chunk(2, -1)
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1)).to(gu.dtype)


def moe_route(h, router_w, top, groups, keep, score=0, correction=None, group_top=1, renorm=True, bias=None):
    T, E = h.shape[0], router_w.shape[0]
    z = h.float() @ router_w.t()
    if bias is not None:
        z = z + bias.float()
    s = torch.sigmoid(z) if score == 1 else torch.softmax(z, -1)
    choice = s if correction is None else s + correction.float()
    masked = choice
    if groups > 1:
        per = E // groups
        best = choice.view(T, groups, per).topk(min(group_top, per), -1).values.sum(-1).topk(keep, -1).indices
        ok = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, best, True)
        masked = choice.masked_fill(~ok.repeat_interleave(per, 1), float("-inf"))
    idx = masked.topk(top, -1).indices
    w = s.gather(1, idx)
    return idx.int(), (w / (w.sum(-1, keepdim=True) + 1e-20) if renorm else w)


def moe_experts(h, idx, wts, w_gu, w_down, limit, alpha, shared, act_kind=0):
    y = torch.zeros(h.shape, dtype=torch.float32)
    for e in idx.unique().tolist():
        tok, k = (idx == e).nonzero(as_tuple=True)
        if act_kind == 0:
            act = clamped_glu(F.linear(h[tok], w_gu[e]), limit, alpha)
        elif act_kind == 3:
            g, u = F.linear(h[tok], w_gu[e]).float().chunk(2, -1)
            g, u = g.clamp(max=limit), u.clamp(-limit, limit)
            act = (g * torch.sigmoid(alpha * g) * u).to(h.dtype)
        else:
            act = F.gelu(F.linear(h[tok], w_gu[e]).float(), approximate="tanh" if act_kind == 2 else "none").to(h.dtype)
        y.index_add_(0, tok, wts[tok, k][:, None] * F.linear(act, w_down[e]).float())
    if shared is not None:
        y = y + shared.float()
    return y.to(h.dtype)


# ---- plumbing counterparts of nanovllm/hy_ops.py --------------------------------------------------------------------
def _unit_rms(x, eps):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def embed_scaled(ids, embed, scale):
    return embed[ids].float() * scale


def sublayer_close(x, y, gate, gate_bias, post_w, mult, next_w, eps, dtype, carry):
    if y is not None:
        z = y.float() * torch.sigmoid(gate.float() + gate_bias.float())
        x.add_(mult * _unit_rms(z, eps) * post_w.float())
    if carry is not None:
        src, state, layer, ctx = carry
        last = (ctx.qstart[1:] - 1).long()
        state[ctx.seq_slot.long(), layer] = src[last].to(state.dtype)
    if next_w is None:
        return None
    return (_unit_rms(x, eps) * next_w.float()).to(dtype)


def token_shift(h, mu, state, layer, ctx):
    hf = h.float()
    prev = torch.cat([torch.zeros_like(hf[:1]), hf[:-1]], 0)
    first = ctx.qstart[:-1].long()
    carried = state[ctx.seq_slot.long(), layer].float()
    carried = carried * (ctx.seq_pos0 > 0).float()[:, None]
    prev[first] = carried
    return (hf + (prev - hf) * mu.float()).to(h.dtype)


def rotate_half_partial(x, pos, inv_freq, mag=1.0):
    """x f32 [T, heads, D]: the first 2 * len(inv_freq) channels of every head turn by pos * inv_freq (cosines and sines
    times ``mag``)."""
    half = inv_freq.numel()
    ang = pos.float()[:, None] * inv_freq[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = x[..., :half], x[..., half:2 * half]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., 2 * half:]], -1)


def rotate_pairs_partial(x, pos, inv_freq, mag):
    """x f32 [T, heads, D]: channels (2i, 2i + 1), i < len(inv_freq), of every head turn by pos * inv_freq[i]; cosines and
    sines times ``mag``."""
    n = inv_freq.numel()
    ang = pos.float()[:, None] * inv_freq[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    out = x.clone()
    out[..., 0:2 * n:2] = a * c - b * s
    out[..., 1:2 * n:2] = b * c + a * s
    return out


def qkv_prepare(qkv, H, G, D, V, q_norm_w, k_norm_w, eps, inv_freq, unit_norm, ctx, k_cache, v_cache, v_first, lam,
                q_head_w=None, k_head_w=None, q_head_scale=None, interleaved=False, rot_mag=1.0, v_unit_norm=False):
    T = qkv.shape[0]

    def turn(x):                                        # (the pairing this call asks for)
        if interleaved:
            return rotate_pairs_partial(x, ctx.tok_pos, inv_freq, rot_mag)
        return rotate_half_partial(x, ctx.tok_pos, inv_freq, rot_mag)
    if k_cache is None:                        # the rows hold q only
        q = qkv.float().reshape(T, H, D)
        if q_head_w is not None:
            q = _unit_rms(q, eps) * q_head_w.float()
        if q_head_scale is not None:
            q = q * q_head_scale.float()[None, :, None]
        if inv_freq is not None:
            q = turn(q)
        if unit_norm:
            q = _unit_rms(q, eps)
        return q.to(qkv.dtype).contiguous()
    q, k, v = qkv.float().split([H * D, G * D, G * V], -1)
    if q_norm_w is not None:
        q, k = _unit_rms(q, eps) * q_norm_w.float(), _unit_rms(k, eps) * k_norm_w.float()
    q, k = q.reshape(T, H, D), k.reshape(T, G, D)
    if q_head_w is not None:
        q, k = _unit_rms(q, eps) * q_head_w.float(), _unit_rms(k, eps) * k_head_w.float()
    if q_head_scale is not None:
        q = q * q_head_scale.float()[None, :, None]
    if inv_freq is not None:
        q, k = turn(q), turn(k)
    if unit_norm:
        q, k = _unit_rms(q, eps), _unit_rms(k, eps)
    if v_first is not None:
        v = (1 - lam.float()) * v + lam.float() * v_first.float()
    if v_unit_norm:
        v = _unit_rms(v.reshape(T, G, V), eps).reshape(T, G * V)
    rows = ctx.slot_mapping.long()
    k_cache.view(-1, G, D)[rows] = k.to(k_cache.dtype)
    v_cache.view(-1, G, V)[rows] = v.reshape(T, G, V).to(v_cache.dtype)
    return q.to(qkv.dtype).contiguous()


def pool_blocks(k_cache, v_cache, kp_cache, vp_cache, pool, ctx):
    bs, pr = k_cache.shape[1], kp_cache.shape[1]
    kr, vr = k_cache.view(-1, *k_cache.shape[2:]), v_cache.view(-1, *v_cache.shape[2:])
    kp, vp = kp_cache.view(-1, *kp_cache.shape[2:]), vp_cache.view(-1, *vp_cache.shape[2:])
    for t in range(ctx.num_tokens):
        pos, b = int(ctx.tok_pos[t]), int(ctx.tok_seq[t])
        if (pos + 1) % pool:
            continue
        e = pos // pool
        j = torch.arange(e * pool, e * pool + pool)
        rows = ctx.block_tables[b, j // bs].long() * bs + j % bs
        prow = int(ctx.block_tables[b, e // pr]) * pr + e % pr
        kp[prow] = kr[rows].float().mean(0).to(kp.dtype)
        vp[prow] = vr[rows].float().mean(0).to(vp.dtype)


def paged_attention(q, k_cache, v_cache, ctx, scale, sink, window, keep_first, pooled=None, chunk=0, sigmoid=False,
                    head_bias=None):
    T, H, D = q.shape
    bs, G, V = k_cache.shape[1], k_cache.shape[2], v_cache.shape[3]
    o = torch.empty((T, H * V), dtype=q.dtype)
    kr, vr = k_cache.view(-1, G, D), v_cache.view(-1, G, V)
    qs = ctx.qstart.tolist()
    for b in range(ctx.num_seqs):
        a, e = qs[b], qs[b + 1]
        if e <= a:
            continue
        n = int(ctx.ctx_lens[b])
        j = torch.arange(n)
        rows = ctx.block_tables[b, j // bs].long() * bs + j % bs
        kk = kr[rows].float().repeat_interleave(H // G, 1)                       # [n, H, D]
        vv = vr[rows].float().repeat_interleave(H // G, 1)
        s = torch.einsum("thd,nhd->thn", q[a:e].float(), kk) * scale
        i = ctx.tok_pos[a:e].long()[:, None]
        ok = j[None, :] <= i
        if window > 0:
            ok &= ((i - j[None, :]) < window) | (j[None, :] < keep_first)
        if chunk > 0:
            ok &= (i // chunk) == (j[None, :] // chunk)
        if sigmoid:
            hb = head_bias.float()[None, :, None] if head_bias is not None else 0.0
            p = torch.sigmoid(s + hb) * ok[:, None, :]
            o[a:e] = torch.einsum("thn,nhv->thv", p, vv).reshape(e - a, H * V).to(q.dtype)
            continue
        s = s.masked_fill(~ok[:, None, :], float("-inf"))
        if pooled is not None and pooled[2] > 0:
            kp_c, vp_c, pool = pooled
            pr = kp_c.shape[1]
            ne = max(0, (n - window) // pool) if n - window > 0 else 0       # entries the last token of the portion sees
            if ne:
                e_ = torch.arange(ne)
                prow = ctx.block_tables[b, e_ // pr].long() * pr + e_ % pr
                kpp = kp_c.view(-1, G, D)[prow].float().repeat_interleave(H // G, 1)
                vpp = vp_c.view(-1, G, V)[prow].float().repeat_interleave(H // G, 1)
                sp = torch.einsum("thd,nhd->thn", q[a:e].float(), kpp) * scale
                seen = torch.clamp((i + 1 - window), min=0) // pool                 # [t, 1]
                sp = sp.masked_fill(~(e_[None, :] < seen)[:, None, :], float("-inf"))
                p = torch.softmax(torch.cat([sp, s], -1), -1)
                o[a:e] = (torch.einsum("thn,nhv->thv", p[..., :ne], vpp) +
                          torch.einsum("thn,nhv->thv", p[..., ne:], vv)).reshape(e - a, H * V).to(q.dtype)
                continue
        if sink is not None:
            s = torch.cat([s, sink.float()[None, :, None].expand(e - a, H, 1)], -1)
        p = torch.softmax(s, -1)[..., :n]
        o[a:e] = torch.einsum("thn,nhv->thv", p, vv).reshape(e - a, H * V).to(q.dtype)
    return o


def delta_prepare(proj, cols, w2, w0, a_bias, H, D, decay_scale):
    T = proj.shape[0]
    pf = proj.float()
    r, k, a_pre, z = (pf[:, c:c + n] for c, n in cols)
    decay = torch.exp(-decay_scale * torch.sigmoid(torch.tanh(z) @ w2.float().t() + w0.float()))
    a = torch.sigmoid(a_pre + a_bias.float())
    kh = k.reshape(T, H, D)
    u = kh / torch.sqrt(kh.pow(2).sum(-1, keepdim=True) + 1e-6)
    return torch.stack([decay.reshape(T, H, D), a.reshape(T, H, D) * u, u, kh, r.reshape(T, H, D)], 2).contiguous()


def delta_recurrence(prep, v, state, ctx):
    T, H, _, D = prep.shape
    o = torch.empty((T, H, D), dtype=torch.float32)
    vf = v.float().reshape(T, H, D)
    qs = ctx.qstart.tolist()
    for b in range(ctx.num_seqs):
        a, e = qs[b], qs[b + 1]
        if e <= a:
            continue
        slot = int(ctx.seq_slot[b])
        S = state[slot].clone() if int(ctx.seq_pos0[b]) > 0 else torch.zeros_like(state[slot])
        for t in range(a, e):
            decay, au, u, k, r = prep[t].unbind(1)
            uS = torch.einsum("hi,hij->hj", u, S)
            S = decay[:, :, None] * S - au[:, :, None] * uS[:, None, :] + k[:, :, None] * vf[t][:, None, :]
            o[t] = torch.einsum("hij,hi->hj", S, r)
        state[slot] = S
    return o


def delta_gate_norm(o, g, norm_w, eps, dtype):
    T, H, D = o.shape
    return (_unit_rms(o, eps).reshape(T, H * D) * norm_w.float() * torch.sigmoid(g.float())).to(dtype)


def relu_squared(z):
    return torch.relu(z.float()).pow(2).to(z.dtype)


def group_norm_residual(x, y, post_w, groups, eps, dtype, next_w, ids, want_h):
    def gnorm(v, w):
        g = v.view(v.shape[0], groups, -1)
        return (g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)).view(v.shape) * w.float()
    if y is not None:
        n = gnorm((y[ids] if ids is not None else y).float(), post_w)
        if ids is not None:
            x = n
        else:
            x += n
    if not want_h:
        return x, None
    h = gnorm(x, next_w).to(dtype) if next_w is not None else (x if dtype == torch.float32 else x.to(dtype))
    return x, h


def scale_softcap_(logits, scale, cap):
    logits.mul_(scale)
    if cap:
        logits.copy_(cap * torch.tanh(logits / cap))
    return logits


def dyt_residual(x, y, post, nxt, dtype, ids, want_h):
    def dyt(v, n):
        w, b, a = n
        return torch.tanh(a.float() * v) * w.float() + b.float()
    if y is not None:
        if ids is not None:
            x = y[ids].float()
        else:
            x += dyt(y.float(), post)
    if not want_h:
        return x, None
    h = dyt(x, nxt).to(dtype) if nxt is not None else (x if dtype == torch.float32 else x.to(dtype))
    return x, h


def lightning_recurrence(proj, q_off, k_off, v_off, H, D, V, decay, state, ctx):
    T = proj.shape[0]
    pf = proj.float()
    q = F.silu(pf[:, q_off:q_off + H * D]).reshape(T, H, D)
    k = F.silu(pf[:, k_off:k_off + H * D]).reshape(T, H, D)
    v = F.silu(pf[:, v_off:v_off + H * V]).reshape(T, H, V)
    o = torch.empty((T, H, V), dtype=torch.float32)
    qs = ctx.qstart.tolist()
    for b in range(ctx.num_seqs):
        a, e = qs[b], qs[b + 1]
        if e <= a:
            continue
        slot = int(ctx.seq_slot[b])
        S = state[slot].clone() if int(ctx.seq_pos0[b]) > 0 else torch.zeros_like(state[slot])
        for t in range(a, e):
            S = decay.float()[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S
    return o
