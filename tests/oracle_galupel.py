"""Plain restatement of the Galupel design in float64 torch: one function per mechanism, whole sequences, no cache, no
batching.  It shares no code with the package; the tests compare the engine and its kernels against it.

A model is (cfg, tensors): cfg the parsed config.json, tensors a dict name -> tensor under the checkpoint's names."""
import math

import torch

F64 = torch.float64


def group_rms_norm(x, w, groups, eps):
    """x [..., W] split into ``groups`` consecutive parts, each divided by its own root mean square, the whole times w."""
    shp = x.shape
    g = x.reshape(*shp[:-1], groups, shp[-1] // groups)
    g = g / torch.sqrt((g * g).mean(-1, keepdim=True) + eps)
    return g.reshape(shp) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def rotate_interleaved(x, pos, dims, base):
    """x [T, ..., D]: channels (2i, 2i+1), i < dims/2, turned by the angle pos * base^(-2i/dims); the rest unchanged."""
    T = x.shape[0]
    i = torch.arange(dims // 2, dtype=F64)
    ang = pos.to(F64)[:, None] * (float(base) ** (-2.0 * i / dims))[None, :]          # [T, dims/2]
    shape = [T] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def pooled_window_attention(q, k, v, scale_h, window, pool):
    """q [T, H, D], k [T, G, D], v [T, G, V] of one sequence; scale_h [H] multiplies head h's scores.  Query i sees the
    tokens j with 0 <= i - j < window and, for every block of ``pool`` tokens whose last token lies at or before
    i - window, the mean key and mean value of the block, all in one softmax.  window <= 0: every j <= i; pool <= 0: no
    blocks."""
    T, H, D = q.shape
    G, V = k.shape[1], v.shape[2]
    out = torch.zeros(T, H, V, dtype=F64)
    nb = T // pool if pool > 0 else 0
    if nb:
        kp = k[:nb * pool].reshape(nb, pool, G, D).mean(1)
        vp = v[:nb * pool].reshape(nb, pool, G, V).mean(1)
    for i in range(T):
        lo = max(0, i - window + 1) if window > 0 else 0
        seen = 0
        if pool > 0 and window > 0:
            seen = max(0, (i - window + 1) // pool) if i - window + 1 > 0 else 0
        for h in range(H):
            g = h // (H // G)
            keys, vals = k[lo:i + 1, g], v[lo:i + 1, g]
            if seen:
                keys, vals = torch.cat([kp[:seen, g], keys]), torch.cat([vp[:seen, g], vals])
            s = (keys @ q[i, h]) * scale_h[h]
            out[i, h] = torch.softmax(s, 0) @ vals
    return out


def attention_keys_values(h, p, m, eps):
    """What an attention layer caches for a whole sequence: normed keys [T, G, D] and values [T, G, V]."""
    T = h.shape[0]
    G, D, V = m["kv_heads"], m["dim"], m["vdim"]
    k = rms_norm((h @ p["mix.k"].T).reshape(T, G, D), p["mix.k.norm"], eps)
    v = (h @ p["mix.v"].T).reshape(T, G, V)
    return k, v


def attention_mixer(h, p, m, eps, kv=None, rounding=None):
    """The 'attention' mixer on one sequence h [T, W].  ``kv``: keys and values of the layer named by kv_from.
    ``rounding``: a function applied to keys and values as a cache of lower precision would hold them."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = rms_norm((h @ p["mix.q"].T).reshape(T, H, D), p["mix.q.norm"], eps)
    k, v = kv if kv is not None else attention_keys_values(h, p, m, eps)
    if rounding is not None:
        k, v = rounding(k), rounding(v)
    mask = m.get("mask") or {}
    o = pooled_window_attention(q, k, v, p["mix.temp"].to(F64) * m["scale"], mask.get("size", 0), mask.get("pool", 0))
    return o.reshape(T, H * V) @ p["mix.o"].T, (k, v)


def latent_attention_mixer(h, p, m, eps):
    """The 'latent_attention' mixer on one sequence: explicit keys and values from the latent, rotated parts, window."""
    T = h.shape[0]
    H, D, Rd, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ p["mix.q"].T).reshape(T, H, D + Rd)
    qn, qr = q[..., :D], rotate_interleaved(q[..., D:], pos, m["rot"]["dims"], m["rot"]["base"])
    ckr = h @ p["mix.dkv"].T
    c = rms_norm(ckr[:, :R], p["mix.dkv.norm"], eps)
    kr = rotate_interleaved(ckr[:, R:], pos, m["rot"]["dims"], m["rot"]["base"])          # [T, Rd], shared by the heads
    kn = (c @ p["mix.uk"].T).reshape(T, H, D)
    v = (c @ p["mix.uv"].T).reshape(T, H, V)
    window = (m.get("mask") or {}).get("size", 0)
    out = torch.zeros(T, H, V, dtype=F64)
    for i in range(T):
        lo = max(0, i - window + 1) if window > 0 else 0
        for hd in range(H):
            s = (kn[lo:i + 1, hd] @ qn[i, hd] + kr[lo:i + 1] @ qr[i, hd]) * m["scale"]
            out[i, hd] = torch.softmax(s, 0) @ v[lo:i + 1, hd]
    return out.reshape(T, H * V) @ p["mix.o"].T


def route(h, router_w, correction, top, groups, keep):
    """Sigmoid router with a correction that only steers the choice: returns (idx [T, top], weights [T, top])."""
    s = torch.sigmoid(h @ router_w.T)                       # [T, E]
    choice = s + correction
    T, E = s.shape
    per = E // groups
    gs = choice.reshape(T, groups, per).topk(min(2, per), dim=-1).values.sum(-1)          # [T, groups]
    kept = gs.topk(keep, dim=-1).indices
    allowed = torch.zeros(T, groups, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = choice.masked_fill(~allowed.repeat_interleave(per, dim=1), -math.inf)
    idx = masked.topk(top, dim=-1).indices
    return idx, s.gather(1, idx)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def moe(h, p, mlp):
    r = mlp["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    idx, wts = route(h, p["mlp.router"], p["mlp.correction"], r["top"], g["count"], g["keep"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            out[t] += wts[t, j] * (gelu_erf(h[t] @ p[f"mlp.e{e}.up"].T) @ p[f"mlp.e{e}.down"].T)
    return out


def layer_params(tensors, i):
    pre = f"l{i}."
    return {k[len(pre):]: v.to(F64) for k, v in tensors.items() if k.startswith(pre)}


def forward(cfg, tensors, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out``: a list that receives the residual after every layer."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    embed = tensors["embed"].to(F64)
    x = group_rms_norm(embed[torch.as_tensor(tokens)], tensors["embed.norm"].to(F64), groups, eps)
    kvs = {}
    for i, spec in enumerate(cfg["layers"]):
        p, m = layer_params(tensors, i), spec["mixer"]
        if spec["type"] == "attention":
            src = m.get("kv_from")
            y, kv = attention_mixer(x, p, m, eps, kvs[src] if src is not None else None)
            kvs[i] = kv
        elif spec["type"] == "latent_attention":
            y = latent_attention_mixer(x, p, m, eps)
        else:
            raise ValueError(spec["type"])
        x = x + group_rms_norm(y, p["norm1"], groups, eps)
        if spec.get("mlp") is not None:
            x = x + group_rms_norm(moe(x, p, spec["mlp"]), p["norm2"], groups, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    hN = group_rms_norm(x, tensors["final.norm"].to(F64), groups, eps)
    logits = hN @ embed.T * cfg.get("logit_scale", 1.0)
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
