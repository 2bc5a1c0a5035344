"""Plain restatement of the Lilevik design in float64 torch: one function per mechanism, whole sequences, no cache, no
batching.  It shares no code with the package; the tests compare the engine and its kernels against it.

A model is (cfg, tensors): cfg the parsed config.json, tensors a dict name -> tensor under the checkpoint's names."""
import math

import torch

F64 = torch.float64


def dyn_tanh(x, w, b, alpha):
    """The design's norm: no statistics, tanh(alpha x) w + b per channel."""
    return torch.tanh(alpha * x) * w + b


def rms_norm(x, w, eps):
    n = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return n if w is None else n * w


def rotary_table(rot):
    """rot = {dims, base, scaling?} -> (frequencies [dims/2], factor on cos and sin).  With ``scaling`` = {factor, original,
    fast, slow} the frequencies of slowly turning pairs are divided by the factor, those of fast pairs are kept, a linear
    ramp over the pair index between them; and cos and sin grow by 0.1 ln(factor) + 1."""
    dims, base = rot["dims"], float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F64), 1.0
    def where(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(where(sc["fast"])), 0)
    hi = min(math.ceil(where(sc["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / sc["factor"] * ramp + fi * (1 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_interleaved(x, pos, freqs, mag=1.0):
    """x [T, ..., D]: channels (2i, 2i+1), i < len(freqs), turned by the angle pos * freqs[i] (cos and sin times ``mag``);
    the rest unchanged."""
    T, n = x.shape[0], freqs.numel()
    ang = pos.to(F64)[:, None] * freqs[None, :]
    shape = [T] + [1] * (x.dim() - 2) + [n]
    c, s = (torch.cos(ang) * mag).reshape(shape), (torch.sin(ang) * mag).reshape(shape)
    u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    out = x.clone()
    out[..., 0:2 * n:2] = u * c - v * s
    out[..., 1:2 * n:2] = v * c + u * s
    return out


def latent_attention_mixer(h, p, m, eps, rounding=None):
    """Keys and values are up-projections of a normed latent; queries come through a normed latent of their own; one
    rotated key part is shared by all heads.  Causal softmax."""
    T = h.shape[0]
    H, D, Rd, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    freqs, mag = rotary_table(m["rot"])
    cq = rms_norm(h @ p["mix.dq"].T, p["mix.dq.norm"], eps)
    q = (cq @ p["mix.uq"].T).reshape(T, H, D + Rd)
    dkv = h @ p["mix.dkv"].T
    c = rms_norm(dkv[:, :R], p["mix.dkv.norm"], eps)
    kr = rotate_interleaved(dkv[:, R:], pos, freqs, mag)                      # [T, Rd], one for all heads
    if rounding is not None:
        c, kr = rounding(c), rounding(kr)
    qr = rotate_interleaved(q[..., D:], pos, freqs, mag)
    k = (c @ p["mix.uk"].T).reshape(T, H, D)
    v = (c @ p["mix.uv"].T).reshape(T, H, V)
    s = (torch.einsum("ihd,jhd->hij", q[..., :D], k) + torch.einsum("ihd,jd->hij", qr, kr)) * m["scale"]
    s = s.masked_fill(pos[None, :, None] < pos[None, None, :], float("-inf"))
    o = torch.einsum("hij,jhv->ihv", torch.softmax(s, -1), v)
    return o.reshape(T, H * V) @ p["mix.o"].T


def sigmoid_chunk_attention(q, k, v, bias, scale, chunk):
    """q [T, H, D], k [T, G, D], v [T, G, V]: query i weighs key j <= i of its own chunk (i // chunk == j // chunk;
    chunk <= 0: every j <= i) by sigmoid(score + bias[h]); the weights are not normalised.  -> [T, H, V]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for i in range(T):
        lo = (i // chunk) * chunk if chunk > 0 else 0
        for hh in range(H):
            g = hh // (H // G)
            w = torch.sigmoid((k[lo:i + 1, g] @ q[i, hh]) * scale + bias[hh])
            out[i, hh] = w @ v[lo:i + 1, g]
    return out


def attention_mixer(h, p, m, eps, rounding=None):
    """Grouped heads; q and k RMS-normed over their whole projections; rotation of the first rot.dims channels of every
    head; every value head divided by its root mean square; chunked mask; sigmoid weights with a number per head."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    freqs, mag = rotary_table(m["rot"])
    q = rms_norm(h @ p["mix.q"].T, p["mix.q.norm"], eps).reshape(T, H, D)
    k = rms_norm(h @ p["mix.k"].T, p["mix.k.norm"], eps).reshape(T, G, D)
    v = rms_norm((h @ p["mix.v"].T).reshape(T, G, V), None, eps)
    q, k = rotate_interleaved(q, pos, freqs, mag), rotate_interleaved(k, pos, freqs, mag)
    if rounding is not None:
        k, v = rounding(k), rounding(v)
    o = sigmoid_chunk_attention(q, k, v, p["mix.pb"], m["scale"], (m.get("mask") or {}).get("size", 0))
    return o.reshape(T, H * V) @ p["mix.o"].T


def lightning_recurrence(q, k, v, decay, S0=None):
    """Per head S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  q, k [T, H, D], v [T, H, V] -> (o [T, H, V], S)."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[2], dtype=F64) if S0 is None else S0.clone()
    o = torch.zeros(T, H, v.shape[2], dtype=F64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o, S


def lightning_mixer(h, p, m, eps):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    silu = torch.nn.functional.silu
    q, k = silu(h @ p["mix.q"].T).reshape(T, H, D), silu(h @ p["mix.k"].T).reshape(T, H, D)
    v = silu(h @ p["mix.v"].T).reshape(T, H, V)
    o, _ = lightning_recurrence(q, k, v, torch.tensor(m["decay"], dtype=F64))
    y = rms_norm(o.reshape(T, H * V), p["mix.norm"], eps) * torch.sigmoid(h @ p["mix.g"].T)
    return y @ p["mix.o"].T


def route(h, w, b, top):
    """Router: logits W h + b, the ``top`` largest chosen, weights = softmax over the chosen logits."""
    z = h @ w.T + b
    val, idx = z.topk(top, -1)
    return idx, torch.softmax(val, -1)


def experts(h, p, mlp):
    idx, wts = route(h, p["mlp.router"], p["mlp.router.b"], mlp["router"]["top"])
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wts[t]):
            a = torch.nn.functional.silu(p[f"mlp.e{e}.gate"] @ h[t]) * (p[f"mlp.e{e}.up"] @ h[t])
            y[t] += w * (p[f"mlp.e{e}.down"] @ a)
    return y


MIXERS = {"latent_attention": latent_attention_mixer, "attention": attention_mixer, "lightning": lightning_mixer}


def forward(cfg, tensors, tokens, rounding=None):
    """tokens [T] of one sequence -> (float64 logits [T, vocab], the residual after every layer [L, T, W]).
    ``rounding``: applied to what the attention layers cache (keys, values, latents)."""
    t = {k: v.to(F64) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    trace = []

    def norm(name, z):
        return dyn_tanh(z, t[name], t[name + ".b"], t[name + ".alpha"])
    for i, spec in enumerate(cfg["layers"]):
        pre = f"l{i}."
        p = {k[len(pre):]: v for k, v in t.items() if k.startswith(pre)}
        h = norm(pre + "norm1", x)
        kw = {"rounding": rounding} if spec["type"] != "lightning" else {}
        x = x + norm(pre + "norm1b", MIXERS[spec["type"]](h, p, spec["mixer"], eps, **kw))
        if spec.get("mlp") is not None:
            x = x + norm(pre + "norm2b", experts(norm(pre + "norm2", x), p, spec["mlp"]))
        trace.append(x.clone())
    return norm("final.norm", x) @ t["embed"].T, torch.stack(trace)
