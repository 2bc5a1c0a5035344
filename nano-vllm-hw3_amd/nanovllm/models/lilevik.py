"""Lilevik: a decoder-only model whose layers are listed one by one in config.json.  A layer has one of three mixers -
latent attention whose queries come through a latent of their own, with a rotated key part shared by the heads
("latent_attention"); grouped-head attention with q and k normalised over their whole projections, interleaved rotation on
a frequency table stretched for long contexts, unit-RMS value heads, a mask that shows a query only its own chunk of
positions, and sigmoid weights with a learned number per head instead of a softmax ("attention"); or linear attention
with a constant decay per head and a float32 state ("lightning") - and optionally a mixture of SiLU-gated experts
behind a biased softmax-over-the-chosen router.  Every sublayer sits between two Dynamic-Tanh norms on a float32
residual, x <- x + dyt_b(f(dyt_a(x))); the logits are products of the final norm's output with the embedding table.

Read from config.json: vocab, width, norm.eps, and per layer
  {type, mixer: {heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot: {dims, base}} |
                {heads, kv_heads, dim, vdim, scale, rot: {dims, base, scaling: {factor, original, fast, slow}}, mask: {size}} |
                {heads, dim, vdim, decay: [per head]},
   mlp: null | {kind: moe, expert: {ff}, router: {experts, top}}}.
Checkpoint tensors: embed, final.norm{, .b, .alpha}, and per layer l<i>.{norm1, norm1b, norm2, norm2b}{, .b, .alpha},
l<i>.mix.*, l<i>.mlp.{router, router.b, e<j>.{gate, up, down}}.

The model is stepped with portions of sequences (nanovllm.seq_ops.StepContext).  It owns a paged key/value cache per
attention layer, a paged cache of [latent | rotated key part] rows per latent layer (all layers share a sequence's block
table) and, per state slot, the float32 state of every lightning layer."""
import re

import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import hy_ops
from nanovllm.layers.dyn_tanh import DynTanh
from nanovllm.layers.feedforward import RoutedExperts
from nanovllm.layers.latent_attention import LatentAttention
from nanovllm.layers.lightning import LightningAttention
from nanovllm.layers.rotary_attention import PagedRotaryAttention


class LilevikLayer(nn.Module):
    def __init__(self, cfg, spec):
        super().__init__()
        W, eps, m = cfg.hidden_size, cfg.norm_eps, spec["mixer"]
        self.kind = spec["type"]
        self.norm1, self.norm1b = DynTanh(W), DynTanh(W)
        rot = m.get("rot") or {}
        if self.kind == "latent_attention":
            if rot.get("scaling"):
                raise ValueError("latent_attention: a stretched frequency table is not part of this mixer")
            self.mixer = LatentAttention(W, m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["scale"], eps,
                                         rot_dim=m.get("rot_dim", 0), rot_dims=rot.get("dims", 0), rot_base=rot.get("base", 10000.0),
                                         q_rank=m.get("q_rank", 0))
        elif self.kind == "attention":
            self.mixer = PagedRotaryAttention(W, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"]),
                                              m["scale"], eps, rot.get("dims", 0), rot.get("base", 10000.0), proj_norm=True, interleaved=True,
                                              rot_scaling=rot.get("scaling"), v_unit_norm=True,
                                              chunk=(m.get("mask") or {}).get("size", 0), weights="sigmoid")
        elif self.kind == "lightning":
            self.mixer = LightningAttention(W, m["heads"], m["dim"], m.get("vdim", m["dim"]), m["decay"], eps)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            if mlp["kind"] != "moe":
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
            r = mlp["router"]
            self.norm2, self.norm2b = DynTanh(W), DynTanh(W)
            self.mlp = RoutedExperts(W, r["experts"], r["top"], mlp["expert"]["ff"], score="softmax", renorm=True, act="silu_glu",
                                     bias=True)


class LilevikForCausalLM(nn.Module):
    runs_portions = True           # stepped with portions; owns its caches and per-sequence state
    default_block_size = 64
    native_library = ("hymix", "seqmix")      # norms, attention and the recurrence; latent attention and experts

    @staticmethod
    def normalize_config(d: dict) -> dict:
        d = dict(d)
        d["vocab_size"], d["hidden_size"] = d["vocab"], d["width"]
        d["max_position_embeddings"] = d.get("max_positions", 1 << 20)
        d["norm_eps"] = d["norm"]["eps"]
        d.setdefault("torch_dtype", "bfloat16")
        return d

    def __init__(self, cfg):
        super().__init__()
        self.cfg = cfg
        W = cfg.hidden_size
        self.dtype = torch.get_default_dtype()
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W), requires_grad=False)
        self.layers = nn.ModuleList([LilevikLayer(cfg, spec) for spec in cfg.layers])
        self.final_norm = DynTanh(W)
        self._f32_out = None       # whether the vendor GEMM writes float32 from 16-bit operands for the head's shape

    # ------------------------------------------------------------------ checkpoint names
    _SIMPLE = {"mix.o": "mixer.o_proj", "mix.q.norm": "mixer.q_norm", "mix.k.norm": "mixer.k_norm", "mix.pb": "mixer.head_bias",
               "mix.dq.norm": "mixer.q_latent_norm", "mix.uq": "mixer.uq", "mix.dkv.norm": "mixer.latent_norm",
               "mix.norm": "mixer.out_norm", "mlp.router": "mlp.router", "mlp.router.b": "mlp.bias"}
    _NORM = {"": "weight", ".b": "bias", ".alpha": "alpha"}

    def load_checkpoint_tensor(self, params, name, tensor):
        """Place one checkpoint tensor; returns False for a name this model does not know."""
        if name == "embed":
            params["embed"].data.copy_(tensor)
            return True
        n = re.fullmatch(r"(final\.norm|l\d+\.norm(?:1|1b|2|2b))(|\.b|\.alpha)", name)
        if n:
            where = "final_norm" if n.group(1) == "final.norm" else "layers." + n.group(1)[1:]
            p = params.get(f"{where}.{self._NORM[n.group(2)]}")
            if p is None:
                return False
            p.data.copy_(tensor.reshape(p.shape))
            return True
        m = re.fullmatch(r"l(\d+)\.(.+)", name)
        if not m or int(m.group(1)) >= len(self.layers):
            return False
        i, rest = int(m.group(1)), m.group(2)
        layer, pre = self.layers[i], f"layers.{i}."
        if rest in self._SIMPLE:
            p = params.get(pre + self._SIMPLE[rest])
            if p is None:
                return False
            p.data.copy_(tensor.reshape(p.shape))
            return True
        mx = layer.mixer
        if isinstance(mx, PagedRotaryAttention) and rest in ("mix.q", "mix.k", "mix.v"):
            a = mx.heads * mx.dim
            b = a + mx.kv_heads * mx.dim
            lo, hi = {"mix.q": (0, a), "mix.k": (a, b), "mix.v": (b, b + mx.kv_heads * mx.vdim)}[rest]
            mx.qkv_proj.data[lo:hi].copy_(tensor)
        elif isinstance(mx, LightningAttention) and rest[4:] in LightningAttention.ROWS and rest.startswith("mix."):
            lo, hi = mx.row_range(rest[4:])
            mx.in_proj.data[lo:hi].copy_(tensor)
        elif isinstance(mx, LatentAttention) and rest in ("mix.dq", "mix.q"):
            mx.qc_proj.data[:mx.q_rows].copy_(tensor)
        elif isinstance(mx, LatentAttention) and rest == "mix.dkv":
            mx.qc_proj.data[mx.q_rows:].copy_(tensor)
        elif isinstance(mx, LatentAttention) and rest == "mix.uk":
            mx.uk.data.copy_(tensor.view(mx.heads, mx.dim, mx.kv_rank))
        elif isinstance(mx, LatentAttention) and rest == "mix.uv":
            mx.uv.data.copy_(tensor.view(mx.heads, mx.vdim, mx.kv_rank))
        else:
            e = re.fullmatch(r"mlp\.e(\d+)\.(gate|up|down)", rest)
            if not e or layer.mlp is None or int(e.group(1)) >= layer.mlp.experts:
                return False
            j, ff = int(e.group(1)), layer.mlp.w_down.shape[2]
            if e.group(2) == "down":
                layer.mlp.w_down.data[j].copy_(tensor)
            else:
                lo = 0 if e.group(2) == "gate" else ff
                layer.mlp.w_gu.data[j, lo:lo + ff].copy_(tensor)
        return True

    def checkpoint_tensors(self, seed=0, std=0.05):
        """Random tensors with the checkpoint's names and shapes (benchmarks and tests without a checkpoint), drawn in
        a fixed order from one seeded generator on the model's device."""
        cfg, dev = self.cfg, self.embed.device
        g = torch.Generator(device=dev).manual_seed(seed)
        W = cfg.hidden_size

        def rnd(*shape, s=std):
            return torch.randn(*shape, generator=g, device=dev, dtype=torch.float32) * s

        def norm(t, name):
            t.update({name: 1 + rnd(W, s=0.1), name + ".b": rnd(W, s=0.1), name + ".alpha": 0.7 + rnd((), s=0.1)})
        t = {"embed": rnd(cfg.vocab_size, W, s=1.0)}
        norm(t, "final.norm")
        for i, spec in enumerate(cfg.layers):
            p, m = f"l{i}.", spec["mixer"]
            norm(t, p + "norm1")
            norm(t, p + "norm1b")
            H, D, V = m["heads"], m["dim"], m.get("vdim", m["dim"])
            if spec["type"] == "attention":
                G = m.get("kv_heads", H)
                t.update({p + "mix.q": rnd(H * D, W, s=W ** -0.5), p + "mix.k": rnd(G * D, W, s=W ** -0.5),
                          p + "mix.v": rnd(G * V, W, s=W ** -0.5), p + "mix.q.norm": 1 + rnd(H * D, s=0.2),
                          p + "mix.k.norm": 1 + rnd(G * D, s=0.2), p + "mix.pb": rnd(H, s=1.0) - 2.0,
                          p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
            elif spec["type"] == "latent_attention":
                R, Rd, Q = m["kv_rank"], m.get("rot_dim", 0), m.get("q_rank", 0)
                if Q:
                    t.update({p + "mix.dq": rnd(Q, W, s=W ** -0.5), p + "mix.dq.norm": 1 + rnd(Q, s=0.2),
                              p + "mix.uq": rnd(H * (D + Rd), Q, s=Q ** -0.5)})
                else:
                    t[p + "mix.q"] = rnd(H * (D + Rd), W, s=W ** -0.5)
                t.update({p + "mix.dkv": rnd(R + Rd, W, s=W ** -0.5), p + "mix.dkv.norm": 1 + rnd(R, s=0.2),
                          p + "mix.uk": rnd(H * D, R, s=R ** -0.5), p + "mix.uv": rnd(H * V, R, s=R ** -0.5),
                          p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
            else:
                for n_, rows in (("q", H * D), ("k", H * D), ("v", H * V), ("g", H * V)):
                    t[p + "mix." + n_] = rnd(rows, W, s=W ** -0.5)
                t.update({p + "mix.norm": 1 + rnd(H * V, s=0.2), p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
            mlp = spec.get("mlp")
            if mlp is None:
                continue
            norm(t, p + "norm2")
            norm(t, p + "norm2b")
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            t.update({p + "mlp.router": rnd(E, W, s=2 * W ** -0.5), p + "mlp.router.b": rnd(E, s=0.3)})
            for e in range(E):
                t.update({f"{p}mlp.e{e}.gate": rnd(ff, W, s=2 * W ** -0.5), f"{p}mlp.e{e}.up": rnd(ff, W, s=2 * W ** -0.5),
                          f"{p}mlp.e{e}.down": rnd(W, ff, s=ff ** -0.5)})
        return {k: v.to(torch.bfloat16) for k, v in t.items()}

    # ------------------------------------------------------------------ cache and state
    def cache_bytes_per_block(self, block_size):
        item, total = self.dtype.itemsize, 0
        for layer in self.layers:
            mx = layer.mixer
            if isinstance(mx, PagedRotaryAttention):
                total += block_size * mx.cache_bytes_per_token(item, block_size)
            elif isinstance(mx, LatentAttention):
                total += block_size * mx.row * item
        return total

    def state_bytes_per_slot(self):
        return sum(l.mixer.state_bytes_per_slot() for l in self.layers if isinstance(l.mixer, LightningAttention))

    def allocate_cache(self, num_blocks, block_size, num_slots, device):
        """A key and a value cache per attention layer, one cache of [latent | rotated key part] rows per latent layer (all
        share the sequences' block tables), one float32 state per state slot and lightning layer."""
        self.num_slots = num_slots
        for layer in self.layers:
            mx = layer.mixer
            if isinstance(mx, PagedRotaryAttention):
                mx.allocate(num_blocks, block_size, self.dtype, device)
            elif isinstance(mx, LatentAttention):
                mx.allocate(0, num_blocks, block_size, self.dtype, device)
            else:
                mx.allocate(num_slots, device)

    def workspaces(self):
        """Scratch buffers that captured decode graphs address."""
        from nanovllm import _hymix, _seqmix
        return [_hymix.decode_workspace, _seqmix.decode_workspace]

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids, positions, trace=None):
        """input_ids int64 [T], positions int32 [T] (the step's context is seq_ops.get_step()) -> final-normed hidden
        [T, width].  ``trace``: a list that receives the residual after every layer (debugging)."""
        dt = self.dtype
        # x = embed[id]; h = what the first mixer reads
        x, h = hy_ops.dyt_residual(None, self.embed, None, self.layers[0].norm1.tensors(), dt, ids=input_ids)
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            y = layer.mixer(h)
            if isinstance(y, tuple):
                y = y[0]
            post = layer.norm1b
            if layer.mlp is not None:
                x, h = hy_ops.dyt_residual(x, y, post.tensors(), layer.norm2.tensors(), dt)
                y, post = layer.mlp(h), layer.norm2b
            # the write of this layer's last sublayer and the norm in front of the next layer's first (or the final norm)
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            x, h = hy_ops.dyt_residual(x, y, post.tensors(), nxt.tensors(), dt)
            if trace is not None:
                trace.append(x.clone())
        return h

    def compute_logits(self, hidden_states):
        """float32 logits of the given rows: products with the embedding table, float32 accumulation AND output."""
        if hidden_states.dtype == torch.float32:
            return F.linear(hidden_states, self.embed)
        if hidden_states.is_cuda and self._f32_out is not False:
            try:
                out = torch.mm(hidden_states, self.embed.t(), out_dtype=torch.float32)
                self._f32_out = True
                return out
            except RuntimeError:
                if self._f32_out:          # it has worked before: this is another fault
                    raise
                self._f32_out = False      # no such GEMM for this shape: the same sums from widened operands
        return F.linear(hidden_states.float(), self.embed.float())
