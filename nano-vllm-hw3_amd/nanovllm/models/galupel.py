"""Galupel: a decoder-only model whose layers are listed one by one in config.json.  A layer has one of two mixers -
grouped-head attention without positions whose queries see a sliding window of tokens and, beside it, one pooled key and
value per block of tokens that lies wholly before the window ("attention"; a layer may read another layer's keys and
values), or latent attention with a rotated key part and a sliding window ("latent_attention") - and optionally a
mixture of GELU experts behind a sigmoid router with a choice correction and group-limited top-k.  The residual is
float32 and normalised on the sublayers' OUTPUT: x <- x + norm(f(x)), f reading x itself, with an RMS norm taken over
groups of channels; the embedding passes through the same norm, the logits are products with the embedding table, scaled
and soft-capped.

Read from config.json: vocab, width, norm.{eps, groups}, logit_scale, logit_softcap, and per layer
  {type, mixer: {heads, kv_heads, dim, vdim, scale, mask: {size, pool}, kv_from} |
                {heads, dim, rot_dim, vdim, kv_rank, scale, rot: {dims, base}, mask: {size}},
   mlp: null | {kind: moe, expert: {ff}, router: {experts, top, groups: {count, keep}}}}.
Checkpoint tensors: embed, embed.norm, final.norm, and per layer l<i>.{norm1, norm2, mix.*, mlp.*}.

The model is stepped with portions of sequences (nanovllm.seq_ops.StepContext).  It owns, per attention layer with keys
of its own, a paged key and value cache and the pooled caches beside them, and per latent layer one paged cache of
[latent | rotated key part] rows; all layers share a sequence's block table.  There is no per-sequence state."""
import re

import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import hy_ops, seq_ops
from nanovllm.layers.feedforward import RoutedExperts
from nanovllm.layers.latent_attention import LatentAttention
from nanovllm.layers.rotary_attention import PagedRotaryAttention

GROUP_TOP = 2          # a group of experts scores the sum of its two largest choice scores


class GalupelLayer(nn.Module):
    def __init__(self, cfg, spec, earlier):
        super().__init__()
        W, eps, m = cfg.hidden_size, cfg.norm_eps, spec["mixer"]
        self.kind = spec["type"]
        mask = m.get("mask") or {}
        self.norm1 = nn.Parameter(torch.ones(W), requires_grad=False)
        if self.kind == "attention":
            src = m.get("kv_from")
            if src is not None and not (0 <= src < len(earlier) and isinstance(earlier[src].mixer, PagedRotaryAttention)):
                raise ValueError(f"kv_from: {src} is not an earlier attention layer")
            source = earlier[src].mixer if src is not None else None
            # a reader's key/value head count and value size are its source's (config.json may repeat them)
            kv_heads = m["kv_heads"] if "kv_heads" in m or source is None else source.kv_heads
            vdim = m["vdim"] if "vdim" in m or source is None else source.vdim
            self.mixer = PagedRotaryAttention(W, m["heads"], kv_heads, m["dim"], vdim, m["scale"], eps, 0, 1.0,
                                              window=mask.get("size", 0), pool=mask.get("pool", 0), head_norm=True,
                                              head_temp=True, kv_source=source)
        elif self.kind == "latent_attention":
            rot = m.get("rot") or {}
            self.mixer = LatentAttention(W, m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["scale"], eps,
                                         rot_dim=m.get("rot_dim", 0), rot_dims=rot.get("dims", 0), rot_base=rot.get("base", 10000.0),
                                         window=mask.get("size", 0))
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            if mlp["kind"] != "moe":
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
            r = mlp["router"]
            g = r.get("groups") or {"count": 1, "keep": 1}
            self.norm2 = nn.Parameter(torch.ones(W), requires_grad=False)
            self.mlp = RoutedExperts(W, r["experts"], r["top"], mlp["expert"]["ff"], groups=g["count"], keep=g["keep"],
                                     score="sigmoid", correction=True, group_top=GROUP_TOP, renorm=False, act="gelu")


class GalupelForCausalLM(nn.Module):
    runs_portions = True           # stepped with portions; owns its caches
    default_block_size = 64
    native_library = ("hymix", "seqmix")      # grouped-norm residual and pooled-window attention; latent attention and experts

    @staticmethod
    def normalize_config(d: dict) -> dict:
        d = dict(d)
        d["vocab_size"], d["hidden_size"] = d["vocab"], d["width"]
        d["max_position_embeddings"] = d.get("max_positions", 1 << 20)
        d["norm_eps"], d["norm_groups"] = d["norm"]["eps"], d["norm"].get("groups", 1)
        d["logit_scale"] = d.get("logit_scale", 1.0)
        d["logit_softcap"] = d.get("logit_softcap") or 0.0
        if d["hidden_size"] % d["norm_groups"]:
            raise ValueError("norm.groups must divide width")
        d.setdefault("torch_dtype", "bfloat16")
        return d

    def __init__(self, cfg):
        super().__init__()
        self.cfg = cfg
        W = cfg.hidden_size
        self.dtype = torch.get_default_dtype()
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W), requires_grad=False)
        self.embed_norm = nn.Parameter(torch.ones(W), requires_grad=False)
        layers = []
        for spec in cfg.layers:
            layers.append(GalupelLayer(cfg, spec, layers))
        self.layers = nn.ModuleList(layers)
        self.final_norm = nn.Parameter(torch.ones(W), requires_grad=False)
        self._f32_out = None       # whether the vendor GEMM writes float32 from 16-bit operands for the head's shape

    # ------------------------------------------------------------------ checkpoint names
    _SIMPLE = {"norm1": "norm1", "norm2": "norm2", "mix.o": "mixer.o_proj", "mix.q.norm": "mixer.q_head_norm",
               "mix.k.norm": "mixer.k_head_norm", "mix.temp": "mixer.temp", "mix.dkv.norm": "mixer.latent_norm",
               "mlp.router": "mlp.router", "mlp.correction": "mlp.correction"}

    def load_checkpoint_tensor(self, params, name, tensor):
        """Place one checkpoint tensor; returns False for a name this model does not know."""
        top = {"embed": "embed", "embed.norm": "embed_norm", "final.norm": "final_norm"}
        if name in top:
            params[top[name]].data.copy_(tensor)
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
            if hi > mx.qkv_proj.shape[0]:
                return False                                   # keys or values for a layer that reads another layer's
            mx.qkv_proj.data[lo:hi].copy_(tensor)
        elif isinstance(mx, LatentAttention) and rest == "mix.q":
            mx.qc_proj.data[:mx.heads * (mx.dim + mx.rot_dim)].copy_(tensor)
        elif isinstance(mx, LatentAttention) and rest == "mix.dkv":
            mx.qc_proj.data[mx.heads * (mx.dim + mx.rot_dim):].copy_(tensor)
        elif isinstance(mx, LatentAttention) and rest == "mix.uk":
            mx.uk.data.copy_(tensor.view(mx.heads, mx.dim, mx.kv_rank))
        elif isinstance(mx, LatentAttention) and rest == "mix.uv":
            mx.uv.data.copy_(tensor.view(mx.heads, mx.vdim, mx.kv_rank))
        else:
            e = re.fullmatch(r"mlp\.e(\d+)\.(up|down)", rest)
            if not e or layer.mlp is None or int(e.group(1)) >= layer.mlp.experts:
                return False
            w = layer.mlp.w_gu if e.group(2) == "up" else layer.mlp.w_down
            w.data[int(e.group(1))].copy_(tensor)
        return True

    def checkpoint_tensors(self, seed=0, std=0.05):
        """Random tensors with the checkpoint's names and shapes (benchmarks and tests without a checkpoint), drawn in
        a fixed order from one seeded generator on the model's device."""
        cfg, dev = self.cfg, self.embed.device
        g = torch.Generator(device=dev).manual_seed(seed)
        W = cfg.hidden_size

        def rnd(*shape, s=std):
            return torch.randn(*shape, generator=g, device=dev, dtype=torch.float32) * s
        t = {"embed": rnd(cfg.vocab_size, W, s=1.0), "embed.norm": 1 + rnd(W), "final.norm": 1 + rnd(W)}
        for i, spec in enumerate(cfg.layers):
            p, m = f"l{i}.", spec["mixer"]
            t[p + "norm1"] = 0.5 + rnd(W)
            H, D, V = m["heads"], m["dim"], m["vdim"]
            if spec["type"] == "attention":
                G = m.get("kv_heads", 1)                       # (not needed by a layer that reads another layer's)
                t.update({p + "mix.q": rnd(H * D, W, s=W ** -0.5), p + "mix.q.norm": 1 + rnd(D, s=0.2),
                          p + "mix.temp": 1 + rnd(H, s=0.2), p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
                if m.get("kv_from") is None:
                    t.update({p + "mix.k": rnd(G * D, W, s=W ** -0.5), p + "mix.v": rnd(G * V, W, s=W ** -0.5),
                              p + "mix.k.norm": 1 + rnd(D, s=0.2)})
            else:
                R, Rd = m["kv_rank"], m.get("rot_dim", 0)
                t.update({p + "mix.q": rnd(H * (D + Rd), W, s=W ** -0.5), p + "mix.dkv": rnd(R + Rd, W, s=W ** -0.5),
                          p + "mix.dkv.norm": 1 + rnd(R, s=0.2), p + "mix.uk": rnd(H * D, R, s=R ** -0.5),
                          p + "mix.uv": rnd(H * V, R, s=R ** -0.5), p + "mix.o": rnd(W, H * V, s=(H * V) ** -0.5)})
            mlp = spec.get("mlp")
            if mlp is None:
                continue
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            t.update({p + "norm2": 0.5 + rnd(W), p + "mlp.router": rnd(E, W, s=2 * W ** -0.5), p + "mlp.correction": rnd(E, s=0.3)})
            for e in range(E):
                t.update({f"{p}mlp.e{e}.up": rnd(ff, W, s=2 * W ** -0.5), f"{p}mlp.e{e}.down": rnd(W, ff, s=ff ** -0.5)})
        return {k: v.to(torch.bfloat16) for k, v in t.items()}

    # ------------------------------------------------------------------ cache and state
    def cache_bytes_per_block(self, block_size):
        item, total = self.dtype.itemsize, 0
        for layer in self.layers:
            mx = layer.mixer
            if isinstance(mx, PagedRotaryAttention):
                total += block_size * mx.cache_bytes_per_token(item, block_size)
            else:
                total += block_size * mx.row * item
        return total

    def state_bytes_per_slot(self):
        return 0

    def allocate_cache(self, num_blocks, block_size, num_slots, device):
        """Per attention layer with keys of its own a key and a value cache and their pooled caches (a layer that reads
        another's takes that layer's; it keeps pooled caches only for a block size of its own); per latent layer one cache
        of [latent | rotated key part] rows.  All share the sequences' block tables."""
        self.num_slots = num_slots
        for layer in self.layers:                  # in order: a reader's source comes before it
            if isinstance(layer.mixer, PagedRotaryAttention):
                layer.mixer.allocate(num_blocks, block_size, self.dtype, device)
            else:
                layer.mixer.allocate(0, num_blocks, block_size, self.dtype, device)

    def workspaces(self):
        """Scratch buffers that captured decode graphs address."""
        from nanovllm import _hymix, _seqmix
        return [_hymix.decode_workspace, _seqmix.decode_workspace]

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids, positions, trace=None):
        """input_ids int64 [T], positions int32 [T] (the step's context is seq_ops.get_step()) -> final-normed hidden
        [T, width].  ``trace``: a list that receives the residual after every layer (debugging)."""
        cfg, dt = self.cfg, self.dtype
        eps, groups = cfg.norm_eps, cfg.norm_groups
        # x = norm(embed[id]); h = x in the storage type, what the first mixer reads
        x, h = hy_ops.group_norm_residual(None, self.embed, self.embed_norm, groups, eps, dt, ids=input_ids)
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            y = layer.mixer(h)
            if isinstance(y, tuple):
                y = y[0]
            last = i + 1 == n
            if layer.mlp is not None:
                x, h = hy_ops.group_norm_residual(x, y, layer.norm1, groups, eps, dt)
                y, post = layer.mlp(h), layer.norm2
            else:
                post = layer.norm1
            # the write of this layer's last sublayer and what the next reader needs (behind the last layer: the final norm)
            x, h = hy_ops.group_norm_residual(x, y, post, groups, eps, dt, next_w=self.final_norm if last else None)
            if trace is not None:
                trace.append(x.clone())
        return h

    def compute_logits(self, hidden_states):
        """float32 logits of the given rows: products with the embedding table (float32 accumulation AND output), times
        logit_scale, soft-capped."""
        if hidden_states.dtype == torch.float32:
            out = F.linear(hidden_states, self.embed)
        else:
            out = None
            if hidden_states.is_cuda and self._f32_out is not False:
                try:
                    out = torch.mm(hidden_states, self.embed.t(), out_dtype=torch.float32)
                    self._f32_out = True
                except RuntimeError:
                    if self._f32_out:          # it has worked before: this is another fault
                        raise
                    self._f32_out = False      # no such GEMM for this shape: the same sums from widened operands
            if out is None:
                out = F.linear(hidden_states.float(), self.embed.float())
        return hy_ops.scale_softcap_(out.contiguous(), self.cfg.logit_scale, self.cfg.logit_softcap)
