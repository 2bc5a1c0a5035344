"""Attention over a paged key/value cache with rotary positions on part of every head and the variations that differ
between designs as constructor arguments:
  proj_norm   RMS norm with a weight over the whole q and the whole k projection, before the rotation
  unit_norm   every rotated q and k head divided by its RMS (no weight)
  sink        "learned": a per-head score that joins the softmax denominator without a value; "zero": the same with score
              0 (one added to the denominator); None: plain softmax
  window, keep_first   window > 0: a query sees the last ``window`` positions and the first ``keep_first`` tokens
  v_mix       values blended with those of the first such layer of the model, (1 - lam) v + lam v_first, before caching
  head_norm   every q and k head RMS-normalised over its own channels with one weight row [dim] shared by the heads
  head_temp   a learned number per query head that multiplies its scores (folded into the normalised query)
  pool        pool > 0 (with a window): beside its window a query sees one key and value per block of ``pool`` tokens that
              lies wholly before the window - the block's mean key and mean value, kept in pooled caches
  kv_source   another PagedRotaryAttention whose keys and values (and, for an equal ``pool``, pooled blocks) this layer
              reads: it has no k/v projection of its own, only queries, mask and output
  rot_dims    0 = positions do not enter the scores
  interleaved the rotation pairs channel 2i with 2i + 1 instead of i with i + rot_dims / 2
  rot_scaling {factor, original, fast, slow}: a frequency table stretched for longer contexts (hy_ops.rotary_table)
  v_unit_norm every value head divided by its RMS (no weight) before it is cached
  chunk       chunk > 0: a query sees a key only inside its own chunk of ``chunk`` positions (counted from position 0)
  weights     "softmax", or "sigmoid": the weight of a visible key is sigmoid(score + b_h) with a learned number per
              query head, not normalised over the keys
Grouped heads: query head h reads key/value head h // (heads / kv_heads).  q, k and v come from ONE merged product."""
import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import hy_ops, seq_ops


class PagedRotaryAttention(nn.Module):
    def __init__(self, width, heads, kv_heads, dim, vdim, scale, eps, rot_dims, rot_base, proj_norm=False, unit_norm=False,
                 sink=None, window=0, keep_first=0, v_mix=False, head_norm=False, head_temp=False, pool=0, kv_source=None,
                 interleaved=False, rot_scaling=None, v_unit_norm=False, chunk=0, weights="softmax"):
        super().__init__()
        assert weights in ("softmax", "sigmoid") and not (weights == "sigmoid" and (sink or pool))
        assert not chunk or (not keep_first and not pool), "a chunked mask goes without kept first tokens and pooled blocks"
        assert not (v_unit_norm and (v_mix or kv_source is not None))
        assert heads % kv_heads == 0 and rot_dims % 2 == 0 and rot_dims <= dim and sink in (None, "learned", "zero")
        assert not pool or (window > 0 and not keep_first), "pooled blocks go with a window that keeps no first tokens"
        assert kv_source is None or (kv_source.kv_heads, kv_source.dim, kv_source.vdim, kv_source.rot_dims) == \
            (kv_heads, dim, vdim, rot_dims), "a layer that reads another layer's keys and values has its head sizes"
        assert kv_source is None or (kv_source.kv_source is None and not v_mix)
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.eps, self.unit_norm = float(scale), eps, unit_norm
        self.window, self.keep_first, self.v_mix = int(window), int(keep_first), v_mix
        self.rot_dims, self.rot_base = rot_dims, rot_base
        self.pool = int(pool)
        self.interleaved, self.rot_scaling, self.rot_mag = bool(interleaved), rot_scaling, 1.0
        self.v_unit_norm, self.chunk, self.sigmoid = bool(v_unit_norm), int(chunk), weights == "sigmoid"
        self.__dict__["kv_source"] = kv_source              # (not a submodule of this layer)
        own_kv = kv_source is None
        self.qkv_proj = nn.Parameter(torch.empty(heads * dim + (kv_heads * (dim + vdim) if own_kv else 0), width),
                                     requires_grad=False)
        self.o_proj = nn.Parameter(torch.empty(width, heads * vdim), requires_grad=False)
        f32 = dict(dtype=torch.float32)
        self.q_norm = nn.Parameter(torch.ones(heads * dim), requires_grad=False) if proj_norm else None
        self.k_norm = nn.Parameter(torch.ones(kv_heads * dim), requires_grad=False) if proj_norm else None
        self.sink = nn.Parameter(torch.zeros(heads, **f32), requires_grad=False) if sink else None
        self.lam = nn.Parameter(torch.zeros(1, **f32), requires_grad=False) if v_mix else None
        self.q_head_norm = nn.Parameter(torch.ones(dim), requires_grad=False) if head_norm else None
        self.k_head_norm = nn.Parameter(torch.ones(dim), requires_grad=False) if head_norm and own_kv else None
        self.temp = nn.Parameter(torch.ones(heads, **f32), requires_grad=False) if head_temp else None
        self.head_bias = nn.Parameter(torch.zeros(heads, **f32), requires_grad=False) if self.sigmoid else None
        self.inv_freq = None       # f32 [rot_dims / 2], made with the cache
        self.k_cache = self.v_cache = self.kp_cache = self.vp_cache = None

    def _pools_own(self):
        """Whether this layer keeps pooled blocks of its own (a reader with the source's block size shares the source's)."""
        return self.pool > 0 and (self.kv_source is None or self.kv_source.pool != self.pool)

    def allocate(self, num_blocks, block_size, dtype, device):
        """Caches for ``num_blocks`` pages.  A layer that reads another layer's keys and values must be allocated after it."""
        src = self.kv_source
        if src is None:
            self.k_cache = torch.zeros(num_blocks, block_size, self.kv_heads, self.dim, dtype=dtype, device=device)
            self.v_cache = torch.zeros(num_blocks, block_size, self.kv_heads, self.vdim, dtype=dtype, device=device)
        else:
            assert src.k_cache is not None
            self.k_cache, self.v_cache = src.k_cache, src.v_cache
        if self._pools_own():
            rows = hy_ops.pool_rows_per_page(block_size, self.pool)
            self.kp_cache = torch.zeros(num_blocks, rows, self.kv_heads, self.dim, dtype=dtype, device=device)
            self.vp_cache = torch.zeros(num_blocks, rows, self.kv_heads, self.vdim, dtype=dtype, device=device)
        elif self.pool > 0:
            self.kp_cache, self.vp_cache = src.kp_cache, src.vp_cache
        if self.rot_dims:
            self.inv_freq, self.rot_mag = hy_ops.rotary_table(self.rot_dims, self.rot_base, device, self.rot_scaling)
        else:
            self.inv_freq = None

    def cache_bytes_per_token(self, itemsize, block_size=64):
        own = self.kv_heads * (self.dim + self.vdim) * itemsize
        pooled = own * hy_ops.pool_rows_per_page(block_size, self.pool) / block_size if self._pools_own() else 0
        return int((own if self.kv_source is None else 0) + pooled + 0.999)

    def forward(self, h, v_first=None):
        """h [T, width] -> (output [T, width], this layer's own values [T, kv_heads * vdim] before any blending)."""
        ctx = seq_ops.get_step()
        qkv = F.linear(h, self.qkv_proj)
        own_kv = self.kv_source is None
        q = hy_ops.qkv_prepare(qkv, self.heads, self.kv_heads, self.dim, self.vdim, self.q_norm, self.k_norm, self.eps,
                               self.inv_freq, self.unit_norm, ctx, self.k_cache if own_kv else None,
                               self.v_cache if own_kv else None, v_first if self.v_mix else None, self.lam,
                               self.q_head_norm, self.k_head_norm, self.temp, self.interleaved, self.rot_mag, self.v_unit_norm)
        if self._pools_own():                  # the blocks this step completes (the keys are in the cache by now)
            hy_ops.pool_blocks(self.k_cache, self.v_cache, self.kp_cache, self.vp_cache, self.pool, ctx)
        pooled = (self.kp_cache, self.vp_cache, self.pool) if self.pool > 0 else None
        o = hy_ops.paged_attention(q, self.k_cache, self.v_cache, ctx, self.scale, self.sink, self.window, self.keep_first,
                                   pooled=pooled, chunk=self.chunk, sigmoid=self.sigmoid, head_bias=self.head_bias)
        return F.linear(o, self.o_proj), (qkv[:, (self.heads + self.kv_heads) * self.dim:] if own_kv else None)
