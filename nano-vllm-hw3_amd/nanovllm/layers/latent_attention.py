"""Latent attention: keys and values are up-projections of one small per-token latent, and only the latent is cached.
The key up-projection is folded into the query ("absorbed": q'_h = W_uk,h^T q_h, so that
q_h . k_h = q'_h . c) and the value up-projection is applied after the attention sum, which makes the cached latent
both key and value of a multi-query attention with ``heads`` query heads of size ``kv_rank``.

Without further arguments positions do not enter.  ``rot_dim`` > 0 adds a rotated part: every query head carries
``rot_dim`` more channels, the down-projection ``rot_dim`` more rows that form ONE key part shared by all heads; the
first ``rot_dims`` channels of both turn with the position (channel 2i pairs with 2i + 1, angle = position *
rot_base^(-2i/rot_dims)) and their product joins the score.  The cache row is then [latent | rotated key part], the
absorbed query [W_uk^T q | rotated q part], and only the latent columns are values.  ``window`` > 0: a query sees itself
and the window - 1 tokens before it.  ``q_rank`` > 0: the queries come through a latent of their own,
q = W_uq rms_norm(W_dq h) with a weight on the norm (the down-projection shares its product with the key/value latent's)."""
import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import seq_ops


class LatentAttention(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, vdim: int, kv_rank: int, scale: float, eps: float,
                 rot_dim: int = 0, rot_dims: int = 0, rot_base: float = 10000.0, window: int = 0, q_rank: int = 0):
        super().__init__()
        assert rot_dims % 2 == 0 and rot_dims <= rot_dim
        self.heads, self.dim, self.vdim, self.kv_rank, self.scale, self.eps = heads, dim, vdim, kv_rank, float(scale), eps
        self.rot_dim, self.rot_dims, self.rot_base, self.window = rot_dim, rot_dims, rot_base, int(window)
        self.row = kv_rank + rot_dim           # columns of a cache row
        self.inv_freq = None                   # f32 [rot_dims / 2], made with the cache
        # query and latent down-projection share one product: rows [0, heads*(dim+rot_dim)) = W_q (per head [dim | rot_dim]),
        # then kv_rank rows of W_dkv and its rot_dim rows of the shared key part
        # with a query latent: rows [0, q_rank) = W_dq instead, and W_uq [heads*(dim+rot_dim), q_rank] follows its norm
        self.q_rank = int(q_rank)
        self.q_rows = self.q_rank or heads * (dim + rot_dim)
        self.qc_proj = nn.Parameter(torch.empty(self.q_rows + kv_rank + rot_dim, width), requires_grad=False)
        self.q_latent_norm = nn.Parameter(torch.ones(q_rank), requires_grad=False) if q_rank else None
        self.uq = nn.Parameter(torch.empty(heads * (dim + rot_dim), q_rank), requires_grad=False) if q_rank else None
        self.latent_norm = nn.Parameter(torch.ones(kv_rank), requires_grad=False)
        self.uk = nn.Parameter(torch.empty(heads, dim, kv_rank), requires_grad=False)      # per head [dim, kv_rank]
        self.uv = nn.Parameter(torch.empty(heads, vdim, kv_rank), requires_grad=False)     # per head [vdim, kv_rank]
        self.o_proj = nn.Parameter(torch.empty(width, heads * vdim), requires_grad=False)
        self.cache = {}            # layer run -> [blocks, block_size, kv_rank + rot_dim]

    def allocate(self, run, num_blocks, block_size, dtype, device):
        self.cache[run] = torch.zeros(num_blocks, block_size, self.row, dtype=dtype, device=device)
        if self.rot_dims and self.inv_freq is None:
            i = torch.arange(self.rot_dims // 2, dtype=torch.float64)
            self.inv_freq = (float(self.rot_base) ** (-2.0 * i / self.rot_dims)).to(torch.float32).to(device)

    def forward(self, h, run: int = 0):
        if self.rot_dim or self.window or self.q_rank:
            return self._forward_rotated(h, run)
        ctx = seq_ops.get_step()
        T = h.shape[0]
        H, D = self.heads, self.dim
        qc = F.linear(h, self.qc_proj)                                     # [T, H*D + R]
        cache = self.cache[run]
        seq_ops.latent_norm_store(qc[:, H * D:], self.latent_norm, self.eps, cache, ctx.slot_mapping)
        q = qc[:, :H * D].view(T, H, D).transpose(0, 1)                    # [H, T, D]
        qa = torch.bmm(q, self.uk).transpose(0, 1).contiguous()            # absorbed queries [T, H, R]
        ol = seq_ops.latent_attention(qa, cache, ctx, self.scale)          # [T, H, R]
        ov = torch.bmm(ol.transpose(0, 1), self.uv.transpose(1, 2))        # [H, T, V]
        return F.linear(ov.transpose(0, 1).reshape(T, H * self.vdim), self.o_proj)

    def _forward_rotated(self, h, run):
        ctx = seq_ops.get_step()
        T = h.shape[0]
        H, D, Rd, R = self.heads, self.dim, self.rot_dim, self.kv_rank
        nq = self.q_rows
        qc = F.linear(h, self.qc_proj)                                     # [T, H*(D+Rd) (or q_rank) + R + Rd]
        cache = self.cache[run]
        qa = torch.empty((T, H, self.row), dtype=h.dtype, device=h.device)  # absorbed queries [T, H, R | Rd]
        if self.q_rank:
            q2 = F.linear(seq_ops.rms_norm_rows(qc[:, :nq], self.q_latent_norm, self.eps), self.uq)
        else:
            q2 = qc[:, :nq]
        q = q2.view(T, H, D + Rd)
        # q'_h = W_uk,h^T q_h straight into the first R columns of every head's row
        torch.bmm(q[..., :D].transpose(0, 1), self.uk, out=qa.transpose(0, 1)[..., :R])
        seq_ops.latent_rope_store(qc[:, nq:], self.latent_norm, self.eps, q2, qa, self.inv_freq, self.rot_dims, H, D, R, Rd,
                                  cache, ctx)
        ol = seq_ops.latent_attention(qa, cache, ctx, self.scale, value_cols=R, window=self.window)      # [T, H, R]
        ov = torch.bmm(ol.transpose(0, 1), self.uv.transpose(1, 2))        # [H, T, V]
        return F.linear(ov.transpose(0, 1).reshape(T, H * self.vdim), self.o_proj)
