"""Linear attention with a constant decay per head ("lightning" attention): a recurrent mixer whose per-head state
S [dim, vdim] forgets at a fixed rate and learns the outer product of key and value,
    S <- decay_h S + k v^T,   o = S^T q,   q, k, v = silu of projections of the input,
with no other scale.  The heads' outputs, side by side, are RMS-normalised together with a weight, gated by
sigmoid(W_g h) and projected.  The state is float32, one [heads, dim, vdim] block per state slot; q, k, v and g come from
ONE merged product."""
import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import hy_ops, seq_ops


class LightningAttention(nn.Module):
    def __init__(self, width, heads, dim, vdim, decay, eps):
        super().__init__()
        assert len(decay) == heads
        self.heads, self.dim, self.vdim, self.eps = heads, dim, vdim, eps
        hd, hv = heads * dim, heads * vdim
        # rows: q | k | v | g
        self.in_proj = nn.Parameter(torch.empty(2 * hd + 2 * hv, width), requires_grad=False)
        self.decay = nn.Parameter(torch.tensor([float(d) for d in decay], dtype=torch.float32), requires_grad=False)
        self.out_norm = nn.Parameter(torch.ones(hv), requires_grad=False)
        self.o_proj = nn.Parameter(torch.empty(width, hv), requires_grad=False)
        self.state = None          # f32 [slots, heads, dim, vdim]

    ROWS = ("q", "k", "v", "g")

    def row_range(self, name):
        hd, hv = self.heads * self.dim, self.heads * self.vdim
        lo = {"q": 0, "k": hd, "v": 2 * hd, "g": 2 * hd + hv}[name]
        return lo, lo + (hd if name in ("q", "k") else hv)

    def allocate(self, num_slots, device):
        self.state = torch.zeros(num_slots, self.heads, self.dim, self.vdim, dtype=torch.float32, device=device)

    def state_bytes_per_slot(self):
        return self.heads * self.dim * self.vdim * 4

    def forward(self, h):
        ctx = seq_ops.get_step()
        hd, hv = self.heads * self.dim, self.heads * self.vdim
        p = F.linear(h, self.in_proj)
        o = hy_ops.lightning_recurrence(p, 0, hd, 2 * hd, self.heads, self.dim, self.vdim, self.decay, self.state, ctx)
        # the norm runs over all heads at once: one "head" of heads * vdim channels
        y = hy_ops.delta_gate_norm(o.view(-1, 1, hv), p[:, 2 * hd + hv:], self.out_norm, self.eps, h.dtype)
        return F.linear(y, self.o_proj)
