"""Feed-forward layers beyond the SiLU-gated MLP: a dense layer with the PolyNorm activation, the clamped GLU expert,
and a routed mixture of such experts with group-limited top-k routing and an optional shared expert."""
import torch
import torch.nn.functional as F
from torch import nn

from nanovllm import seq_ops


class PolyNormMLP(nn.Module):
    """down(PolyNorm(up(h))): PolyNorm(z) = a N(z) + b N(z^2) + c N(z^3) + e with N = division by the row's RMS."""

    def __init__(self, width: int, ff: int, eps: float):
        super().__init__()
        self.eps = eps
        self.up = nn.Parameter(torch.empty(ff, width), requires_grad=False)
        self.down = nn.Parameter(torch.empty(width, ff), requires_grad=False)
        self.coef = nn.Parameter(torch.zeros(4, dtype=torch.float32), requires_grad=False)     # a, b, c, e

    def forward(self, h):
        return F.linear(seq_ops.poly_norm(F.linear(h, self.up), self.coef, self.eps), self.down)


class ClampedGLU(nn.Module):
    """down(g * sigmoid(alpha g) * (u + 1)) with g = min(gate(h), limit), u = clamp(up(h), +-limit); no biases."""

    def __init__(self, width: int, ff: int, limit: float, alpha: float = 1.702):
        super().__init__()
        self.ff, self.limit, self.alpha = ff, float(limit), alpha
        self.gate_up = nn.Parameter(torch.empty(2 * ff, width), requires_grad=False)          # gate rows, then up rows
        self.down = nn.Parameter(torch.empty(width, ff), requires_grad=False)

    def forward(self, h):
        return F.linear(seq_ops.clamped_glu(F.linear(h, self.gate_up), self.limit, self.alpha), self.down)


class RoutedExperts(nn.Module):
    """Softmax router in float32; experts in ``groups`` equal groups of neighbours, only the ``keep`` groups with the
    largest member score are eligible; the ``top`` best eligible experts run, weighted by their renormalised scores.
    A shared expert (its own size and limit) runs for every token and is added.

    Variations: ``score`` = "sigmoid" (independent scores instead of a softmax); ``correction``: a learned per-expert
    number added to the scores for the CHOICE of groups and experts only (the weights stay the scores); ``group_top``: a
    group scores the sum of that many of its largest choice scores instead of the largest; ``renorm`` = False: the chosen
    scores weigh as they are; ``act`` = "gelu" / "gelu_tanh": an expert is down(gelu(up h)), no gate, no clamp;
    ``act`` = "silu_glu": an expert is down(silu(gate h) * up h), no clamp; ``bias``: a learned number per expert added to
    the router's logits (with softmax scores and ``renorm`` the weights are the softmax over the chosen logits)."""

    ACTS = {"clamped_glu": seq_ops.ACT_CLAMPED_GLU, "gelu": seq_ops.ACT_GELU, "gelu_tanh": seq_ops.ACT_GELU_TANH,
            "silu_glu": seq_ops.ACT_SILU_GLU}

    def __init__(self, width: int, experts: int, top: int, ff: int, limit: float = 0.0, groups: int = 1, keep: int = 1,
                 shared: ClampedGLU = None, alpha: float = 1.702, score: str = "softmax", correction: bool = False,
                 group_top: int = 1, renorm: bool = True, act: str = "clamped_glu", bias: bool = False):
        super().__init__()
        if act == "silu_glu":                  # the gated form with nothing clamped and a plain sigmoid
            limit, alpha = float("inf"), 1.0
        self.experts, self.top, self.groups, self.keep, self.limit, self.alpha = experts, top, groups, keep, float(limit), alpha
        self.score = {"softmax": seq_ops.ROUTE_SOFTMAX, "sigmoid": seq_ops.ROUTE_SIGMOID}[score]
        self.group_top, self.renorm, self.act_kind = group_top, renorm, self.ACTS[act]
        self.parts = 2 if self.act_kind in seq_ops.GATED_ACTS else 1           # gate and up rows, or up rows alone
        self.bias = nn.Parameter(torch.zeros(experts, dtype=torch.float32), requires_grad=False) if bias else None
        self.correction = nn.Parameter(torch.zeros(experts, dtype=torch.float32), requires_grad=False) if correction else None
        self.router = nn.Parameter(torch.empty(experts, width, dtype=torch.float32), requires_grad=False)
        self.w_gu = nn.Parameter(torch.empty(experts, self.parts * ff, width), requires_grad=False)
        self.w_down = nn.Parameter(torch.empty(experts, width, ff), requires_grad=False)
        self.shared = shared
        self._tiled = None         # the expert weights in the layout the matrix-core kernels stream (made at the first step)

    def forward(self, h):
        if self._tiled is None and h.is_cuda and h.dtype == torch.bfloat16:
            self._tiled = (seq_ops.tile_expert_weights(self.w_gu, self.parts), seq_ops.tile_expert_weights(self.w_down))
        idx, wts = seq_ops.moe_route(h, self.router, self.top, self.groups, self.keep, self.score, self.correction,
                                     self.group_top, self.renorm, self.bias)
        shared = self.shared(h) if self.shared is not None else None
        return seq_ops.moe_experts(h, idx, wts, self.w_gu, self.w_down, self.limit, self.alpha, shared, tiled=self._tiled,
                                   act_kind=self.act_kind)


class ReluSquaredMLP(nn.Module):
    """down(relu(up(h))^2).  ``extra_rows`` more rows of the up product belong to the caller (a gate that reads the same
    h): forward returns (result, those columns of the product)."""

    def __init__(self, width: int, ff: int, extra_rows: int = 0):
        super().__init__()
        self.ff = ff
        self.up = nn.Parameter(torch.empty(ff + extra_rows, width), requires_grad=False)
        self.down = nn.Parameter(torch.empty(width, ff), requires_grad=False)

    def forward(self, h):
        from nanovllm import hy_ops
        z = F.linear(h, self.up)
        return F.linear(hy_ops.relu_squared(z[:, :self.ff]), self.down), z[:, self.ff:]
