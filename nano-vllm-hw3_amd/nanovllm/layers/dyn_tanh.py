"""Dynamic Tanh: a norm without statistics, dyt(z) = tanh(alpha z) * w + b per channel with a learned scalar alpha.
``DynTanh`` holds one norm's tensors (alpha in float32 on the device, so that no step waits for its value);
hy_ops.dyt_residual applies them at the boundary between two sublayers of a float32 residual:
    h = dyt_pre(x);   x <- x + dyt_post(sublayer(h))."""
import torch
from torch import nn


class DynTanh(nn.Module):
    def __init__(self, width: int):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(width), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(width), requires_grad=False)
        self.alpha = nn.Parameter(torch.ones(1, dtype=torch.float32), requires_grad=False)

    def tensors(self):
        return self.weight, self.bias, self.alpha
