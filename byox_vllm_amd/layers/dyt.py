"""Dynamic Tanh: a norm that computes no mean or variance, y = tanh(alpha * x) * weight + b, with a learned scalar
``alpha``.  It reads the fp32 residual stream and, in the same launch, first adds the previous sublayer's output to it
(pre-norm blocks: x <- x + f(norm(x)) means every norm follows a residual add).  The arithmetic is fp32, the result is
rounded to the model dtype for the projections that consume it."""

import torch
from torch import nn

from byox_vllm_amd import kernels


class DynamicTanh(nn.Module):
    def __init__(self, size: int):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(size), requires_grad=False)
        self.b = nn.Parameter(torch.zeros(size), requires_grad=False)
        # fp32 whatever the model dtype: a checkpoint's 16-bit scalar widens exactly, and the kernel reads it as fp32
        self.alpha = nn.Parameter(torch.ones(1, dtype=torch.float32), requires_grad=False)
        self.alpha.weight_loader = lambda p, t: p.data.copy_(t.reshape(1).to(torch.float32))

    def forward(self, residual: torch.Tensor, delta: torch.Tensor | None = None, rows_idx: torch.Tensor | None = None):
        """``residual`` fp32 [T, size], updated in place by ``delta``; ``rows_idx`` picks rows (and leaves the residual
        as it is)."""
        return kernels.dyt_norm(residual, self.alpha.data, self.weight.data, self.b.data, delta=delta, rows_idx=rows_idx)
