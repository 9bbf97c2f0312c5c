"""Token sampler (interface of nanovllm/layers/sampler.py:5-15).

Gumbel-max sampling as in the reference, with two additions: temperature 0
means argmax, and the Exp(1) draws can be injected (``noise``) so a test can
replay the reference's random numbers.
"""

import torch
from torch import nn

from byox_vllm_amd import kernels


class Sampler(nn.Module):
    def __init__(self, seed: int = 0):
        super().__init__()
        self.seed = seed
        self.calls = 0

    def forward(self, logits: torch.Tensor, temperatures: torch.Tensor, noise: torch.Tensor | None = None):
        self.calls += 1
        if logits.dtype == torch.float32:      # models that hand over fp32 logits (fp32 residual stream)
            assert noise is None
            return kernels.sample_f32(logits, temperatures, seed=(self.seed << 32) + self.calls)
        return kernels.sample(logits, temperatures, noise=noise, seed=(self.seed << 32) + self.calls)
