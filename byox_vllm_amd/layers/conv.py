"""Short causal convolution per channel, out[t] = act(b + sum_j w[:, j] x[t - (taps - 1 - j)]), with zeros before a
sequence's start.  The last taps - 1 inputs are a request's state (fp32 [taps - 1, channels] in a state slot), so a
prompt may arrive in pieces of any size and decoding continues from it (csrc/scan.hip)."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.utils.context import get_context


class CausalConv1d(nn.Module):
    def __init__(self, channels: int, taps: int, activation: str | None = None):
        super().__init__()
        self.channels, self.taps = channels, taps
        self.act = {None: 0, "silu": 1}[activation]
        self.weight = nn.Parameter(torch.empty(channels, taps), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(channels), requires_grad=False)
        self.state = torch.tensor([])          # fp32 [slots, taps - 1, channels], bound by the runner

    def state_spec(self) -> dict:
        return {"shape": (self.taps - 1, self.channels)}

    def forward(self, x: torch.Tensor, want_f32: bool = True, want_t: bool = False, x_bias: torch.Tensor | None = None):
        """``x`` fp32 [T, channels] (a column slice of a wider buffer is fine; ``x_bias`` is added to it first)
        -> (fp32 rows, rows in the model dtype)."""
        ctx = get_context()
        return kernels.causal_conv(x, self.weight.data, self.bias.data, self.state, ctx.cu_seqlens_q, ctx.past_lens,
                                   ctx.state_slots, ctx.seq_of_token, act=self.act, want_f32=want_f32, want_t=want_t, x_bias=x_bias)
