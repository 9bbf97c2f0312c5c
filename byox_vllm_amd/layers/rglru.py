"""Real-gated linear recurrent unit (the recurrence of Griffin's recurrent block): per channel, with u the output of a
short causal convolution,

    r = sigmoid(W_a u + b_a),  i = sigmoid(W_i u + b_i)            W_a, W_i block-diagonal ('blocks' square blocks)
    a = exp(-c r softplus(lam)),   S_t = a S_(t-1) + sqrt(1 - a^2) (i u),   c = 8

and the block's output is S_t * gelu(y_t) with y the second branch.  The state S (fp32 [channels]) and the convolution's
last inputs live in a request's state slot.  Gate logits are one batched product over the blocks (both gates' rows merged
per block), left in fp32; gates, decay and recurrence are fp32 (csrc/scan.hip).

The module owns no in/out projection: it takes the fp32 x and y columns of a (possibly merged) projection and writes
into a column slice of the caller's buffer."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.conv import CausalConv1d
from byox_vllm_amd.utils.context import get_context


class RealGatedLRU(nn.Module):
    def __init__(self, channels: int, blocks: int, taps: int, c: float = 8.0):
        super().__init__()
        assert channels % blocks == 0
        self.channels, self.blocks, self.bw, self.c = channels, blocks, channels // blocks, float(c)
        bw = self.bw
        self.conv = CausalConv1d(channels, taps)
        # per block: bw rows of the recurrence gate, then bw rows of the input gate
        self.gates = nn.Parameter(torch.empty(blocks, 2 * bw, bw), requires_grad=False)
        self.gates_bias = nn.Parameter(torch.zeros(blocks, 2 * bw), requires_grad=False)
        self.gates.weight_loader = self.gates_bias.weight_loader = self._load_gate
        self.lam = nn.Parameter(torch.zeros(channels), requires_grad=False)
        self.state = torch.tensor([])          # fp32 [slots, channels], bound by the runner

    def _load_gate(self, param, tensor, which: str):
        at = 0 if which == "a" else self.bw
        param.data[:, at:at + self.bw].copy_(tensor.reshape(self.blocks, self.bw, *param.shape[2:]))

    def state_spec(self) -> dict:
        return {"shape": (self.channels,)}

    def state_modules(self):
        return [self.conv, self]

    def forward(self, x: torch.Tensor, y: torch.Tensor, out: torch.Tensor, out_scale: float = 1.0,
                x_bias: torch.Tensor | None = None, y_bias: torch.Tensor | None = None) -> torch.Tensor:
        """``x``, ``y`` fp32 [T, channels] (column slices are fine; their biases may still be to add); ``out``
        [T, >= channels] in the model dtype."""
        ctx = get_context()
        u32, ut = self.conv(x, want_f32=True, want_t=self.lam.dtype != torch.float32, x_bias=x_bias)
        ut = u32 if ut is None else ut
        bw = self.bw
        g = kernels.linear(ut, self.gates.data, self.gates_bias.data, out_dtype=torch.float32, batch=self.blocks,
                           a_batch_stride=bw, w_batch_stride=2 * bw * bw, out_batch_stride=2 * bw)
        return kernels.rglru_scan(u32, g, y, self.lam.data, self.state, ctx.cu_seqlens_q, ctx.past_lens, ctx.state_slots,
                                  bw, out, c=self.c, out_scale=out_scale, y_bias=y_bias)
