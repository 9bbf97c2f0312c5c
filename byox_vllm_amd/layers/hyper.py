"""A residual kept as several fp32 streams ("hyper-connections"), its RMS norm, and the token shift.

Instead of one residual x a model carries S copies x_1 .. x_S, all equal at the start.  A sublayer f with the learned
numbers in[S], out[S], mix[S, S] reads one weighted sum of them and writes back into all of them:

    u = sum_s in[s] x_s;   y = f(norm(u));   x_t <- sum_s mix[s, t] x_s + out[t] y     (mix indexed [from, to])

With S = 1 and in = out = mix = 1 this is the pre-norm residual x <- x + f(norm(x)).  ``StreamNorm`` is the norm of
such a sublayer: it first folds the PREVIOUS sublayer's output into the streams (so streams are read and written once
per sublayer), then normalises this sublayer's weighted sum: u / sqrt(mean(u^2) + eps) * (1 + w), weight stored around
zero.  All of it is fp32 (csrc/streams.hip); the result is rounded to the model dtype for the projections that read it.

``TokenShift`` mixes a row with its predecessor, h_t + (h_(t-1) - h_t) * mu, with zeros before a sequence's first token;
the last row of a step is a request's state (fp32 [width] in a slot of the engine's StateSlotManager)."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.utils.context import get_context


class StreamNorm(nn.Module):
    def __init__(self, width: int, streams: int, eps: float, connections: bool = True, one_plus: bool = True):
        super().__init__()
        self.streams, self.eps, self.one_plus = streams, eps, one_plus
        self.weight = nn.Parameter(torch.zeros(width) if one_plus else torch.ones(width), requires_grad=False)
        if connections:
            # in | out | mix, fp32 whatever the model dtype (16-bit checkpoint values widen exactly)
            S = streams
            init = torch.cat([torch.ones(2 * S, dtype=torch.float32), torch.eye(S, dtype=torch.float32).flatten()])
            self.hc = nn.Parameter(init, requires_grad=False)
            self.hc.weight_loader = self._load_hc
            self.hc.keep_init = True              # random initialisation leaves the identity in place
        else:
            self.register_parameter("hc", None)

    def _load_hc(self, param, tensor, part: str):
        S = self.streams
        at, n = {"in": (0, S), "out": (S, S), "mix": (2 * S, S * S)}[part]
        assert tensor.numel() == n, f"{part}: {tuple(tensor.shape)} for {S} streams"
        param.data[at:at + n].copy_(tensor.reshape(-1).to(torch.float32))

    def forward(self, x, pending=None, rows_idx=None, out_dtype=None):
        """``x`` fp32 [T, S, width]; ``pending`` = (output of the previous sublayer, that sublayer's norm) or None."""
        delta, prev = pending if pending is not None else (None, None)
        hc_prev = prev.hc.data if prev is not None and prev.hc is not None else None
        hc_in = self.hc.data if self.hc is not None else None
        return kernels.hc_norm(x, self.weight.data, self.eps, hc_in=hc_in, delta=delta, hc_prev=hc_prev,
                               rows_idx=rows_idx, one_plus=self.one_plus, out_dtype=out_dtype)


class TokenShift(nn.Module):
    def __init__(self, width: int):
        super().__init__()
        self.width = width
        self.mu = nn.Parameter(torch.zeros(width), requires_grad=False)
        self.state = torch.tensor([])          # fp32 [slots, width], bound by the runner

    def state_spec(self) -> dict:
        return {"shape": (self.width,)}

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        """``h`` fp32 [T, width] -> shifted rows in the model dtype."""
        ctx = get_context()
        return kernels.token_shift(h, self.mu.data, self.state, ctx.cu_seqlens_q, ctx.past_lens, ctx.state_slots,
                                   ctx.seq_of_token)
