"""Mamba-2 mixer (state-space duality, Dao & Gu) in its recurrent form.  With inner = heads * vdim, N = state, G groups,
one projection gives [z: inner | x: inner | B: G N | C: G N | dt: heads]; x, B, C pass a short causal convolution and
SiLU; per head h (sharing B, C with the heads of its group)

    dt = softplus(dt + dt_bias),  S_t = exp(-exp(A_log_h) dt) S_(t-1) + dt B_t x_t^T  (S is N x vdim),  y_t = S_t^T C_t + D_h x_t

then y * silu(z), an RMS norm over 'norm_groups' equal parts of the inner dimension (gate before norm), and the output
projection.  S (fp32 [heads, N, vdim]) and the convolution's last inputs live in a request's state slot; everything
after the projection and before the output projection is fp32 (csrc/scan.hip, csrc/streams.hip)."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.conv import CausalConv1d
from byox_vllm_amd.layers.linear import DenseLinear
from byox_vllm_amd.utils.context import get_context


class Mamba2Mixer(nn.Module):
    def __init__(self, width: int, heads: int, vdim: int, state: int, groups: int, taps: int, norm_groups: int,
                 eps: float):
        super().__init__()
        assert heads % groups == 0 and (heads * vdim) % norm_groups == 0
        self.heads, self.vdim, self.n, self.groups, self.norm_groups, self.eps = heads, vdim, state, groups, norm_groups, eps
        self.inner = inner = heads * vdim
        self.inp = DenseLinear(width, 2 * inner + 2 * groups * state + heads)
        self.conv = CausalConv1d(inner + 2 * groups * state, taps, "silu")
        self.dt_bias = nn.Parameter(torch.zeros(heads), requires_grad=False)
        self.A_log = nn.Parameter(torch.zeros(heads), requires_grad=False)
        self.D = nn.Parameter(torch.ones(heads), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(inner), requires_grad=False)
        self.o = DenseLinear(inner, width)
        self.state = torch.tensor([])          # fp32 [slots, heads, N, vdim], bound by the runner

    def state_spec(self) -> dict:
        return {"shape": (self.heads, self.n, self.vdim)}

    def state_modules(self):
        return [self.conv, self]

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        inner, gn = self.inner, self.groups * self.n
        proj = self.inp(h, out_dtype=torch.float32)
        xbc, _ = self.conv(proj[:, inner:2 * inner + 2 * gn])
        y = kernels.ssd_scan(xbc, proj[:, :inner], proj[:, 2 * inner + 2 * gn:], self.dt_bias.data, self.A_log.data,
                             self.D.data, self.state, ctx.cu_seqlens_q, ctx.past_lens, ctx.state_slots, self.heads,
                             self.groups, self.n, self.vdim, max_q=ctx.max_seqlen_q)
        y = kernels.group_rms_norm_f32(y, self.norm.data, self.norm_groups, self.eps)
        return self.o(y, out_dtype=torch.float32)
