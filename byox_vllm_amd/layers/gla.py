"""Gated linear attention mixer: linear attention with a matrix state per head and a learned, data-dependent decay per
key channel (Yang et al.'s gated linear attention family).  For head states S [dim, vdim]:

    a_t = sigmoid(W_a2 (W_a1 h_t) + b_a)^(1/tau)           decay per (head, key channel), low-rank parameterised
    S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t  with q_t = W_q h_t / sqrt(dim)
    y_t = W_o (RMSNorm_vdim(o_t) * silu(W_g h_t))

The state is the only thing a request keeps between steps: fp32 [heads, dim, vdim] in a slot of a pool that the engine's
StateSlotManager hands out; a request's first tokens start from zero instead of reading the slot, so slots need no
clearing when they are given to the next request.  Projections run in the model dtype with fp32 accumulation and are
handed to the recurrence in fp32; decay, state, output norm and gate are fp32 (csrc/gla.hip)."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.linear import DenseLinear
from byox_vllm_amd.utils.context import get_context


class GatedLinearAttention(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay_rank: int, tau: float, eps: float):
        super().__init__()
        self.heads, self.dim, self.vdim, self.tau, self.eps = heads, dim, vdim, float(tau), eps
        self.qkvg = DenseLinear(width, shards={"q": heads * dim, "k": heads * dim, "v": heads * vdim, "g": heads * vdim})
        self.a1 = DenseLinear(width, decay_rank)
        self.a2 = DenseLinear(decay_rank, heads * dim, bias=True)
        self.norm = nn.Parameter(torch.ones(vdim), requires_grad=False)
        self.o = DenseLinear(heads * vdim, width)
        self.offsets = tuple(self.qkvg.offset(s) for s in "qkvg")
        self.state = torch.tensor([])          # [slots, heads, dim, vdim] fp32, bound by the runner

    def state_spec(self) -> dict:
        return {"shape": (self.heads, self.dim, self.vdim)}

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        proj = self.qkvg(h, out_dtype=torch.float32)
        z = self.a2(self.a1(h), out_dtype=torch.float32)
        o = kernels.gla_recurrent(proj, self.offsets, z, self.state, ctx.cu_seqlens_q, ctx.past_lens, ctx.state_slots,
                                  self.norm.data, self.heads, self.dim, self.vdim, self.tau, self.dim ** -0.5, self.eps)
        return self.o(o, out_dtype=torch.float32)
