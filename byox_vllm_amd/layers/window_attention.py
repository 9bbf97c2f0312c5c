"""Softmax attention with grouped key/value heads over a paged cache, with the score shaped before the softmax:

    s_ij = cap(q_i . k_j * scale * temp_h) - slope_h (i - j),   cap(z) = c tanh(z / c),   slope_h = 2^(-8 (h + 1) / H)

q and k are RMS-normed per head (weights shared by the heads), there is no rotation: positions enter through the
distance term only.  Position i sees the keys 0 <= i - j < window (window 0: all earlier keys).  Key and value sizes may
differ.  Cache rows [k: G * dim | v: G * vdim] live in pages of the engine's BlockManager in the model dtype; norms,
scores and softmax are fp32 (csrc/window_attn.hip).

The module owns no projection: it takes the fp32 q | k | v columns of a (possibly merged) projection and writes into a
column slice of the caller's buffer, so a block that runs another branch beside it projects once in and once out."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.utils.context import get_context


class WindowAttention(nn.Module):
    def __init__(self, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, window: int, softcap: float | None,
                 eps: float):
        super().__init__()
        assert heads % kv_heads == 0
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.window, self.softcap, self.eps = float(scale), int(window), float(softcap or 0.0), eps
        self.q_norm = nn.Parameter(torch.ones(dim), requires_grad=False)
        self.k_norm = nn.Parameter(torch.ones(dim), requires_grad=False)
        self.temp = nn.Parameter(torch.ones(heads), requires_grad=False)
        self.cache = torch.tensor([])          # [pages * block_size, G * (dim + vdim)], bound by the runner
        self.block_size = 0

    def page_spec(self) -> dict:
        return {"width": self.kv_heads * (self.dim + self.vdim)}

    def sizes(self) -> dict:
        return {"q": self.heads * self.dim, "k": self.kv_heads * self.dim, "v": self.kv_heads * self.vdim}

    def forward(self, proj: torch.Tensor, offsets: tuple, out: torch.Tensor, out_scale: float = 1.0,
                bias: torch.Tensor | None = None) -> torch.Tensor:
        """``proj`` fp32 [T, *] with q | k | v at ``offsets`` (``bias``, over the same columns, is still to be added);
        ``out`` [T, >= heads * vdim] in the model dtype."""
        ctx = get_context()
        q = kernels.qk_norm_store(proj, offsets, self.q_norm.data, self.k_norm.data, self.temp.data, self.scale, self.eps,
                                  ctx.slot_mapping, self.cache, self.heads, self.kv_heads, self.dim, self.vdim, bias=bias)
        return kernels.window_attn(q, self.cache, ctx.block_tables, ctx.cu_seqlens_q, ctx.past_lens, ctx.seq_of_token,
                                   ctx.max_seqlen_q, self.heads, self.kv_heads, self.dim, self.vdim, self.block_size,
                                   self.window, self.softcap, out, out_scale)
