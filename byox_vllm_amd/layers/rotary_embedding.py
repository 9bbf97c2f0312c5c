"""NeoX rotary embedding (interface of nanovllm/layers/rotary_embedding.py:18-61).

The fp32 cos/sin table is built exactly as the reference builds it
(rotary_embedding.py:29-35); the rotation itself runs in nv_rope_kv_store.
"""

from functools import lru_cache

import torch
from torch import nn

from byox_vllm_amd import kernels


class RotaryEmbedding(nn.Module):
    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: float) -> None:
        super().__init__()
        assert rotary_dim == head_size
        self.head_size = head_size
        inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float) / rotary_dim))
        t = torch.arange(max_position_embeddings, dtype=torch.float)
        freqs = torch.einsum("i,j -> ij", t, inv_freq)
        cache = torch.cat((freqs.cos(), freqs.sin()), dim=-1).unsqueeze_(1)
        self.register_buffer("cos_sin_cache", cache, persistent=False)

    def forward(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor):
        """Stand-alone form: rotates contiguous query [T, H, D] and key [T, Hkv, D] in place."""
        d = self.head_size
        for x in (query, key):
            assert x.is_contiguous()
            kernels.rope_kv_store(x.view(x.size(0), -1), positions, self.cos_sin_cache, x.size(1), 0, d)
        return query, key


@lru_cache(1)
def get_rope(head_size: int, rotary_dim: int, max_position: int, base: float, rope_scaling: dict | None = None):
    assert rope_scaling is None
    return RotaryEmbedding(head_size, rotary_dim, max_position, base)


def scaled_inv_freq(dims: int, base: float, scaling: dict | None = None) -> tuple[torch.Tensor, float]:
    """Rotation frequencies of the 'rotate half' layout (dimension i pairs with i + dims/2) -> (fp32 [dims/2], the
    factor that multiplies both cosine and sine).  Without ``scaling``: base^(-2i/dims) and 1.

    With YaRN-style scaling {factor, original, fast, slow}: a rotation count t (turns over the original context) maps
    to the dimension index dims * ln(original / (2 pi t)) / (2 ln base); between the indices of ``fast`` (floor, at
    least 0) and ``slow`` (ceil, at most dims - 1) a linear ramp blends the plain frequency (ramp 0, fast-rotating
    dimensions keep theirs) into the frequency divided by ``factor`` (ramp 1); the magnitude factor is
    0.1 ln(factor) + 1.  The rotation itself (angle = position * frequency in fp32) runs inside the kernels."""
    import math
    i = torch.arange(dims // 2, dtype=torch.float64)
    freq = torch.as_tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    magnitude = 1.0
    if scaling:
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def index_of(turns: float) -> float:
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        freq = freq / factor * ramp + freq * (1.0 - ramp)
        magnitude = 0.1 * math.log(factor) + 1.0
    return freq.to(torch.float32), magnitude
