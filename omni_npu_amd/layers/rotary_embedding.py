"""Rotary embedding of the 64 rope dims as the MLA layers use it (pairs (2i, 2i+1), the non-neox convention).

Mirrors the table construction of the reference's rotary classes (cos / sin rows per position, handed to the fused ops as
cat(c, c): src/omni_npu/layers/rotary_embedding/rotary_embedding_torch_npu.py:166-173, deepseek_scaling_rope.py:51-87) and
their result layout: the rotated vector is DE-INTERLEAVED, cat(o1, o2) (rotary_embedding_torch_npu.py:146-163).  Query and
key get the same permutation, so every q.k is unchanged; nothing downstream looks at single rope dims."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import kernels as K


class HIPRotaryEmbedding(torch.nn.Module):
    def __init__(self, rotary_dim: int = 64, max_position: int = 8192, base: float = 10000.0, mscale: float = 1.0,
                 dtype: torch.dtype = torch.bfloat16, device=None):
        super().__init__()
        if rotary_dim != K.D_ROPE:
            raise NotImplementedError("the HIP kernels rotate 64 dims")
        inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
        freqs = torch.outer(torch.arange(max_position, dtype=torch.float32), inv_freq)
        emb = torch.cat((freqs, freqs), dim=-1)
        self.register_buffer("cos_cached", (emb.cos() * mscale).to(dtype).to(device), persistent=False)
        self.register_buffer("sin_cached", (emb.sin() * mscale).to(dtype).to(device), persistent=False)
        self.rotary_dim = rotary_dim

    def get_cos_sin(self, positions: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """[T, 64] rows of cat(c, c) for ``positions`` (layers/rotary_embedding/common.py:43-64)."""
        pos = positions.flatten()
        return self.cos_cached.index_select(0, pos), self.sin_cached.index_select(0, pos)

    def forward(self, positions: torch.Tensor, query: torch.Tensor, key: Optional[torch.Tensor] = None):
        """query [T, N, 64], key [T, 1, 64] (strided views are fine) -> rotated copies, same shapes."""
        cos, sin = self.get_cos_sin(positions)
        q = K.interleave_rope(query, cos, sin, table="half")
        k = K.interleave_rope(key, cos, sin, table="half") if key is not None else None
        return q, k
