"""Rotary embedding of the 64 rope dims as the MLA layers use it (pairs (2i, 2i+1), the non-neox convention).

Mirrors the table construction of the reference's rotary classes (cos / sin rows per position, handed to the fused ops as
cat(c, c): src/omni_npu/layers/rotary_embedding/rotary_embedding_torch_npu.py:166-173, deepseek_scaling_rope.py:51-87) and
their result layout: the rotated vector is DE-INTERLEAVED, cat(o1, o2) (rotary_embedding_torch_npu.py:146-163).  Query and
key get the same permutation, so every q.k is unchanged; nothing downstream looks at single rope dims."""
from __future__ import annotations

import math
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


def yarn_find_correction_dim(num_rotations: float, dim: int, base: float, max_position_embeddings: int) -> float:
    """The (fractional) pair index whose wavelength makes ``num_rotations`` turns over the original context: the published
    YaRN formula the reference takes from vLLM (yarn_find_correction_range, imported at deepseek_scaling_rope.py:7-10)."""
    return (dim * math.log(max_position_embeddings / (num_rotations * 2 * math.pi))) / (2 * math.log(base))


def yarn_find_correction_range(low_rot: float, high_rot: float, dim: int, base: float, max_position_embeddings: int):
    low = math.floor(yarn_find_correction_dim(low_rot, dim, base, max_position_embeddings))
    high = math.ceil(yarn_find_correction_dim(high_rot, dim, base, max_position_embeddings))
    return max(low, 0), min(high, dim - 1)


def yarn_linear_ramp_mask(low: float, high: float, dim: int) -> torch.Tensor:
    if low == high:
        high += 0.001                                          # no division by zero
    return torch.clamp((torch.arange(dim, dtype=torch.float32) - low) / (high - low), 0, 1)


def yarn_get_mscale(scale: float = 1, mscale: float = 1) -> float:
    return 1.0 if scale <= 1 else 0.1 * mscale * math.log(scale) + 1.0


class HIPDeepseekScalingRotaryEmbedding(HIPRotaryEmbedding):
    """YaRN-scaled tables as DeepSeek-V2/V3 run with (reference NPUDeepseekScalingRotaryEmbedding,
    layers/rotary_embedding/deepseek_scaling_rope.py:16-87): the inverse frequencies blend the original ones
    (extrapolation, fast-rotating pairs) with those divided by ``scaling_factor`` (interpolation, slow pairs) through a
    linear ramp between the pairs that make ``beta_fast`` and ``beta_slow`` turns over the original context; the table
    covers ``max_position_embeddings * scaling_factor`` positions and cos / sin are multiplied by
    yarn_get_mscale(factor, mscale) / yarn_get_mscale(factor, mscale_all_dim) * attn_factor.  Argument names and order
    are the reference's; the kernels take any table, so forward() is the plain class's."""

    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: float, is_neox_style: bool,
                 scaling_factor: float, dtype: torch.dtype = torch.bfloat16, *, extrapolation_factor: float = 1,
                 attn_factor: float = 1, beta_fast: int = 32, beta_slow: int = 1, mscale: float = 1,
                 mscale_all_dim: float = 0, device=None) -> None:
        torch.nn.Module.__init__(self)
        if rotary_dim != K.D_ROPE:
            raise NotImplementedError("the HIP kernels rotate 64 dims")
        if is_neox_style:
            raise NotImplementedError("the MLA layers rotate pairs (2i, 2i+1): is_neox_style must be False")
        self.head_size, self.rotary_dim, self.base = head_size, rotary_dim, base
        self.max_position_embeddings, self.scaling_factor = max_position_embeddings, scaling_factor
        self.extrapolation_factor, self.attn_factor = extrapolation_factor, attn_factor
        self.beta_fast, self.beta_slow = beta_fast, beta_slow
        self.mscale = float(yarn_get_mscale(scaling_factor, float(mscale))
                            / yarn_get_mscale(scaling_factor, float(mscale_all_dim)) * attn_factor)
        self._set_cos_sin_cache(max_position_embeddings, device, dtype)

    def _set_cos_sin_cache(self, seq_len: int, device, dtype: torch.dtype) -> None:
        self.max_seq_len_cached = seq_len
        dim = self.rotary_dim
        pos_freqs = self.base ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim)
        freq_extra, freq_inter = 1.0 / pos_freqs, 1.0 / (self.scaling_factor * pos_freqs)
        low, high = yarn_find_correction_range(self.beta_fast, self.beta_slow, dim, self.base, self.max_position_embeddings)
        inv_freq_mask = 1.0 - yarn_linear_ramp_mask(low, high, dim // 2)     # (deepseek_scaling_rope.py:73: no extrapolation factor)
        inv_freq = freq_inter * (1 - inv_freq_mask) + freq_extra * inv_freq_mask
        self.register_buffer("inv_freq", inv_freq.to(device), persistent=False)
        t = torch.arange(int(seq_len * self.scaling_factor), dtype=torch.float32)
        freqs = torch.outer(t, inv_freq)
        emb = torch.cat((freqs, freqs), dim=-1)
        self.register_buffer("cos_cached", (emb.cos() * self.mscale).to(dtype).to(device), persistent=False)
        self.register_buffer("sin_cached", (emb.sin() * self.mscale).to(dtype).to(device), persistent=False)
