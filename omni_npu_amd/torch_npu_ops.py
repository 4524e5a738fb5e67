"""The vendor ops of the step in front of the attention path, under the names and argument order the reference calls
them with (``torch_npu.npu_kv_rmsnorm_rope_cache`` at src/omni_npu/v1/layers/attention/npu_mla.py:196-206, 296-309 and
npu_dsa.py:410-424, 517-527; ``torch_npu.npu_interleave_rope`` at npu_mla.py:210, 316; ``torch_npu.npu_rotary_mul`` at
npu_dsa.py:120, 130; ``torch_npu.npu_attention_update`` at attention/backends/mla.py:683-687), backed by the HIP kernels.

Differences a caller must know: the cache layout is the plain paged one (``cache_mode="PA"``); the Ascend fractal layout
("PA_NZ") has no meaning for these kernels and is rejected.  Quantisation scales / offsets are rejected (the reference
passes None everywhere).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import kernels as K


def npu_kv_rmsnorm_rope_cache(kv: torch.Tensor, gamma: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                              index: torch.Tensor, k_cache: torch.Tensor, ckv_cache: torch.Tensor, *,
                              k_rope_scale=None, c_kv_scale=None, k_rope_offset=None, c_kv_offset=None,
                              epsilon: float = 1e-5, cache_mode: str = "PA", is_output_kv: bool = False
                              ) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """kv [T,1,1,576] -> RMSNorm(kv[..., :512]) * gamma into ``ckv_cache`` and the rotated kv[..., 512:] into ``k_cache`` at
    the rows ``index`` (slot mapping) names.  Returns ``(k_cache, ckv_cache, k_rope, c_kv)``; the last two are the
    [T,1,1,64] / [T,1,1,512] results when ``is_output_kv`` is set, else None."""
    if any(a is not None for a in (k_rope_scale, c_kv_scale, k_rope_offset, c_kv_offset)):
        raise NotImplementedError("npu_kv_rmsnorm_rope_cache: quantisation scales / offsets are not supported")
    if cache_mode != "PA":
        raise NotImplementedError(f"npu_kv_rmsnorm_rope_cache: cache_mode {cache_mode!r} (only the plain paged layout 'PA')")
    t = kv.shape[0]
    k_rope = c_kv = None
    if is_output_kv:
        k_rope = torch.empty(t, K.D_ROPE, dtype=kv.dtype, device=kv.device)
        c_kv = torch.empty(t, K.D_NOPE, dtype=kv.dtype, device=kv.device)
    K.kv_rmsnorm_rope_cache(kv, gamma, cos, sin, index, ckv_cache, k_cache, eps=epsilon, table="half",
                            kv_a_out=c_kv, k_pe_out=k_rope)
    if is_output_kv:
        k_rope, c_kv = k_rope.view(t, 1, 1, K.D_ROPE), c_kv.view(t, 1, 1, K.D_NOPE)
    return k_cache, ckv_cache, k_rope, c_kv


def npu_interleave_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [B, N, S, 64] (or [T, N, 64]) with interleaved pairs; cos / sin [B, 1, S, 64] rows of cat(c, c).  Returns the
    rotated tensor in the de-interleaved layout cat(o1, o2), same shape as x."""
    shape = x.shape
    if x.dim() == 4:
        if x.shape[2] != 1:
            raise NotImplementedError("npu_interleave_rope: one position per (batch, head) row (S = 1)")
        x3 = x.squeeze(2)
    else:
        x3 = x
    return K.interleave_rope(x3, cos, sin, table="half").view(shape)


def npu_rotary_mul(x: torch.Tensor, r1: torch.Tensor, r2: torch.Tensor) -> torch.Tensor:
    """x * r1 + rotate_half(x) * r2 for x [B, N, S, 64] (or [T, N, 64]) and cos / sin rows r1 / r2 [B, 1, S, 64] whose two
    halves are equal (cat(c, c), as the reference builds them): the half-rotation rotary embedding of the indexer
    (npu_dsa.py:116-131).  Same shape as x."""
    shape = x.shape
    if x.dim() == 4:
        if x.shape[2] != 1:
            raise NotImplementedError("npu_rotary_mul: one position per (batch, head) row (S = 1)")
        x3 = x.squeeze(2)
    else:
        x3 = x
    return K.rotary_mul(x3, r1, r2, table="half").view(shape)


def npu_attention_update(lse, local_out, update_type: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    """N-way log-sum-exp merge of partial attention results: ``lse`` a list of n fp32 [R] vectors, ``local_out`` a list
    of n [R, D] matrices -> (merged fp32 [R, D], merged lse fp32 [R]) (attention/backends/mla.py:683-687; the same
    formula as attention/ops.py:109-141).  One launch for any n."""
    if update_type != 0:
        raise NotImplementedError(f"npu_attention_update: update_type {update_type}")
    from .attention.ops import attention_update_torch
    return attention_update_torch(list(local_out), [v.reshape(-1) for v in lse])
