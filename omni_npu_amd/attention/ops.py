"""HIP counterparts of the reference's torch helpers (src/omni_npu/attention/ops.py), same names and argument order.

Every function launches a gfx950 kernel through the C-ABI; tensors must live on the GPU.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import kernels as K


def gather_and_maybe_dequant_cache(
    src_cache: Tuple[torch.Tensor, torch.Tensor],
    dst: torch.Tensor,
    block_table: torch.Tensor,
    cu_seq_lens: torch.Tensor,
    batch_size: int,
    kv_cache_dtype: str,
    scale: Optional[torch.Tensor],
    seq_starts: Optional[torch.Tensor] = None,
    total_rows: Optional[int] = None,
) -> None:
    """dst[cu[i]:cu[i+1]] = cat(nope, rope) rows of positions seq_starts[i] .. of sequence i
    (reference ops.py:5-41).  Over the bf16 caches ``kv_cache_dtype`` and ``scale`` are accepted and unused, as in the
    reference: no dequantisation happens there.  ``src_cache`` may also be this build's fp8 block-scaled cache (one
    uint8 tensor [num_blocks, page, 656], alone or as the only member of a tuple): its rows carry their own scales and are
    dequantised to bf16 on the way."""
    dev = dst.device
    cu = cu_seq_lens.to(device=dev, dtype=torch.int32).contiguous()
    st = None if seq_starts is None else seq_starts.to(device=dev, dtype=torch.int32).contiguous()
    if torch.is_tensor(src_cache) or len(src_cache) == 1:
        cache = src_cache if torch.is_tensor(src_cache) else src_cache[0]
        K.gather_paged_fp8(cache, dst, block_table, cu, batch_size, st, total_rows)
        return
    K.gather_paged(src_cache[0], src_cache[1], dst, block_table, cu, batch_size, st, total_rows)


def merge_attn_states(
    output: torch.Tensor,
    prefix_output: torch.Tensor,
    prefix_lse: torch.Tensor,
    suffix_output: torch.Tensor,
    suffix_lse: torch.Tensor,
    output_lse: Optional[torch.Tensor] = None,
) -> None:
    """Two-way LSE merge of (T, N, D) outputs with (T, N, 1) log-sum-exps (reference ops.py:44-106)."""
    assert output.dim() == 3, f"output should have 3 dimensions, but got shape {output.shape}."
    assert prefix_lse.dim() == 3 and prefix_lse.size(-1) == 1, \
        f"LSE should have 3 dimensions and the last should be 1, but got shape {prefix_lse.shape}."
    K.merge_states(prefix_output, prefix_lse.float().contiguous(), suffix_output, suffix_lse.float().contiguous(),
                   output, output_lse)


def attention_update_torch(outs, lses):
    """N-way merge (reference ops.py:109-141): outs [n, T, D] (or list), lses [n, T] -> (out fp32 [T, D], lse fp32 [T]).
    One launch of the N-way merge kernel for any n."""
    if type(outs) is list:
        assert type(lses) is list and len(outs) == len(lses)
        outs = torch.stack(outs, dim=0)
        lses = torch.stack(lses, dim=0)
    assert outs.dim() == 3 and lses.dim() == 2
    assert outs.size(0) == lses.size(0) and outs.size(1) == lses.size(1)
    if outs.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        outs = outs.float()
    if outs.stride(-1) != 1:
        outs = outs.contiguous()
    return K.merge_n_states(outs, lses)
