"""torch-tensor front end of the C-ABI: validates shapes on the host, passes raw device pointers,
strides and the current HIP stream, and never allocates behind the caller's back except for the
split-KV workspace, which is cached per (device, size)."""
from __future__ import annotations

import math
from typing import Optional

import torch

from . import _lib

PAGE = 128
D_NOPE = 512
D_ROPE = 64


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("this op runs HIP kernels only: every tensor must live on a GPU (there is no CPU path)")


def _cache3(c: torch.Tensor, width: int) -> torch.Tensor:
    """[nblk, page, (1,) width] -> [nblk, page, width] view."""
    if c.dim() == 4 and c.shape[2] == 1:
        c = c.squeeze(2)
    if c.dim() != 3 or c.shape[-1] != width or c.stride(-1) != 1:
        raise ValueError(f"cache must be [num_blocks, page, {width}] with a contiguous last dim, got {tuple(c.shape)}")
    return c


# ------------------------------------------------------------------------------------------------
def cache_write(kv_c: torch.Tensor, k_pe: torch.Tensor, slot_mapping: torch.Tensor,
                nope_cache: torch.Tensor, rope_cache: torch.Tensor) -> None:
    """nope.flatten(0,1)[slot[t]] = kv_c[t]; rope.flatten(0,1)[slot[t]] = k_pe[t]; negative slots skipped
    (reference: store_kv, src/omni_npu/attention/backends/mla.py:868-881)."""
    _need_cuda(kv_c, k_pe, slot_mapping, nope_cache, rope_cache)
    lib = _lib.load()
    nope, rope = _cache3(nope_cache, D_NOPE), _cache3(rope_cache, D_ROPE)
    k_pe = k_pe.reshape(k_pe.shape[0], -1) if k_pe.dim() == 3 else k_pe
    t = min(slot_mapping.numel(), kv_c.shape[0])
    if kv_c.shape[-1] != D_NOPE or k_pe.shape[-1] != D_ROPE or kv_c.stride(-1) != 1 or k_pe.stride(-1) != 1:
        raise ValueError(f"kv_c must be [T,512] and k_pe [T,64], got {tuple(kv_c.shape)} {tuple(k_pe.shape)}")
    if kv_c.dtype != torch.bfloat16 or k_pe.dtype != torch.bfloat16 or nope.dtype != torch.bfloat16 or rope.dtype != torch.bfloat16:
        raise TypeError("cache_write: bf16 only")
    if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous():
        slot_mapping = slot_mapping.to(torch.int64).contiguous()
    if nope.shape[0] != rope.shape[0] or nope.shape[1] != rope.shape[1]:
        raise ValueError("nope and rope caches disagree on [num_blocks, page]")
    rc = lib.mla_cache_write_bf16(kv_c.data_ptr(), kv_c.stride(0), k_pe.data_ptr(), k_pe.stride(0),
                                  slot_mapping.data_ptr(), t, nope.data_ptr(), nope.stride(0), nope.stride(1),
                                  rope.data_ptr(), rope.stride(0), rope.stride(1), nope.shape[1], nope.shape[0],
                                  _stream(kv_c))
    _lib.check(rc, "mla_cache_write_bf16")


def scatter_rows(src: torch.Tensor, slot_mapping: torch.Tensor, cache: torch.Tensor) -> None:
    """cache.flatten(0,1)[slot[t]] = src[t] for one cache of any 16-byte-multiple row width
    (indexer K: vllm_patches/patches/models/deepseek/patch_dsv32_indexer.py:116-121)."""
    _need_cuda(src, slot_mapping, cache)
    lib = _lib.load()
    if cache.dim() == 4 and cache.shape[2] == 1:
        cache = cache.squeeze(2)
    src = src.reshape(src.shape[0], -1)
    es = cache.element_size()
    if cache.dim() != 3 or cache.stride(-1) != 1 or src.stride(-1) != 1 or src.shape[-1] != cache.shape[-1] or src.dtype != cache.dtype:
        raise ValueError("scatter_rows: src [T,W] and cache [num_blocks,page,W] must agree in width and dtype")
    if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous():
        slot_mapping = slot_mapping.to(torch.int64).contiguous()
    t = min(slot_mapping.numel(), src.shape[0])
    rc = lib.mla_scatter_rows(src.data_ptr(), src.stride(0) * es, src.shape[-1] * es, slot_mapping.data_ptr(), t,
                              cache.data_ptr(), cache.stride(0) * es, cache.stride(1) * es, cache.shape[1],
                              cache.shape[0], _stream(src))
    _lib.check(rc, "mla_scatter_rows")


FP8_ROW_BYTES = 656      # 512 e4m3 + 4 fp32 block scales + 64 bf16 rope


def cache_write_fp8(kv_c: torch.Tensor, k_pe: torch.Tensor, slot_mapping: torch.Tensor, cache: torch.Tensor) -> None:
    """Quantise the new tokens' latent to e4m3 with one fp32 scale per 128 elements and write 656-byte rows
    (512 fp8 | 4 fp32 scales | 64 bf16 rope) into ``cache`` = uint8 [num_blocks, page, 656]."""
    _need_cuda(kv_c, k_pe, slot_mapping, cache)
    lib = _lib.load()
    k_pe = k_pe.reshape(k_pe.shape[0], -1) if k_pe.dim() == 3 else k_pe
    if cache.dtype != torch.uint8 or cache.dim() != 3 or cache.shape[-1] != FP8_ROW_BYTES or cache.stride(-1) != 1:
        raise ValueError(f"fp8 cache must be uint8 [num_blocks, page, {FP8_ROW_BYTES}], got {cache.dtype} {tuple(cache.shape)}")
    if kv_c.shape[-1] != D_NOPE or k_pe.shape[-1] != D_ROPE or kv_c.dtype != torch.bfloat16 or k_pe.dtype != torch.bfloat16 \
            or kv_c.stride(-1) != 1 or k_pe.stride(-1) != 1:
        raise ValueError("cache_write_fp8: kv_c must be bf16 [T,512] and k_pe bf16 [T,64]")
    if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous():
        slot_mapping = slot_mapping.to(torch.int64).contiguous()
    t = min(slot_mapping.numel(), kv_c.shape[0])
    rc = lib.mla_cache_write_fp8(kv_c.data_ptr(), kv_c.stride(0), k_pe.data_ptr(), k_pe.stride(0), slot_mapping.data_ptr(),
                                 t, cache.data_ptr(), cache.stride(0), cache.stride(1), cache.shape[1], cache.shape[0],
                                 _stream(kv_c))
    _lib.check(rc, "mla_cache_write_fp8")


def _table_step(cos: torch.Tensor, sin: torch.Tensor, t: int, table: str):
    """cos / sin rows [T, W] (singleton dims dropped) and the entry step of pair i: 'half' = the reference's cat(c, c)
    rows or plain [T,32] rows (entry i), 'repeat' = rows that repeat every entry (entry 2i)."""
    cos, sin = cos.reshape(cos.shape[0], -1), sin.reshape(sin.shape[0], -1)
    step = {"half": 1, "repeat": 2}[table]
    if cos.shape != sin.shape or cos.shape[0] < t or cos.shape[1] < 31 * step + 1 or cos.stride(-1) != 1 or sin.stride(-1) != 1 \
            or cos.stride(0) != sin.stride(0) or cos.dtype != torch.bfloat16 or sin.dtype != torch.bfloat16:
        raise ValueError(f"cos / sin must be bf16 [T, >= {31 * step + 1}] rows with equal strides, got {tuple(cos.shape)}")
    return cos, sin, step


def kv_rmsnorm_rope_cache(kv: torch.Tensor, gamma: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                          slot_mapping: Optional[torch.Tensor], nope_cache: Optional[torch.Tensor],
                          rope_cache: Optional[torch.Tensor],
                          eps: float = 1e-6, table: str = "half", interleaved_out: bool = False,
                          kv_a_out: Optional[torch.Tensor] = None, k_pe_out: Optional[torch.Tensor] = None,
                          q_rope: Optional[torch.Tensor] = None, q_out: Optional[torch.Tensor] = None) -> None:
    """RMSNorm(kv[:, :512]) * gamma and the rotary embedding of kv[:, 512:] written into the paged cache rows
    ``slot_mapping`` names, in one launch (reference: torch_npu.npu_kv_rmsnorm_rope_cache,
    src/omni_npu/v1/layers/attention/npu_mla.py:196-206).  ``rope_cache=None`` selects the fp8 cache
    (``nope_cache`` = uint8 [num_blocks, page, 656]); ``slot_mapping=None`` caches nothing and only fills ``kv_a_out`` / ``k_pe_out``.
    ``q_rope`` (bf16 [T, N, 64], any strides with a contiguous last dim): the rotary embedding of the same tokens' query
    heads (npu_interleave_rope, npu_mla.py:210) runs in the same launch, into ``q_out`` (default: in place)."""
    _need_cuda(kv, gamma, cos, sin, slot_mapping, nope_cache)
    lib = _lib.load()
    kv = kv.reshape(kv.shape[0], -1)
    if kv.shape[-1] != D_NOPE + D_ROPE or kv.dtype != torch.bfloat16 or kv.stride(-1) != 1:
        raise ValueError(f"kv must be bf16 [T, 576] with a contiguous last dim, got {kv.dtype} {tuple(kv.shape)}")
    if gamma.shape != (D_NOPE,) or gamma.dtype != torch.bfloat16 or not gamma.is_contiguous():
        raise ValueError("gamma must be a contiguous bf16 [512] vector")
    if slot_mapping is not None and (slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous()):
        slot_mapping = slot_mapping.to(torch.int64).contiguous()
    t = min(slot_mapping.numel(), kv.shape[0]) if slot_mapping is not None else kv.shape[0]
    cos, sin, step = _table_step(cos, sin, t, table)
    for o, w, name in ((kv_a_out, D_NOPE, "kv_a_out"), (k_pe_out, D_ROPE, "k_pe_out")):
        if o is not None and (o.dim() != 2 or o.shape[0] < t or o.shape[1] != w or o.dtype != torch.bfloat16 or o.stride(-1) != 1
                              or not o.is_cuda):
            raise ValueError(f"{name} must be a bf16 GPU tensor [T, {w}]")
    outs = (kv_a_out.data_ptr() if kv_a_out is not None else None, kv_a_out.stride(0) if kv_a_out is not None else 0,
            k_pe_out.data_ptr() if k_pe_out is not None else None, k_pe_out.stride(0) if k_pe_out is not None else 0)
    k_pe = kv[:, D_NOPE:]
    qargs, sfx = (), ""
    if q_rope is not None:
        _need_cuda(q_rope, q_out)
        q_out = q_rope if q_out is None else q_out
        if q_rope.dim() != 3 or q_rope.shape[0] < t or q_rope.shape[-1] != D_ROPE or q_rope.dtype != torch.bfloat16 \
                or q_rope.stride(-1) != 1 or q_out.shape != q_rope.shape or q_out.dtype != q_rope.dtype or q_out.stride(-1) != 1:
            raise ValueError("q_rope / q_out must be bf16 [T, N, 64] with a contiguous last dim")
        qargs = (q_rope.data_ptr(), q_rope.stride(0), q_rope.stride(1), q_rope.shape[1], q_out.data_ptr(), q_out.stride(0),
                 q_out.stride(1))
        sfx = "_q"
    if slot_mapping is None:
        if kv_a_out is None or k_pe_out is None:
            raise ValueError("without a slot mapping both kv_a_out and k_pe_out are required")
        name = "mla_kv_rmsnorm_rope_cache" + sfx
        rc = getattr(lib, name)(kv.data_ptr(), kv.stride(0), k_pe.data_ptr(), kv.stride(0), gamma.data_ptr(),
                                cos.data_ptr(), sin.data_ptr(), cos.stride(0), step, int(interleaved_out), None, t,
                                float(eps), None, 0, 0, None, 0, 0, 1, 1, *outs, *qargs, _stream(kv))
        _lib.check(rc, name)
        return
    if rope_cache is None:
        c = nope_cache
        if c.dtype != torch.uint8 or c.dim() != 3 or c.shape[-1] != FP8_ROW_BYTES or c.stride(-1) != 1:
            raise ValueError(f"fp8 cache must be uint8 [num_blocks, page, {FP8_ROW_BYTES}], got {c.dtype} {tuple(c.shape)}")
        name = "mla_kv_rmsnorm_rope_cache" + sfx + "_fp8"
        rc = getattr(lib, name)(kv.data_ptr(), kv.stride(0), k_pe.data_ptr(), kv.stride(0), gamma.data_ptr(),
                                cos.data_ptr(), sin.data_ptr(), cos.stride(0), step, int(interleaved_out),
                                slot_mapping.data_ptr(), t, float(eps), c.data_ptr(), c.stride(0), c.stride(1),
                                c.shape[1], c.shape[0], *outs, *qargs, _stream(kv))
        _lib.check(rc, name)
        return
    _need_cuda(rope_cache)
    nope, rope = _cache3(nope_cache, D_NOPE), _cache3(rope_cache, D_ROPE)
    if nope.dtype != torch.bfloat16 or rope.dtype != torch.bfloat16 or nope.shape[:2] != rope.shape[:2]:
        raise ValueError("nope / rope caches must be bf16 and agree on [num_blocks, page]")
    name = "mla_kv_rmsnorm_rope_cache" + sfx
    rc = getattr(lib, name)(kv.data_ptr(), kv.stride(0), k_pe.data_ptr(), kv.stride(0), gamma.data_ptr(),
                            cos.data_ptr(), sin.data_ptr(), cos.stride(0), step, int(interleaved_out),
                            slot_mapping.data_ptr(), t, float(eps), nope.data_ptr(), nope.stride(0), nope.stride(1),
                            rope.data_ptr(), rope.stride(0), rope.stride(1), nope.shape[1], nope.shape[0], *outs, *qargs,
                            _stream(kv))
    _lib.check(rc, name)


def interleave_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, out: Optional[torch.Tensor] = None,
                    table: str = "half", interleaved_out: bool = False) -> torch.Tensor:
    """Rotary embedding of x [T, N, 64] (pairs (2i, 2i+1)), result cat(o1, o2) like the reference's
    torch_npu.npu_interleave_rope (src/omni_npu/v1/layers/attention/npu_mla.py:210) or, with ``interleaved_out``, pairs in
    place.  Returns ``out`` (a new tensor unless given)."""
    _need_cuda(x, cos, sin)
    lib = _lib.load()
    if x.dim() != 3 or x.shape[-1] != D_ROPE or x.dtype != torch.bfloat16 or x.stride(-1) != 1:
        raise ValueError(f"x must be bf16 [T, N, 64] with a contiguous last dim, got {x.dtype} {tuple(x.shape)}")
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    if out.shape != x.shape or out.dtype != x.dtype or out.stride(-1) != 1 or not out.is_cuda:
        raise ValueError("out must match x")
    cos, sin, step = _table_step(cos, sin, x.shape[0], table)
    rc = lib.mla_interleave_rope(x.data_ptr(), x.stride(0), x.stride(1), x.shape[0], x.shape[1], cos.data_ptr(), sin.data_ptr(),
                                 cos.stride(0), step, int(interleaved_out), out.data_ptr(), out.stride(0), out.stride(1),
                                 _stream(x))
    _lib.check(rc, "mla_interleave_rope")
    return out


def rotary_mul(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, out: Optional[torch.Tensor] = None,
               table: str = "half") -> torch.Tensor:
    """Rotary embedding of x [T, N, 64] with the half-rotation pairing (element i with i + 32), result in the input's
    layout, like torch_npu.npu_rotary_mul in the indexer (src/omni_npu/v1/layers/attention/npu_dsa.py:120, 130).
    ``out`` may be ``x`` (in place); returns ``out`` (a new tensor unless given)."""
    _need_cuda(x, cos, sin)
    lib = _lib.load()
    if x.dim() != 3 or x.shape[-1] != D_ROPE or x.dtype != torch.bfloat16 or x.stride(-1) != 1:
        raise ValueError(f"x must be bf16 [T, N, 64] with a contiguous last dim, got {x.dtype} {tuple(x.shape)}")
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    if out.shape != x.shape or out.dtype != x.dtype or out.stride(-1) != 1 or not out.is_cuda:
        raise ValueError("out must match x")
    cos, sin, step = _table_step(cos, sin, x.shape[0], table)
    rc = lib.mla_rotary_mul(x.data_ptr(), x.stride(0), x.stride(1), x.shape[0], x.shape[1], cos.data_ptr(), sin.data_ptr(),
                            cos.stride(0), step, out.data_ptr(), out.stride(0), out.stride(1), _stream(x))
    _lib.check(rc, "mla_rotary_mul")
    return out


def gather_paged(nope_cache: torch.Tensor, rope_cache: torch.Tensor, dst: torch.Tensor, block_table: torch.Tensor,
                 cu_seq_lens: torch.Tensor, batch_size: int, seq_starts: Optional[torch.Tensor] = None,
                 total_rows: Optional[int] = None) -> None:
    """dst[cu[i]:cu[i+1]] = cat(nope[blk, slot], rope[blk, slot]) for positions seq_starts[i] .. +len_i
    (reference: gather_and_maybe_dequant_cache, src/omni_npu/attention/ops.py:5-41).  cu_seq_lens / seq_starts are
    int32 device tensors; ``total_rows`` bounds the launch (defaults to dst.shape[0]) so no host sync is needed."""
    _need_cuda(nope_cache, rope_cache, dst, block_table, cu_seq_lens, seq_starts)
    lib = _lib.load()
    nope, rope = _cache3(nope_cache, D_NOPE), _cache3(rope_cache, D_ROPE)
    if dst.dim() != 2 or dst.shape[1] < D_NOPE + D_ROPE or dst.stride(1) != 1 or dst.dtype != nope.dtype or nope.dtype != torch.bfloat16:
        raise ValueError("gather_paged: dst must be bf16 [rows, >=576] like the caches")
    if block_table.dtype != torch.int32 or cu_seq_lens.dtype != torch.int32 or not cu_seq_lens.is_contiguous():
        raise TypeError("gather_paged: block_table and cu_seq_lens must be int32 (cu_seq_lens contiguous)")
    if seq_starts is not None and (seq_starts.dtype != torch.int32 or not seq_starts.is_contiguous()):
        raise TypeError("gather_paged: seq_starts must be contiguous int32")
    if cu_seq_lens.numel() < batch_size + 1:
        raise ValueError("gather_paged: cu_seq_lens needs batch_size + 1 entries")
    rows = dst.shape[0] if total_rows is None else min(int(total_rows), dst.shape[0])
    rc = lib.mla_gather_paged(nope.data_ptr(), nope.stride(0), nope.stride(1), rope.data_ptr(), rope.stride(0), rope.stride(1),
                              nope.shape[0], nope.shape[1], dst.data_ptr(), dst.stride(0), dst.shape[0],
                              block_table.data_ptr(), block_table.stride(0), block_table.shape[1], cu_seq_lens.data_ptr(),
                              seq_starts.data_ptr() if seq_starts is not None else None, batch_size, rows, _stream(dst))
    _lib.check(rc, "mla_gather_paged")


def gather_paged_fp8(cache: torch.Tensor, dst: torch.Tensor, block_table: torch.Tensor, cu_seq_lens: torch.Tensor,
                     batch_size: int, seq_starts: Optional[torch.Tensor] = None, total_rows: Optional[int] = None) -> None:
    """gather_paged out of the fp8 block-scaled cache (uint8 [num_blocks, page, 656], see cache_write_fp8):
    dst[cu[i] + j] = cat(bf16(e4m3 * block scale), rope) of position seq_starts[i] + j, the values the fp8 decode attends
    over (the chunked-context prefill of the reference, attention/backends/mla.py:377-450, over a quantised cache)."""
    _need_cuda(cache, dst, block_table, cu_seq_lens, seq_starts)
    lib = _lib.load()
    if cache.dtype != torch.uint8 or cache.dim() != 3 or cache.shape[-1] != FP8_ROW_BYTES or cache.stride(-1) != 1:
        raise ValueError(f"fp8 cache must be uint8 [num_blocks, page, {FP8_ROW_BYTES}], got {cache.dtype} {tuple(cache.shape)}")
    if dst.dim() != 2 or dst.shape[1] < D_NOPE + D_ROPE or dst.stride(1) != 1 or dst.dtype != torch.bfloat16:
        raise ValueError("gather_paged_fp8: dst must be bf16 [rows, >=576]")
    if block_table.dtype != torch.int32 or cu_seq_lens.dtype != torch.int32 or not cu_seq_lens.is_contiguous():
        raise TypeError("gather_paged_fp8: block_table and cu_seq_lens must be int32 (cu_seq_lens contiguous)")
    if block_table.dim() != 2 or block_table.stride(1) != 1 or block_table.shape[0] < batch_size:
        raise ValueError("gather_paged_fp8: block_table must be [>= batch, max_blocks] with contiguous rows")
    if seq_starts is not None and (seq_starts.dtype != torch.int32 or not seq_starts.is_contiguous()):
        raise TypeError("gather_paged_fp8: seq_starts must be contiguous int32")
    if cu_seq_lens.numel() < batch_size + 1:
        raise ValueError("gather_paged_fp8: cu_seq_lens needs batch_size + 1 entries")
    rows = dst.shape[0] if total_rows is None else min(int(total_rows), dst.shape[0])
    rc = lib.mla_gather_paged_fp8(cache.data_ptr(), cache.stride(0), cache.stride(1), cache.shape[0], cache.shape[1],
                                  dst.data_ptr(), dst.stride(0), dst.shape[0], block_table.data_ptr(), block_table.stride(0),
                                  block_table.shape[1], cu_seq_lens.data_ptr(),
                                  seq_starts.data_ptr() if seq_starts is not None else None, batch_size, rows, _stream(dst))
    _lib.check(rc, "mla_gather_paged_fp8")


_DT = {torch.bfloat16: 0, torch.float32: 1}


def merge_states(prefix_out: torch.Tensor, prefix_lse: torch.Tensor, suffix_out: torch.Tensor, suffix_lse: torch.Tensor,
                 out: torch.Tensor, out_lse: Optional[torch.Tensor] = None) -> None:
    """Two-way log-sum-exp merge (reference: merge_attn_states, src/omni_npu/attention/ops.py:44-106).
    outputs [T,N,D] (bf16 or fp32, any token/head strides), lse fp32 [T,N] or [T,N,1] contiguous."""
    _need_cuda(prefix_out, prefix_lse, suffix_out, suffix_lse, out, out_lse)
    lib = _lib.load()
    t, n, d = out.shape
    if prefix_out.shape != out.shape or suffix_out.shape != out.shape or prefix_out.dtype != suffix_out.dtype:
        raise ValueError("merge_states: prefix, suffix and out must share [T,N,D]; prefix and suffix share a dtype")
    if prefix_out.dtype not in _DT or out.dtype not in _DT:
        raise TypeError("merge_states: bf16 / fp32 only")
    for x in (prefix_out, suffix_out, out):
        if x.stride(-1) != 1:
            raise ValueError("merge_states: last dim must be contiguous")
    for l in (prefix_lse, suffix_lse, out_lse):
        if l is not None and (l.dtype != torch.float32 or l.numel() != t * n or not l.is_contiguous()):
            raise TypeError("merge_states: lse tensors must be contiguous fp32 with T*N elements")
    rc = lib.mla_merge_states(prefix_out.data_ptr(), prefix_out.stride(0), prefix_out.stride(1), prefix_lse.data_ptr(),
                              suffix_out.data_ptr(), suffix_out.stride(0), suffix_out.stride(1), suffix_lse.data_ptr(),
                              _DT[prefix_out.dtype], out.data_ptr(), out.stride(0), out.stride(1), _DT[out.dtype],
                              out_lse.data_ptr() if out_lse is not None else None, t, n, d, _stream(out))
    _lib.check(rc, "mla_merge_states")


def merge_n_states(outs: torch.Tensor, lses: torch.Tensor, out: Optional[torch.Tensor] = None,
                   lse_out: Optional[torch.Tensor] = None):
    """N-way log-sum-exp merge in one launch (reference: attention_update_torch, src/omni_npu/attention/ops.py:109-141).
    outs [n,T,D] bf16 / fp16 / fp32 (last dim contiguous), lses fp32 [n,T] -> (out fp32 [T,D], lse fp32 [T])."""
    _need_cuda(outs, lses, out, lse_out)
    if outs.dim() != 3 or lses.dim() != 2 or outs.shape[:2] != lses.shape:
        raise ValueError("merge_n_states: outs [n,T,D] and lses [n,T] expected")
    codes = {torch.bfloat16: 0, torch.float32: 1, torch.float16: 2}
    if outs.dtype not in codes:
        raise TypeError("merge_n_states: bf16 / fp16 / fp32 partials only")
    if outs.stride(-1) != 1:
        raise ValueError("merge_n_states: last dim must be contiguous")
    n, t, d = outs.shape
    lses = lses.float()
    if lses.stride(-1) != 1:
        lses = lses.contiguous()
    if out is None:
        out = torch.empty(t, d, dtype=torch.float32, device=outs.device)
    if lse_out is None:
        lse_out = torch.empty(t, dtype=torch.float32, device=outs.device)
    if out.dtype != torch.float32 or out.shape != (t, d) or out.stride(-1) != 1 or lse_out.dtype != torch.float32 or \
            lse_out.numel() != t or not lse_out.is_contiguous():
        raise TypeError("merge_n_states: out fp32 [T,D] (rows contiguous) and lse_out fp32 [T] expected")
    if n == 0:
        raise ValueError("merge_n_states: at least one partial")
    rc = _lib.load().mla_merge_n_states(outs.data_ptr(), outs.stride(0), outs.stride(1), codes[outs.dtype], lses.data_ptr(),
                                        lses.stride(0), out.data_ptr(), out.stride(0), lse_out.data_ptr(), n, t, d,
                                        _stream(out))
    _lib.check(rc, "mla_merge_n_states")
    return out, lse_out


# ------------------------------------------------------------------------------------------------
_workspaces: dict = {}


def _workspace(dev: torch.device, nbytes: int, tag: str = "decode") -> torch.Tensor:
    """Scratch memory of at least ``nbytes``, kept per (device, stream, tag).

    A buffer handed out once is NEVER freed: a HIP graph captured earlier holds its address, and memory returned to the
    caching allocator would be given to other tensors while replays of that graph still write split-KV partials into it.
    When a later call needs more, a new buffer (at least 1.5 x the old size) is allocated next to the old ones, which stay
    alive; an earlier graph keeps using the buffer it captured.  Buffers are not shared between streams, so steps running
    concurrently on different streams do not write into each other's partials.  Callers that want to own the lifetime pass
    ``workspace=`` instead."""
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream, tag)
    bufs = _workspaces.setdefault(key, [])
    size = _workspace_growth(bufs[-1].numel() if bufs else 0, nbytes)
    if size:
        bufs.append(torch.empty(size, dtype=torch.uint8, device=dev))
    return bufs[-1]


def _workspace_growth(have: int, nbytes: int) -> int:
    """Size of the buffer to allocate next to one of ``have`` bytes for a request of ``nbytes`` (0: the one there is
    enough).  Every new buffer is at least 1.5 x its predecessor, so a key that has seen requests up to M bytes holds at
    most 2 + log1.5(M / first request) buffers and less than 4.5 M bytes in total (the newest is below 1.5 M, the one
    before it below M, the older ones shrink geometrically)."""
    if have >= max(nbytes, 1):
        return 0
    return max(nbytes, 1, (have * 3) // 2)


def retained_workspace_bytes() -> int:
    """Bytes of scratch this process holds in all (device, stream, tag) keys; they are released at process end only."""
    return sum(b.numel() for bufs in _workspaces.values() for b in bufs)


# Sparse MLA over many tokens (a DSA prefill chunk) runs in launches of at most this much split-KV scratch, so the scratch
# does not grow with the prefill chunk (128 heads, one split: about 970 tokens per launch)
SPARSE_WORKSPACE_CAP = 256 << 20


def default_num_splits(batch: int, max_q_len: int, num_heads: int, max_seq_len: int, num_cus: int = 256) -> int:
    """Static split count (a function of shapes only, so a captured graph stays valid)."""
    groups = batch * math.ceil(max_q_len * num_heads / 128)
    # a chunk should hold at least eight 32-key blocks: that is what starting a segment costs
    by_length = max(1, math.ceil(max_seq_len / 256))
    want = max(1, math.ceil(num_cus / max(groups, 1)))
    return int(max(1, min(want, by_length, 256)))


def _vup_out(out: torch.Tensor, w_uv: torch.Tensor, t: int, n: int) -> torch.Tensor:
    """The [T,N,128] view of the output of a decode with the value up-projection fused in, after checking w_uv."""
    _need_cuda(w_uv)
    if w_uv.dtype != torch.bfloat16 or w_uv.shape != (n, D_NOPE, 128) or w_uv.stride(2) != 1:
        raise TypeError(f"w_uv must be bf16 [{n},512,128] with contiguous rows, got {tuple(w_uv.shape)}")
    o3 = out.view(t, n, 128) if out.dim() == 2 else out
    if o3.shape != (t, n, 128) or o3.dtype != torch.bfloat16 or o3.stride(-1) != 1:
        raise ValueError(f"with w_uv the output must be bf16 [T, N*128] or [T,N,128], got {tuple(out.shape)}")
    return o3


# The fused merge + up-projection gives a row to ONE wavefront (six partials per round trip).  Past this many partials per
# sequence (few sequences with long contexts) the separate merge, which puts a workgroup on every row, followed by the
# library GEMM is faster ...
VUP_MAX_SPLITS = 11
# ... and past this many query tokens a workgroup of the fused kernel walks through many passes of 16 tokens one after
# the other, while the separate merge keeps every row in flight (measured break-even at 128 heads: 256 tokens)
VUP_MAX_TOKENS = 256


def _reduce_vup(lib, ws_args, seq_lens, qsl, b, q_len, n, num_splits, t, w_uv, o3, st) -> None:
    if num_splits > VUP_MAX_SPLITS or t > VUP_MAX_TOKENS:
        o = torch.empty(n, t, D_NOPE, dtype=torch.bfloat16, device=o3.device)
        rc = lib.mla_splitkv_reduce(*ws_args, seq_lens.data_ptr(), qsl, b, q_len, n, num_splits, o.data_ptr(), o.stride(1),
                                    o.stride(0), None, st)
        _lib.check(rc, "mla_splitkv_reduce")
        o3.copy_(torch.bmm(o, w_uv).transpose(0, 1))
        return
    rc = lib.mla_splitkv_reduce_vup(*ws_args, seq_lens.data_ptr(), qsl, b, q_len, n, num_splits, t, w_uv.data_ptr(),
                                    w_uv.stride(0), w_uv.stride(1), o3.data_ptr(), o3.stride(0), o3.stride(1), st)
    _lib.check(rc, "mla_splitkv_reduce_vup")


def _decode_args(q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, scale, out, out_width, q_len,
                 query_start_loc, lse_out, num_splits, max_seq_len, workspace):
    """Checks shared by decode() and decode_vup(); returns what the C calls need."""
    _need_cuda(q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, out)
    lib = _lib.load()
    nope, rope = _cache3(nope_cache, D_NOPE), _cache3(rope_cache, D_ROPE)
    t, n, _ = q_nope.shape
    b = seq_lens.numel()
    if q_nope.shape != (t, n, D_NOPE) or q_rope.shape != (t, n, D_ROPE) or out.shape != (t, n, out_width):
        raise ValueError(f"decode: q_nope {tuple(q_nope.shape)} q_rope {tuple(q_rope.shape)} out {tuple(out.shape)} (want [T,N,{out_width}])")
    for x in (q_nope, q_rope, out, nope, rope):
        if x.dtype != torch.bfloat16 or x.stride(-1) != 1:
            raise TypeError("decode: bf16 tensors with a contiguous last dim only")
    if block_table.dtype != torch.int32 or seq_lens.dtype != torch.int32 or block_table.stride(-1) != 1:
        raise TypeError("decode: block_table and seq_lens must be int32")
    if not seq_lens.is_contiguous():
        seq_lens = seq_lens.contiguous()
    if block_table.shape[0] < b:
        raise ValueError("decode: block_table has fewer rows than seq_lens")
    if query_start_loc is None and t != b * q_len:
        raise ValueError(f"decode: {t} query tokens != batch {b} x q_len {q_len}")
    if query_start_loc is not None and (query_start_loc.dtype != torch.int32 or query_start_loc.numel() != b + 1):
        raise TypeError("decode: query_start_loc must be int32 [B+1]")
    if lse_out is not None and (lse_out.dtype != torch.float32 or lse_out.shape != (t, n) or not lse_out.is_contiguous()):
        raise TypeError("decode: lse_out must be contiguous fp32 [T,N]")
    if max_seq_len is None:
        max_seq_len = block_table.shape[1] * nope.shape[1]
    if nope.shape[1] != PAGE:
        raise ValueError("decode: page size must be 128")
    if num_splits is None:
        num_splits = default_num_splits(b, q_len, n, max_seq_len)
    need = lib.mla_decode_workspace_bytes(b, q_len, n, num_splits)
    ws = workspace if workspace is not None else _workspace(q_nope.device, need)
    qsl = query_start_loc.data_ptr() if query_start_loc is not None else None
    front = (q_nope.data_ptr(), q_nope.stride(0), q_nope.stride(1), q_rope.data_ptr(), q_rope.stride(0), q_rope.stride(1),
             nope.data_ptr(), nope.stride(0), nope.stride(1), rope.data_ptr(), rope.stride(0), rope.stride(1),
             nope.shape[0], block_table.data_ptr(), block_table.stride(0), block_table.shape[1], seq_lens.data_ptr(),
             qsl, b, q_len, n, float(scale))
    ws_args = (ws.data_ptr(), ws.numel() * ws.element_size())
    lse_p = lse_out.data_ptr() if lse_out is not None else None
    st = _stream(q_nope)
    return lib, front, ws_args, lse_p, st, qsl, seq_lens, b, n, num_splits


def decode(q_nope: torch.Tensor, q_rope: torch.Tensor, nope_cache: torch.Tensor, rope_cache: torch.Tensor,
           block_table: torch.Tensor, seq_lens: torch.Tensor, scale: float, out: torch.Tensor,
           q_len: int = 1, query_start_loc: Optional[torch.Tensor] = None, lse_out: Optional[torch.Tensor] = None,
           num_splits: Optional[int] = None, max_seq_len: Optional[int] = None,
           workspace: Optional[torch.Tensor] = None, phase: str = "both",
           w_uv: Optional[torch.Tensor] = None, sink_len: int = 0, window: Optional[int] = None,
           new_rows: Optional[tuple] = None) -> torch.Tensor:
    """Absorbed-MLA paged decode (reference: FIA decode call, src/omni_npu/attention/backends/mla.py:781-804).

    q_nope [T,N,512], q_rope [T,N,64] (any token/head strides), caches [nblk,128,512] / [nblk,128,64],
    block_table int32 [B,maxblk], seq_lens int32 [B] on the device, ``out`` a bf16 tensor viewed as
    [T,N,512] through its strides: pass ``o.transpose(0,1)`` of an [N,T,512] buffer for the reference's
    head-major result.  Sequence b owns query tokens [b*q_len, (b+1)*q_len) unless query_start_loc
    (int32 [B+1], device) says otherwise; token i of a request sees keys [0, L - s + i].
    ``phase`` = "both" | "split" | "reduce" runs the split-KV kernel, the reduction, or both (one C call).
    With ``w_uv`` (bf16 [N,512,128], the reference's W_UV) the value up-projection of mla.py:309-315 is fused into the
    reduction: ``out`` is then [T, N*128] (or a [T,N,128] view) and holds o[t,n,:] @ w_uv[n]; no lse_out.
    With ``window`` the call is the static-sink + sliding-window decode of mla.py:705-779 as one attention: the first
    ``sink_len`` keys of every block-table row are the sink, ``seq_lens`` counts the keys behind them, and a token sees
    the sink plus the newest ``window`` keys it may see.
    ``new_rows`` = (kv_c [T,512], k_pe [T,64] or [T,1,64], slot_mapping int64 [T]): the step's cache write
    (mla.py:868-881) rides in the split kernel instead of being a launch of its own; the caches must hold the rows
    of every earlier token, and ``seq_lens`` counts the new ones.
    """
    if new_rows is not None:
        if window is not None or w_uv is not None or phase not in ("both", "split"):
            raise ValueError("decode: new_rows goes with the plain decode (both phases, or the split phase alone)")
        kv_c, k_pe, slots = new_rows
        k_pe = k_pe.reshape(k_pe.shape[0], -1)
        t = q_nope.shape[0]
        _need_cuda(kv_c, k_pe, slots)
        if kv_c.shape != (t, D_NOPE) or k_pe.shape != (t, D_ROPE) or kv_c.dtype != torch.bfloat16 or \
                k_pe.dtype != torch.bfloat16 or kv_c.stride(-1) != 1 or k_pe.stride(-1) != 1:
            raise ValueError(f"decode: new rows must be bf16 [T,{D_NOPE}] and [T,{D_ROPE}] with contiguous last dims")
        if slots.dtype != torch.int64 or slots.numel() < t or not slots.is_contiguous():
            raise TypeError("decode: slot_mapping must be contiguous int64 with an entry per query token")
        lib, front, ws_args, lse_p, st, qsl, seq_lens, b, n, num_splits = _decode_args(
            q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, scale, out, D_NOPE, q_len, query_start_loc,
            lse_out, num_splits, max_seq_len, workspace)
        rc = lib.mla_decode_bf16_step(*front[:13], kv_c.data_ptr(), kv_c.stride(0), k_pe.data_ptr(), k_pe.stride(0),
                                      slots.data_ptr(), *front[13:], out.data_ptr() if phase == "both" else None,
                                      out.stride(0), out.stride(1), lse_p, *ws_args, num_splits, st)
        _lib.check(rc, "mla_decode_bf16_step")
        return out
    if window is not None:
        return _decode_window(q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, scale, out, q_len,
                              query_start_loc, lse_out, num_splits, max_seq_len, workspace, phase, w_uv, sink_len, window)
    if sink_len:
        raise ValueError("decode: sink_len goes with window (without one, pass seq_lens + sink_len)")
    if w_uv is not None:
        if lse_out is not None or phase == "split":
            raise ValueError("decode: w_uv goes with the reduction and without lse_out")
        t, n, _ = q_nope.shape
        o3 = _vup_out(out, w_uv, t, n)
        lib, front, ws_args, _, st, qsl, seq_lens, b, n, num_splits = _decode_args(
            q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, scale, o3, 128, q_len, query_start_loc, None,
            num_splits, max_seq_len, workspace)
        if phase == "both":
            _lib.check(lib.mla_decode_bf16_split(*front, *ws_args, num_splits, st), "mla_decode_bf16_split")
        elif phase != "reduce":
            raise ValueError(f"decode: unknown phase {phase!r}")
        _reduce_vup(lib, ws_args, seq_lens, qsl, b, q_len, n, num_splits, t, w_uv, o3, st)
        return out
    lib, front, ws_args, lse_p, st, qsl, seq_lens, b, n, num_splits = _decode_args(
        q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, scale, out, D_NOPE, q_len, query_start_loc, lse_out,
        num_splits, max_seq_len, workspace)
    if phase == "both":
        rc = lib.mla_decode_bf16(*front, out.data_ptr(), out.stride(0), out.stride(1), lse_p, *ws_args, num_splits, st)
        _lib.check(rc, "mla_decode_bf16")
    elif phase == "split":
        _lib.check(lib.mla_decode_bf16_split(*front, *ws_args, num_splits, st), "mla_decode_bf16_split")
    elif phase == "reduce":
        rc = lib.mla_splitkv_reduce(*ws_args, seq_lens.data_ptr(), qsl, b, q_len, n, num_splits, out.data_ptr(), out.stride(0), out.stride(1),
                                    lse_p, st)
        _lib.check(rc, "mla_splitkv_reduce")
    else:
        raise ValueError(f"decode: unknown phase {phase!r}")
    return out


def _decode_window(q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, scale, out, q_len, query_start_loc,
                   lse_out, num_splits, max_seq_len, workspace, phase, w_uv, sink_len, window):
    """decode() with static sink keys and a sliding window: a plan kernel shortens every sequence to sink + window
    blocks, the dense split kernel walks the shortened sequences, and the ordinary merge (or merge + up-projection)
    follows with the shortened lengths."""
    if phase != "both":
        raise ValueError("decode: the windowed decode runs both phases")
    if window < 1 or sink_len < 0 or sink_len % PAGE != 0:
        raise ValueError(f"decode: window {window} must be positive and sink_len {sink_len} a whole number of pages")
    if w_uv is not None and lse_out is not None:
        raise ValueError("decode: w_uv goes without lse_out")
    t, n, _ = q_nope.shape
    o3 = _vup_out(out, w_uv, t, n) if w_uv is not None else None
    longest = sink_len + window + 32 + q_len                  # keys of a shortened sequence
    max_seq_len = longest if max_seq_len is None else min(max_seq_len, longest)
    lib, front, ws_args, lse_p, st, qsl, seq_lens, b, n, num_splits = _decode_args(
        q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, scale, out if o3 is None else o3,
        D_NOPE if o3 is None else 128, q_len, query_start_loc, lse_out, num_splits, max_seq_len, workspace)
    plan = torch.empty(2, b, dtype=torch.int32, device=q_nope.device)      # shortened lengths, blocks left out
    short, skip = plan[0], plan[1]
    _lib.check(lib.mla_window_plan(seq_lens.data_ptr(), qsl, b, q_len, sink_len, window, short.data_ptr(), skip.data_ptr(), st),
               "mla_window_plan")
    rc = lib.mla_decode_bf16_window_split(*front[:16], short.data_ptr(), skip.data_ptr(), qsl, b, q_len, n, sink_len, window,
                                          float(scale), *ws_args, num_splits, st)
    _lib.check(rc, "mla_decode_bf16_window_split")
    if o3 is not None:
        _reduce_vup(lib, ws_args, short, qsl, b, q_len, n, num_splits, t, w_uv, o3, st)
    else:
        rc = lib.mla_splitkv_reduce(*ws_args, short.data_ptr(), qsl, b, q_len, n, num_splits, out.data_ptr(), out.stride(0),
                                    out.stride(1), lse_p, st)
        _lib.check(rc, "mla_splitkv_reduce")
    return out


# ------------------------------------------------------------------------------------------------
# DSA: lightning indexer, top-k, sparse decode
def indexer_logits_stride(max_seq_len: int) -> int:
    return (int(max_seq_len) + 31) // 32 * 32


def indexer_scores(q8: torch.Tensor, weights: torch.Tensor, k8_cache: torch.Tensor, k_scale_cache: torch.Tensor,
                   block_table: torch.Tensor, seq_lens: torch.Tensor, logits: torch.Tensor, q_len: int = 1,
                   q_scale: Optional[torch.Tensor] = None, query_start_loc: Optional[torch.Tensor] = None,
                   max_seq_len: Optional[int] = None) -> torch.Tensor:
    """logits[t, s] = k_scale[s] * sum_h w[t,h] (* q_scale[t,h]) * relu(q8[t,h] . k8[s]) for the visible keys s of token t.

    q8 [T,64,128] float8_e4m3fn (or uint8 bits), weights fp32 [T,64], k8_cache [nblk,page,128] fp8, k_scale_cache fp32
    [nblk,page], logits fp32 [T, >= round_up(max_seq_len, 32)] (reference call site:
    src/omni_npu/v1/layers/attention/npu_dsa.py:92-103)."""
    _need_cuda(q8, weights, k8_cache, k_scale_cache, block_table, seq_lens, logits, q_scale)
    lib = _lib.load()
    if k8_cache.dim() == 4 and k8_cache.shape[2] == 1:
        k8_cache = k8_cache.squeeze(2)
    t, h, d = q8.shape
    b = seq_lens.numel()
    if d != 128 or k8_cache.dim() != 3 or k8_cache.shape[-1] != 128 or q8.element_size() != 1 or k8_cache.element_size() != 1:
        raise ValueError("indexer_scores: q8 [T,H,128] and k8_cache [nblk,page,128] must be 1-byte fp8 tensors")
    if q8.stride(-1) != 1 or k8_cache.stride(-1) != 1:
        raise ValueError("indexer_scores: fp8 rows must be contiguous")
    if weights.dtype != torch.float32 or weights.shape != (t, h) or weights.stride(-1) != 1:
        raise TypeError("indexer_scores: weights must be fp32 [T,H]")
    if q_scale is not None and (q_scale.dtype != torch.float32 or q_scale.shape != (t, h) or q_scale.stride(-1) != 1):
        raise TypeError("indexer_scores: q_scale must be fp32 [T,H]")
    if k_scale_cache.dtype != torch.float32 or k_scale_cache.shape[:2] != k8_cache.shape[:2] or k_scale_cache.reshape(
            k8_cache.shape[0], k8_cache.shape[1]).stride(-1) != 1:
        raise TypeError("indexer_scores: k_scale_cache must be fp32 [nblk,page]")
    k_scale_cache = k_scale_cache.reshape(k8_cache.shape[0], k8_cache.shape[1])
    if block_table.dtype != torch.int32 or seq_lens.dtype != torch.int32 or logits.dtype != torch.float32:
        raise TypeError("indexer_scores: int32 tables / lens, fp32 logits")
    if max_seq_len is None:
        max_seq_len = min(block_table.shape[1] * k8_cache.shape[1], logits.shape[1])
    if logits.shape[0] < t or logits.stride(1) != 1 or logits.shape[1] < indexer_logits_stride(max_seq_len):
        raise ValueError("indexer_scores: logits must be [T, >= round_up(max_seq_len, 32)]")
    if query_start_loc is None and t != b * q_len:
        raise ValueError(f"indexer_scores: {t} query tokens != batch {b} x q_len {q_len}")
    rc = lib.dsa_indexer_scores_fp8(
        q8.data_ptr(), q8.stride(0), q8.stride(1), weights.data_ptr(), weights.stride(0),
        q_scale.data_ptr() if q_scale is not None else None, q_scale.stride(0) if q_scale is not None else 0,
        k8_cache.data_ptr(), k8_cache.stride(0), k8_cache.stride(1), k_scale_cache.data_ptr(), k_scale_cache.stride(0),
        k8_cache.shape[0], k8_cache.shape[1], block_table.data_ptr(), block_table.stride(0), block_table.shape[1],
        seq_lens.data_ptr(), query_start_loc.data_ptr() if query_start_loc is not None else None, b, q_len, h,
        int(max_seq_len), logits.data_ptr(), logits.stride(0), _stream(q8))
    _lib.check(rc, "dsa_indexer_scores_fp8")
    return logits


def topk(logits: torch.Tensor, seq_lens: torch.Tensor, k: int, out: torch.Tensor, q_len: int = 1,
         query_start_loc: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
         single_workgroup: bool = False, block_table: Optional[torch.Tensor] = None, page_size: int = PAGE,
         num_pages: int = 0, rows: Optional[torch.Tensor] = None, counts: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Positions of the k largest logits among each token's visible keys, ties to the lower position, ascending
    position order, -1 padding; out int32 [T,k] or [T,1,k] (patch_dsv32_indexer.py:133-146).
    single_workgroup=True runs the variant that needs no scratch memory (one workgroup per token).
    With block_table / num_pages / rows [T,k] / counts [T] the same launch also fills the flat cache rows and the pick
    counts that build_sparse_rows would produce from `out`."""
    _need_cuda(logits, seq_lens, out)
    lib = _lib.load()
    o2 = out.reshape(out.shape[0], -1) if out.dim() == 3 else out
    if o2.data_ptr() != out.data_ptr():
        raise ValueError("topk: out must be viewable as [T,k]")
    if logits.dtype != torch.float32 or logits.stride(-1) != 1 or o2.dtype != torch.int32 or o2.stride(-1) != 1 or o2.shape[1] < k:
        raise TypeError("topk: fp32 logits [T,S], int32 out [T,>=k]")
    b = seq_lens.numel()
    ws_ptr, ws_bytes = None, 0
    if not single_workgroup:
        need = lib.dsa_topk_workspace_bytes(b, q_len, logits.stride(0))
        ws = workspace if workspace is not None else _workspace(logits.device, need, tag="topk")
        ws_ptr, ws_bytes = ws.data_ptr(), ws.numel() * ws.element_size()
    qsl = query_start_loc.data_ptr() if query_start_loc is not None else None
    if rows is not None:
        _need_cuda(block_table, rows, counts)
        if block_table is None or counts is None or rows.dtype != torch.int32 or rows.dim() != 2 or rows.shape[1] < k or \
                rows.stride(-1) != 1 or counts.dtype != torch.int32 or not counts.is_contiguous() or \
                block_table.dtype != torch.int32 or num_pages < 1:
            raise TypeError("topk: rows int32 [T,>=k], counts int32 [T], int32 block_table and num_pages go together")
        rc = lib.dsa_topk_rows(logits.data_ptr(), logits.stride(0), seq_lens.data_ptr(), qsl, b, q_len, k, o2.data_ptr(),
                               o2.stride(0), block_table.data_ptr(), block_table.stride(0), block_table.shape[1], page_size,
                               num_pages, rows.data_ptr(), rows.stride(0), counts.data_ptr(), ws_ptr, ws_bytes,
                               _stream(logits))
        _lib.check(rc, "dsa_topk_rows")
        return out
    rc = lib.dsa_topk(logits.data_ptr(), logits.stride(0), seq_lens.data_ptr(), qsl, b, q_len, k, o2.data_ptr(),
                      o2.stride(0), ws_ptr, ws_bytes, _stream(logits))
    _lib.check(rc, "dsa_topk")
    return out


def build_sparse_rows(indices: torch.Tensor, block_table: torch.Tensor, seq_lens: torch.Tensor, page_size: int,
                      num_pages: int, rows: torch.Tensor, counts: torch.Tensor, q_len: int = 1,
                      query_start_loc: Optional[torch.Tensor] = None) -> None:
    """Translate logical key positions [T,(1,)K] (-1 = unused) into flat cache rows, compacted, plus a count per token."""
    _need_cuda(indices, block_table, seq_lens, rows, counts)
    lib = _lib.load()
    idx = indices.reshape(indices.shape[0], -1)
    if idx.dtype != torch.int32 or idx.stride(-1) != 1 or rows.dtype != torch.int32 or rows.shape != idx.shape or \
            rows.stride(-1) != 1 or counts.dtype != torch.int32 or counts.numel() < idx.shape[0] or not counts.is_contiguous():
        raise TypeError("build_sparse_rows: int32 indices [T,K], rows [T,K], counts [T]")
    b = seq_lens.numel()
    rc = lib.dsa_build_rows(idx.data_ptr(), idx.stride(0), block_table.data_ptr(), block_table.stride(0),
                            block_table.shape[1], seq_lens.data_ptr(),
                            query_start_loc.data_ptr() if query_start_loc is not None else None, b, q_len, idx.shape[1],
                            page_size, num_pages, rows.data_ptr(), rows.stride(0), counts.data_ptr(), _stream(idx))
    _lib.check(rc, "dsa_build_rows")


def sparse_decode(q_nope: torch.Tensor, q_rope: torch.Tensor, nope_cache: torch.Tensor, rope_cache: torch.Tensor,
                  rows: torch.Tensor, counts: torch.Tensor, scale: float, out: torch.Tensor,
                  lse_out: Optional[torch.Tensor] = None, num_splits: Optional[int] = None,
                  workspace: Optional[torch.Tensor] = None, w_uv: Optional[torch.Tensor] = None,
                  counts_bounded: bool = False, method: str = "auto") -> torch.Tensor:
    """Absorbed MLA of token t over cache rows rows[t, :counts[t]] (reference: npu_sparse_flash_attention call,
    src/omni_npu/attention/backends/dsa.py:259-291).  out bf16 viewed as [T,N,512]; with ``w_uv`` (bf16 [N,512,128])
    the value up-projection of dsa.py:233-240 is fused into the merge and out is [T, N*128] / [T,N,128].

    ``method``: "keys" cuts every token's keys into ``num_splits`` chunks (split-KV partials + merge: the form for few
    heads or few tokens); "heads" gives every (token, 16 heads) a workgroup that walks all of the token's keys and
    writes the result itself (one launch, no scratch, every probability carried as two bf16 numbers; heads a multiple
    of 16, no ``w_uv``).  Measured at 32 tokens x 128 heads x 2048 keys: 56 us against 50 us for "keys" (split + merge),
    so "auto" is "keys"; the form is there for callers without scratch memory.

    counts[t] must not exceed rows.shape[1]; unless the caller vouches for that (``counts_bounded``: the counts come from
    build_sparse_rows / topk_rows) they are clamped here.  Many tokens (a prefill chunk) run as several launches so that
    the split-KV scratch stays below SPARSE_WORKSPACE_CAP and the launch below the grid limit."""
    _need_cuda(q_nope, q_rope, nope_cache, rope_cache, rows, counts, out)
    lib = _lib.load()
    nope, rope = _cache3(nope_cache, D_NOPE), _cache3(rope_cache, D_ROPE)
    t, n, _ = q_nope.shape
    o3 = None
    if w_uv is not None:
        if lse_out is not None:
            raise ValueError("sparse_decode: w_uv goes without lse_out")
        o3 = _vup_out(out, w_uv, t, n)
    if q_rope.shape != (t, n, D_ROPE) or (o3 is None and out.shape != (t, n, D_NOPE)) or rows.shape[0] < t or counts.numel() < t:
        raise ValueError("sparse_decode: shape mismatch")
    for x in (q_nope, q_rope, out, nope, rope):
        if x.dtype != torch.bfloat16 or x.stride(-1) != 1:
            raise TypeError("sparse_decode: bf16 tensors with a contiguous last dim only")
    if rows.dtype != torch.int32 or counts.dtype != torch.int32 or rows.stride(-1) != 1 or not counts.is_contiguous():
        raise TypeError("sparse_decode: int32 rows [T,K] and counts [T]")
    if lse_out is not None and (lse_out.dtype != torch.float32 or lse_out.numel() != t * n or not lse_out.is_contiguous()):
        raise TypeError("sparse_decode: lse_out must be contiguous fp32 [T,N]")
    if not counts_bounded:
        counts = counts[:t].clamp(max=rows.shape[1])
    if method not in ("auto", "keys", "heads"):
        raise ValueError(f"sparse_decode: unknown method {method!r}")
    heads_ok = w_uv is None and n % 16 == 0 and nope.stride(0) == nope.shape[1] * nope.stride(1) and \
        rope.stride(0) == rope.shape[1] * rope.stride(1)
    if method == "heads" and not heads_ok:
        raise ValueError("sparse_decode: the heads form wants a multiple of 16 heads, contiguous cache pages and no w_uv")
    if method == "heads":
        st = _stream(q_nope)
        for t0 in range(0, t, 1 << 20):
            t1 = min(t, t0 + (1 << 20))
            qn, qr, rw, ct, oc = q_nope[t0:t1], q_rope[t0:t1], rows[t0:t1], counts[t0:t1], out[t0:t1]
            rc = lib.dsa_sparse_decode_heads_bf16(
                qn.data_ptr(), qn.stride(0), qn.stride(1), qr.data_ptr(), qr.stride(0), qr.stride(1), nope.data_ptr(),
                nope.stride(1), rope.data_ptr(), rope.stride(1), nope.shape[0] * nope.shape[1], rw.data_ptr(), rw.stride(0),
                ct.data_ptr(), t1 - t0, n, float(scale), oc.data_ptr(), oc.stride(0), oc.stride(1),
                lse_out.view(t, n)[t0:t1].data_ptr() if lse_out is not None else None, st)
            _lib.check(rc, "dsa_sparse_decode_heads_bf16")
        return out
    if num_splits is None:
        num_splits = default_num_splits(t, 1, n, rows.shape[1])
    per_token = lib.mla_decode_workspace_bytes(1, 1, n, num_splits)
    cap = workspace.numel() * workspace.element_size() if workspace is not None else SPARSE_WORKSPACE_CAP
    step = max(1, min(t, cap // max(per_token, 1), 32768))
    need = lib.mla_decode_workspace_bytes(min(step, max(t, 1)), 1, n, num_splits)
    ws = workspace if workspace is not None else _workspace(q_nope.device, need)
    ws_args = (ws.data_ptr(), ws.numel() * ws.element_size())
    st = _stream(q_nope)
    lse2 = lse_out.view(t, n) if lse_out is not None else None
    for t0 in range(0, t, step):
        t1 = min(t, t0 + step)
        qn, qr, rw, ct = q_nope[t0:t1], q_rope[t0:t1], rows[t0:t1], counts[t0:t1]
        oc = out[t0:t1] if o3 is None else None
        rc = lib.dsa_sparse_decode_bf16(
            qn.data_ptr(), qn.stride(0), qn.stride(1), qr.data_ptr(), qr.stride(0), qr.stride(1),
            nope.data_ptr(), nope.stride(0), nope.stride(1), rope.data_ptr(), rope.stride(0), rope.stride(1), nope.shape[0],
            nope.shape[1], rw.data_ptr(), rw.stride(0), ct.data_ptr(), t1 - t0, n, float(scale),
            oc.data_ptr() if oc is not None else None, oc.stride(0) if oc is not None else 0,
            oc.stride(1) if oc is not None else 0, lse2[t0:t1].data_ptr() if lse2 is not None else None, *ws_args,
            num_splits, st)
        _lib.check(rc, "dsa_sparse_decode_bf16")
        if o3 is not None:
            _reduce_vup(lib, ws_args, ct, None, t1 - t0, 1, n, num_splits, t1 - t0, w_uv, o3[t0:t1], st)
    return out


# ------------------------------------------------------------------------------------------------
_PREFILL_KV_F16 = 16                                       # added to the output dtype code: k_nope, k_pe, v hold fp16


def prefill_varlen(q_nope: torch.Tensor, q_pe: torch.Tensor, k_nope: torch.Tensor, k_pe: torch.Tensor, v: torch.Tensor,
                   cu_q: torch.Tensor, cu_k: torch.Tensor, max_q_len: int, scale: float, causal: bool,
                   out: torch.Tensor, lse_out: Optional[torch.Tensor] = None, window: Optional[int] = None,
                   prev_out: Optional[torch.Tensor] = None, prev_lse: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Varlen non-absorbed MLA attention (reference: the prefill FIA calls, src/omni_npu/attention/backends/mla.py:574-590
    and :415-431).  q_nope [T,N,128], q_pe [T,N,64], k_nope [Tk,N,128], k_pe [Tk,64] (shared by the heads), v [Tk,N,128],
    cu_q / cu_k int32 [B+1] device tensors, out [T,N,128] bf16 or fp32, lse_out fp32 [T,N].  ``window`` keeps only the
    newest ``window`` visible keys of each row (the sliding-window band of mla.py:525-541).
    ``prev_out`` (fp32 [T,N,128]) / ``prev_lse`` (fp32 [T,N]): the result of an earlier call over OTHER keys of the same
    rows; the call then returns the attention over the union, i.e. what this attention followed by merge_attn_states
    (src/omni_npu/attention/ops.py:5-42) gives, in one launch.  ``out`` may be ``prev_out``.
    k_nope, k_pe and v may all three be fp16 (a caller that makes them with an fp16 GEMM): both products then run on fp16
    and the kernel skips the conversion of the value tiles it otherwise does (the queries stay bf16)."""
    if window is not None and window < 1:
        raise ValueError(f"prefill_varlen: window must be positive (got {window})")
    _need_cuda(q_nope, q_pe, k_nope, k_pe, v, cu_q, cu_k, out, lse_out)
    lib = _lib.load()
    t, n, p = q_nope.shape
    k_pe = k_pe.reshape(k_pe.shape[0], 64)
    if p != 128 or q_pe.shape != (t, n, 64) or k_nope.shape[1:] != (n, 128) or v.shape != k_nope.shape or \
            k_pe.shape != (k_nope.shape[0], 64) or out.shape != (t, n, 128):
        raise ValueError("prefill_varlen: shapes must be q_nope [T,N,128], q_pe [T,N,64], k_nope/v [Tk,N,128], k_pe [Tk,64]")
    kv_half = k_nope.dtype == torch.float16
    for x, want in ((q_nope, torch.bfloat16), (q_pe, torch.bfloat16), (k_nope, None), (k_pe, k_nope.dtype), (v, k_nope.dtype)):
        if x.dtype != (want or x.dtype) or x.dtype not in (torch.bfloat16, torch.float16) or x.stride(-1) != 1:
            raise TypeError("prefill_varlen: bf16 queries, keys and values all bf16 or all fp16, with a contiguous last dim")
    kv_code = _PREFILL_KV_F16 if kv_half else 0
    if out.dtype not in _DT or out.stride(-1) != 1:
        raise TypeError("prefill_varlen: out must be bf16 or fp32")
    if cu_q.dtype != torch.int32 or cu_k.dtype != torch.int32 or cu_q.numel() != cu_k.numel() or \
            not cu_q.is_contiguous() or not cu_k.is_contiguous():
        raise TypeError("prefill_varlen: cu_q / cu_k must be contiguous int32 [B+1]")
    if lse_out is not None and (lse_out.dtype != torch.float32 or lse_out.numel() != t * n or not lse_out.is_contiguous()):
        raise TypeError("prefill_varlen: lse_out must be contiguous fp32 [T,N]")
    if (prev_out is None) != (prev_lse is None):
        raise ValueError("prefill_varlen: prev_out and prev_lse go together")
    if prev_out is not None:
        _need_cuda(prev_out, prev_lse)
        if prev_out.dtype != torch.float32 or prev_out.shape != (t, n, 128) or prev_out.stride(-1) != 1 or \
                prev_lse.dtype != torch.float32 or prev_lse.numel() != t * n or not prev_lse.is_contiguous():
            raise TypeError("prefill_varlen: prev_out must be fp32 [T,N,128], prev_lse contiguous fp32 [T,N]")
    if k_nope.shape[0] == 0 or t == 0:
        # no keys at all (a context chunk in which every sequence is empty): zeros and lse = -inf, as the kernel gives for
        # an empty key range (the earlier result itself when there is one); empty tensors have no address to hand over
        if prev_out is not None:
            if out.data_ptr() != prev_out.data_ptr():
                out.copy_(prev_out)
            if lse_out is not None and lse_out.data_ptr() != prev_lse.data_ptr():
                lse_out.copy_(prev_lse.view_as(lse_out))
            return out
        out.zero_()
        if lse_out is not None:
            lse_out.fill_(float("-inf"))
        return out
    if prev_out is not None:
        rc = lib.mla_prefill_varlen_continue(
            q_nope.data_ptr(), q_nope.stride(0), q_nope.stride(1), q_pe.data_ptr(), q_pe.stride(0), q_pe.stride(1),
            k_nope.data_ptr(), k_nope.stride(0), k_nope.stride(1), k_pe.data_ptr(), k_pe.stride(0), v.data_ptr(), v.stride(0),
            v.stride(1), cu_q.data_ptr(), cu_k.data_ptr(), cu_q.numel() - 1, n, int(max_q_len), 1 if causal else 0,
            int(window or 0), float(scale), out.data_ptr(), out.stride(0), out.stride(1), _DT[out.dtype] | kv_code,
            lse_out.data_ptr() if lse_out is not None else None, prev_out.data_ptr(), prev_out.stride(0), prev_out.stride(1),
            prev_lse.data_ptr(), _stream(q_nope))
        _lib.check(rc, "mla_prefill_varlen_continue")
        return out
    rc = lib.mla_prefill_varlen(q_nope.data_ptr(), q_nope.stride(0), q_nope.stride(1), q_pe.data_ptr(), q_pe.stride(0),
                                q_pe.stride(1), k_nope.data_ptr(), k_nope.stride(0), k_nope.stride(1), k_pe.data_ptr(),
                                k_pe.stride(0), v.data_ptr(), v.stride(0), v.stride(1), cu_q.data_ptr(), cu_k.data_ptr(),
                                cu_q.numel() - 1, n, int(max_q_len), 1 if causal else 0, int(window or 0), float(scale),
                                out.data_ptr(),
                                out.stride(0), out.stride(1), _DT[out.dtype] | kv_code,
                                lse_out.data_ptr() if lse_out is not None else None, _stream(q_nope))
    _lib.check(rc, "mla_prefill_varlen")
    return out


def decode_fp8(q_nope: torch.Tensor, q_rope: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor,
               seq_lens: torch.Tensor, scale: float, out: torch.Tensor, q_len: int = 1,
               query_start_loc: Optional[torch.Tensor] = None, lse_out: Optional[torch.Tensor] = None,
               num_splits: Optional[int] = None, max_seq_len: Optional[int] = None,
               workspace: Optional[torch.Tensor] = None, w_uv: Optional[torch.Tensor] = None, sink_len: int = 0,
               window: Optional[int] = None) -> torch.Tensor:
    """Absorbed-MLA paged decode over the fp8 block-scaled cache (uint8 [num_blocks, 128, 656], see cache_write_fp8).
    With ``w_uv`` (bf16 [N,512,128]) the value up-projection is fused into the merge: out is [T, N*128] / [T,N,128].
    ``sink_len`` / ``window``: static sink keys + sliding window as in decode()."""
    if window is None and sink_len:
        raise ValueError("decode_fp8: sink_len goes with window (without one, pass seq_lens + sink_len)")
    if window is not None and (window < 1 or sink_len < 0 or sink_len % PAGE != 0):
        raise ValueError(f"decode_fp8: window {window} must be positive and sink_len {sink_len} a whole number of pages")
    _need_cuda(q_nope, q_rope, cache, block_table, seq_lens, out)
    lib = _lib.load()
    t, n, _ = q_nope.shape
    b = seq_lens.numel()
    o3 = None
    if w_uv is not None:
        if lse_out is not None:
            raise ValueError("decode_fp8: w_uv goes without lse_out")
        o3 = _vup_out(out, w_uv, t, n)
    if cache.dtype != torch.uint8 or cache.dim() != 3 or cache.shape[1:] != (PAGE, FP8_ROW_BYTES) or cache.stride(-1) != 1:
        raise ValueError(f"decode_fp8: cache must be uint8 [num_blocks, {PAGE}, {FP8_ROW_BYTES}]")
    if q_nope.shape != (t, n, D_NOPE) or q_rope.shape != (t, n, D_ROPE) or (o3 is None and out.shape != (t, n, D_NOPE)):
        raise ValueError("decode_fp8: q_nope [T,N,512], q_rope [T,N,64], out [T,N,512]")
    for x in (q_nope, q_rope, out):
        if x.dtype != torch.bfloat16 or x.stride(-1) != 1:
            raise TypeError("decode_fp8: bf16 queries / output with a contiguous last dim")
    if block_table.dtype != torch.int32 or seq_lens.dtype != torch.int32:
        raise TypeError("decode_fp8: block_table and seq_lens must be int32")
    if block_table.dim() != 2 or block_table.shape[0] < b or block_table.stride(-1) != 1:
        raise ValueError(f"decode_fp8: block_table must be [>= {b}, max_blocks] with contiguous rows, got {tuple(block_table.shape)}")
    if not seq_lens.is_contiguous():
        seq_lens = seq_lens.contiguous()
    if query_start_loc is not None and (query_start_loc.dtype != torch.int32 or query_start_loc.numel() < b + 1 or
                                        not query_start_loc.is_contiguous()):
        raise TypeError("decode_fp8: query_start_loc must be contiguous int32 [B+1]")
    if lse_out is not None and (lse_out.dtype != torch.float32 or lse_out.numel() != t * n or not lse_out.is_contiguous()):
        raise TypeError("decode_fp8: lse_out must be contiguous fp32 [T,N]")
    if query_start_loc is None and t != b * q_len:
        raise ValueError(f"decode_fp8: {t} query tokens != batch {b} x q_len {q_len}")
    if max_seq_len is None:
        max_seq_len = block_table.shape[1] * PAGE
    if window is not None:
        max_seq_len = min(max_seq_len, sink_len + window + 32 + q_len)         # keys of a shortened sequence
    if num_splits is None:
        num_splits = default_num_splits(b, q_len, n, max_seq_len)
    need = lib.mla_decode_workspace_bytes(b, q_len, n, num_splits)
    ws = workspace if workspace is not None else _workspace(q_nope.device, need)
    if window is not None:
        if not seq_lens.is_contiguous():
            seq_lens = seq_lens.contiguous()
        st = _stream(q_nope)
        qsl = query_start_loc.data_ptr() if query_start_loc is not None else None
        ws_args = (ws.data_ptr(), ws.numel() * ws.element_size())
        plan = torch.empty(2, b, dtype=torch.int32, device=q_nope.device)  # shortened lengths, blocks left out
        short, skip = plan[0], plan[1]
        _lib.check(lib.mla_window_plan(seq_lens.data_ptr(), qsl, b, q_len, sink_len, window, short.data_ptr(),
                                       skip.data_ptr(), st), "mla_window_plan")
        rc = lib.mla_decode_fp8_window_split(
            q_nope.data_ptr(), q_nope.stride(0), q_nope.stride(1), q_rope.data_ptr(), q_rope.stride(0), q_rope.stride(1),
            cache.data_ptr(), cache.stride(0), cache.stride(1), cache.shape[0], block_table.data_ptr(), block_table.stride(0),
            block_table.shape[1], short.data_ptr(), skip.data_ptr(), qsl, b, q_len, n, sink_len, window, float(scale),
            *ws_args, num_splits, st)
        _lib.check(rc, "mla_decode_fp8_window_split")
        if o3 is not None:
            _reduce_vup(lib, ws_args, short, qsl, b, q_len, n, num_splits, t, w_uv, o3, st)
        else:
            rc = lib.mla_splitkv_reduce(*ws_args, short.data_ptr(), qsl, b, q_len, n, num_splits, out.data_ptr(), out.stride(0),
                                        out.stride(1), lse_out.data_ptr() if lse_out is not None else None, st)
            _lib.check(rc, "mla_splitkv_reduce")
        return out
    rc = lib.mla_decode_fp8(q_nope.data_ptr(), q_nope.stride(0), q_nope.stride(1), q_rope.data_ptr(), q_rope.stride(0),
                            q_rope.stride(1), cache.data_ptr(), cache.stride(0), cache.stride(1), cache.shape[0],
                            block_table.data_ptr(), block_table.stride(0), block_table.shape[1], seq_lens.data_ptr(),
                            query_start_loc.data_ptr() if query_start_loc is not None else None, b, q_len, n, float(scale),
                            out.data_ptr() if o3 is None else None, out.stride(0) if o3 is None else 0,
                            out.stride(1) if o3 is None else 0,
                            lse_out.data_ptr() if lse_out is not None else None, ws.data_ptr(),
                            ws.numel() * ws.element_size(), num_splits, _stream(q_nope))
    _lib.check(rc, "mla_decode_fp8")
    if o3 is not None:
        if not seq_lens.is_contiguous():
            seq_lens = seq_lens.contiguous()
        _reduce_vup(lib, (ws.data_ptr(), ws.numel() * ws.element_size()), seq_lens,
                    query_start_loc.data_ptr() if query_start_loc is not None else None, b, q_len, n, num_splits, t, w_uv, o3,
                    _stream(q_nope))
    return out


def quant_qk_fp8(q: torch.Tensor, q8: torch.Tensor, q_scale: torch.Tensor, k: torch.Tensor, k8_cache: torch.Tensor,
                 scale_cache: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """quant_rows_fp8(q, q8, q_scale) and quant_rows_fp8(k, k8_cache, scale_cache, slot_mapping) in one launch: the
    indexer's two quantisations of a step (src/omni_npu/vllm_patches/patches/models/deepseek/patch_dsv32_indexer.py:116-131)."""
    _need_cuda(q, q8, q_scale, k, k8_cache, scale_cache, slot_mapping)
    lib = _lib.load()
    q2, k2 = q.reshape(-1, q.shape[-1]), k.reshape(-1, k.shape[-1])
    o8, sc = q8.reshape(-1, 128), q_scale.reshape(-1)
    if k8_cache.dim() == 4 and k8_cache.shape[2] == 1:
        k8_cache = k8_cache.squeeze(2)
    for x in (q2, k2):
        if x.shape[-1] != 128 or x.dtype != torch.bfloat16 or x.stride(-1) != 1:
            raise TypeError("quant_qk_fp8: bf16 rows of 128")
    if o8.data_ptr() != q8.data_ptr() or not o8.is_contiguous() or o8.element_size() != 1 or o8.shape[0] < q2.shape[0] or \
            sc.dtype != torch.float32 or not sc.is_contiguous() or sc.numel() < q2.shape[0]:
        raise ValueError("quant_qk_fp8: q8 / q_scale must be contiguous 1-byte [R,128] / fp32 [R]")
    if k8_cache.dim() != 3 or k8_cache.element_size() != 1 or k8_cache.stride(-1) != 1 or scale_cache.dtype != torch.float32 or \
            scale_cache.shape[:2] != k8_cache.shape[:2]:
        raise ValueError("quant_qk_fp8: paged outputs must be 1-byte [nblk,page,128] and fp32 [nblk,page]")
    ksc = scale_cache.reshape(k8_cache.shape[0], k8_cache.shape[1])
    if ksc.stride(-1) != 1:
        raise ValueError("quant_qk_fp8: scale rows must be contiguous")
    if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous():
        slot_mapping = slot_mapping.to(torch.int64).contiguous()
    n = min(k2.shape[0], slot_mapping.numel())
    rc = lib.dsa_quant_qk_fp8(q2.data_ptr(), q2.stride(0), q2.shape[0], o8.data_ptr(), sc.data_ptr(), k2.data_ptr(),
                              k2.stride(0), n, slot_mapping.data_ptr(), k8_cache.data_ptr(), k8_cache.stride(0),
                              k8_cache.stride(1), ksc.data_ptr(), ksc.stride(0), k8_cache.shape[1], k8_cache.shape[0],
                              _stream(q))
    _lib.check(rc, "dsa_quant_qk_fp8")


def quant_rows_fp8(x: torch.Tensor, out8: torch.Tensor, out_scale: torch.Tensor,
                   slot_mapping: Optional[torch.Tensor] = None) -> None:
    """Per-row e4m3 quantisation of bf16 rows [R,128] (scale = amax/448).  Without ``slot_mapping``: out8 [R,128] (1-byte
    dtype), out_scale fp32 [R].  With it: out8 is a paged cache [nblk,page,128] and out_scale [nblk,page]; row r goes to
    flat slot slot_mapping[r] (negative slots skipped) - the fused indexer-K quantise-and-write."""
    _need_cuda(x, out8, out_scale, slot_mapping)
    lib = _lib.load()
    x2 = x.reshape(-1, x.shape[-1])
    if x2.shape[-1] != 128 or x2.dtype != torch.bfloat16 or x2.stride(-1) != 1 or out8.element_size() != 1 or \
            out_scale.dtype != torch.float32 or out8.stride(-1) != 1:
        raise TypeError("quant_rows_fp8: bf16 [R,128] in, 1-byte [.,128] and fp32 scales out")
    if slot_mapping is None:
        o8, sc = out8.reshape(-1, 128), out_scale.reshape(-1)
        if o8.data_ptr() != out8.data_ptr() or o8.shape[0] < x2.shape[0] or sc.numel() < x2.shape[0] or not sc.is_contiguous():
            raise ValueError("quant_rows_fp8: outputs must be contiguous and hold R rows")
        rc = lib.dsa_quant_rows_fp8(x2.data_ptr(), x2.stride(0), x2.shape[0], None, o8.data_ptr(), 0, o8.stride(0),
                                    sc.data_ptr(), 0, x2.shape[0], 1, _stream(x))
    else:
        if out8.dim() == 4 and out8.shape[2] == 1:
            out8 = out8.squeeze(2)
        if out8.dim() != 3 or out_scale.shape[:2] != out8.shape[:2]:
            raise ValueError("quant_rows_fp8: paged outputs must be [nblk,page,128] and [nblk,page]")
        sc = out_scale.reshape(out8.shape[0], out8.shape[1])
        if sc.stride(-1) != 1:
            raise ValueError("quant_rows_fp8: scale rows must be contiguous")
        if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous():
            slot_mapping = slot_mapping.to(torch.int64).contiguous()
        n = min(x2.shape[0], slot_mapping.numel())
        rc = lib.dsa_quant_rows_fp8(x2.data_ptr(), x2.stride(0), n, slot_mapping.data_ptr(), out8.data_ptr(), out8.stride(0),
                                    out8.stride(1), sc.data_ptr(), sc.stride(0), out8.shape[1], out8.shape[0], _stream(x))
    _lib.check(rc, "dsa_quant_rows_fp8")
