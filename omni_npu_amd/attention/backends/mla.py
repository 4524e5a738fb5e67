"""MLA attention backend for MI355X behind the reference's vLLM plugin contract.

Mirrors src/omni_npu/attention/backends/mla.py (class names, methods, metadata fields, error behaviour) for the
single-GPU path; every vendor op there is replaced by a HIP kernel of libmla_hip.so:
  store_kv (mla.py:868-881)                  -> kernels.cache_write / cache_write_fp8   (one launch for both caches)
  FIA decode (mla.py:781-804)                -> kernels.decode / decode_fp8             (split-KV + reduce)
  FIA prefill (mla.py:574-590, 415-431)      -> kernels.prefill_varlen
  gather / merge (ops.py)                    -> kernels.gather_paged / merge_states
The absorb and up-projection GEMMs stay torch.bmm (hipBLASLt), as in the reference (mla.py:309-315, 900-912).
Static sink tokens with or without a sliding window (mla.py:463-560, 705-779) run as ONE attention over the union of
the keys: without a window the sink pages are simply the first pages of the block table; with one the dense decode
kernel leaves out the blocks between the sink and the window (prefill: kernels.prefill_varlen with a band).  Out of scope and rejected loudly: decode context parallelism, mc2 masks.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import ClassVar, Optional, Tuple

import torch

from ... import kernels as K
from ..._vllm_compat import (AttentionCGSupport, AttentionType, MLACommonBackend, MLACommonBaseImpl,
                             MLACommonDecodeMetadata, MLACommonMetadata, MLACommonMetadataBuilder,
                             MLACommonPrefillMetadata, QueryLenSupport, get_current_vllm_config)
from .. import ops

FP8_CACHE_DTYPES = ("fp8", "fp8_e4m3")


class NPUMLABackend(MLACommonBackend):
    @staticmethod
    def get_name() -> str:
        return "NPUMLA"

    @staticmethod
    def get_metadata_cls() -> type["NPUMLAMetadata"]:
        return NPUMLAMetadata

    @staticmethod
    def get_builder_cls() -> type["NPUMLAMetadataBuilder"]:
        return NPUMLAMetadataBuilder

    @staticmethod
    def get_impl_cls() -> type["NPUMLAImpl"]:
        return NPUMLAImpl

    @staticmethod
    def reshape_kv_cache(
        raw_tensor: torch.Tensor,
        num_blocks: int,
        block_size: int,
        num_kv_heads: int,
        head_size: int,
        dtype: torch.dtype = torch.bfloat16,
    ) -> Tuple[torch.Tensor, ...]:
        """View the per-layer raw allocation as the cache tensors (reference mla.py:59-74): all nope pages
        [num_blocks, block, 512] first, then all rope pages [num_blocks, block, 64].  With dtype uint8 and head size
        656 the allocation is one fp8 block-scaled cache [num_blocks, block, 656] (see kernels.cache_write_fp8)."""
        if dtype == torch.uint8 and head_size == K.FP8_ROW_BYTES:
            raw = raw_tensor.view(dtype=torch.uint8)
            if raw.numel() != num_blocks * block_size * K.FP8_ROW_BYTES:
                raise RuntimeError(f"Raw tensor has {raw.numel()} elements, while the expected size for the fp8 KV cache"
                                   f" is {num_blocks * block_size * K.FP8_ROW_BYTES}.")
            return (raw.view(num_blocks, block_size, K.FP8_ROW_BYTES),)
        raw_tensor = raw_tensor.view(dtype=dtype)
        shapes = [(num_blocks, block_size, 512), (num_blocks, block_size, 64)]
        sizes = [math.prod(shape) for shape in shapes]
        if raw_tensor.numel() != sum(sizes):
            raise RuntimeError(f"Raw tensor has {raw_tensor.numel()} elements, while"
                               f" the expected sizes for KV cache are {sizes}.")
        tensors = torch.split(raw_tensor, sizes)
        return tuple(t.view(shape) for t, shape in zip(tensors, shapes))


@dataclass
class NPUMLAPrefillMetadata(MLACommonPrefillMetadata):
    query_cumlens: list = None
    seq_lens: list = None


@dataclass
class NPUMLADecodeMetadata(MLACommonDecodeMetadata):
    # Unlike the reference (host lists, mla.py:137-138) the lengths stay on the device so that a captured HIP graph
    # reads fresh values on every replay.  Nothing on the GPU path reads host lists; a caller that wants the
    # reference's gets them from seq_lens_list / query_cumlens_list, which are only built when asked for.
    query_cumlens: torch.Tensor = None
    query_start_loc: torch.Tensor = None
    seq_lens_cpu: torch.Tensor = None
    query_start_loc_cpu: torch.Tensor = None
    q_len: int = 1
    max_seq_len: int = 0
    mc2_mask: torch.Tensor = None
    # static sink tokens (reference mla.py:152-153): the sink keys sit in the first pages of every block-table row and
    # ``seq_lens`` counts the keys behind them (the reference passes it next to block_table[:, num_sink_blocks:]).
    seq_sink_len: list = None

    @property
    def seq_lens_list(self) -> list:
        return self.seq_lens_cpu.tolist()

    @property
    def query_cumlens_list(self) -> list:
        return self.query_start_loc_cpu[1:].tolist()


@dataclass
class NPUMLAMetadata(MLACommonMetadata[NPUMLADecodeMetadata]):
    pass


def _persistent_int32(owner, name: str, t: torch.Tensor) -> torch.Tensor:
    """``t`` itself when it is int32 already (the runner's persistent buffer: captured graphs read it in place).  A
    runner that keeps its lengths in another integer type (the reference widens them, npu_model_runner.py:81-86) gets
    them copied into ONE int32 buffer owned by the builder, which only ever grows, so that a graph captured over a step
    reads the lengths of every later step from the same address instead of from a fresh tensor per build."""
    if t.dtype == torch.int32:
        return t
    buf = getattr(owner, name, None)
    if buf is None or buf.numel() < t.numel() or buf.device != t.device:
        buf = torch.zeros(max(t.numel(), 2 * (buf.numel() if buf is not None else 0)), dtype=torch.int32,
                          device=t.device)
        setattr(owner, name, buf)
    view = buf[:t.numel()]
    view.copy_(t)
    return view


class NPUMLAMetadataBuilder(MLACommonMetadataBuilder[NPUMLAMetadata]):
    _cudagraph_support: ClassVar[AttentionCGSupport] = AttentionCGSupport.ALWAYS
    supports_uniform_spec_as_decode: ClassVar[bool] = True
    query_len_support: ClassVar[QueryLenSupport] = QueryLenSupport.VARLEN

    def __init__(self, kv_cache_spec, layer_names, vllm_config, device):
        super().__init__(kv_cache_spec, layer_names, vllm_config, device, NPUMLAMetadata)
        self.prefill_metadata_cls = NPUMLAPrefillMetadata
        if self._use_fi_prefill:
            raise ValueError("Flashinfer should not be enabled.")
        if self._use_cudnn_prefill:
            raise ValueError("CUDNN should not be enabled.")
        if self.dcp_local_block_size != 1:
            raise ValueError("DCP only support cp_kv_cache_interleave_size == 1.")
        if self.dcp_world_size > 1:
            raise ValueError("Decode context parallelism is not part of the single-GPU build.")
        if self.aot_schedule:
            raise ValueError("AOT schedule should be enabled.")
        if self.compilation_config is not None:
            cap = getattr(self.compilation_config, "max_cudagraph_capture_size", None) or 0
            self.reorder_batch_threshold = max(cap, self.reorder_batch_threshold)

    def _build_decode(self, block_table_tensor, seq_lens_cpu, seq_lens_device, query_start_loc_cpu,
                      query_start_loc_device, num_decode_tokens, dcp_tot_seq_lens_device) -> NPUMLADecodeMetadata:
        num_decodes = seq_lens_cpu.numel()
        qlens = (query_start_loc_cpu[1:] - query_start_loc_cpu[:-1])
        max_q = int(qlens.max()) if num_decodes else 1
        uniform = num_decodes > 0 and int(qlens.min()) == max_q
        return NPUMLADecodeMetadata(
            block_table=block_table_tensor,
            seq_lens=_persistent_int32(self, "_seq_lens_i32", seq_lens_device),
            dcp_tot_seq_lens=dcp_tot_seq_lens_device,
            query_cumlens=query_start_loc_device[1:],
            query_start_loc=None if uniform else query_start_loc_device.to(torch.int32).contiguous(),
            seq_lens_cpu=seq_lens_cpu,
            query_start_loc_cpu=query_start_loc_cpu,
            q_len=max_q,
            max_seq_len=int(seq_lens_cpu.max()) if num_decodes else 0,
        )

    def build(self, common_prefix_len: int, common_attn_metadata, fast_build: bool = False) -> NPUMLAMetadata:
        metadata = super().build(common_prefix_len, common_attn_metadata, fast_build)
        sink_len = getattr(self.kv_cache_spec, "sink_len", 0) or 0
        if metadata.decode is not None and sink_len > 0:
            metadata.decode.seq_sink_len = [sink_len] * metadata.num_decodes
        if metadata.prefill is not None:
            metadata.prefill.query_start_loc_list = metadata.prefill.query_start_loc.tolist()
            metadata.prefill.query_cumlens = common_attn_metadata.query_start_loc_cpu[1:].tolist()
            metadata.prefill.seq_lens = metadata.prefill.query_cumlens
        return metadata


def _caller_wrote_cache(impl, attn_metadata, num_tokens: int) -> bool:
    """Consumes ``impl.cache_written_for``: True when the caller's fused norm + rope launch has written the cache rows
    of this very metadata object and at least ``num_tokens`` of them (the mark is ``(metadata, rows written)``)."""
    mark, impl.cache_written_for = impl.cache_written_for, None
    if mark is None:
        return False
    meta, rows = mark
    return meta is attn_metadata and rows >= num_tokens


class NPUMLAImpl(MLACommonBaseImpl[NPUMLAMetadata]):
    can_return_lse_for_decode: bool = True
    # Set by a caller whose fused norm + rope launch has already written the step's rows into the cache: the metadata
    # object of that step.  forward() then skips its own write once and clears the mark.
    cache_written_for = None

    def __init__(self, num_heads: int, head_size: int, scale: float, num_kv_heads: int,
                 alibi_slopes: Optional[list], sliding_window: Optional[int], kv_cache_dtype: str,
                 logits_soft_cap: Optional[float], attn_type: str, kv_sharing_target_layer_name: Optional[str],
                 **mla_args) -> None:
        super().__init__(num_heads, head_size, scale, num_kv_heads, alibi_slopes, sliding_window, kv_cache_dtype,
                         logits_soft_cap, attn_type, kv_sharing_target_layer_name, **mla_args)
        cfg = get_current_vllm_config()
        self.chunked_prefill_workspace_size = (
            MLACommonMetadataBuilder.determine_chunked_prefill_workspace_size(cfg) if cfg is not None else 0)
        self.sliding_window = sliding_window
        unsupported_features = [alibi_slopes, logits_soft_cap]
        if any(unsupported_features):
            raise NotImplementedError(
                "NPUMLAImpl does not support one of the following: "
                "alibi_slopes, logits_soft_cap")
        if sliding_window is not None and sliding_window < 1:
            raise ValueError(f"NPUMLAImpl: sliding_window must be positive (got {sliding_window})")
        # static sink tokens (reference mla.py:278-281); the window only acts together with them, as in the reference
        self.sink_k_pe = None
        self.sink_compressed_kv = None
        self.sink_len = 0
        if attn_type != AttentionType.DECODER:
            raise NotImplementedError(
                "Encoder self-attention and "
                "encoder/decoder cross-attention "
                "are not implemented for "
                "NPUMLAImpl")
        self.fp8_cache = kv_cache_dtype in FP8_CACHE_DTYPES

    def update_sink_kv(self, sink_k_pe: torch.Tensor, sink_compressed_kv: torch.Tensor) -> None:
        """The latents of the static sink tokens, [S,64] and [S,512] (reference mla.py:304-307)."""
        self.sink_k_pe = sink_k_pe.unsqueeze(1)
        self.sink_compressed_kv = sink_compressed_kv
        self.sink_len = sink_compressed_kv.shape[0]

    # ---- GEMMs around the kernels (library GEMMs, as in the reference) ----
    def _v_up_proj(self, x: torch.Tensor) -> torch.Tensor:
        """[N*T, 512] N-major (or [N,T,512]) -> [T, N*V]  (reference mla.py:309-315)."""
        x = x.view(self.num_heads, -1, self.kv_lora_rank)
        out2 = torch.bmm(x, self.W_UV)
        return out2.transpose(0, 1).contiguous().view(-1, self.num_heads * self.v_head_dim)

    # The prefill kernel multiplies the probabilities with fp16 values (the bf16 bar of the output leaves no room for bf16
    # probabilities), so it converts every value tile it is given in bf16.  Where the up-projection is a plain weight the
    # keys and values are made in fp16 in the first place - the same GEMM on fp16 copies of its operands, no extra pass -
    # and the kernel converts nothing (configs of 4 x 2048 over 16k: 13.2 -> 12.2 ms).  fp16 holds every bf16 number of
    # magnitude 2^-14 .. 65504 exactly; set prefill_kv_fp16 = False for a model whose keys or values can exceed that range.
    prefill_kv_fp16 = True

    def _kv_up(self, kv_c: torch.Tensor, allow_fp16: bool = False):
        """(k_nope [T,N,128], v [T,N,128]) of latent rows kv_c [T,512] (reference: ``self.kv_b_proj(kv_c_normed)[0]``,
        mla.py:405-413, 566-571).  With ``allow_fp16`` both may come back as fp16."""
        n, d = self.num_heads, self.qk_nope_head_dim + self.v_head_dim
        w = getattr(self.kv_b_proj, "weight", None)
        if (allow_fp16 and self.prefill_kv_fp16 and isinstance(w, torch.Tensor) and w.dtype in (torch.bfloat16, torch.float16)
                and tuple(w.shape) == (n * d, kv_c.shape[-1]) and getattr(self.kv_b_proj, "bias", None) is None
                and kv_c.dtype in (torch.bfloat16, torch.float16)):
            kv = torch.matmul(kv_c.to(torch.float16), w.to(torch.float16).t())
        else:
            kv = self.kv_b_proj(kv_c)
            kv = kv[0] if isinstance(kv, tuple) else kv
        kv = kv.view(-1, n, d)
        return kv[..., :self.qk_nope_head_dim], kv[..., self.qk_nope_head_dim:]

    # ---- prefill ----
    def _compute_prefill_context(self, q_nope, q_pe, kv_c_cache, k_pe_cache, attn_metadata, k_scale):
        """Chunked context: gather -> up-project -> unmasked attention with LSE (reference mla.py:377-450).  The reference
        merges every chunk's result into a running one (merge_attn_states); here a chunk's launch continues from the
        running result, so the merge is part of the attention kernel and there is no merge launch."""
        prefill = attn_metadata.prefill
        cc = prefill.chunked_context
        assert cc is not None
        t, n = q_nope.shape[0], self.num_heads
        cu_q = prefill.query_start_loc.to(torch.int32).contiguous()
        output = output_lse = None
        for i in range(len(cc.seq_tot)):
            toks = int(cc.seq_tot[i])
            if toks == 0:
                continue
            ops.gather_and_maybe_dequant_cache(src_cache=(kv_c_cache,) if k_pe_cache is None else (kv_c_cache, k_pe_cache),
                                               dst=cc.workspace,
                                               block_table=prefill.block_table, cu_seq_lens=cc.cu_seq_lens[i],
                                               batch_size=attn_metadata.num_prefills, kv_cache_dtype=self.kv_cache_dtype,
                                               scale=k_scale, seq_starts=cc.starts[i], total_rows=toks)
            kv_c_normed = cc.workspace[:toks][..., :self.kv_lora_rank]
            k_pe = cc.workspace[:toks][..., self.kv_lora_rank:]
            k_nope, v = self._kv_up(kv_c_normed, allow_fp16=True)
            k_pe = k_pe.to(k_nope.dtype)
            # running results stay fp32: each bf16 rounding in between would add 2^-10 of mean relative error to the
            # layer's output
            first = output is None
            if first:
                output = torch.empty(t, n, self.v_head_dim, dtype=torch.float32, device=q_nope.device)
                output_lse = torch.empty(t, n, dtype=torch.float32, device=q_nope.device)
            K.prefill_varlen(q_nope, q_pe, k_nope, k_pe, v, cu_q, cc.cu_seq_lens[i].to(torch.int32).contiguous(),
                             prefill.max_query_len, self.scale, False, output, output_lse,
                             prev_out=None if first else output, prev_lse=None if first else output_lse)
        return output, output_lse

    def _forward_prefill(self, q, kv_c_normed, k_pe, kv_cache, attn_metadata, k_scale) -> torch.Tensor:
        """Causal suffix attention merged with the chunked context (reference mla.py:452-483, 573-616): the context chunks
        first, then the suffix launch continues from their result (the reference's final merge_attn_states, inside the
        kernel)."""
        prefill = attn_metadata.prefill
        assert prefill is not None
        if self.sink_len > 0:
            return self._forward_prefill_sink(q, kv_c_normed, k_pe, prefill)
        t, n = q.shape[0], self.num_heads
        has_context = prefill.chunked_context is not None
        q_nope, q_pe = q[..., :self.qk_nope_head_dim], q[..., self.qk_nope_head_dim:]
        k_nope, v = self._kv_up(kv_c_normed, allow_fp16=True)
        cu_q = prefill.query_start_loc.to(torch.int32).contiguous()
        ctx_out = ctx_lse = None
        if has_context:
            # (the fp8 cache is one tensor whose rows hold latent, scales and rope; the gather dequantises it)
            ctx_out, ctx_lse = self._compute_prefill_context(q_nope, q_pe, kv_cache[0],
                                                             None if self.fp8_cache else kv_cache[1], attn_metadata, k_scale)
        output = torch.empty(t, n, self.v_head_dim, dtype=torch.bfloat16, device=q.device)
        K.prefill_varlen(q_nope, q_pe, k_nope, k_pe.reshape(t, -1).to(k_nope.dtype), v, cu_q, cu_q, prefill.max_query_len,
                         self.scale, True, output, prev_out=ctx_out, prev_lse=ctx_lse)
        return output.flatten(start_dim=-2)

    def _forward_prefill_sink(self, q, kv_c_normed, k_pe, prefill) -> torch.Tensor:
        """Prefill with static sink tokens (reference mla.py:463-560): the cached context is not read (mla.py:497).
        Without a window the sink latents go in front of every sequence's new latents and one right-down causal attention
        runs over sink_len + s_b keys.  With a window the reference runs a sink attention and a banded attention and merges
        them by LSE; that is the same softmax over sink keys + band: here the banded launch continues from the sink result."""
        t, n, s_len = q.shape[0], self.num_heads, self.sink_len
        q_nope, q_pe = q[..., :self.qk_nope_head_dim], q[..., self.qk_nope_head_dim:]
        starts = prefill.query_start_loc_list
        nb = len(starts) - 1
        cu_q = prefill.query_start_loc.to(torch.int32).contiguous()
        sink_pe = self.sink_k_pe.reshape(s_len, -1)
        output = torch.empty(t, n, self.v_head_dim, dtype=q.dtype, device=q.device)
        if self.sliding_window is None:
            lat = self._insert_tensor_by_start_loc(kv_c_normed, self.sink_compressed_kv, starts)
            pe = self._insert_tensor_by_start_loc(k_pe.reshape(t, -1), sink_pe, starts)
            k_nope, v = self._kv_up(lat)
            cu_k = cu_q + s_len * torch.arange(nb + 1, dtype=torch.int32, device=q.device)
            K.prefill_varlen(q_nope, q_pe, k_nope, pe, v, cu_q, cu_k, prefill.max_query_len, self.scale, True, output)
            return output.flatten(start_dim=-2)
        ks_nope, vs = self._kv_up(self.sink_compressed_kv)
        cu_s = s_len * torch.arange(nb + 1, dtype=torch.int32, device=q.device)
        out_sink = torch.empty(t, n, self.v_head_dim, dtype=torch.float32, device=q.device)     # the running result stays fp32
        lse_sink = torch.empty(t, n, dtype=torch.float32, device=q.device)
        K.prefill_varlen(q_nope, q_pe, ks_nope.repeat(nb, 1, 1), sink_pe.repeat(nb, 1), vs.repeat(nb, 1, 1), cu_q, cu_s,
                         prefill.max_query_len, self.scale, False, out_sink, lse_sink)
        k_nope, v = self._kv_up(kv_c_normed)
        # the banded launch continues from the sink result: the reference's merge of the two, inside the kernel
        K.prefill_varlen(q_nope, q_pe, k_nope, k_pe.reshape(t, -1), v, cu_q, cu_q, prefill.max_query_len, self.scale, True,
                         output, window=self.sliding_window, prev_out=out_sink, prev_lse=lse_sink)
        return output.flatten(start_dim=-2)

    @staticmethod
    def _insert_tensor_by_start_loc(raw_tensor: torch.Tensor, insert_segment: torch.Tensor, start_loc: list) -> torch.Tensor:
        """insert_segment in front of every raw_tensor[start_loc[i]:start_loc[i+1]] (reference mla.py:929-949)."""
        pieces = []
        for i in range(len(start_loc) - 1):
            pieces.append(insert_segment)
            pieces.append(raw_tensor[start_loc[i]:start_loc[i + 1]])
        return torch.cat(pieces, 0)

    # ---- decode ----
    def _fusable_w_uv(self, out: torch.Tensor) -> bool:
        """The fused merge + up-projection kernel takes bf16 W_UV [N,512,128] with contiguous rows and writes rows of 128."""
        w = self.W_UV
        return (w.dtype == torch.bfloat16 and w.dim() == 3 and w.shape[1:] == (512, 128) and w.stride(2) == 1
                and w.stride(0) % 8 == 0 and w.stride(1) % 8 == 0 and w.data_ptr() % 16 == 0
                and out.dtype == torch.bfloat16 and out.stride(-1) == 1 and out.stride(0) % 4 == 0 and out.data_ptr() % 8 == 0)

    def _forward_decode(self, decode_ql_nope, decode_q_pe, kv_cache, attn_metadata, layer=None,
                        proj_out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Absorbed paged decode; returns the head-major [N, T, 512] tensor of the reference (mla.py:781-804).  With
        ``proj_out`` ([T, N*V]) the value up-projection (mla.py:309-315) is fused into the merge of the split-KV
        partials: the result goes straight into ``proj_out`` and nothing is returned."""
        d = attn_metadata.decode
        assert d is not None
        t = decode_ql_nope.shape[0]
        if self.sink_len > 0:
            return self._forward_decode_sink(decode_ql_nope, decode_q_pe, kv_cache, d, proj_out)
        kw = dict(q_len=d.q_len, query_start_loc=d.query_start_loc, max_seq_len=d.block_table.shape[1] * K.PAGE)
        if proj_out is not None:
            if self.fp8_cache:
                K.decode_fp8(decode_ql_nope, decode_q_pe, kv_cache[0], d.block_table, d.seq_lens, self.scale, proj_out,
                             w_uv=self.W_UV, **kw)
            else:
                K.decode(decode_ql_nope, decode_q_pe, kv_cache[0], kv_cache[1], d.block_table, d.seq_lens, self.scale,
                         proj_out, w_uv=self.W_UV, **kw)
            return None
        o = torch.empty(self.num_heads, t, self.kv_lora_rank, dtype=decode_ql_nope.dtype, device=decode_ql_nope.device)
        if self.fp8_cache:
            K.decode_fp8(decode_ql_nope, decode_q_pe, kv_cache[0], d.block_table, d.seq_lens, self.scale,
                         o.transpose(0, 1), **kw)
        else:
            K.decode(decode_ql_nope, decode_q_pe, kv_cache[0], kv_cache[1], d.block_table, d.seq_lens, self.scale,
                     o.transpose(0, 1), **kw)
        return o

    def _forward_decode_sink(self, ql_nope, q_pe, kv_cache, d, proj_out: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """Decode with static sink tokens (reference mla.py:705-779).  The reference attends to the sink pages and to the
        sequence's own pages separately and merges the two by LSE; the result is one softmax over the union of the keys,
        and that is what runs here: the sink pages are the first pages of every block-table row, so without a window it is
        the plain decode over sink_len + seq_len keys, and with a window the dense kernel walks each sequence with the
        blocks between the sink and the window left out (kernels.decode(..., sink_len=, window=))."""
        if self.sink_len % K.PAGE != 0:
            raise ValueError(f"sink_len {self.sink_len} must align with block size")
        t, dev = ql_nope.shape[0], ql_nope.device
        o = None
        if proj_out is None:
            o = torch.empty(self.num_heads, t, self.kv_lora_rank, dtype=ql_nope.dtype, device=dev)
        out = proj_out if proj_out is not None else o.transpose(0, 1)
        w_uv = self.W_UV if proj_out is not None else None
        if self.sliding_window is None:
            kw = dict(q_len=d.q_len, query_start_loc=d.query_start_loc, max_seq_len=d.block_table.shape[1] * K.PAGE, w_uv=w_uv)
            if self.fp8_cache:
                K.decode_fp8(ql_nope, q_pe, kv_cache[0], d.block_table, d.seq_lens + self.sink_len, self.scale, out, **kw)
            else:
                K.decode(ql_nope, q_pe, kv_cache[0], kv_cache[1], d.block_table, d.seq_lens + self.sink_len, self.scale, out,
                         **kw)
            return o
        kw = dict(q_len=d.q_len, query_start_loc=d.query_start_loc, w_uv=w_uv, sink_len=self.sink_len, window=self.sliding_window)
        if self.fp8_cache:
            K.decode_fp8(ql_nope, q_pe, kv_cache[0], d.block_table, d.seq_lens, self.scale, out, **kw)
        else:
            K.decode(ql_nope, q_pe, kv_cache[0], kv_cache[1], d.block_table, d.seq_lens, self.scale, out, **kw)
        return o

    def forward(self, layer, q: torch.Tensor, k_c_normed: torch.Tensor, k_pe: torch.Tensor,
                kv_cache: Tuple[torch.Tensor, ...], attn_metadata: NPUMLAMetadata,
                output: Optional[torch.Tensor] = None, output_scale: Optional[torch.Tensor] = None,
                output_block_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
        assert output is not None, "Output tensor must be provided."
        if output_scale is not None or output_block_scale is not None:
            raise NotImplementedError("fused output quantization is not yet supported for NPUMLAImpl")

        if attn_metadata is None:
            # profile run: reserve the worst-case up-projection scratch, zero the output (reference mla.py:825-842)
            _ = torch.empty((self.chunked_prefill_workspace_size, self.num_heads,
                             self.qk_nope_head_dim + self.v_head_dim), device=k_c_normed.device, dtype=k_c_normed.dtype)
            return output.fill_(0)

        num_actual_toks = attn_metadata.num_actual_tokens
        assert isinstance(kv_cache, (list, tuple)), f"{type(kv_cache)=}."
        want = 1 if self.fp8_cache else 2
        assert len(kv_cache) == want, f"{len(kv_cache)=}."
        assert all(isinstance(c, torch.Tensor) and c.numel() > 0 for c in kv_cache), \
            f"{[getattr(c, 'shape', None) for c in kv_cache]}"

        output_padded = output
        assert (attn_metadata.num_decodes is not None and attn_metadata.num_prefills is not None
                and attn_metadata.num_decode_tokens is not None)
        has_decode = attn_metadata.num_decodes > 0
        has_prefill = attn_metadata.num_prefills > 0
        num_decode_tokens = attn_metadata.num_decode_tokens
        decode_q = q[:num_decode_tokens]

        # write the latent and rope rows of the new tokens (one launch), unless the caller's fused norm + rope launch has
        # put them there already and said so for this very metadata object
        written = _caller_wrote_cache(self, attn_metadata, num_actual_toks)
        if written:
            pass
        elif self.fp8_cache:
            K.cache_write_fp8(k_c_normed, k_pe, attn_metadata.slot_mapping, kv_cache[0])
        else:
            K.cache_write(k_c_normed, k_pe, attn_metadata.slot_mapping, kv_cache[0], kv_cache[1])

        if has_prefill:
            output = output[:num_actual_toks, ...]
            q = q[:num_actual_toks, ...]
            k_c_normed = k_c_normed[:num_actual_toks, ...]
            k_pe = k_pe[:num_actual_toks, ...]
            output[num_decode_tokens:] = self._forward_prefill(
                q[num_decode_tokens:], k_c_normed[num_decode_tokens:], k_pe[num_decode_tokens:], kv_cache, attn_metadata,
                getattr(layer, "_k_scale", None))

        if has_decode:
            assert attn_metadata.decode is not None
            decode_q_nope, decode_q_pe = decode_q.split([self.qk_nope_head_dim, self.qk_rope_head_dim], dim=-1)
            # (B, N, P) -> (N, B, P) x (N, P, L) -> (N, B, L) -> (B, N, L) view
            decode_ql_nope = torch.bmm(decode_q_nope.transpose(0, 1), self.W_UK_T).transpose(0, 1)
            ndt = decode_ql_nope.shape[0]
            if self._fusable_w_uv(output[:ndt]):
                self._forward_decode(decode_ql_nope, decode_q_pe, kv_cache, attn_metadata, layer, proj_out=output[:ndt])
            else:
                attn_out = self._forward_decode(decode_ql_nope, decode_q_pe, kv_cache, attn_metadata, layer)
                out_proj = self._v_up_proj(attn_out)
                output[:out_proj.shape[0]].copy_(out_proj)
        return output_padded
