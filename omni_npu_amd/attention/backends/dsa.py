"""DSA (sparse MLA) attention backend for MI355X behind the reference's vLLM plugin contract.

Mirrors src/omni_npu/attention/backends/dsa.py.  Vendor ops replaced:
  npu_scatter_nd_update_ x2 (dsa.py:359-362)          -> kernels.cache_write
  npu_lightning_indexer (patch_dsv32_indexer.py:133-146,
                         v1/layers/attention/npu_dsa.py:92-103)  -> LightningIndexer: quant + fp8 score MFMA + exact top-k
  npu_sparse_flash_attention (dsa.py:259-291)         -> kernels.build_sparse_rows + kernels.sparse_decode
The third cache tensor holds the indexer keys.  The reference keeps them in bf16; here the same bytes hold float8_e4m3fn
keys and one fp32 scale per key, per page: [page*128 B keys | page*4 B scales | unused], see indexer_cache_views().
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import ClassVar, Optional, Tuple

import torch

from ... import kernels as K
from .mla import _caller_wrote_cache, _persistent_int32
from ..._vllm_compat import (PAD_SLOT_ID, AttentionCGSupport, AttentionType, MLACommonBackend, MLACommonBaseImpl,
                             MLACommonDecodeMetadata, MLACommonMetadata, MLACommonMetadataBuilder,
                             MLACommonPrefillMetadata, QueryLenSupport, get_current_vllm_config)

INDEX_HEAD_DIM = 128


def indexer_cache_views(index_cache: torch.Tensor):
    """(k8 [nblk, page, 128] float8 view, k_scale [nblk, page] fp32 view) of the third cache tensor
    ([nblk, page, 1, 128] in a 2-byte dtype, reference dsa.py:67)."""
    nblk, page = index_cache.shape[0], index_cache.shape[1]
    raw = index_cache.reshape(nblk, -1).view(torch.uint8)                    # [nblk, page*256]
    k8 = raw[:, : page * INDEX_HEAD_DIM].view(nblk, page, INDEX_HEAD_DIM)
    ks = raw[:, page * INDEX_HEAD_DIM: page * (INDEX_HEAD_DIM + 4)].view(torch.float32)
    return k8, ks


class NPUDSABackend(MLACommonBackend):
    @staticmethod
    def get_name() -> str:
        return "NPUDSA"

    @staticmethod
    def get_metadata_cls() -> type["NPUDSAMetadata"]:
        return NPUDSAMetadata

    @staticmethod
    def get_builder_cls() -> type["NPUDSAMetadataBuilder"]:
        return NPUDSAMetadataBuilder

    @staticmethod
    def get_impl_cls() -> type["NPUDSAImpl"]:
        return NPUDSAImpl

    @staticmethod
    def reshape_kv_cache(raw_tensor: torch.Tensor, num_blocks: int, block_size: int, num_kv_heads: int, head_size: int,
                         dtype: torch.dtype = torch.bfloat16) -> Tuple[torch.Tensor, ...]:
        """Three contiguous tensors out of one raw allocation (reference dsa.py:58-73)."""
        raw_tensor = raw_tensor.view(dtype=dtype)
        shapes = [(num_blocks, block_size, 1, 512), (num_blocks, block_size, 1, 64), (num_blocks, block_size, 1, 128)]
        sizes = [math.prod(shape) for shape in shapes]
        if raw_tensor.numel() != sum(sizes):
            raise RuntimeError(f"Raw tensor has {raw_tensor.numel()} elements, while"
                               f" the expected sizes for KV cache are {sizes}.")
        tensors = torch.split(raw_tensor, sizes)
        return tuple(t.view(shape) for t, shape in zip(tensors, shapes))


@dataclass
class NPUDSAPrefillMetadata(MLACommonPrefillMetadata):
    query_cumlens: torch.Tensor = None
    seq_lens: torch.Tensor = None


@dataclass
class NPUDSADecodeMetadata(MLACommonDecodeMetadata):
    query_cumlens: torch.Tensor = None
    query_start_loc: torch.Tensor = None
    q_len: int = 1
    mc2_mask: torch.Tensor = None


@dataclass
class NPUDSAMetadata(MLACommonMetadata[NPUDSADecodeMetadata]):
    pass


class NPUDSAMetadataBuilder(MLACommonMetadataBuilder[NPUDSAMetadata]):
    _cudagraph_support: ClassVar[AttentionCGSupport] = AttentionCGSupport.UNIFORM_BATCH
    query_len_support: ClassVar[QueryLenSupport] = QueryLenSupport.VARLEN

    def __init__(self, kv_cache_spec, layer_names, vllm_config, device):
        super().__init__(kv_cache_spec, layer_names, vllm_config, device, NPUDSAMetadata)
        self.prefill_metadata_cls = NPUDSAPrefillMetadata
        if self._use_fi_prefill:
            raise ValueError("Flashinfer should not be enabled.")
        if self._use_cudnn_prefill:
            raise ValueError("CUDNN should not be enabled.")
        if self.dcp_world_size > 1:
            raise ValueError("DCP should not be enabled.")
        if self.aot_schedule:
            raise ValueError("AOT schedule should be enabled.")
        spec = getattr(vllm_config, "speculative_config", None)
        self.uniform_decode_query_len = 1 if not spec else 1 + spec.num_speculative_tokens
        if self.compilation_config is not None:
            cap = getattr(self.compilation_config, "max_cudagraph_capture_size", None) or 0
            self.reorder_batch_threshold = max(cap, self.reorder_batch_threshold, self.uniform_decode_query_len)

    def _build_decode(self, block_table_tensor, seq_lens_cpu, seq_lens_device, query_start_loc_cpu,
                      query_start_loc_device, num_decode_tokens, dcp_tot_seq_lens_device) -> NPUDSADecodeMetadata:
        qlens = query_start_loc_cpu[1:] - query_start_loc_cpu[:-1]
        n = qlens.numel()
        max_q = int(qlens.max()) if n else 1
        uniform = n > 0 and int(qlens.min()) == max_q
        return NPUDSADecodeMetadata(block_table=block_table_tensor, seq_lens=_persistent_int32(self, "_seq_lens_i32", seq_lens_device),
                                    dcp_tot_seq_lens=dcp_tot_seq_lens_device, query_cumlens=query_start_loc_device[1:],
                                    query_start_loc=None if uniform else query_start_loc_device.to(torch.int32).contiguous(),
                                    q_len=max_q)

    def build(self, common_prefix_len: int, common_attn_metadata, fast_build: bool = False) -> NPUDSAMetadata:
        metadata = super().build(common_prefix_len, common_attn_metadata, fast_build)
        if metadata.decode is not None and getattr(self.vllm_config, "kv_transfer_config", None) is not None:
            metadata.slot_mapping = self._align_slot_mapping(metadata.slot_mapping, metadata.num_reqs)
        if metadata.prefill is not None:
            qsl = metadata.prefill.query_start_loc
            metadata.prefill.seq_lens = qsl[1:] - qsl[:-1]
            metadata.prefill.query_cumlens = torch.cumsum(qsl[1:] - qsl[:-1], dim=0)
            # sparse attention over the cache needs each prefill request's total cached length
            nd = metadata.num_decodes
            metadata.prefill.kv_lens = common_attn_metadata.seq_lens[nd:].to(torch.int32)
        if metadata.prefill is not None and metadata.prefill.chunked_context is not None:
            raise RuntimeError("Chunked prefill is not enabled yet.")
        return metadata

    def _align_slot_mapping(self, slot_mapping: torch.Tensor, num_reqs) -> torch.Tensor:
        num_tokens_padded = num_reqs * self.uniform_decode_query_len
        if slot_mapping.numel() < num_tokens_padded:
            slot_mapping = torch.nn.functional.pad(slot_mapping, (0, num_tokens_padded - slot_mapping.numel()),
                                                   value=PAD_SLOT_ID)
        return slot_mapping


class LightningIndexer:
    """The selection step of the DeepSeek-V3.2 indexer on the GPU: quantise q, quantise-and-cache the new keys, fp8
    score GEMM, exact top-k into ``topk_indices_buffer`` (the tail of the reference's patched Indexer.forward,
    patch_dsv32_indexer.py:104-146; the projections, LayerNorm and RoPE before it are the caller's)."""

    def __init__(self, topk_tokens: int, n_head: int = 64, head_dim: int = INDEX_HEAD_DIM, max_tokens: int = 1,
                 device=None):
        self.topk_tokens, self.n_head, self.head_dim = topk_tokens, n_head, head_dim
        self.topk_indices_buffer = torch.full((max_tokens, topk_tokens), -1, dtype=torch.int32, device=device)
        # what the sparse attention reads: the picks as flat cache rows and their number per token, written by the same
        # launch that writes the positions (the block ids of the three DSA cache tensors are the same)
        self.rows_buffer = torch.zeros((max_tokens, topk_tokens), dtype=torch.int32, device=device)
        self.counts_buffer = torch.zeros((max_tokens,), dtype=torch.int32, device=device)
        self._rows_meta = None       # the metadata object the row buffers were filled for
        self._logits = None
        self._logits_kept = []       # outgrown score buffers: a captured graph may still hold their address, never freed

    def __call__(self, q: torch.Tensor, k: torch.Tensor, weights: torch.Tensor, kv_cache, attn_metadata):
        if attn_metadata is None:                                   # profile run (patch_dsv32_indexer.py:104-112)
            return self.topk_indices_buffer
        assert len(kv_cache) >= 3, f"Expected kv_cache to have at least 3 elements, but got {len(kv_cache)}"
        k8, ks = indexer_cache_views(kv_cache[2])
        t = q.shape[0]
        q8 = torch.empty(t, self.n_head, self.head_dim, dtype=torch.uint8, device=q.device)
        qs = torch.empty(t, self.n_head, dtype=torch.float32, device=q.device)
        # the new keys into the cache and the queries into plain buffers: one launch
        K.quant_qk_fp8(q.reshape(t * self.n_head, self.head_dim), q8, qs, k.reshape(-1, self.head_dim), k8, ks,
                       attn_metadata.slot_mapping)
        w = weights.float().contiguous()
        out = self.topk_indices_buffer[:t]
        off = 0
        for meta, nreq in ((attn_metadata.decode, attn_metadata.num_decodes), (attn_metadata.prefill, attn_metadata.num_prefills)):
            if meta is None or nreq == 0:
                continue
            if meta is attn_metadata.decode:
                ntok, lens, q_len, qsl = attn_metadata.num_decode_tokens, meta.seq_lens, meta.q_len, meta.query_start_loc
            else:
                ntok = t - off
                lens, q_len = meta.kv_lens, meta.max_query_len
                qsl = meta.query_start_loc.to(torch.int32).contiguous()
            max_len = meta.block_table.shape[1] * k8.shape[1]
            stride = K.indexer_logits_stride(max_len)
            if self._logits is None or self._logits.shape[0] < ntok or self._logits.shape[1] < stride:
                if self._logits is not None:
                    self._logits_kept.append(self._logits)
                    ntok_a, stride_a = max(ntok, self._logits.shape[0]), max(stride, self._logits.shape[1])
                else:
                    ntok_a, stride_a = max(ntok, 1), stride
                self._logits = torch.empty(ntok_a, stride_a, dtype=torch.float32, device=q.device)
            lg = self._logits[:ntok, :stride]
            sl = slice(off, off + ntok)
            K.indexer_scores(q8[sl], w[sl], k8, ks, meta.block_table, lens, lg, q_len=q_len, q_scale=qs[sl],
                             query_start_loc=qsl, max_seq_len=max_len)
            K.topk(lg, lens, self.topk_tokens, out[sl], q_len=q_len, query_start_loc=qsl, block_table=meta.block_table,
                   page_size=k8.shape[1], num_pages=k8.shape[0], rows=self.rows_buffer[sl], counts=self.counts_buffer[sl])
            off += ntok
        self._rows_meta = attn_metadata
        return out.view(t, 1, self.topk_tokens)

    def rows_for(self, attn_metadata):
        """(cache rows [max_tokens, k], counts [max_tokens]) of the picks if the last selection ran for this very metadata
        object, else None (the caller then translates ``topk_indices_buffer`` itself)."""
        if attn_metadata is not None and self._rows_meta is attn_metadata:
            return self.rows_buffer, self.counts_buffer
        return None


class NPUDSAImpl(MLACommonBaseImpl[NPUDSAMetadata]):
    can_return_lse_for_decode: bool = False
    cache_written_for = None     # see NPUMLAImpl.cache_written_for

    def __init__(self, num_heads: int, head_size: int, scale: float, num_kv_heads: int, alibi_slopes: Optional[list],
                 sliding_window: Optional[int], kv_cache_dtype: str, logits_soft_cap: Optional[float], attn_type: str,
                 kv_sharing_target_layer_name: Optional[str], **mla_args) -> None:
        super().__init__(num_heads, head_size, scale, num_kv_heads, alibi_slopes, sliding_window, kv_cache_dtype,
                         logits_soft_cap, attn_type, kv_sharing_target_layer_name, **mla_args)
        cfg = get_current_vllm_config()
        self.chunked_prefill_workspace_size = (
            MLACommonMetadataBuilder.determine_chunked_prefill_workspace_size(cfg) if cfg is not None else 0)
        unsupported_features = [alibi_slopes, sliding_window, logits_soft_cap]
        if any(unsupported_features):
            raise NotImplementedError(
                "NPUDSAImpl does not support one of the following: "
                "alibi_slopes, sliding_window, logits_soft_cap")
        if attn_type != AttentionType.DECODER:
            raise NotImplementedError(
                "Encoder self-attention and "
                "encoder/decoder cross-attention "
                "are not implemented for "
                "NPUDSAImpl")
        if kv_cache_dtype in ("fp8", "fp8_e4m3"):
            raise NotImplementedError("NPUDSAImpl writes the bf16 cache layout (latent, rope, indexer keys) only: "
                                      "an fp8 KV cache is not supported for DSA models")

    def _v_up_proj(self, x: torch.Tensor, out: torch.Tensor):
        """[T,N,512] token-major -> out [T, N*V]  (reference dsa.py:233-240)."""
        x = x.transpose(0, 1)
        out2 = torch.bmm(x, self.W_UV)
        out.copy_(out2.transpose(0, 1).reshape(-1, self.num_heads * self.v_head_dim))

    def _absorb_prolog(self, q: torch.Tensor):
        q_nope, q_pe = q.split([self.qk_nope_head_dim, self.qk_rope_head_dim], dim=-1)
        ql_nope = torch.bmm(q_nope.transpose(0, 1), self.W_UK_T).transpose(0, 1)
        return ql_nope, q_pe

    def _fusable_w_uv(self, out: torch.Tensor) -> bool:
        """The fused merge + up-projection kernel takes bf16 W_UV [N,512,128] with contiguous rows and writes rows of 128."""
        w = self.W_UV
        return (w.dtype == torch.bfloat16 and w.dim() == 3 and w.shape[1:] == (512, 128) and w.stride(2) == 1
                and w.stride(0) % 8 == 0 and w.stride(1) % 8 == 0 and w.data_ptr() % 16 == 0
                and out.dtype == torch.bfloat16 and out.stride(-1) == 1 and out.stride(0) % 4 == 0 and out.data_ptr() % 8 == 0)

    def _apply_sparse_attention(self, q_nope, q_pe, kv_cache, meta, lens, q_len, qsl, topk_indices,
                                proj_out: Optional[torch.Tensor] = None, rows_counts=None) -> Optional[torch.Tensor]:
        """Absorbed MLA over the indexer's positions (reference dsa.py:259-291); token-major [T,N,512].  With
        ``proj_out`` ([T, N*V]) the value up-projection (dsa.py:233-240) is fused into the merge of the partials and
        nothing is returned.  ``rows_counts``: the picks of these tokens already translated into cache rows, with their
        counts (LightningIndexer.rows_for); without it the positions are translated here."""
        bs = q_nope.shape[0]
        k = topk_indices.shape[-1]
        nope, rope = kv_cache[0], kv_cache[1]
        if rows_counts is not None:
            rows, counts = rows_counts
        else:
            rows = torch.empty(bs, k, dtype=torch.int32, device=q_nope.device)
            counts = torch.empty(bs, dtype=torch.int32, device=q_nope.device)
            K.build_sparse_rows(topk_indices.reshape(bs, k), meta.block_table, lens, nope.shape[1], nope.shape[0], rows,
                                counts, q_len=q_len, query_start_loc=qsl)
        if proj_out is not None:
            K.sparse_decode(q_nope, q_pe, nope, rope, rows, counts, self.scale, proj_out, w_uv=self.W_UV, counts_bounded=True)
            return None
        out = torch.empty(bs, self.num_heads, self.kv_lora_rank, dtype=q_nope.dtype, device=q_nope.device)
        K.sparse_decode(q_nope, q_pe, nope, rope, rows, counts, self.scale, out, counts_bounded=True)
        return out

    def forward(self, layer, q: torch.Tensor, k_c_normed: torch.Tensor, k_pe: torch.Tensor,
                kv_cache: Tuple[torch.Tensor, torch.Tensor, torch.Tensor], attn_metadata: NPUDSAMetadata,
                output: Optional[torch.Tensor] = None, output_scale: Optional[torch.Tensor] = None,
                output_block_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
        assert output is not None, "Output tensor must be provided."
        if output_scale is not None or output_block_scale is not None:
            raise NotImplementedError("fused output quantization is not yet supported for NPUDSAImpl")
        if attn_metadata is None:
            _ = torch.empty((self.chunked_prefill_workspace_size, self.num_heads,
                             self.qk_nope_head_dim + self.v_head_dim), device=k_c_normed.device, dtype=k_c_normed.dtype)
            # the profile run sizes the KV cache: the split-KV scratch a real prefill will need (bounded by
            # SPARSE_WORKSPACE_CAP whatever the chunk size) is allocated now, so that it is counted
            # (for the split count the real steps will pick; scratch is kept per stream, so a runner that captures its graphs
            # on another stream pays this once more there: at most SPARSE_WORKSPACE_CAP per stream that runs steps)
            if k_c_normed.is_cuda:
                toks = max(int(k_c_normed.shape[0]), 1)
                k_sel = int(self.indexer.topk_indices_buffer.shape[-1]) if self.indexer is not None else 2048
                splits = K.default_num_splits(toks, 1, self.num_heads, k_sel)
                need = K._lib.load().mla_decode_workspace_bytes(min(toks, 32768), 1, self.num_heads, splits)
                K._workspace(k_c_normed.device, min(need, K.SPARSE_WORKSPACE_CAP))
            return output.fill_(0)

        num_actual_toks = attn_metadata.num_actual_tokens
        assert isinstance(kv_cache, (list, tuple)), f"{type(kv_cache)=}."
        assert len(kv_cache) == 3, f"{len(kv_cache)=}."
        k_nope, k_rope, _ = kv_cache
        assert isinstance(k_nope, torch.Tensor) and isinstance(k_rope, torch.Tensor), f"{type(k_nope)=}, {type(k_rope)=}."
        assert k_nope.numel() > 0 and k_rope.numel() > 0, f"{k_nope.shape=}, {k_rope.shape=}"

        output_padded = output
        output = output[:num_actual_toks, ...]
        q = q[:num_actual_toks, ...]
        assert (attn_metadata.num_decodes is not None and attn_metadata.num_prefills is not None
                and attn_metadata.num_decode_tokens is not None)
        has_decode = attn_metadata.num_decodes > 0
        has_prefill = attn_metadata.num_prefills > 0
        ndt = attn_metadata.num_decode_tokens
        written = _caller_wrote_cache(self, attn_metadata, num_actual_toks)
        if not written:                                            # (else the caller's fused norm + rope launch wrote them)
            K.cache_write(k_c_normed, k_pe, attn_metadata.slot_mapping, k_nope, k_rope)
        topk = self.indexer.topk_indices_buffer
        rows_for = getattr(self.indexer, "rows_for", None)
        rc = rows_for(attn_metadata) if rows_for is not None else None
        part = lambda a, b: None if rc is None else (rc[0][a:b], rc[1][a:b])

        if has_prefill:
            p = attn_metadata.prefill
            assert p is not None
            q_nope, q_pe = self._absorb_prolog(q[ndt:])
            fused = output[ndt:] if self._fusable_w_uv(output[ndt:]) else None
            attn_out = self._apply_sparse_attention(q_nope, q_pe, kv_cache, p, p.kv_lens, p.max_query_len,
                                                    p.query_start_loc.to(torch.int32).contiguous(),
                                                    topk[ndt:num_actual_toks], proj_out=fused,
                                                    rows_counts=part(ndt, num_actual_toks))
            if fused is None:
                self._v_up_proj(attn_out, out=output[ndt:])
        if has_decode:
            d = attn_metadata.decode
            assert d is not None
            q_nope, q_pe = self._absorb_prolog(q[:ndt])
            fused = output[:ndt] if self._fusable_w_uv(output[:ndt]) else None
            attn_out = self._apply_sparse_attention(q_nope, q_pe, kv_cache, d, d.seq_lens, d.q_len, d.query_start_loc,
                                                    topk[:ndt], proj_out=fused, rows_counts=part(0, ndt))
            if fused is None:
                self._v_up_proj(attn_out, out=output[:ndt])
        return output_padded
