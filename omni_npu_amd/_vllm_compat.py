"""The vLLM 0.12 side of the plugin contract.

When vLLM is importable its own classes are used.  When it is not (CPU test boxes, kernel benchmarks) this module
provides small stand-ins with the same names, fields and call signatures that the backend consumes, so the
backend, builder, impl and graph wrapper can be exercised without vLLM.  The stand-ins restate only what the
reference relies on:
  * CommonAttentionMetadata fields as constructed in the reference's
    tests/integration/attention/test_mla_chunked_prefill.py:450-462;
  * decode requests come first in the batch; a request is a decode iff its query length is at most the
    builder's reorder_batch_threshold (src/omni_npu/attention/backends/mla.py:96, 119-120, 862-866);
  * the chunked-context schedule fields seq_tot / workspace / cu_seq_lens / starts
    (src/omni_npu/attention/backends/mla.py:391-405).
"""
from __future__ import annotations

import enum
from dataclasses import dataclass, field
from typing import Any, Generic, Optional, TypeVar

import torch

try:  # pragma: no cover - exercised only where vLLM is installed
    from vllm.attention.backends.abstract import AttentionType  # noqa: F401
    from vllm.config import CUDAGraphMode  # noqa: F401
    from vllm.forward_context import BatchDescriptor, get_forward_context  # noqa: F401
    from vllm.platforms.interface import Platform, PlatformEnum  # noqa: F401
    from vllm.v1.attention.backends.mla.common import (MLACommonBackend, MLACommonBaseImpl,  # noqa: F401
                                                      MLACommonDecodeMetadata, MLACommonMetadata,
                                                      MLACommonMetadataBuilder, MLACommonPrefillMetadata,
                                                      QueryLenSupport)
    from vllm.v1.attention.backends.utils import AttentionCGSupport, CommonAttentionMetadata  # noqa: F401
    from vllm.v1.kv_cache_interface import AttentionSpec, MLAAttentionSpec  # noqa: F401
    HAVE_VLLM = True
except Exception:  # vLLM absent: stand-ins
    HAVE_VLLM = False

    class AttentionType:
        DECODER = "decoder"
        ENCODER = "encoder"
        ENCODER_ONLY = "encoder_only"
        ENCODER_DECODER = "encoder_decoder"

    class CUDAGraphMode(enum.Enum):
        NONE = 0
        PIECEWISE = 1
        FULL = 2

    class AttentionCGSupport(enum.Enum):
        NEVER = 0
        UNIFORM_SINGLE_TOKEN_DECODE = 1
        UNIFORM_BATCH = 2
        ALWAYS = 3

    class QueryLenSupport(enum.Enum):
        SINGLE_ONLY = "single_only"
        UNIFORM = "uniform"
        VARLEN = "varlen"

    class PlatformEnum(enum.Enum):
        CUDA = enum.auto()
        ROCM = enum.auto()
        OOT = enum.auto()
        UNSPECIFIED = enum.auto()

    class Platform:
        _enum = PlatformEnum.UNSPECIFIED
        device_name: str = ""
        device_type: str = ""
        dispatch_key: str = "CPU"
        ray_device_key: str = ""
        dist_backend: str = ""
        device_control_env_var: str = ""

        def __init__(self):
            pass

    @dataclass(frozen=True)
    class BatchDescriptor:
        num_tokens: int
        num_reqs: Optional[int] = None
        uniform: bool = False
        has_lora: bool = False

    @dataclass
    class _ForwardContext:
        attn_metadata: Any = None
        batch_descriptor: Optional[BatchDescriptor] = None
        cudagraph_runtime_mode: CUDAGraphMode = CUDAGraphMode.NONE
        virtual_engine: int = 0
        capturing: bool = False

    _forward_context: Optional[_ForwardContext] = None

    def get_forward_context() -> _ForwardContext:
        assert _forward_context is not None, "forward context is not set"
        return _forward_context

    class set_forward_context:  # context manager, same role as vllm.forward_context.set_forward_context
        def __init__(self, attn_metadata=None, batch_descriptor=None, cudagraph_runtime_mode=CUDAGraphMode.NONE):
            self.ctx = _ForwardContext(attn_metadata, batch_descriptor, cudagraph_runtime_mode)

        def __enter__(self):
            global _forward_context
            self.prev = _forward_context
            _forward_context = self.ctx
            return self.ctx

        def __exit__(self, *exc):
            global _forward_context
            _forward_context = self.prev
            return False

    @dataclass
    class AttentionSpec:
        block_size: int
        num_kv_heads: int
        head_size: int
        dtype: torch.dtype

        @property
        def page_size_bytes(self) -> int:
            # keys and values: twice the row (vLLM's AttentionSpec)
            return 2 * self.block_size * self.num_kv_heads * self.head_size * torch.empty((), dtype=self.dtype).element_size()

    @dataclass
    class MLAAttentionSpec(AttentionSpec):
        cache_dtype_str: Optional[str] = None

        @property
        def page_size_bytes(self) -> int:
            # one latent row per token serves as key and value (vLLM's MLAAttentionSpec)
            return self.block_size * self.num_kv_heads * self.head_size * torch.empty((), dtype=self.dtype).element_size()

    @dataclass
    class CommonAttentionMetadata:
        query_start_loc: torch.Tensor
        query_start_loc_cpu: torch.Tensor
        seq_lens: torch.Tensor
        seq_lens_cpu: torch.Tensor
        num_computed_tokens_cpu: torch.Tensor
        num_reqs: int
        num_actual_tokens: int
        max_query_len: int
        max_seq_len: int
        block_table_tensor: torch.Tensor
        slot_mapping: torch.Tensor
        causal: bool = True

    @dataclass
    class ChunkedContextMetadata:
        cu_seq_lens: torch.Tensor            # int32 [iters, B+1]
        starts: torch.Tensor                 # int32 [iters, B]
        seq_tot: list
        max_seq_lens: list
        seq_lens: torch.Tensor               # int32 [iters, B]
        workspace: torch.Tensor              # [>= max(seq_tot), 576]

    @dataclass
    class MLACommonPrefillMetadata:
        block_table: torch.Tensor
        query_start_loc: torch.Tensor
        max_query_len: int
        chunked_context: Optional[ChunkedContextMetadata] = None
        query_start_loc_list: Optional[list] = None

    @dataclass
    class MLACommonDecodeMetadata:
        block_table: torch.Tensor
        seq_lens: Any
        dcp_tot_seq_lens: Optional[torch.Tensor] = None

    D = TypeVar("D")

    @dataclass
    class MLACommonMetadata(Generic[D]):
        num_reqs: int
        max_query_len: int
        max_seq_len: int
        num_actual_tokens: int
        query_start_loc: torch.Tensor
        slot_mapping: torch.Tensor
        num_decodes: int
        num_decode_tokens: int
        num_prefills: int
        head_dim: Optional[int] = None
        decode: Optional[D] = None
        prefill: Optional[MLACommonPrefillMetadata] = None

    class MLACommonBackend:
        accept_output_buffer: bool = True

        @staticmethod
        def get_supported_head_sizes() -> list:
            return [576]

        @staticmethod
        def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int,
                               cache_dtype_str: str = "auto") -> tuple:
            return (num_blocks, block_size, head_size)

    def split_decodes_and_prefills(common: CommonAttentionMetadata, decode_threshold: int = 1):
        """(num_decodes, num_prefills, num_decode_tokens, num_prefill_tokens); decodes come first in the batch."""
        q = common.query_start_loc_cpu
        lens = (q[1:] - q[:-1]).tolist()
        nd = 0
        while nd < len(lens) and lens[nd] <= decode_threshold:
            nd += 1
        ndt = int(q[nd])
        return nd, len(lens) - nd, ndt, common.num_actual_tokens - ndt

    class MLACommonMetadataBuilder(Generic[D]):
        """Stand-in for vLLM's builder: decode/prefill split and the chunked-context schedule."""
        reorder_batch_threshold: int = 1

        def __init__(self, kv_cache_spec, layer_names, vllm_config, device, metadata_cls=None):
            self.kv_cache_spec = kv_cache_spec
            self.layer_names = layer_names
            self.vllm_config = vllm_config
            self.device = device
            self.metadata_cls = metadata_cls or MLACommonMetadata
            self.prefill_metadata_cls = MLACommonPrefillMetadata
            self.compilation_config = getattr(vllm_config, "compilation_config", None)
            pc = getattr(vllm_config, "parallel_config", None)
            self.dcp_world_size = getattr(pc, "decode_context_parallel_size", 1) or 1
            self.dcp_local_block_size = getattr(pc, "cp_kv_cache_interleave_size", 1) or 1
            self._use_fi_prefill = False
            self._use_cudnn_prefill = False
            self.aot_schedule = False
            self.page_size = kv_cache_spec.block_size
            self.chunked_prefill_workspace_size = self.determine_chunked_prefill_workspace_size(vllm_config)
            self.chunked_prefill_workspace = None

        @staticmethod
        def determine_chunked_prefill_workspace_size(vllm_config) -> int:
            sc = getattr(vllm_config, "scheduler_config", None)
            mc = getattr(vllm_config, "model_config", None)
            cc = getattr(vllm_config, "cache_config", None)
            max_num_seqs = getattr(sc, "max_num_seqs", 1) or 1
            max_model_len = getattr(mc, "max_model_len", 4096) or 4096
            block = getattr(cc, "block_size", 128) or 128
            size = min(max(8 * max_model_len, 4 * max_num_seqs * block), 64 * 1024)
            return max(size, max_num_seqs * block)

        def _build_decode(self, block_table_tensor, seq_lens_cpu, seq_lens_device, query_start_loc_cpu,
                          query_start_loc_device, num_decode_tokens, dcp_tot_seq_lens_device):
            return MLACommonDecodeMetadata(block_table=block_table_tensor, seq_lens=seq_lens_device,
                                           dcp_tot_seq_lens=dcp_tot_seq_lens_device)

        def build(self, common_prefix_len: int, common_attn_metadata: CommonAttentionMetadata, fast_build: bool = False):
            c = common_attn_metadata
            nd, npf, ndt, _ = split_decodes_and_prefills(c, self.reorder_batch_threshold)
            prefill = decode = None
            if npf > 0:
                qsl = c.query_start_loc[nd:] - c.query_start_loc[nd]
                ctx_cpu = c.num_computed_tokens_cpu[nd:].to(torch.int32)
                chunked = None
                if int(ctx_cpu.max()) > 0:
                    n_ctx = int((ctx_cpu > 0).sum())
                    chunk = max(self.chunked_prefill_workspace_size // max(n_ctx, 1), 1)
                    if chunk >= self.page_size:
                        chunk = chunk // self.page_size * self.page_size
                    iters = -(-int(ctx_cpu.max()) // chunk)
                    starts = (torch.arange(iters, dtype=torch.int32).view(-1, 1) * chunk).expand(-1, npf)
                    ends = torch.minimum(ctx_cpu.view(1, -1), starts + chunk)
                    lens = (ends - starts).clamp_min(0)
                    cu = torch.zeros(iters, npf + 1, dtype=torch.int32)
                    cu[:, 1:] = torch.cumsum(lens, 1)
                    if self.chunked_prefill_workspace is None:
                        self.chunked_prefill_workspace = torch.empty(self.chunked_prefill_workspace_size, 576,
                                                                     dtype=self.kv_cache_spec.dtype, device=self.device)
                    chunked = ChunkedContextMetadata(cu_seq_lens=cu.to(self.device), starts=starts.contiguous().to(self.device),
                                                     seq_tot=lens.sum(1).tolist(), max_seq_lens=lens.max(1)[0].tolist(),
                                                     seq_lens=lens, workspace=self.chunked_prefill_workspace)
                prefill = self.prefill_metadata_cls(block_table=c.block_table_tensor[nd:], query_start_loc=qsl,
                                                    max_query_len=int((c.query_start_loc_cpu[nd + 1:] -
                                                                       c.query_start_loc_cpu[nd:-1]).max()),
                                                    chunked_context=chunked)
            if nd > 0:
                decode = self._build_decode(c.block_table_tensor[:nd], c.seq_lens_cpu[:nd], c.seq_lens[:nd],
                                            c.query_start_loc_cpu[:nd + 1], c.query_start_loc[:nd + 1], ndt, None)
            return self.metadata_cls(num_reqs=c.num_reqs, max_query_len=c.max_query_len, max_seq_len=c.max_seq_len,
                                     num_actual_tokens=c.num_actual_tokens, query_start_loc=c.query_start_loc,
                                     slot_mapping=c.slot_mapping, num_decodes=nd, num_decode_tokens=ndt,
                                     num_prefills=npf, head_dim=576, decode=decode, prefill=prefill)

    class MLACommonBaseImpl(Generic[D]):
        """Stand-in: stores the MLA hyper-parameters; W_UK_T [N,P,L] and W_UV [N,L,V] are set by
        process_weights_after_loading from kv_b_proj (weight viewed [L, N, P+V], reference
        tests/integration/attention/test_npu_mla_math.py:302-313)."""

        def __init__(self, num_heads, head_size, scale, num_kv_heads, alibi_slopes, sliding_window, kv_cache_dtype,
                     logits_soft_cap, attn_type, kv_sharing_target_layer_name, q_lora_rank=None, kv_lora_rank=512,
                     qk_nope_head_dim=128, qk_rope_head_dim=64, qk_head_dim=192, v_head_dim=128, kv_b_proj=None,
                     indexer=None, q_pad_num_heads=None, **_):
            self.num_heads = num_heads
            self.head_size = head_size
            self.scale = float(scale)
            self.num_kv_heads = num_kv_heads
            self.kv_cache_dtype = kv_cache_dtype
            self.q_lora_rank = q_lora_rank
            self.kv_lora_rank = kv_lora_rank
            self.qk_nope_head_dim = qk_nope_head_dim
            self.qk_rope_head_dim = qk_rope_head_dim
            self.qk_head_dim = qk_head_dim
            self.v_head_dim = v_head_dim
            self.kv_b_proj = kv_b_proj
            self.indexer = indexer
            self.dcp_world_size = 1

        def process_weights_after_loading(self, act_dtype: torch.dtype):
            w = self.kv_b_proj.weight.t() if self.kv_b_proj.weight.shape[0] != self.kv_lora_rank else self.kv_b_proj.weight
            kv = w.reshape(self.kv_lora_rank, self.num_heads, self.qk_nope_head_dim + self.v_head_dim)
            w_uk, w_uv = kv.split([self.qk_nope_head_dim, self.v_head_dim], dim=-1)
            self.W_UK_T = w_uk.permute(1, 2, 0).contiguous().to(act_dtype)
            self.W_UV = w_uv.transpose(0, 1).contiguous().to(act_dtype)

    _current_vllm_config = None

    def get_current_vllm_config():
        return _current_vllm_config

    def set_current_vllm_config(cfg):
        global _current_vllm_config
        _current_vllm_config = cfg

if HAVE_VLLM:  # pragma: no cover
    from vllm.config import get_current_vllm_config  # noqa: F401
    from vllm.forward_context import set_forward_context  # noqa: F401
    from vllm.v1.attention.backends.utils import split_decodes_and_prefills  # noqa: F401

PAD_SLOT_ID = -1


class _DeviceBytes:
    """A span of device memory named by address only, for ``torch.as_tensor``: the tensor built over it owns nothing."""

    def __init__(self, ptr: int, nbytes: int):
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (ptr, False), "version": 3,
                                         "strides": None}


def _weak_ref_tensor(t):
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.numel() == 0:
        return t
    # the smallest span of the storage the view can touch
    span = 1 + sum((n - 1) * st for n, st in zip(t.shape, t.stride()))
    with torch.cuda.device(t.device):
        raw = torch.as_tensor(_DeviceBytes(t.data_ptr(), span * t.element_size()), device=t.device)
    return raw.view(t.dtype).as_strided(t.shape, t.stride())


def weak_ref_tensors(out):
    """Aliases of ``out`` (a tensor, or a list / tuple of them) that do not keep its storage alive, as vLLM's helper of the
    same name gives: a captured graph's output then lives in the graph's memory pool alone, and the pool can hand the
    bytes to the next graph (reference acl_graph.py:209-222).  Without vLLM the alias is built over the bare address."""
    if HAVE_VLLM:  # pragma: no cover
        from vllm.utils.torch_utils import weak_ref_tensors as _w
        return _w(out)
    if isinstance(out, (list, tuple)):
        return type(out)(weak_ref_tensors(o) for o in out)
    return _weak_ref_tensor(out)
