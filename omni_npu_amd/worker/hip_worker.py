"""Worker-side hooks of the plugin contract that touch the attention path (reference:
src/omni_npu/worker/npu_model_runner.py:125-187 and npu_worker.py:38-60).

The reference's NPUModelRunner subclasses vLLM's GPUModelRunner wholesale after swapping torch.cuda for torch.npu;
on ROCm the stock runner already drives HIP, so only the two cache hooks differ and they are provided here as a mixin
that is combined with vLLM's classes when vLLM is importable.
"""
from __future__ import annotations

from typing import Any

import torch

from .. import kernels as K
from .._vllm_compat import HAVE_VLLM, AttentionSpec, MLAAttentionSpec

INDEX_HEAD_DIM_DEFAULT = 128


def kv_cache_dtype_and_head_size(cache_dtype: str, model_dtype: torch.dtype, head_size: int, index_head_dim: int = 0):
    """fp8 cache: 656 bytes per token in a uint8 tensor (512 e4m3 | 4 fp32 scales | 64 bf16 rope); otherwise
    head_size + index_head_dim elements of the model dtype (the DSA layout keeps the indexer keys in the same pages).
    An fp8 latent cache for a DSA model is refused: the 656-byte row has no room for the indexer keys and NPUDSAImpl writes
    the bf16 layout only."""
    if cache_dtype in ("fp8", "fp8_e4m3"):
        if index_head_dim:
            raise NotImplementedError("an fp8 KV cache is not supported for DSA (indexer) models: the fp8 row layout holds "
                                      "the 512 + 64 latent only; use kv_cache_dtype='auto'")
        return torch.uint8, K.FP8_ROW_BYTES
    return model_dtype, head_size + index_head_dim


class KVCacheHooksMixin:
    """get_kv_cache_spec / _reshape_kv_cache_tensors as the reference overrides them."""

    def get_kv_cache_spec(self) -> dict:
        mc = self.vllm_config.model_config
        cc = self.vllm_config.cache_config
        if not getattr(mc, "use_mla", False):
            return super().get_kv_cache_spec()
        is_dsa = hasattr(mc.hf_config, "index_topk")
        extra = getattr(mc.hf_config, "index_head_dim", INDEX_HEAD_DIM_DEFAULT) if is_dsa else 0
        specs = {}
        for layer_name, attn_module in self._attention_layers().items():
            dtype, head = kv_cache_dtype_and_head_size(cc.cache_dtype, mc.dtype, attn_module.head_size, extra)
            specs[layer_name] = MLAAttentionSpec(block_size=cc.block_size, num_kv_heads=1, head_size=head, dtype=dtype,
                                                 cache_dtype_str=cc.cache_dtype)
        return specs

    def _reshape_kv_cache_tensors(self, kv_cache_config: Any, kv_cache_raw_tensors: dict, kernel_block_sizes=None) -> dict:
        kv_caches = {}
        for group in self._kv_cache_spec_attn_group_iterator():
            spec, backend = group.kv_cache_spec, group.backend
            for layer_name in group.layer_names:
                if layer_name in getattr(self, "runner_only_attn_layers", ()):
                    continue
                raw = kv_cache_raw_tensors[layer_name]
                assert raw.numel() % spec.page_size_bytes == 0
                num_blocks = raw.numel() // spec.page_size_bytes
                if not isinstance(spec, AttentionSpec):
                    raise NotImplementedError
                kv_caches[layer_name] = backend.reshape_kv_cache(raw, num_blocks, spec.block_size, spec.num_kv_heads,
                                                                 spec.head_size, dtype=spec.dtype)
        return kv_caches


if HAVE_VLLM:  # pragma: no cover - needs vLLM
    from vllm.v1.worker.gpu_model_runner import GPUModelRunner
    from vllm.v1.worker.gpu_worker import Worker as _GPUWorker

    class HIPModelRunner(KVCacheHooksMixin, GPUModelRunner):
        def _attention_layers(self):
            from vllm.attention.layer import AttentionLayerBase
            from vllm.config import get_layers_from_vllm_config
            return get_layers_from_vllm_config(self.vllm_config, AttentionLayerBase)

    class HIPWorker(_GPUWorker):
        """Worker(vllm_config, local_rank, rank, distributed_init_method, is_driver_worker=False)."""

        def init_device(self):
            super().init_device()
            self.model_runner.__class__ = type("HIPModelRunnerBound", (KVCacheHooksMixin, self.model_runner.__class__), {
                "_attention_layers": HIPModelRunner._attention_layers})
else:
    class HIPWorker:
        """Placeholder with the reference's constructor signature (npu_worker.py:41-60); the real class needs vLLM."""

        def __init__(self, vllm_config, local_rank: int, rank: int, distributed_init_method: str,
                     is_driver_worker: bool = False):
            raise ImportError("HIPWorker wraps vLLM's GPU worker; vLLM 0.12 is not importable in this environment")
