"""vLLM Platform for MI355X (reference: src/omni_npu/platform.py:45-187).

Selects the worker, the attention backends and the graph wrapper by dotted class path, exactly as the reference's
NPUPlatform does; device shims go to torch.cuda, which is HIP on PyTorch-ROCm; the distributed backend name is
"nccl" (RCCL), unused on the single-GPU path.
"""
from __future__ import annotations

from typing import Optional

import torch

from ._vllm_compat import Platform, PlatformEnum


class MI355XPlatform(Platform):
    _enum = getattr(PlatformEnum, "OOT", None)
    device_name: str = "cuda"
    device_type: str = "cuda"
    dispatch_key: str = "CUDA"
    ray_device_key: str = "GPU"
    dist_backend: str = "nccl"
    device_control_env_var: str = "HIP_VISIBLE_DEVICES"

    def __init__(self):
        super().__init__()

    @classmethod
    def set_device(cls, device: torch.device) -> None:
        torch.cuda.set_device(device)

    @classmethod
    def get_device_name(cls, device_id: int = 0) -> str:
        return torch.cuda.get_device_name(device_id)

    @classmethod
    def inference_mode(cls):
        return torch.no_grad()

    @classmethod
    def import_kernels(cls):
        from . import _lib
        _lib.load()                      # fail at start-up, not at the first token, if the HIP library is missing

    @classmethod
    def get_current_memory_usage(cls, device: Optional[torch.types.Device] = None) -> float:
        torch.cuda.reset_peak_memory_stats(device)
        return torch.cuda.max_memory_allocated(device)

    @classmethod
    def device_count(cls) -> int:
        return torch.cuda.device_count()

    @classmethod
    def mem_get_info(cls) -> tuple:
        return torch.cuda.mem_get_info()

    @classmethod
    def pre_register_and_update(cls, parser=None) -> None:
        return None

    @classmethod
    def check_and_update_config(cls, vllm_config) -> None:
        """Worker class, default block size 128, fusion passes off (reference platform.py:115-128)."""
        vllm_config.parallel_config.worker_cls = "omni_npu_amd.worker.hip_worker.HIPWorker"
        cache_config = vllm_config.cache_config
        if cache_config and cache_config.block_size is None:
            cache_config.block_size = 128
        pass_config = getattr(getattr(vllm_config, "compilation_config", None), "pass_config", None)
        if pass_config is not None:
            pass_config.fuse_norm_quant = False
            pass_config.fuse_act_quant = False
            pass_config.fuse_attn_quant = False

    @classmethod
    def get_punica_wrapper(cls) -> str:
        return "vllm.lora.punica_wrapper.punica_gpu.PunicaWrapperGPU"

    @classmethod
    def get_device_communicator_cls(cls) -> str:
        return "vllm.distributed.device_communicators.cuda_communicator.CudaCommunicator"

    @classmethod
    def get_attn_backend_cls(cls, selected_backend, head_size: int, dtype: torch.dtype, kv_cache_dtype: Optional[str],
                             block_size: int, use_mla: bool, has_sink: bool, use_sparse: bool,
                             attn_type: "str | None" = None) -> str:
        """MLA -> NPUMLABackend, sparse MLA -> NPUDSABackend (reference platform.py:140-162).  Non-MLA attention is not
        part of this build."""
        if use_mla:
            if use_sparse:
                return "omni_npu_amd.attention.backends.dsa.NPUDSABackend"
            return "omni_npu_amd.attention.backends.mla.NPUMLABackend"
        raise NotImplementedError("omni_npu_amd provides the MLA / DSA attention backends only")

    @property
    def simple_compile_backend(self):
        return "eager"

    @classmethod
    def support_static_graph_mode(cls) -> bool:
        return True

    @classmethod
    def get_static_graph_wrapper_cls(cls) -> str:
        return "omni_npu_amd.compilation.acl_graph.HIPGraphWrapper"


NPUPlatform = MI355XPlatform          # the reference's class name
