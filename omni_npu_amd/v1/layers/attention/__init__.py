from .npu_dsa import NPUDeepseekSparseAttention
from .npu_mla import NPUDeepseekMLAAttention

__all__ = ["NPUDeepseekMLAAttention", "NPUDeepseekSparseAttention"]
