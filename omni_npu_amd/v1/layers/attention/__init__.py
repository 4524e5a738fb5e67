from .npu_mla import NPUDeepseekMLAAttention

__all__ = ["NPUDeepseekMLAAttention"]
