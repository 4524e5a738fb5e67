"""Counterparts of the reference's custom-model route (src/omni_npu/v1): modules that call the kernels directly."""
