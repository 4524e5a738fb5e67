def plugin() -> "str | None":
    """Entry point of the ``vllm.platform_plugins`` group (reference src/omni_npu/vllm_plugin.py:1-23).

    Returns the dotted path of the Platform class when this process runs PyTorch-ROCm and sees a gfx950 device,
    otherwise None so that vLLM falls back to its other platforms.
    """
    try:
        import torch
    except Exception:
        return None
    if getattr(torch.version, "hip", None) is None:
        return None
    try:
        if torch.cuda.device_count() < 1:
            return None
        arch = torch.cuda.get_device_properties(0).gcnArchName
    except Exception:
        return None
    if not str(arch).startswith("gfx950"):
        return None
    return "omni_npu_amd.platform.MI355XPlatform"
