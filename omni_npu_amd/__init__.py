"""MI355X (gfx950) MLA / DSA attention backend behind the omni-npu vLLM plugin surface.

The package mirrors the part of the reference tree that sits on the attention hot path
(src/omni_npu/{vllm_plugin,platform}.py, attention/backends/{mla,dsa}.py, attention/ops.py,
compilation/acl_graph.py); every kernel underneath is a hand-written HIP kernel in
``csrc/`` reached through the C-ABI of ``libmla_hip.so`` (declared in include/mla_hip.h).
"""
__version__ = "0.1.0"
