"""ctypes binding of libmla_hip.so.

There is no fallback: if the library is missing or a symbol is absent this module raises, and so
does every op built on it.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int32, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmla_hip.so")

P, I32, I64, F32, SZ = c_void_p, c_int32, c_int64, c_float, c_size_t

# name -> (restype, argtypes); mirrors include/mla_hip.h one to one
SIGNATURES = {
    "mlahip_version": (c_int32, []),
    "mlahip_last_error_string": (c_char_p, []),
    "mla_cache_write_bf16": (c_int32, [P, I64, P, I64, P, I32, P, I64, I64, P, I64, I64, I32, I64, P]),
    "mla_scatter_rows": (c_int32, [P, I64, I32, P, I32, P, I64, I64, I32, I64, P]),
    "mla_cache_write_fp8": (c_int32, [P, I64, P, I64, P, I32, P, I64, I64, I32, I64, P]),
    "mla_kv_rmsnorm_rope_cache": (c_int32, [P, I64, P, I64, P, P, P, I64, I32, I32, P, I32, F32, P, I64, I64, P, I64, I64,
                                            I32, I64, P, I64, P, I64, P]),
    "mla_kv_rmsnorm_rope_cache_fp8": (c_int32, [P, I64, P, I64, P, P, P, I64, I32, I32, P, I32, F32, P, I64, I64, I32, I64,
                                                P, I64, P, I64, P]),
    "mla_kv_rmsnorm_rope_cache_q": (c_int32, [P, I64, P, I64, P, P, P, I64, I32, I32, P, I32, F32, P, I64, I64, P, I64, I64,
                                              I32, I64, P, I64, P, I64, P, I64, I64, I32, P, I64, I64, P]),
    "mla_kv_rmsnorm_rope_cache_q_fp8": (c_int32, [P, I64, P, I64, P, P, P, I64, I32, I32, P, I32, F32, P, I64, I64, I32,
                                                  I64, P, I64, P, I64, P, I64, I64, I32, P, I64, I64, P]),
    "mla_interleave_rope": (c_int32, [P, I64, I64, I64, I32, P, P, I64, I32, I32, P, I64, I64, P]),
    "mla_rotary_mul": (c_int32, [P, I64, I64, I64, I32, P, P, I64, I32, P, I64, I64, P]),
    "mla_decode_fp8": (c_int32, [P, I64, I64, P, I64, I64, P, I64, I64, I64, P, I64, I32, P, P, I32, I32, I32, F32, P, I64,
                                 I64, P, P, SZ, I32, P]),
    "mla_gather_paged": (c_int32, [P, I64, I64, P, I64, I64, I64, I32, P, I64, I64, P, I64, I32, P, P, I32, I64, P]),
    "mla_gather_paged_fp8": (c_int32, [P, I64, I64, I64, I32, P, I64, I64, P, I64, I32, P, P, I32, I64, P]),
    "mla_merge_states": (c_int32, [P, I64, I64, P, P, I64, I64, P, I32, P, I64, I64, I32, P, I32, I32, I32, P]),
    "mla_merge_n_states": (c_int32, [P, I64, I64, I32, P, I64, P, I64, P, I32, I32, I32, P]),
    "mla_decode_workspace_bytes": (SZ, [I32, I32, I32, I32]),
    "mla_decode_bf16_split": (c_int32, [P, I64, I64, P, I64, I64, P, I64, I64, P, I64, I64, I64, P, I64, I32, P, P, I32,
                                        I32, I32, F32, P, SZ, I32, P]),
    "mla_window_plan": (c_int32, [P, P, I32, I32, I32, I32, P, P, P]),
    "mla_decode_bf16_window_split": (c_int32, [P, I64, I64, P, I64, I64, P, I64, I64, P, I64, I64, I64, P, I64, I32, P, P, P,
                                               I32, I32, I32, I32, I32, F32, P, SZ, I32, P]),
    "mla_decode_fp8_window_split": (c_int32, [P, I64, I64, P, I64, I64, P, I64, I64, I64, P, I64, I32, P, P, P, I32, I32, I32,
                                              I32, I32, F32, P, SZ, I32, P]),
    "mla_splitkv_reduce": (c_int32, [P, SZ, P, P, I32, I32, I32, I32, P, I64, I64, P, P]),
    "mla_splitkv_reduce_vup": (c_int32, [P, SZ, P, P, I32, I32, I32, I32, I32, P, I64, I64, P, I64, I64, P]),
    "mla_decode_bf16": (c_int32, [P, I64, I64, P, I64, I64, P, I64, I64, P, I64, I64, I64, P, I64, I32, P, P, I32,
                                  I32, I32, F32, P, I64, I64, P, P, SZ, I32, P]),
    "mla_decode_bf16_step": (c_int32, [P, I64, I64, P, I64, I64, P, I64, I64, P, I64, I64, I64, P, I64, P, I64, P, P, I64,
                                       I32, P, P, I32, I32, I32, F32, P, I64, I64, P, P, SZ, I32, P]),
    "mla_decode_bf16_static": (c_int32, [P, I64, I64, P, I64, I64, P, I64, I64, P, I64, I64, I64, P, I64, I32, P, P, I32,
                                         I32, I32, F32, P, I64, I64, P, I32, P]),
    "mla_prefill_varlen": (c_int32, [P, I64, I64, P, I64, I64, P, I64, I64, P, I64, P, I64, I64, P, P, I32, I32, I32, I32,
                                     I32, F32, P, I64, I64, I32, P, P]),
    "mla_prefill_varlen_continue": (c_int32, [P, I64, I64, P, I64, I64, P, I64, I64, P, I64, P, I64, I64, P, P, I32, I32, I32,
                                              I32, I32, F32, P, I64, I64, I32, P, P, I64, I64, P, P]),
    "dsa_indexer_scores_fp8": (c_int32, [P, I64, I64, P, I64, P, I64, P, I64, I64, P, I64, I64, I32, P, I64, I32, P, P, I32,
                                         I32, I32, I32, P, I64, P]),
    "dsa_quant_rows_fp8": (c_int32, [P, I64, I64, P, P, I64, I64, P, I64, I32, I64, P]),
    "dsa_quant_qk_fp8": (c_int32, [P, I64, I64, P, P, P, I64, I64, P, P, I64, I64, P, I64, I32, I64, P]),
    "dsa_topk_workspace_bytes": (SZ, [I32, I32, I64]),
    "dsa_topk": (c_int32, [P, I64, P, P, I32, I32, I32, P, I64, P, SZ, P]),
    "dsa_topk_rows": (c_int32, [P, I64, P, P, I32, I32, I32, P, I64, P, I64, I32, I32, I64, P, I64, P, P, SZ, P]),
    "dsa_build_rows": (c_int32, [P, I64, P, I64, I32, P, P, I32, I32, I32, I32, I64, P, I64, P, P]),
    "dsa_sparse_decode_bf16": (c_int32, [P, I64, I64, P, I64, I64, P, I64, I64, P, I64, I64, I64, I32, P, I64, P, I32, I32,
                                         F32, P, I64, I64, P, P, SZ, I32, P]),
    "dsa_sparse_decode_heads_bf16": (c_int32, [P, I64, I64, P, I64, I64, P, I64, P, I64, I64, P, I64, P, I32, I32, F32, P, I64,
                                               I64, P, P]),
}


class MlaHipError(RuntimeError):
    """A C-ABI entry point returned a negative code."""


_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C omni_npu_amd/csrc`). There is no non-HIP fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().mlahip_last_error_string()
        raise MlaHipError(f"{what} failed with code {rc}: {msg.decode() if msg else ''}")
