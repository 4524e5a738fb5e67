"""The C-ABI library loads on a box without a GPU and exports every symbol include/mla_hip.h declares;
argument validation answers with error codes (no compute is launched here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mla_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:mla|mlahip|dsa)_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_path():
    syms = declared_symbols()
    for must in ("mla_cache_write_bf16", "mla_cache_write_fp8", "mla_decode_bf16", "mla_splitkv_reduce",
                 "mla_decode_workspace_bytes", "mla_gather_paged", "mla_merge_states", "dsa_indexer_scores_fp8",
                 "dsa_topk", "dsa_topk_rows", "dsa_topk_workspace_bytes", "dsa_sparse_decode_bf16", "mlahip_version", "mlahip_last_error_string"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    from omni_npu_amd import _lib
    lib = _lib.load()
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in include/mla_hip.h but not exported"
    assert set(_lib.SIGNATURES) == set(declared_symbols()), "ctypes table and header disagree"
    assert lib.mlahip_version() >= 100


def test_bad_arguments_return_codes_not_crashes():
    from omni_npu_amd import _lib
    lib = _lib.load()
    assert lib.mla_decode_workspace_bytes(64, 1, 128, 4) == 64 * (4 + 1) * 128 * (512 * 2 + 4 + 4 + 8) + 64 * 8
    assert lib.mla_decode_workspace_bytes(0, 1, 128, 4) == 0
    rc = lib.mla_cache_write_bf16(None, 512, None, 64, None, 4, None, 0, 0, None, 0, 0, 128, 1, None)
    assert rc == -1 and b"null" in lib.mlahip_last_error_string()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf) // 16 * 16 + 16
    rc = lib.mla_cache_write_bf16(p, 513, p, 64, p, 4, p, 65536, 512, p, 8192, 64, 128, 1, None)   # odd row stride
    assert rc == -2
    rc = lib.dsa_topk(p, 1 << 23, p, None, 1, 1, 16, p, 16, None, 0, None)                                  # too many keys per row
    assert rc == -2
    rc = lib.mla_merge_states(p, 1, 1, p, p, 1, 1, p, 7, p, 1, 1, 0, None, 1, 1, 1, None)          # unknown dtype code
    assert rc == -3
    with pytest.raises(_lib.MlaHipError):
        _lib.check(rc, "mla_merge_states")


def test_ops_refuse_cpu_tensors():
    """The product path has no CPU fallback: host tensors are rejected before any launch."""
    import torch
    from omni_npu_amd import kernels as K
    with pytest.raises(ValueError, match="no CPU path"):
        K.cache_write(torch.zeros(1, 512, dtype=torch.bfloat16), torch.zeros(1, 64, dtype=torch.bfloat16),
                      torch.zeros(1, dtype=torch.int64), torch.zeros(1, 128, 512, dtype=torch.bfloat16),
                      torch.zeros(1, 128, 64, dtype=torch.bfloat16))
