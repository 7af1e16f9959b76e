"""The C-ABI library loads and exports every symbol include/f8mi.h declares (no GPU, no compute)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "f8mi.h")
LIB = os.path.join(ROOT, "float8_experimental_amd", "libf8mi.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(f8mi_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for must in ("f8mi_amax_scale", "f8mi_cast", "f8mi_gemm_nt", "f8mi_sync", "f8mi_delayed_init", "f8mi_version"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    if not os.path.exists(LIB):
        pytest.fail(f"{LIB} has not been built (run __graft_entry__.build())")
    lib = ctypes.CDLL(LIB)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, f"declared in f8mi.h but not exported: {missing}"
    lib.f8mi_version.restype = ctypes.c_int
    assert lib.f8mi_version() >= 100
    lib.f8mi_workspace_bytes.restype = ctypes.c_size_t
    assert 8 <= lib.f8mi_workspace_bytes() <= 4096


def test_binding_lists_the_same_symbols():
    from float8_experimental_amd import _native

    assert sorted(_native.EXPORTS) == declared_symbols()


def test_host_side_argument_checks_need_no_gpu():
    """Invalid arguments are rejected on the host before anything touches a device."""
    lib = ctypes.CDLL(LIB)
    lib.f8mi_last_error.restype = ctypes.c_char_p
    i64 = ctypes.c_int64
    rc = lib.f8mi_gemm_nt(None, 0, i64(8), None, 0, i64(8), i64(4), i64(4), i64(16), None, None, None, 0, i64(4), None, None)
    assert rc == -1 and b"lda" in lib.f8mi_last_error()
    rc = lib.f8mi_cast(None, i64(-1), i64(4), i64(4), 0, None, 0, 0, None, None, None, None, None)
    assert rc == -1
    rc = lib.f8mi_amax_scale(None, i64(4), i64(4), i64(4), 7, 0, 0, 0, None, None, None, None)
    assert rc == -1
    rc = lib.f8mi_sync(None, -1, 16, 0, 0, None)
    assert rc == -1
    # k-blocked operands: k must be a multiple of 64 and at least 384 (unsupported, not invalid)
    rc = lib.f8mi_gemm_nt_kb(None, 0, None, 0, i64(4), i64(4), i64(100), None, None, None, 0, i64(4), None, None)
    assert rc == -2 and b"k-blocked" in lib.f8mi_last_error()
    # the workspace variants check their arguments like the plain ones
    rc = lib.f8mi_gemm_nt_kb_ws(None, 0, None, 0, i64(4), i64(4), i64(100), None, None, None, 0, i64(4), None, None, i64(0), None)
    assert rc == -2 and b"k-blocked" in lib.f8mi_last_error()
    rc = lib.f8mi_gemm_nt_ws(None, 0, i64(8), None, 0, i64(8), i64(-1), i64(4), i64(8), None, None, None, 0, i64(4), None, None, i64(0), None)
    assert rc == -1
    # transposed operands: (a transposed, bt not) is not built; row counts must be multiples of 64
    rc = lib.f8mi_gemm_kb_ex(None, 0, 1, None, 0, 0, i64(64), i64(64), i64(384), None, None, None, 0, i64(64), None, None)
    assert rc == -2
    rc = lib.f8mi_gemm_kb_ex(None, 0, 0, None, 0, 1, i64(64), i64(100), i64(384), None, None, None, 0, i64(100), None, None)
    assert rc == -2 and b"multiple of 64" in lib.f8mi_last_error()
    rc = lib.f8mi_cast_layout(None, i64(4), i64(100), i64(100), 0, ctypes.c_void_p(8), 0, 0, ctypes.c_void_p(8), 1, None, 0, None, None)
    assert rc == -2 and b"cols % 64" in lib.f8mi_last_error()
    rc = lib.f8mi_cast_layout(None, i64(4), i64(64), i64(64), 0, ctypes.c_void_p(8), 0, 0, ctypes.c_void_p(8), 5, None, 0, None, None)
    assert rc == -1
    rc = lib.f8mi_cast_dynamic(None, i64(4), i64(4), i64(4), 0, 0, None, None, 0, None, 0, None, None)
    assert rc == -1 and b"scale" in lib.f8mi_last_error()
    rc = lib.f8mi_amax_scale_multi(None, 5000, i64(5000), 0, 0, 0, 0, ctypes.c_void_p(8), None, None, None)
    assert rc == -1 and b"at most" in lib.f8mi_last_error()


def test_cpu_tensors_are_refused_loudly():
    import torch

    from float8_experimental_amd import _native

    with pytest.raises(_native.Float8NativeError):
        _native.amax_scale(torch.ones(4, 4, dtype=torch.bfloat16), torch.float8_e4m3fn)
    with pytest.raises(_native.Float8NativeError):
        _native.cast(torch.ones(4, 4, dtype=torch.bfloat16), torch.tensor(1.0), torch.float8_e4m3fn)
