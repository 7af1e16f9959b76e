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


def test_benchmark_probe_is_not_part_of_the_library():
    """The register-only MFMA probe synchronises and copies from the host: it lives in its own shared object."""
    lib = ctypes.CDLL(LIB)
    assert not hasattr(lib, "f8mi_probe_mfma")
    probe = os.path.join(ROOT, "float8_experimental_amd", "libf8mi_probe.so")
    assert os.path.exists(probe), f"{probe} has not been built (run __graft_entry__.build())"
    assert hasattr(ctypes.CDLL(probe), "f8mi_probe_mfma")


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
    rc = lib.f8mi_sync_host(None, 3, 16, 0, 0, None)
    assert rc == -1
    bad = (ctypes.c_int64 * 4)(8, 0, 8, 0)  # null history pointer
    rc = lib.f8mi_sync_host(bad, 1, 16, 0, 0, None)
    assert rc == -1 and b"entry 0" in lib.f8mi_last_error()
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
    rc = lib.f8mi_cast_dynamic_static(ctypes.c_void_p(16), i64(1 << 20), i64(1 << 20), i64(1 << 20), 0, 0, ctypes.c_void_p(16),
                                      ctypes.c_void_p(16), 0, None, 0, None)
    assert rc == -1 and b"at most" in lib.f8mi_last_error()
    rc = lib.f8mi_amax_scale_multi(None, 5000, i64(5000), 0, 0, 0, 0, ctypes.c_void_p(8), None, None, None)
    assert rc == -1 and b"at most" in lib.f8mi_last_error()


def test_cpu_tensors_are_refused_loudly():
    import torch

    from float8_experimental_amd import _native

    with pytest.raises(_native.Float8NativeError):
        _native.amax_scale(torch.ones(4, 4, dtype=torch.bfloat16), torch.float8_e4m3fn)
    with pytest.raises(_native.Float8NativeError):
        _native.cast(torch.ones(4, 4, dtype=torch.bfloat16), torch.tensor(1.0), torch.float8_e4m3fn)


def test_gemm_plan_names_the_kernel_each_shape_class_takes():
    """f8mi_gemm_plan needs no GPU: the shape classes the GPU tests are written for really take the kernel they name."""
    from float8_experimental_amd import _native as nat

    plan = nat.gemm_plan
    # training shapes of the benchmark: whole rounds of 256 x 256 tiles
    for m, n, k in ((16384, 10240, 8192), (16384, 8192, 8192), (16384, 57344, 8192), (16384, 8192, 28672), (8192, 57344, 16384)):
        assert plan(m, n, k) == ("tiles256", 0, 0), (m, n, k)
    # decode steps stream the weight once; so does a narrow weight up to 256 rows
    for m, n, k in ((1, 8192, 8192), (16, 57344, 8192), (32, 8192, 8192), (128, 4096, 4096), (200, 4096, 4096)):
        assert plan(m, n, k)[0] == "few_rows", (m, n, k)
    # a wide weight at 17 - 256 rows, and outputs of at most 256 small tiles: 128-row tiles
    assert plan(64, 28672, 512) == ("tiles128", 0, 1) and plan(20, 16384, 256) == ("tiles128", 0, 1)
    assert plan(200, 8192, 512) == ("tiles128", 0, 1) and plan(300, 520, 1024) == ("tiles128", 0, 1)
    assert plan(1024, 8192, 1024) == ("tiles128", 0, 2) and plan(8192, 1024, 4096) == ("tiles128", 0, 2)
    # few tiles and a long k: split over k when there is scratch memory, and only then
    for m, n, k in ((256, 2048, 16384), (512, 1024, 8192), (100, 4096, 16384), (128, 8192, 28672)):
        name, parts, mid = plan(m, n, k)
        assert name == "tiles128_split_k" and parts in (2, 4, 8) and k % (128 * parts) == 0 and parts * m * n * 4 <= nat.GEMM_WORKSPACE_BYTES
        assert plan(m, n, k, split_k=False)[0] in ("few_rows", "tiles128")
    # a sparse last round goes to 128-row tiles
    assert plan(4352, 4096, 512) == ("tiles256_and_128", 0, 1) and plan(6144, 4096, 640) == ("tiles256_and_128", 0, 2)
    # the other contraction lengths and unaligned operands
    assert plan(4096, 4096, 448)[0] == "tiles256_mfma32" and plan(4096, 4096, 200)[0] == "staged"
    assert plan(4096, 4096, 4096, aligned=False)[0] == "staged" and plan(64, 4096, 4096, aligned=False)[0] == "staged"
    assert plan(0, 4096, 4096) == (None, 0, 0)


def test_ragged_layers_stay_off_the_register_staged_gemm():
    """The padding benchmark's shapes (reference benchmarks/bench_padding.py:117-132: dimensions that are no multiple
    of 16) and the stress configuration's two layers: on the fused route every product whose contraction reaches 384
    once padded runs on zero-padded k-blocked copies, i.e. on the LDS-DMA kernels, not on the register-staged one."""
    from float8_experimental_amd import _native as nat

    assert nat.lib().f8mi_padded_k(4097) == 4224 == nat.padded_k(4097) and nat.padded_k(128) == 128 and nat.padded_k(0) == 0
    assert nat.kblock_layout(8192) == nat.KBLOCK and nat.kblock_layout(448) == nat.KBLOCK
    assert nat.kblock_layout(4097) == nat.KBLOCK_PAD and nat.kblock_layout(1000) == nat.KBLOCK_PAD and nat.kblock_layout(257) == nat.KBLOCK_PAD
    assert nat.kblock_layout(256) == nat.ROWMAJOR and nat.kblock_layout(200) == nat.ROWMAJOR
    shapes = [(4099, 4097, 11007), (4099, 1000, 3000)]                                  # (tokens, in, out): config 5
    shapes += [(8193, 2501, 5008), (65, 253, 4096), (1023, 1029, 2512), (4095, 511, 10000), (2047, 3073, 8192),
               (511, 769, 7504), (127, 4097, 12288), (32769, 15, 15024), (9217, 8191, 20480),
               (16385, 1025, 25008)]                                                     # (M, K, N) of the padding benchmark
    for m, k, n in shapes:
        route = nat.linear_route(m, k, n)
        for name in ("output", "grad_input", "grad_weight"):
            layout, kc, (kernel, parts, mid) = route[name]
            short = {"output": k, "grad_input": n, "grad_weight": m}[name] <= 256
            if short:
                assert layout == nat.ROWMAJOR
                continue
            assert layout in (nat.KBLOCK, nat.KBLOCK_PAD) and kc % 128 in (0, 64), (m, k, n, name, route[name])
            assert kernel != "staged", (m, k, n, name, route[name])
    # the layers of the benchmark keep one fp8 copy per tensor
    assert nat.linear_route(16384, 8192, 10240)["one_copy"] and not nat.linear_route(4099, 4097, 11007)["one_copy"]
