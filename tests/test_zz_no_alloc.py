"""f8mi_cast_dynamic_static -- the entry point that allocates nothing -- against f8mi_cast_dynamic.

Both are called through the C ABI with raw pointers into tensors allocated beforehand.  The static variant keeps
its per-workgroup partial maxima in an array inside the library; that array keeps the previous call's contents, so
the second call is made on a smaller tensor with a smaller maximum: a stale word read back would show as a wrong
scale.  Bar: identical bits (scale and every fp8 byte)."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def native():
    if not torch.cuda.is_available():
        pytest.fail("these tests need a GPU (run with -m gpu on an MI355X box)")
    from float8_experimental_amd import _native

    _native.lib()
    return _native


def _both(native, x, f8, kblock):
    """(scale, out, out_t) from the workspace entry point and from the static one, on the same input."""
    lib = native.lib()
    rows, cols = x.shape
    code_dt, code_f8 = native._DT[x.dtype], native._F8[f8]
    ws = torch.full((lib.f8mi_workspace_bytes() // 4,), -1, dtype=torch.int32, device=DEV)
    res = []
    for static in (False, True):
        scale = torch.full((1,), float("nan"), dtype=torch.float32, device=DEV)
        out = torch.zeros(rows * cols, dtype=torch.uint8, device=DEV)
        out_t = torch.zeros(rows * cols, dtype=torch.uint8, device=DEV)
        stream = torch.cuda.current_stream().cuda_stream
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        if static:
            rc = lib.f8mi_cast_dynamic_static(x.data_ptr(), rows, cols, x.stride(0), code_dt, code_f8, scale.data_ptr(),
                                              out.data_ptr(), int(kblock), out_t.data_ptr(), int(kblock), stream)
        else:
            rc = lib.f8mi_cast_dynamic(x.data_ptr(), rows, cols, x.stride(0), code_dt, code_f8, scale.data_ptr(),
                                       out.data_ptr(), int(kblock), out_t.data_ptr(), int(kblock), ws.data_ptr(), stream)
        assert rc == 0, lib.f8mi_last_error()
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before  # nothing asked of torch's allocator either
        torch.cuda.synchronize()
        res.append((scale.cpu(), out.cpu(), out_t.cpu()))
    return res


@pytest.mark.parametrize("dtype,f8,kblock", [(torch.bfloat16, torch.float8_e4m3fn, True),
                                              (torch.bfloat16, torch.float8_e5m2, False),
                                              (torch.float32, torch.float8_e4m3fn, False)])
def test_static_entry_point_matches_the_workspace_one_twice_in_a_row(native, dtype, f8, kblock):
    torch.manual_seed(5)
    # first call: 512 workgroups' worth of data (every word of the static array that a dense pass can use is written)
    big = (torch.randn(4096, 8192, device=DEV) * 37.0).to(dtype)
    # second call: smaller, and with a smaller maximum; rows a multiple of 64 for the k-blocked transpose
    small = (torch.randn(192, 1024, device=DEV) * 0.02).to(dtype)
    for x in (big, small):
        (s0, o0, t0), (s1, o1, t1) = _both(native, x, f8, kblock)
        want = (x.abs().max().to(dtype).clamp(min=1e-12).reciprocal() * torch.finfo(f8).max).float().cpu()
        assert s0.item() == want.item(), (s0.item(), want.item())
        assert s1.item() == s0.item(), (s1.item(), s0.item(), tuple(x.shape))
        assert torch.equal(o1, o0) and torch.equal(t1, t0), tuple(x.shape)
        assert int(o0.count_nonzero()) > 0.5 * o0.numel()  # and the bytes are an actual cast, not the zero fill


def test_static_entry_point_small_tensor_and_strided_rows(native):
    """The one-workgroup path (<= 32 K elements) and a row stride larger than the row."""
    torch.manual_seed(6)
    base = torch.randn(300, 520, device=DEV).to(torch.bfloat16)
    for x in (base[:40, :512], base[:, :512]):
        (s0, o0, t0), (s1, o1, t1) = _both(native, x, torch.float8_e4m3fn, False)
        assert s1.item() == s0.item() and torch.equal(o1, o0) and torch.equal(t1, t0)


def test_static_entry_point_refuses_what_it_cannot_take(native):
    lib = native.lib()
    i64 = C.c_int64
    one = torch.zeros(1, dtype=torch.float32, device=DEV)
    rc = lib.f8mi_cast_dynamic_static(C.c_void_p(16), i64(1 << 20), i64(1 << 20), i64(1 << 20), 0, 0, one.data_ptr(),
                                      C.c_void_p(16), 0, None, 0, None)
    assert rc == -1 and b"at most" in lib.f8mi_last_error()
    rc = lib.f8mi_cast_dynamic_static(C.c_void_p(16), i64(4), i64(4), i64(4), 0, 0, None, C.c_void_p(16), 0, None, 0, None)
    assert rc == -1 and b"scale" in lib.f8mi_last_error()


def test_static_entry_point_captured_in_a_graph_and_replayed(native):
    """The use the entry point is for: captured into a HIP graph (after one ordinary call on the device, which looks
    the array's address up) and replayed on new contents of the same input buffer -- every replay against
    f8mi_cast_dynamic on the same contents, with eager work and synchronisation between the replays."""
    lib = native.lib()
    torch.manual_seed(7)
    rows, cols = 1024, 2048
    x = torch.randn(rows, cols, device=DEV).to(torch.bfloat16)
    scale = torch.zeros(1, dtype=torch.float32, device=DEV)
    out = torch.zeros(rows * cols, dtype=torch.uint8, device=DEV)
    out_t = torch.zeros(rows * cols, dtype=torch.uint8, device=DEV)
    ws = torch.zeros(lib.f8mi_workspace_bytes() // 4, dtype=torch.int32, device=DEV)

    def static_call(stream):
        rc = lib.f8mi_cast_dynamic_static(x.data_ptr(), rows, cols, cols, 0, 0, scale.data_ptr(), out.data_ptr(), 1, out_t.data_ptr(), 1, stream)
        assert rc == 0, lib.f8mi_last_error()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        static_call(side.cuda_stream)            # the warm-up call, outside any capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_call(torch.cuda.current_stream().cuda_stream)
    for i in range(4):
        x.copy_((torch.randn(rows, cols, device=DEV) * (0.01 * 10.0 ** i)).to(torch.bfloat16))   # eager work between replays
        out.zero_()
        out_t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        s_ref = torch.zeros(1, dtype=torch.float32, device=DEV)
        o_ref, t_ref = torch.zeros_like(out), torch.zeros_like(out_t)
        rc = lib.f8mi_cast_dynamic(x.data_ptr(), rows, cols, cols, 0, 0, s_ref.data_ptr(), o_ref.data_ptr(), 1, t_ref.data_ptr(), 1,
                                   ws.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        assert scale.item() == s_ref.item(), (i, scale.item(), s_ref.item())
        assert torch.equal(out, o_ref) and torch.equal(out_t, t_ref), i
