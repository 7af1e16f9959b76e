"""ctypes binding of ``libf8mi.so`` (the C ABI declared in ``include/f8mi.h``).

Torch is used here for device memory and streams only: every function takes
torch tensors, checks them on the host, and hands raw device pointers plus the
current HIP stream to the library.  There is no fallback: if the library is
missing, cannot be loaded, or the tensors are not on a GPU, the call raises.
"""
import ctypes as C
import os
import threading
from typing import Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# F8MI_LIB names another build of the library (same ABI) to load instead of the in-tree one: a switch for measurements
# (tile walks, cache policies).  Such a build says so through f8mi_build_knobs() and is refused unless
# F8MI_ALLOW_MEASUREMENT_BUILD=1 is set as well.
LIB_PATH = os.environ.get("F8MI_LIB") or os.path.join(_HERE, "libf8mi.so")

BF16, FP16, FP32 = 0, 1, 2
E4M3FN, E5M2 = 0, 1
K_AMAX, K_CAST, K_GEMM, K_SYNC = 0, 1, 2, 3

_DT = {torch.bfloat16: BF16, torch.float16: FP16, torch.float32: FP32}
_F8 = {torch.float8_e4m3fn: E4M3FN, torch.float8_e5m2: E5M2}

EXPORTS = (
    "f8mi_version",
    "f8mi_last_error",
    "f8mi_build_knobs",
    "f8mi_padded_k",
    "f8mi_device_info",
    "f8mi_workspace_bytes",
    "f8mi_gemm_nt_ws",
    "f8mi_gemm_nt_kb_ws",
    "f8mi_gemm_plan",
    "f8mi_amax_scale",
    "f8mi_amax_scale_multi",
    "f8mi_amax_tile_elems",
    "f8mi_cast",
    "f8mi_cast_layout",
    "f8mi_cast_delayed",
    "f8mi_delayed_workspace_bytes",
    "f8mi_cast_dynamic",
    "f8mi_cast_dynamic_static",
    "f8mi_gemm_nt",
    "f8mi_gemm_nt_kb",
    "f8mi_gemm_kb_ex",
    "f8mi_gemm_ex",
    "f8mi_sync",
    "f8mi_sync_host",
    "f8mi_delayed_init",
    "f8mi_prof_enable",
    "f8mi_prof_reset",
    "f8mi_prof_read",
)

_lib = None
_lock = threading.Lock()


class Float8NativeError(RuntimeError):
    pass


def lib() -> C.CDLL:
    """Loads libf8mi.so once.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise Float8NativeError(
                f"{LIB_PATH} not found: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(or `python float8_experimental_amd/_build.py`); there is no fallback path"
            )
        L = C.CDLL(LIB_PATH)
        vp, i64, i32, fp = C.c_void_p, C.c_int64, C.c_int, C.c_void_p
        L.f8mi_version.restype = i32
        L.f8mi_version.argtypes = []
        L.f8mi_last_error.restype = C.c_char_p
        L.f8mi_last_error.argtypes = []
        L.f8mi_build_knobs.restype = C.c_char_p
        L.f8mi_build_knobs.argtypes = []
        L.f8mi_padded_k.restype = i64
        L.f8mi_padded_k.argtypes = [i64]
        L.f8mi_device_info.restype = i32
        L.f8mi_device_info.argtypes = [i32, C.POINTER(i32), C.POINTER(i32), C.c_char_p, i32]
        L.f8mi_workspace_bytes.restype = C.c_size_t
        L.f8mi_workspace_bytes.argtypes = []
        L.f8mi_amax_scale.restype = i32
        L.f8mi_amax_scale.argtypes = [vp, i64, i64, i64, i32, i32, i32, i32, fp, fp, vp, vp]
        L.f8mi_amax_scale_multi.restype = i32
        L.f8mi_amax_scale_multi.argtypes = [vp, i32, i64, i32, i32, i32, i32, fp, fp, vp, vp]
        L.f8mi_amax_tile_elems.restype = i64
        L.f8mi_amax_tile_elems.argtypes = [i32]
        L.f8mi_cast.restype = i32
        L.f8mi_cast.argtypes = [vp, i64, i64, i64, i32, fp, i32, i32, vp, vp, fp, vp, vp]
        L.f8mi_cast_layout.restype = i32
        L.f8mi_cast_layout.argtypes = [vp, i64, i64, i64, i32, fp, i32, i32, vp, i32, vp, i32, fp, vp]
        L.f8mi_delayed_workspace_bytes.restype = C.c_size_t
        L.f8mi_delayed_workspace_bytes.argtypes = []
        L.f8mi_cast_delayed.restype = i32
        L.f8mi_cast_delayed.argtypes = [vp, i64, i64, i64, i32, fp, i32, vp, i32, vp, i32, fp, vp, vp]
        L.f8mi_cast_dynamic.restype = i32
        L.f8mi_cast_dynamic.argtypes = [vp, i64, i64, i64, i32, i32, fp, vp, i32, vp, i32, vp, vp]
        L.f8mi_cast_dynamic_static.restype = i32
        L.f8mi_cast_dynamic_static.argtypes = [vp, i64, i64, i64, i32, i32, fp, vp, i32, vp, i32, vp]
        L.f8mi_gemm_nt_kb.restype = i32
        L.f8mi_gemm_nt_kb.argtypes = [vp, i32, vp, i32, i64, i64, i64, fp, fp, vp, i32, i64, vp, vp]
        L.f8mi_gemm_kb_ex.restype = i32
        L.f8mi_gemm_kb_ex.argtypes = [vp, i32, i32, vp, i32, i32, i64, i64, i64, fp, fp, vp, i32, i64, vp, vp]
        L.f8mi_gemm_ex.restype = i32
        L.f8mi_gemm_ex.argtypes = [vp, i32, i32, i64, vp, i32, i32, i64, i64, i64, i64, fp, fp, vp, i32, i64, vp, vp]
        L.f8mi_gemm_nt.restype = i32
        L.f8mi_gemm_nt.argtypes = [vp, i32, i64, vp, i32, i64, i64, i64, i64, fp, fp, vp, i32, i64, vp, vp]
        L.f8mi_gemm_nt_ws.restype = i32
        L.f8mi_gemm_nt_ws.argtypes = [vp, i32, i64, vp, i32, i64, i64, i64, i64, fp, fp, vp, i32, i64, vp, vp, i64, vp]
        L.f8mi_gemm_plan.restype = i32
        L.f8mi_gemm_plan.argtypes = [i64, i64, i64, i32, i64]
        L.f8mi_gemm_nt_kb_ws.restype = i32
        L.f8mi_gemm_nt_kb_ws.argtypes = [vp, i32, vp, i32, i64, i64, i64, fp, fp, vp, i32, i64, vp, vp, i64, vp]
        L.f8mi_sync.restype = i32
        L.f8mi_sync.argtypes = [vp, i32, i32, i32, i32, vp]
        L.f8mi_sync_host.restype = i32
        L.f8mi_sync_host.argtypes = [vp, i32, i32, i32, i32, vp]
        L.f8mi_delayed_init.restype = i32
        L.f8mi_delayed_init.argtypes = [fp, fp, fp, i32, i32, i32, vp]
        L.f8mi_prof_enable.restype = i32
        L.f8mi_prof_enable.argtypes = [i32]
        L.f8mi_prof_reset.restype = i32
        L.f8mi_prof_reset.argtypes = []
        L.f8mi_prof_read.restype = i32
        L.f8mi_prof_read.argtypes = [i32, C.POINTER(C.c_uint64), C.POINTER(C.c_double), C.POINTER(C.c_double)]
        knobs = L.f8mi_build_knobs().decode()
        if knobs and os.environ.get("F8MI_ALLOW_MEASUREMENT_BUILD") != "1":
            raise Float8NativeError(
                f"{LIB_PATH} is a measurement build ({knobs}), not the library as shipped; set "
                "F8MI_ALLOW_MEASUREMENT_BUILD=1 to load it anyway")
        _lib = L
    return _lib


def build_knobs() -> str:
    """Measurement knobs the loaded library was compiled with ("" for the shipped build).  See f8mi_build_knobs."""
    return lib().f8mi_build_knobs().decode()


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().f8mi_last_error().decode(errors="replace")
        raise Float8NativeError(f"{what} failed with code {rc}: {msg}")


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise Float8NativeError(
            f"{name} is on {t.device}: float8_experimental_amd computes on MI355X device tensors only "
            "(no CPU fallback)"
        )
    if t.device.index is not None and t.device.index != torch.cuda.current_device():
        # the library launches on the tensor's stream with whatever device is current: one process per GPU, or
        # `with torch.cuda.device(t.device):` around the call, keeps the two the same
        raise Float8NativeError(f"{name} is on {t.device} but the current device is cuda:{torch.cuda.current_device()}: "
                                "make the tensor's device current (torch.cuda.set_device / torch.cuda.device)")


def _raw_stream(dev: torch.device) -> int:
    """hipStream_t of torch's current stream on ``dev`` as an integer (the raw accessor: no Stream object is built)."""
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(idx)


def _stream(t: torch.Tensor) -> int:
    return _raw_stream(t.device)


_checked_devices = set()


def _check_device(dev: torch.device) -> None:
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    if idx in _checked_devices:
        return
    arch = C.create_string_buffer(64)
    cu, lds = C.c_int(0), C.c_int(0)
    _check(lib().f8mi_device_info(idx, C.byref(cu), C.byref(lds), arch, 64), "f8mi_device_info")
    _checked_devices.add(idx)


_workspaces = {}
_tls = threading.local()


class transient_workspaces:
    """While active (per thread), ``workspace`` and ``gemm_workspace`` hand out fresh tensors instead of the cached
    per-(device, stream) ones.  The custom ops that ``torch.compile`` calls run under it: a node of a compiled graph must
    not leave a tensor of its own behind in the graph's memory pool (``mode="reduce-overhead"`` checks that), while a
    temporary that dies with the call is fine -- the allocator hands its memory out again in stream order."""

    def __enter__(self):
        self.prev = getattr(_tls, "transient", False)
        _tls.transient = True

    def __exit__(self, *exc):
        _tls.transient = self.prev
        if not self.prev:
            _tls.gemm_ws = None  # the kernels that use it are already queued; its memory is reused in stream order


def workspace(dev: torch.device) -> torch.Tensor:
    """Reduction workspace of f8mi_amax_scale (per-block partial maxima), one per (device, stream)."""
    _check_device(dev)
    if getattr(_tls, "transient", False):
        return torch.empty(lib().f8mi_workspace_bytes() // 4, dtype=torch.int32, device=dev)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), _raw_stream(dev))
    ws = _workspaces.get(key)
    if ws is None:
        ws = torch.zeros(lib().f8mi_workspace_bytes() // 4, dtype=torch.int32, device=dev)
        _workspaces[key] = ws
    return ws


_delayed_workspaces = {}


def delayed_workspace(dev: torch.device) -> torch.Tensor:
    """The zeroed words f8mi_cast_delayed folds the amax into (and leaves zeroed), one per (device, stream)."""
    _check_device(dev)
    words = lib().f8mi_delayed_workspace_bytes() // 4
    if getattr(_tls, "transient", False):
        return torch.zeros(words, dtype=torch.int32, device=dev)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), _raw_stream(dev))
    ws = _delayed_workspaces.get(key)
    if ws is None:
        ws = torch.zeros(words, dtype=torch.int32, device=dev)
        # under stream capture the fill is recorded, not run: such a tensor is zero only inside replays of that graph,
        # so it serves this call and is not kept for later, eager calls on a stream with the same handle
        if not torch.cuda.is_current_stream_capturing():
            _delayed_workspaces[key] = ws
    return ws


GEMM_WORKSPACE_BYTES = 32 << 20  # F8MI_GEMM_WORKSPACE_BYTES
_GEMM_WS_MIN_ROWS, _GEMM_WS_MIN_K = 17, 2048  # below these no GEMM is ever split over k
_gemm_workspaces = {}


def gemm_workspace(dev: torch.device, m: int, k: int, n: int = 0):
    """(pointer, bytes) of the scratch that lets a few-row GEMM with a long contraction split k over workgroups; one
    allocation per (device, stream), made the first time a shape that could use it comes by; (None, 0) for shapes
    that never do."""
    if m < _GEMM_WS_MIN_ROWS or k < _GEMM_WS_MIN_K:
        return None, 0
    if getattr(_tls, "transient", False):
        # a temporary, and only for a product the library would actually split over k
        if (lib().f8mi_gemm_plan(m, n, k, 1, GEMM_WORKSPACE_BYTES) & 0xff) != 1:
            return None, 0
        _tls.gemm_ws = torch.empty(GEMM_WORKSPACE_BYTES // 4, dtype=torch.float32, device=dev)
        return _tls.gemm_ws.data_ptr(), GEMM_WORKSPACE_BYTES
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), _raw_stream(dev))
    ws = _gemm_workspaces.get(key)
    if ws is None:
        ws = _gemm_workspaces[key] = torch.empty(GEMM_WORKSPACE_BYTES // 4, dtype=torch.float32, device=dev)
    return ws.data_ptr(), GEMM_WORKSPACE_BYTES


PLAN_NAMES = {1: "tiles128_split_k", 2: "few_rows", 3: "tiles128", 4: "tiles256", 5: "tiles256_and_128", 6: "tiles256_mfma32",
              7: "staged"}


def gemm_plan(m: int, n: int, k: int, aligned: bool = True, split_k: bool = True):
    """(kernel name, parts of k, 0 / 1 / 2 for none / 128 x 128 / 128 x 256 tiles) the library picks for an m x n x k
    product, as gemm_nt / gemm_nt_kb call it (``split_k``: with the scratch buffer they pass).  Needs no GPU."""
    ws = GEMM_WORKSPACE_BYTES if split_k and m >= _GEMM_WS_MIN_ROWS and k >= _GEMM_WS_MIN_K else 0
    code = lib().f8mi_gemm_plan(m, n, k, int(aligned), ws)
    return PLAN_NAMES.get(code & 0xff), (code >> 8) & 0xff, (code >> 16) & 0xff


def _as_2d(x: torch.Tensor) -> Tuple[torch.Tensor, int, int, int]:
    """(tensor whose memory is read, rows, cols, row stride) -- copies only when the layout needs it.  A tensor
    expanded over all its leading dimensions (what autograd hands to backward after ``y.sum()``) is passed as ONE row
    with row stride 0: the kernels read that row for every output row, nothing of rows x cols is materialised."""
    if x.dim() == 2 and x.stride(1) == 1 and x.stride(0) >= x.shape[1] and x.shape[0] > 0 and x.shape[1] > 0:
        return x, x.shape[0], x.shape[1], x.stride(0)
    if x.dim() >= 2 and x.shape[-1] > 0 and x.numel() > x.shape[-1] and all(
            st == 0 or sz == 1 for st, sz in zip(x.stride()[:-1], x.shape[:-1])):
        row = x[(0,) * (x.dim() - 1)].contiguous()
        return row, x.numel() // x.shape[-1], x.shape[-1], 0
    if not x.is_contiguous():
        x = x.contiguous()
    cols = x.shape[-1] if x.dim() > 0 else 1
    rows = x.numel() // cols if cols else 0
    return x, rows, cols, cols


def amax_scale(x: torch.Tensor, float8_dtype: torch.dtype, math_dtype: Optional[torch.dtype] = None,
               orig_is_fp16: Optional[bool] = None, want_amax: bool = True, want_scale: bool = True,
               amax_out: Optional[torch.Tensor] = None, scale_out: Optional[torch.Tensor] = None):
    """max|x| (fp32, 0-dim) and its fp8 scale (fp32, 0-dim) in one pass.  See f8mi_amax_scale."""
    _require_gpu(x, "x")
    xs, rows, cols, ld = _as_2d(x)
    if math_dtype is None:
        math_dtype = x.dtype
    if orig_is_fp16 is None:
        orig_is_fp16 = x.dtype == torch.float16
    amax = amax_out if amax_out is not None else (torch.empty((), dtype=torch.float32, device=x.device) if want_amax else None)
    scale = scale_out if scale_out is not None else (torch.empty((), dtype=torch.float32, device=x.device) if want_scale else None)
    for o in (amax, scale):
        if o is not None:
            assert o.dtype == torch.float32 and o.numel() == 1 and o.device == x.device
    ws = workspace(x.device)
    rc = lib().f8mi_amax_scale(xs.data_ptr(), rows, cols, ld, _DT[x.dtype], _F8[float8_dtype], _DT[math_dtype],
                               int(orig_is_fp16), amax.data_ptr() if amax is not None else None,
                               scale.data_ptr() if scale is not None else None, ws.data_ptr(), _stream(x))
    _check(rc, "f8mi_amax_scale")
    return amax, scale


_multi_tables = {}


def amax_scale_multi(tensors, float8_dtype: torch.dtype, math_dtype: Optional[torch.dtype] = None,
                     orig_is_fp16: Optional[bool] = None):
    """(amaxes [n] fp32, scales [n] fp32) of n dense tensors of one dtype on one device, in three launches
    whatever n is.  See f8mi_amax_scale_multi.  The device table of (pointer, numel, first tile) rows is kept
    for as long as the same tensors (same storage, same sizes) are passed again."""
    tensors = list(tensors)
    assert tensors, "no tensors"
    x0 = tensors[0]
    for t in tensors:
        _require_gpu(t, "tensor")
        assert t.dtype == x0.dtype and t.device == x0.device, "tensors must share dtype and device"
        assert t.is_contiguous() and t.data_ptr() % 16 == 0, "tensors must be dense and 16-byte aligned"
    if math_dtype is None:
        math_dtype = x0.dtype
    if orig_is_fp16 is None:
        orig_is_fp16 = x0.dtype == torch.float16
    L = lib()
    limit = L.f8mi_workspace_bytes() // 4
    tile = L.f8mi_amax_tile_elems(_DT[x0.dtype])
    amaxes = torch.empty(len(tensors), dtype=torch.float32, device=x0.device)
    scales = torch.empty(len(tensors), dtype=torch.float32, device=x0.device)
    ws = workspace(x0.device)
    for lo in range(0, len(tensors), limit):
        part = tensors[lo:lo + limit]
        key = (x0.device.index, x0.dtype) + tuple((t.data_ptr(), t.numel()) for t in part)
        hit = _multi_tables.get(key)
        if hit is None:
            rows, first = [], 0
            for t in part:
                rows.append([t.data_ptr(), t.numel(), first])
                first += t.numel() // tile + 1
            if len(_multi_tables) > 64:
                _multi_tables.clear()
            hit = (torch.tensor(rows, dtype=torch.int64, device="cpu").to(x0.device), first)
            _multi_tables[key] = hit
        table, total_tiles = hit
        rc = L.f8mi_amax_scale_multi(table.data_ptr(), len(part), total_tiles, _DT[x0.dtype], _F8[float8_dtype],
                                     _DT[math_dtype], int(orig_is_fp16), amaxes[lo:].data_ptr(), scales[lo:].data_ptr(),
                                     ws.data_ptr(), _stream(x0))
        _check(rc, "f8mi_amax_scale_multi")
    return amaxes, scales


KB = 64          # depth of one block of the k-blocked operand layout
KB_MIN_K = 384   # shortest contraction the k-blocked GEMM takes
ROWMAJOR, KBLOCK, KBLOCK_PAD = 0, 1, 2  # F8MI_LAYOUT_ROWMAJOR / _KBLOCK64 / _KBLOCK64_PAD128


def padded_k(k: int) -> int:
    """Contraction length of a zero-padded k-blocked operand: k rounded up to a multiple of 128 (f8mi_padded_k)."""
    return -(-k // 128) * 128 if k > 0 else 0


def kblock_layout(k: int) -> int:
    """Layout code of the fp8 copies that a GEMM contracting over k reads fastest: k-blocked as it is when k is a
    multiple of 64 (and at least 384), k-blocked with the contraction zero-padded to a multiple of 128 for any other k
    that reaches 384 that way (a ragged layer: zeros add nothing to the product, which is the reference's own argument
    for pad_tensor_for_matmul, float8_utils.py:206-247), row-major for a short contraction."""
    if k % KB == 0 and k >= KB_MIN_K:
        return KBLOCK
    return KBLOCK_PAD if padded_k(k) >= KB_MIN_K else ROWMAJOR


def linear_route(m: int, k: int, n: int):
    """How the fused Float8Linear computes a layer of m tokens, k in_features, n out_features (needs no GPU):
    {"one_copy": bool, product: (operand layout code, contraction length the GEMM runs over, kernel plan)} for the
    products "output" (m x n over k), "grad_input" (m x k over n) and "grad_weight" (n x k over m)."""
    route = {"one_copy": tn_ok(m, k, n)}
    for name, (rows, cols, kc) in (("output", (m, n, k)), ("grad_input", (m, k, n)), ("grad_weight", (n, k, m))):
        layout = KBLOCK if route["one_copy"] else kblock_layout(kc)
        kc_run = padded_k(kc) if layout == KBLOCK_PAD else kc
        route[name] = (layout, kc_run, gemm_plan(rows, cols, kc_run, aligned=layout != ROWMAJOR or kc % 16 == 0))
    return route


def _kb_alloc(rows: int, kc: int, layout: int, float8_dtype, device) -> torch.Tensor:
    """Uninitialised k-blocked operand of ``rows`` rows contracting over ``kc``: [kc/64, rows, 64], kc padded for KBLOCK_PAD."""
    if layout == KBLOCK:
        assert kc % KB == 0, f"a k-blocked copy needs a contraction length that is a multiple of {KB}, got {kc} (use KBLOCK_PAD)"
    else:
        kc = padded_k(kc)
    return torch.empty((kc // KB, rows, KB), dtype=float8_dtype, device=device)


def tn_ok(m: int, k: int, n: int) -> bool:
    """True if a linear layer with m tokens, k in_features and n out_features should keep one k-blocked fp8 copy per
    tensor and let the backward GEMMs read it transposed (f8mi_gemm_kb_ex): every dimension a multiple of 128 and at
    least 384 -- and grad_input and grad_weight large enough for the 256 x 256-tile kernels, the only ones that read
    transposed operands (smaller outputs are faster from transposed copies through the 128 x 128-tile kernel)."""
    if not all(d % 128 == 0 and d >= KB_MIN_K for d in (m, k, n)):
        return False
    tiles = lambda rows, cols: -(-rows // 128) * -(-cols // 128)  # of 128 x 128: at most one per CU -> that kernel
    return tiles(m, k) > 256 and tiles(n, k) > 256


def kblock_ok(k: int) -> bool:
    """True if a contraction of length k can use the k-blocked layout ([k/64][rows][64], see f8mi.h)."""
    return k % KB == 0 and k >= KB_MIN_K


def cast(x: torch.Tensor, scale: torch.Tensor, float8_dtype: torch.dtype, product_dtype: Optional[torch.dtype] = None,
         want_out: bool = True, want_out_t: bool = False, amax_out: Optional[torch.Tensor] = None,
         out_kblock: int = 0, out_t_kblock: int = 0):
    """Saturated fp8 cast of a tensor viewed as [rows, cols=last dim].

    Returns (out, out_t): ``out`` has x's shape; ``out_t`` is the dense [cols, rows]
    transpose of the flattened 2-D view.  ``amax_out`` (fp32, 1 element), if given,
    receives max|x| computed in the same pass.  With ``out_kblock`` / ``out_t_kblock``
    the respective output is k-blocked instead: shape [cols/64, rows, 64] for ``out``
    (``out[b, r, j] == rowmajor[r, 64*b + j]``), [rows/64, cols, 64] for ``out_t``; the value
    ``KBLOCK_PAD`` (2) instead of True pads the contraction with zero bytes to a multiple of 128 first
    (any shape: [padded_k(cols)/64, rows, 64] and [padded_k(rows)/64, cols, 64]).
    See f8mi_cast / f8mi_cast_layout.
    """
    _require_gpu(x, "x")
    assert scale.dtype == torch.float32 and scale.numel() == 1 and scale.device == x.device, "scale: 1 fp32 element on x's device"
    xs, rows, cols, ld = _as_2d(x)
    if product_dtype is None:
        product_dtype = x.dtype
    out = out_t = None
    if want_out:
        out = _kb_alloc(rows, cols, int(out_kblock), float8_dtype, x.device) if out_kblock else torch.empty(x.shape, dtype=float8_dtype, device=x.device)
    if want_out_t:
        out_t = _kb_alloc(cols, rows, int(out_t_kblock), float8_dtype, x.device) if out_t_kblock else torch.empty((cols, rows), dtype=float8_dtype, device=x.device)
    if amax_out is not None:
        assert amax_out.dtype == torch.float32 and amax_out.numel() == 1 and amax_out.device == x.device
    _check_device(x.device)
    if rows * cols == 0:  # nothing to convert (an empty batch); torch hands out null pointers for empty tensors
        if amax_out is not None:
            amax_out.zero_()
        return out, out_t
    if amax_out is not None and product_dtype == torch.float32:  # the delayed-scaling cast
        rc = lib().f8mi_cast_delayed(xs.data_ptr(), rows, cols, ld, _DT[x.dtype], scale.data_ptr(), _F8[float8_dtype],
                                     out.data_ptr() if out is not None else None, int(out_kblock),
                                     out_t.data_ptr() if out_t is not None else None, int(out_t_kblock),
                                     amax_out.data_ptr(), delayed_workspace(x.device).data_ptr(), _stream(x))
        _check(rc, "f8mi_cast_delayed")
        return out, out_t
    rc = lib().f8mi_cast_layout(xs.data_ptr(), rows, cols, ld, _DT[x.dtype], scale.data_ptr(), _DT[product_dtype],
                                _F8[float8_dtype], out.data_ptr() if out is not None else None, int(out_kblock),
                                out_t.data_ptr() if out_t is not None else None, int(out_t_kblock),
                                amax_out.data_ptr() if amax_out is not None else None, _stream(x))
    _check(rc, "f8mi_cast_layout")
    return out, out_t


def cast_dynamic(x: torch.Tensor, float8_dtype: torch.dtype, want_out: bool = True, want_out_t: bool = False,
                 out_kblock: int = 0, out_t_kblock: int = 0):
    """(out, out_t, scale): ``amax_scale`` in x's dtype followed by ``cast`` with that scale, as one library call
    (hp_tensor_to_float8_dynamic of the reference); small tensors take a single launch.  See f8mi_cast_dynamic."""
    _require_gpu(x, "x")
    xs, rows, cols, ld = _as_2d(x)
    scale = torch.empty((), dtype=torch.float32, device=x.device)
    out = out_t = None
    if want_out:
        out = _kb_alloc(rows, cols, int(out_kblock), float8_dtype, x.device) if out_kblock else torch.empty(x.shape, dtype=float8_dtype, device=x.device)
    if want_out_t:
        out_t = _kb_alloc(cols, rows, int(out_t_kblock), float8_dtype, x.device) if out_t_kblock else torch.empty((cols, rows), dtype=float8_dtype, device=x.device)
    ws = workspace(x.device)
    empty = rows * cols == 0  # torch hands out null pointers for empty tensors: only the scale is computed
    rc = lib().f8mi_cast_dynamic(xs.data_ptr() if not empty else None, rows, cols, ld, _DT[x.dtype], _F8[float8_dtype],
                                 scale.data_ptr(), out.data_ptr() if out is not None and not empty else None, int(out_kblock),
                                 out_t.data_ptr() if out_t is not None and not empty else None, int(out_t_kblock),
                                 ws.data_ptr(), _stream(x))
    _check(rc, "f8mi_cast_dynamic")
    return out, out_t, scale


def cast_dynamic_static(x: torch.Tensor, scale_out: torch.Tensor, out: Optional[torch.Tensor] = None,
                        out_t: Optional[torch.Tensor] = None, out_kblock: int = 0, out_t_kblock: int = 0) -> None:
    """``cast_dynamic`` into tensors the caller already holds, through the library's own static scratch: this
    function and the library call behind it allocate nothing (see f8mi_cast_dynamic_static).  ``x`` must be a 2-D
    view with unit column stride; ``out`` / ``out_t`` are fp8 tensors of rows*cols elements, ``scale_out`` one fp32
    element.  Calls on one GPU must not overlap in time."""
    _require_gpu(x, "x")
    assert x.dim() == 2 and x.stride(1) == 1 and x.stride(0) >= x.shape[1], "x: 2-D with unit column stride (no copy is made here)"
    rows, cols = x.shape
    assert out is not None or out_t is not None, "no output requested"
    f8 = (out if out is not None else out_t).dtype
    for o in (out, out_t):
        if o is not None:
            assert o.dtype == f8 and o.dtype in _F8 and o.numel() == rows * cols and o.is_contiguous() and o.device == x.device
    assert scale_out.dtype == torch.float32 and scale_out.numel() == 1 and scale_out.device == x.device
    _check_device(x.device)
    rc = lib().f8mi_cast_dynamic_static(x.data_ptr(), rows, cols, x.stride(0), _DT[x.dtype], _F8[f8], scale_out.data_ptr(),
                                        out.data_ptr() if out is not None else None, int(out_kblock),
                                        out_t.data_ptr() if out_t is not None else None, int(out_t_kblock), _stream(x))
    _check(rc, "f8mi_cast_dynamic_static")


def gemm_nt_kb(a_kb: torch.Tensor, a_scale: torch.Tensor, bt_kb: torch.Tensor, b_scale: torch.Tensor,
               out_dtype: torch.dtype, bias: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
               split_k: bool = True) -> torch.Tensor:
    """gemm_nt on k-blocked operands: ``a_kb`` fp8 [k/64, m, 64], ``bt_kb`` fp8 [k/64, n, 64], both contiguous.

    Same result bits as gemm_nt on the row-major operands (with the same ``split_k``).  See f8mi_gemm_nt_kb_ws.
    """
    _require_gpu(a_kb, "a_kb")
    _require_gpu(bt_kb, "bt_kb")
    assert a_kb.dim() == 3 and bt_kb.dim() == 3 and a_kb.shape[2] == KB and bt_kb.shape[2] == KB and a_kb.shape[0] == bt_kb.shape[0], \
        f"k-blocked operands are [k/64, rows, 64], got {tuple(a_kb.shape)} and {tuple(bt_kb.shape)}"
    assert a_kb.is_contiguous() and bt_kb.is_contiguous(), "k-blocked operands must be contiguous"
    assert a_kb.dtype in _F8 and bt_kb.dtype in _F8, "operands must be float8_e4m3fn / float8_e5m2"
    m, n, k = a_kb.shape[1], bt_kb.shape[1], a_kb.shape[0] * KB
    for s in (a_scale, b_scale):
        assert s.dtype == torch.float32 and s.numel() == 1 and s.device == a_kb.device, "scales: 1 fp32 element on the operands' device"
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=a_kb.device)
    else:
        assert out.shape == (m, n) and out.dtype == out_dtype and out.is_contiguous()
    if bias is not None:
        assert bias.dtype == out_dtype and bias.numel() == n and bias.is_contiguous() and bias.device == a_kb.device
    _check_device(a_kb.device)
    ws, ws_bytes = gemm_workspace(a_kb.device, m, k, n) if split_k else (None, 0)
    rc = lib().f8mi_gemm_nt_kb_ws(a_kb.data_ptr(), _F8[a_kb.dtype], bt_kb.data_ptr(), _F8[bt_kb.dtype], m, n, k,
                                  a_scale.data_ptr(), b_scale.data_ptr(), out.data_ptr(), _DT[out_dtype], max(n, 1),
                                  bias.data_ptr() if bias is not None else None, ws, ws_bytes, _stream(a_kb))
    _check(rc, "f8mi_gemm_nt_kb_ws")
    return out


def gemm_kb_ex(a_kb: torch.Tensor, a_transposed: bool, a_scale: torch.Tensor, bt_kb: torch.Tensor, b_transposed: bool,
               b_scale: torch.Tensor, out_dtype: torch.dtype, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """gemm_nt_kb whose operands may be given transposed (see f8mi_gemm_kb_ex).

    ``a_kb`` is [k/64, m, 64] (not transposed) or [m/64, k, 64] (transposed: the k-blocked copy of the [k, m]
    matrix, as the GEMM that contracts over m holds it); ``bt_kb`` likewise with n."""
    _require_gpu(a_kb, "a_kb")
    _require_gpu(bt_kb, "bt_kb")
    for t in (a_kb, bt_kb):
        assert t.dim() == 3 and t.shape[2] == KB and t.is_contiguous() and t.dtype in _F8, "k-blocked fp8 operands are contiguous [x/64, y, 64]"
    m, k = (a_kb.shape[0] * KB, a_kb.shape[1]) if a_transposed else (a_kb.shape[1], a_kb.shape[0] * KB)
    n, k2 = (bt_kb.shape[0] * KB, bt_kb.shape[1]) if b_transposed else (bt_kb.shape[1], bt_kb.shape[0] * KB)
    assert k == k2, f"contraction lengths differ: {k} and {k2}"
    for s in (a_scale, b_scale):
        assert s.dtype == torch.float32 and s.numel() == 1 and s.device == a_kb.device, "scales: 1 fp32 element on the operands' device"
    out = torch.empty((m, n), dtype=out_dtype, device=a_kb.device)
    if bias is not None:
        assert bias.dtype == out_dtype and bias.numel() == n and bias.is_contiguous() and bias.device == a_kb.device
    _check_device(a_kb.device)
    rc = lib().f8mi_gemm_kb_ex(a_kb.data_ptr(), _F8[a_kb.dtype], int(a_transposed), bt_kb.data_ptr(), _F8[bt_kb.dtype],
                               int(b_transposed), m, n, k, a_scale.data_ptr(), b_scale.data_ptr(), out.data_ptr(),
                               _DT[out_dtype], max(n, 1), bias.data_ptr() if bias is not None else None, _stream(a_kb))
    _check(rc, "f8mi_gemm_kb_ex")
    return out


def gemm_nt(a: torch.Tensor, a_scale: torch.Tensor, bt: torch.Tensor, b_scale: torch.Tensor, out_dtype: torch.dtype,
            bias: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None, split_k: bool = True) -> torch.Tensor:
    """out[m, n] = (a[m, :] . bt[n, :]) / (a_scale * b_scale) (+ bias[n]).

    ``a`` is fp8 [m, k], ``bt`` is fp8 [n, k]; both must have unit stride along k.  ``split_k``: hand the library
    this stream's scratch buffer, with which it may split a long contraction of a few-row product over workgroups
    (deterministic, but another summation order than without).  See f8mi_gemm_nt_ws.
    """
    _require_gpu(a, "a")
    _require_gpu(bt, "bt")
    assert a.dim() == 2 and bt.dim() == 2 and a.shape[1] == bt.shape[1], f"shape mismatch {tuple(a.shape)} x {tuple(bt.shape)}^T"
    assert a.dtype in _F8 and bt.dtype in _F8, "operands must be float8_e4m3fn / float8_e5m2"
    m, k = a.shape
    n = bt.shape[0]

    def rowmajor(t):
        if t.shape[1] <= 1 or t.stride(1) == 1:
            if t.shape[0] <= 1 or t.stride(0) >= max(t.shape[1], 1):
                return t, (t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1))
        t = t.view(torch.uint8).contiguous().view(t.dtype)  # byte copy: not every fp8 dtype has copy kernels
        return t, max(t.shape[1], 1)

    a, lda = rowmajor(a)
    bt, ldb = rowmajor(bt)
    lda, ldb = max(lda, k), max(ldb, k)
    for s in (a_scale, b_scale):
        assert s.dtype == torch.float32 and s.numel() == 1 and s.device == a.device, "scales: 1 fp32 element on the operands' device"
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    else:
        assert out.shape == (m, n) and out.dtype == out_dtype and out.is_contiguous()
    if bias is not None:
        assert bias.dtype == out_dtype and bias.numel() == n and bias.is_contiguous() and bias.device == a.device
    _check_device(a.device)
    ws, ws_bytes = gemm_workspace(a.device, m, k, n) if split_k else (None, 0)
    rc = lib().f8mi_gemm_nt_ws(a.data_ptr(), _F8[a.dtype], lda, bt.data_ptr(), _F8[bt.dtype], ldb, m, n, k,
                               a_scale.data_ptr(), b_scale.data_ptr(), out.data_ptr(), _DT[out_dtype], max(n, 1),
                               bias.data_ptr() if bias is not None else None, ws, ws_bytes, _stream(a))
    _check(rc, "f8mi_gemm_nt_ws")
    return out


ERR_UNSUPPORTED = -2  # F8MI_ERR_UNSUPPORTED


def scaled_mm(a: torch.Tensor, a_scale: torch.Tensor, b: torch.Tensor, b_scale: torch.Tensor, out_dtype: torch.dtype,
              bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``(a @ b) / (a_scale * b_scale) (+ bias)`` for fp8 ``a`` [m, k] and ``b`` [k, n] in ANY layout: what
    ``torch._scaled_mm`` computes, without its rule that ``a`` be row-major and ``b`` column-major.  Row-major ``b``
    (and column-major ``a`` next to it) are read transposed by the kernel where it can (f8mi_gemm_ex); where it
    cannot -- small or ragged products -- the operand is copied into the layout ``gemm_nt`` takes, which is the copy
    the reference always makes (float8_ops.py:150-153).  Same bits either way."""
    _require_gpu(a, "a")
    _require_gpu(b, "b")
    assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[0], f"shape mismatch {tuple(a.shape)} @ {tuple(b.shape)}"
    assert a.dtype in _F8 and b.dtype in _F8, "operands must be float8_e4m3fn / float8_e5m2"
    m, k = a.shape
    n = b.shape[1]
    unit = lambda t, d: t.shape[d] <= 1 or t.stride(d) == 1
    a_rowmajor = unit(a, 1) and (m <= 1 or a.stride(0) >= k)   # [m][k] in memory
    a_colmajor = unit(a, 0) and (k <= 1 or a.stride(1) >= m)   # [k][m] in memory
    b_colmajor = unit(b, 0) and (n <= 1 or b.stride(1) >= k)   # [n][k] in memory: gemm_nt's bt
    b_rowmajor = unit(b, 1) and (k <= 1 or b.stride(0) >= n)   # [k][n] in memory
    if a_rowmajor and b_colmajor:
        return gemm_nt(a, a_scale, b.t(), b_scale, out_dtype, bias=bias)
    if b_rowmajor and (a_rowmajor or a_colmajor) and m > 0 and n > 0 and k > 1 and n > 1 and (a_rowmajor or m > 1):
        for s in (a_scale, b_scale):
            assert s.dtype == torch.float32 and s.numel() == 1 and s.device == a.device, "scales: 1 fp32 element on the operands' device"
        if bias is not None:
            assert bias.dtype == out_dtype and bias.numel() == n and bias.is_contiguous() and bias.device == a.device
        _check_device(a.device)
        out = torch.empty((m, n), dtype=out_dtype, device=a.device)
        a_tr = not a_rowmajor
        lda = a.stride(1) if a_tr else (a.stride(0) if m > 1 else k)
        rc = lib().f8mi_gemm_ex(a.data_ptr(), _F8[a.dtype], int(a_tr), lda, b.data_ptr(), _F8[b.dtype], 1, b.stride(0), m, n, k,
                                a_scale.data_ptr(), b_scale.data_ptr(), out.data_ptr(), _DT[out_dtype], n,
                                bias.data_ptr() if bias is not None else None, _stream(a))
        if rc == 0:
            return out
        if rc != ERR_UNSUPPORTED:
            _check(rc, "f8mi_gemm_ex")
    # the copies: gemm_nt makes an operand contiguous along k when it is not
    return gemm_nt(a, a_scale, b.t(), b_scale, out_dtype, bias=bias)


def sync_table(entries, device: torch.device) -> torch.Tensor:
    """Device pointer table for f8mi_sync.  entries: iterable of (amax, history, scale, float8_dtype)."""
    rows = []
    for amax, hist, scale, f8 in entries:
        for t in (amax, hist, scale):
            _require_gpu(t, "buffer")
            assert t.dtype == torch.float32 and t.is_contiguous()
        rows.append([amax.data_ptr(), hist.data_ptr(), scale.data_ptr(), _F8[f8]])
    return torch.tensor(rows, dtype=torch.int64, device="cpu").to(device)


_sync_tables = {}


def sync_table_cached(entries) -> torch.Tensor:
    """``sync_table`` of the same buffers as last time without rebuilding it: the table is rebuilt only when a
    buffer has moved (``.to()``, ``load_state_dict`` into new storage, ...)."""
    entries = list(entries)
    key = tuple((a.data_ptr(), h.data_ptr(), s.data_ptr(), _F8[f8]) for a, h, s, f8 in entries)
    hit = _sync_tables.get(key)
    if hit is None:
        if len(_sync_tables) > 64:
            _sync_tables.clear()
        hit = _sync_tables[key] = sync_table(entries, entries[0][0].device)
    return hit


def sync(table: torch.Tensor, hist_len: int, orig_is_fp16: bool, writeback_history: bool = False) -> None:
    _require_gpu(table, "table")
    assert table.dtype == torch.int64 and table.dim() == 2 and table.shape[1] == 4 and table.is_contiguous()
    _check_device(table.device)
    rc = lib().f8mi_sync(table.data_ptr(), table.shape[0], hist_len, int(orig_is_fp16), int(writeback_history),
                         _stream(table))
    _check(rc, "f8mi_sync")


def sync_host(entries, hist_len: int, orig_is_fp16: bool, writeback_history: bool = False) -> None:
    """``sync`` without a device table: ``entries`` (iterable of (amax, history, scale, float8_dtype)) go to the GPU as
    kernel arguments.  Allocates no tensor, which is what a compiled graph with its own memory pool needs."""
    rows = []
    dev = None
    for amax, hist, scale, f8 in entries:
        for t in (amax, hist, scale):
            _require_gpu(t, "buffer")
            assert t.dtype == torch.float32 and t.is_contiguous()
        assert hist.numel() == hist_len
        rows += [amax.data_ptr(), hist.data_ptr(), scale.data_ptr(), _F8[f8]]
        dev = amax.device
    if not rows:
        return
    _check_device(dev)
    arr = (C.c_int64 * len(rows))(*rows)
    rc = lib().f8mi_sync_host(arr, len(rows) // 4, hist_len, int(orig_is_fp16), int(writeback_history), _raw_stream(dev))
    _check(rc, "f8mi_sync_host")


def delayed_init(amax: torch.Tensor, history: torch.Tensor, scale: torch.Tensor, float8_dtype: torch.dtype,
                 orig_is_fp16: bool) -> None:
    for t in (amax, history, scale):
        _require_gpu(t, "buffer")
        assert t.dtype == torch.float32 and t.is_contiguous()
    _check_device(amax.device)
    rc = lib().f8mi_delayed_init(amax.data_ptr(), history.data_ptr(), scale.data_ptr(), history.numel(),
                                 _F8[float8_dtype], int(orig_is_fp16), _stream(amax))
    _check(rc, "f8mi_delayed_init")


def prof_enable(on: bool) -> None:
    _check(lib().f8mi_prof_enable(int(on)), "f8mi_prof_enable")


def prof_reset() -> None:
    _check(lib().f8mi_prof_reset(), "f8mi_prof_reset")


def prof_read(kernel: int):
    n, ms, work = C.c_uint64(0), C.c_double(0), C.c_double(0)
    _check(lib().f8mi_prof_read(kernel, C.byref(n), C.byref(ms), C.byref(work)), "f8mi_prof_read")
    return n.value, ms.value, work.value
