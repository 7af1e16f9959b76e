"""The kernels as ``torch.library`` custom ops, so that ``torch.compile`` sees opaque nodes with known shapes
instead of tracing into the ctypes calls (which it cannot): the fused linear as one node per direction, and the
primitives the Float8Tensor-level API is made of -- amax + scale, the saturated cast, the scaled matmul -- as one
node each (``f8mi::amax_scale``, ``f8mi::cast``, ``f8mi::gemm_nt``), which is what lets code that produces or
consumes a ``Float8Tensor`` compile (graph inputs, graph outputs, breaks in the middle; reference
test/test_compile.py:173-254).

The reference keeps its float8 pieces traceable with ``torch._dynamo.allow_in_graph``
(float8_linear.py:43, float8_tensor.py:131,198) and lets inductor generate the casts; here the kernels
are hand-written, so the compiler only has to know shapes and dtypes (the fake implementations below) and how
gradients flow (``register_autograd``).  Each of the three tensors is scaled dynamically (no buffers passed)
or with the delayed-scaling buffers of the module: the cast then uses the existing scale and records this
step's amax.  The ops are functional (an op that writes its arguments cannot carry an autograd formula): they
return the new amax as a one-element tensor and the caller copies it into the module's buffer, an in-place
update of a buffer that the compiler knows how to trace.
What stays outside the graph (``torch._dynamo.disable`` on the module) is everything that keeps *Python* state:
the first-iteration amax initialisation and the pre/post-forward flags -- configure
``enable_amax_init=False, enable_pre_and_post_forward=False`` for a graph without breaks, as with the reference.
"""
from typing import List, Optional, Tuple

import torch

from . import _native

e4m3_dtype, e5m2_dtype = torch.float8_e4m3fn, torch.float8_e5m2  # as float8_utils (which imports this module)
_KB = _native.KB


# ---- the primitives ------------------------------------------------------------------------------------------

@torch.library.custom_op("f8mi::amax_scale", mutates_args=())
def amax_scale(x: torch.Tensor, float8_dtype: torch.dtype, math_dtype: torch.dtype, orig_is_fp16: bool) -> Tuple[
        torch.Tensor, torch.Tensor]:
    """(max|x|, fp8 scale of it), both 0-dim fp32, in one pass over x: ``tensor_to_amax`` + ``amax_to_scale`` of the
    reference (float8_utils.py:35-57, 102-120) with the scale arithmetic rounded to ``math_dtype``."""
    with _native.transient_workspaces():
        return _native.amax_scale(x, float8_dtype, math_dtype=math_dtype, orig_is_fp16=orig_is_fp16)


@amax_scale.register_fake
def _(x, float8_dtype, math_dtype, orig_is_fp16):
    return (torch.empty((), dtype=torch.float32, device=x.device), torch.empty((), dtype=torch.float32, device=x.device))


@torch.library.custom_op("f8mi::cast", mutates_args=())
def cast(x: torch.Tensor, scale: torch.Tensor, float8_dtype: torch.dtype, product_dtype: torch.dtype,
         want_amax: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """(fp8 bytes of clamp(x * scale) with x's shape, max|x| as [1] fp32 or an empty tensor): the saturated cast of
    the reference (float8_tensor.py:158-159, float8_utils.py:123-139), optionally with the amax pass of delayed
    scaling (float8_scaling_utils.py:89) folded in.  ``product_dtype``: what ``x * scale`` is rounded to."""
    amax = torch.empty(1 if want_amax else 0, dtype=torch.float32, device=x.device)
    with _native.transient_workspaces():
        bits, _ = _native.cast(x, scale, float8_dtype, product_dtype=product_dtype, amax_out=amax if want_amax else None)
    return bits, amax


@cast.register_fake
def _(x, scale, float8_dtype, product_dtype, want_amax):
    return (torch.empty(x.shape, dtype=float8_dtype, device=x.device),
            torch.empty(1 if want_amax else 0, dtype=torch.float32, device=x.device))


@torch.library.custom_op("f8mi::gemm_nt", mutates_args=())
def gemm_nt(a: torch.Tensor, a_scale: torch.Tensor, bt: torch.Tensor, b_scale: torch.Tensor, out_dtype: torch.dtype,
            bias: Optional[torch.Tensor]) -> torch.Tensor:
    """``(a @ bt^T) / (a_scale * b_scale) (+ bias)`` on the matrix cores: ``torch._scaled_mm`` as the reference calls it
    (float8_python_api.py:24-64), with the second operand given as [n, k]."""
    with _native.transient_workspaces():
        return _native.gemm_nt(a, a_scale, bt, b_scale, out_dtype, bias=bias)


@gemm_nt.register_fake
def _(a, a_scale, bt, b_scale, out_dtype, bias):
    return torch.empty((a.shape[0], bt.shape[0]), dtype=out_dtype, device=a.device)


@torch.library.custom_op("f8mi::scaled_mm", mutates_args=())
def scaled_mm(a: torch.Tensor, a_scale: torch.Tensor, b: torch.Tensor, b_scale: torch.Tensor, out_dtype: torch.dtype,
              bias: Optional[torch.Tensor]) -> torch.Tensor:
    """``(a @ b) / (a_scale * b_scale) (+ bias)`` for fp8 operands in whatever layout they have: ``torch._scaled_mm`` as
    the reference calls it (float8_python_api.py:24-64) without the layout rule that makes float8_ops.preprocess_addmm
    copy (float8_ops.py:150-153) -- a row-major second operand is read transposed by the kernel where it can."""
    with _native.transient_workspaces():
        return _native.scaled_mm(a, a_scale, b, b_scale, out_dtype, bias=bias)


@scaled_mm.register_fake
def _(a, a_scale, b, b_scale, out_dtype, bias):
    return torch.empty((a.shape[0], b.shape[1]), dtype=out_dtype, device=a.device)


# ---- the fused linear ----------------------------------------------------------------------------------------


def _layout(t_rows: int, t_cols: int, layout: int):
    """Shape of an fp8 operand with ``t_rows`` rows contracting over ``t_cols`` in layout ``_native.ROWMAJOR / KBLOCK /
    KBLOCK_PAD``."""
    if layout == _native.ROWMAJOR:
        return (t_rows, t_cols)
    return ((t_cols if layout == _native.KBLOCK else _native.padded_k(t_cols)) // _KB, t_rows, _KB)


def _cast(t2d, float8_dtype, scale_buf, want_row, want_t, row_kb, t_kb):
    """(row copy, transposed copy, scale used, new amax): dynamic scaling without a scale buffer (new amax: empty),
    else the delayed-scaling cast (existing scale, fp32 product, this step's amax in a fresh one-element tensor;
    float8_scaling_utils.py:65-96)."""
    if scale_buf is None:
        row, tr, scale = _native.cast_dynamic(t2d, float8_dtype, want_out=want_row, want_out_t=want_t, out_kblock=row_kb,
                                              out_t_kblock=t_kb)
        return row, tr, scale, torch.empty(0, dtype=torch.float32, device=t2d.device)
    amax = torch.empty(1, dtype=torch.float32, device=t2d.device)
    row, tr = _native.cast(t2d, scale_buf, float8_dtype, product_dtype=torch.float32, want_out=want_row, want_out_t=want_t,
                           amax_out=amax, out_kblock=row_kb, out_t_kblock=t_kb)
    return row, tr, scale_buf, amax


def _gemm(a8, sa, b8, sb, out_dtype, kb):
    return _native.gemm_nt_kb(a8, sa, b8, sb, out_dtype) if kb else _native.gemm_nt(a8, sa, b8, sb, out_dtype)


@torch.library.custom_op("f8mi::linear_fwd", mutates_args=())
def linear_fwd(x2: torch.Tensor, weight: torch.Tensor, need_dx: bool, need_dw: bool,
               scale_x: Optional[torch.Tensor], scale_w: Optional[torch.Tensor]) -> Tuple[
        torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """y = x2 W^T in fp8; also the fp8 copies and the dynamic scales backward needs, and the amaxes delayed scaling records.

    Returns (y, xs, ws, sx, sw, amax_x, amax_w).  When the sizes allow it (``_native.tn_ok``) xs / ws are the
    forward's own k-blocked operands (backward reads them transposed); otherwise they are the transposed copies,
    and one that backward will not need is an empty tensor.  sx / sw are the scales of dynamically scaled
    tensors; for a tensor with delayed scaling (``scale_*`` given: the module's scale buffer) the slot holds an empty
    tensor and ``amax_*`` this step's amax, [1] fp32 (empty for dynamic scaling)."""
    with _native.transient_workspaces():
        return _linear_fwd_impl(x2, weight, need_dx, need_dw, scale_x, scale_w)


def _linear_fwd_impl(x2, weight, need_dx, need_dw, scale_x, scale_w):
    m, k = x2.shape
    n = weight.shape[0]
    none = lambda dt: torch.empty(0, dtype=dt, device=x2.device)
    out_s = lambda s, buf: s if buf is None else none(torch.float32)
    if _native.tn_ok(m, k, n):
        x8, _, sx, ax = _cast(x2, e4m3_dtype, scale_x, True, False, True, False)
        w8, _, sw, aw = _cast(weight, e4m3_dtype, scale_w, True, False, True, False)
        return _native.gemm_nt_kb(x8, sx, w8, sw, x2.dtype), x8, w8, out_s(sx, scale_x), out_s(sw, scale_w), ax, aw
    kb_fwd, kb_dx, kb_dw = _native.kblock_layout(k), _native.kblock_layout(n), _native.kblock_layout(m)
    x8, x8t, sx, ax = _cast(x2, e4m3_dtype, scale_x, True, need_dw, kb_fwd, kb_dw)
    w8, w8t, sw, aw = _cast(weight, e4m3_dtype, scale_w, True, need_dx, kb_fwd, kb_dx)
    y = _gemm(x8, sx, w8, sw, x2.dtype, kb_fwd)
    return (y, (x8t if need_dw else none(e4m3_dtype)), (w8t if need_dx else none(e4m3_dtype)),
            out_s(sx, scale_x), out_s(sw, scale_w), ax, aw)


@linear_fwd.register_fake
def _(x2, weight, need_dx, need_dw, scale_x, scale_w):
    m, k = x2.shape
    n = weight.shape[0]
    f8 = lambda shape: torch.empty(shape, dtype=e4m3_dtype, device=x2.device)
    s = lambda buf: torch.empty(() if buf is None else (0,), dtype=torch.float32, device=x2.device)
    a = lambda buf: torch.empty((0,) if buf is None else (1,), dtype=torch.float32, device=x2.device)
    y = torch.empty((m, n), dtype=x2.dtype, device=x2.device)
    if _native.tn_ok(m, k, n):
        return y, f8((k // _KB, m, _KB)), f8((k // _KB, n, _KB)), s(scale_x), s(scale_w), a(scale_x), a(scale_w)
    kb_dx, kb_dw = _native.kblock_layout(n), _native.kblock_layout(m)
    return (y, f8(_layout(k, m, kb_dw)) if need_dw else f8((0,)), f8(_layout(k, n, kb_dx)) if need_dx else f8((0,)),
            s(scale_x), s(scale_w), a(scale_x), a(scale_w))


@torch.library.custom_op("f8mi::linear_bwd", mutates_args=())
def linear_bwd(dy2: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, sx: torch.Tensor, sw: torch.Tensor,
               k: int, need_dx: bool, need_dw: bool, scale_g: Optional[torch.Tensor]) -> Tuple[
        torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dx, dw, amax_g): (dY W, dY^T x) in fp8, dY cast to e5m2 with a dynamic scale or the delayed-scaling scale
    buffer (then amax_g is this step's amax of dY, [1] fp32; else empty); an unneeded gradient is empty."""
    with _native.transient_workspaces():
        return _linear_bwd_impl(dy2, xs, ws, sx, sw, k, need_dx, need_dw, scale_g)


def _linear_bwd_impl(dy2, xs, ws, sx, sw, k, need_dx, need_dw, scale_g):
    m, n = dy2.shape
    empty = lambda: torch.empty(0, dtype=dy2.dtype, device=dy2.device)
    if _native.tn_ok(m, k, n):
        g8, _, sg, ag = _cast(dy2, e5m2_dtype, scale_g, True, False, True, False)
        dx = _native.gemm_kb_ex(g8, False, sg, ws, True, sw, dy2.dtype) if need_dx else empty()
        dw = _native.gemm_kb_ex(g8, True, sg, xs, True, sx, dy2.dtype) if need_dw else empty()
        return dx, dw, ag
    kb_dx, kb_dw = _native.kblock_layout(n), _native.kblock_layout(m)
    g8, g8t, sg, ag = _cast(dy2, e5m2_dtype, scale_g, need_dx, need_dw, kb_dx, kb_dw)
    dx = _gemm(g8, sg, ws, sw, dy2.dtype, kb_dx) if need_dx else empty()
    dw = _gemm(g8t, sg, xs, sx, dy2.dtype, kb_dw) if need_dw else empty()
    return dx, dw, ag


@linear_bwd.register_fake
def _(dy2, xs, ws, sx, sw, k, need_dx, need_dw, scale_g):
    m, n = dy2.shape
    e = lambda shape: torch.empty(shape, dtype=dy2.dtype, device=dy2.device)
    return (e((m, k)) if need_dx else e((0,)), e((n, k)) if need_dw else e((0,)),
            torch.empty((0,) if scale_g is None else (1,), dtype=torch.float32, device=dy2.device))


class _LinearFn(torch.autograd.Function):
    """Autograd around the two functional ops; the amax buffers of delayed scaling are updated in place here, where
    the compiler traces ordinary tensor operations."""

    @staticmethod
    def forward(ctx, x2, weight, bufs_x, bufs_w, bufs_g):
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        sx_buf = bufs_x[1] if bufs_x is not None else None
        sw_buf = bufs_w[1] if bufs_w is not None else None
        y, xs, ws, sx, sw, ax, aw = linear_fwd(x2, weight, need_dx, need_dw, sx_buf, sw_buf)
        if bufs_x is not None:
            bufs_x[0].copy_(ax)
        if bufs_w is not None:
            bufs_w[0].copy_(aw)
        ctx.k = x2.shape[1]
        ctx.bufs_g = bufs_g
        # a delayed tensor's scale is the module's buffer, a dynamic one's comes out of the forward op
        ctx.save_for_backward(xs, ws, sx if sx_buf is None else sx_buf, sw if sw_buf is None else sw_buf)
        return y

    @staticmethod
    def backward(ctx, gy):
        xs, ws, sx, sw = ctx.saved_tensors
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        bufs_g = ctx.bufs_g
        dx, dw, ag = linear_bwd(gy, xs, ws, sx, sw, ctx.k, need_dx, need_dw,
                                bufs_g[1] if bufs_g is not None else None)
        if bufs_g is not None:
            bufs_g[0].copy_(ag)
        return (dx if need_dx else None), (dw if need_dw else None), None, None, None


def linear(x: torch.Tensor, weight: torch.Tensor, bufs_x=None, bufs_w=None, bufs_g=None) -> torch.Tensor:
    """y = x W^T with fp8 matmuls in both directions, traceable by ``torch.compile`` as one node per direction.
    ``bufs_*``: (amax, scale) buffers of a tensor with delayed scaling, None for dynamic scaling."""
    k = x.shape[-1]
    y = _LinearFn.apply(x.reshape(-1, k), weight, bufs_x, bufs_w, bufs_g)
    return y.reshape(*x.shape[:-1], weight.shape[0])


def linear_dynamic(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``linear`` with all three tensors dynamically scaled."""
    return linear(x, weight)


@torch.library.custom_op("f8mi::sync", mutates_args=("scales",))
def sync(amaxes: List[torch.Tensor], histories: List[torch.Tensor], scales: List[torch.Tensor], is_e5m2: List[bool],
         orig_is_fp16: bool) -> None:
    """The delayed-scaling sync of all listed buffers as one node (and one kernel launch): for each i,
    ``scales[i] = fmax / max(amaxes[i], histories[i][:-1])`` in the reference's rounding
    (float8_linear_utils.py:287-319).  No autograd: the buffers carry none."""
    # the entries travel as kernel arguments: a node of a compiled graph must not allocate a tensor that outlives it
    # (torch.compile(mode="reduce-overhead") keeps the graph's memory in a pool of its own)
    _native.sync_host(((a, h, s, e5m2_dtype if e else e4m3_dtype) for a, h, s, e in zip(amaxes, histories, scales, is_e5m2)),
                      histories[0].numel(), orig_is_fp16, writeback_history=False)


@sync.register_fake
def _(amaxes, histories, scales, is_e5m2, orig_is_fp16):
    return None
