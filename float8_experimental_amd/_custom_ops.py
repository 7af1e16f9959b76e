"""The fused dynamic-scaling linear as two ``torch.library`` custom ops, so that ``torch.compile`` sees
one opaque node per direction instead of tracing into the ctypes calls (which it cannot).

The reference keeps its float8 pieces traceable with ``torch._dynamo.allow_in_graph``
(float8_linear.py:43, float8_tensor.py:131,198) and lets inductor generate the casts; here the kernels
are hand-written, so the compiler only has to know shapes and dtypes (the fake implementations below)
and how gradients flow (``register_autograd``).  Modules with delayed scaling keep state on the module
(flags, amax / scale buffers) and are run outside the graph instead (``torch._dynamo.disable``).
"""
from typing import Tuple

import torch

from . import _native
from .float8_utils import e4m3_dtype, e5m2_dtype

_KB = _native.KB


def _layout(t_rows: int, t_cols: int, kblock: bool):
    """Shape of an fp8 operand with ``t_rows`` rows contracting over ``t_cols``."""
    return (t_cols // _KB, t_rows, _KB) if kblock else (t_rows, t_cols)


def _cast_dynamic(t2d, float8_dtype, want_row, want_t, row_kb, t_kb):
    return _native.cast_dynamic(t2d, float8_dtype, want_out=want_row, want_out_t=want_t, out_kblock=row_kb, out_t_kblock=t_kb)


def _gemm(a8, sa, b8, sb, out_dtype, kb):
    return _native.gemm_nt_kb(a8, sa, b8, sb, out_dtype) if kb else _native.gemm_nt(a8, sa, b8, sb, out_dtype)


@torch.library.custom_op("f8mi::linear_dynamic_fwd", mutates_args=())
def linear_dynamic_fwd(x2: torch.Tensor, weight: torch.Tensor, need_dx: bool, need_dw: bool) -> Tuple[
        torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """y = x2 W^T in fp8 with dynamic scales; also the fp8 copies and scales backward needs.

    Returns (y, xs, ws, sx, sw).  When every dimension allows it (``_native.tn_ok``) xs / ws are the forward's
    own k-blocked operands (backward reads them transposed); otherwise they are the transposed copies, and
    one that backward will not need is an empty tensor."""
    m, k = x2.shape
    n = weight.shape[0]
    if _native.tn_ok(m, k, n):
        x8, _, sx = _cast_dynamic(x2, e4m3_dtype, True, False, True, False)
        w8, _, sw = _cast_dynamic(weight, e4m3_dtype, True, False, True, False)
        return _native.gemm_nt_kb(x8, sx, w8, sw, x2.dtype), x8, w8, sx, sw
    kb_fwd, kb_dx, kb_dw = _native.kblock_ok(k), _native.kblock_ok(n), _native.kblock_ok(m)
    x8, x8t, sx = _cast_dynamic(x2, e4m3_dtype, True, need_dw, kb_fwd, kb_dw)
    w8, w8t, sw = _cast_dynamic(weight, e4m3_dtype, True, need_dx, kb_fwd, kb_dx)
    y = _gemm(x8, sx, w8, sw, x2.dtype, kb_fwd)
    empty = lambda: torch.empty(0, dtype=e4m3_dtype, device=x2.device)
    return y, (x8t if need_dw else empty()), (w8t if need_dx else empty()), sx, sw


@linear_dynamic_fwd.register_fake
def _(x2, weight, need_dx, need_dw):
    m, k = x2.shape
    n = weight.shape[0]
    f8 = lambda shape: torch.empty(shape, dtype=e4m3_dtype, device=x2.device)
    s = lambda: torch.empty((), dtype=torch.float32, device=x2.device)
    y = torch.empty((m, n), dtype=x2.dtype, device=x2.device)
    if _native.tn_ok(m, k, n):
        return y, f8((k // _KB, m, _KB)), f8((k // _KB, n, _KB)), s(), s()
    kb_dx, kb_dw = _native.kblock_ok(n), _native.kblock_ok(m)
    return (y, f8(_layout(k, m, kb_dw)) if need_dw else f8((0,)), f8(_layout(k, n, kb_dx)) if need_dx else f8((0,)), s(), s())


@torch.library.custom_op("f8mi::linear_dynamic_bwd", mutates_args=())
def linear_dynamic_bwd(dy2: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, sx: torch.Tensor, sw: torch.Tensor,
                       k: int, need_dx: bool, need_dw: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """(dx, dw) = (dY W, dY^T x) in fp8, dY cast to e5m2 with a dynamic scale; an unneeded one is empty."""
    m, n = dy2.shape
    empty = lambda: torch.empty(0, dtype=dy2.dtype, device=dy2.device)
    if _native.tn_ok(m, k, n):
        g8, _, sg = _cast_dynamic(dy2, e5m2_dtype, True, False, True, False)
        dx = _native.gemm_kb_ex(g8, False, sg, ws, True, sw, dy2.dtype) if need_dx else empty()
        dw = _native.gemm_kb_ex(g8, True, sg, xs, True, sx, dy2.dtype) if need_dw else empty()
        return dx, dw
    kb_dx, kb_dw = _native.kblock_ok(n), _native.kblock_ok(m)
    g8, g8t, sg = _cast_dynamic(dy2, e5m2_dtype, need_dx, need_dw, kb_dx, kb_dw)
    dx = _gemm(g8, sg, ws, sw, dy2.dtype, kb_dx) if need_dx else empty()
    dw = _gemm(g8t, sg, xs, sx, dy2.dtype, kb_dw) if need_dw else empty()
    return dx, dw


@linear_dynamic_bwd.register_fake
def _(dy2, xs, ws, sx, sw, k, need_dx, need_dw):
    m, n = dy2.shape
    e = lambda shape: torch.empty(shape, dtype=dy2.dtype, device=dy2.device)
    return (e((m, k)) if need_dx else e((0,)), e((n, k)) if need_dw else e((0,)))


def _setup_context(ctx, inputs, output):
    x2, weight, need_dx, need_dw = inputs
    _, x8t, w8t, sx, sw = output
    ctx.k = x2.shape[1]
    ctx.need = (need_dx, need_dw)
    ctx.save_for_backward(x8t, w8t, sx, sw)


def _backward(ctx, gy, *_unused):
    x8t, w8t, sx, sw = ctx.saved_tensors
    need_dx, need_dw = ctx.need
    dx, dw = linear_dynamic_bwd(gy.contiguous(), x8t, w8t, sx, sw, ctx.k, need_dx, need_dw)
    return (dx if need_dx else None), (dw if need_dw else None), None, None


linear_dynamic_fwd.register_autograd(_backward, setup_context=_setup_context)


def linear_dynamic(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """y = x W^T, all three tensors dynamically scaled; traceable by ``torch.compile`` as one node."""
    k = x.shape[-1]
    y = linear_dynamic_fwd(x.reshape(-1, k), weight, x.requires_grad, weight.requires_grad)[0]
    return y.reshape(*x.shape[:-1], weight.shape[0])
