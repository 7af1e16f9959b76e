"""Torch-CPU restatement of the Float8Linear hot path -- TEST INFRASTRUCTURE ONLY.

Each function below re-expresses one step of pytorch-labs/float8_experimental
with the same torch operators in the same dtypes, as free functions on plain
tensors (no tensor subclass, no autograd), so that intermediate fp8 bytes,
amaxes and scales can be compared bit for bit with the HIP kernels.  Reference
locations are quoted per function (paths relative to the reference checkout).

The shipped package never imports this module.
"""
from typing import Dict, List, Optional

import torch

EPS = 1e-12  # float8_utils.py:19
E4M3 = torch.float8_e4m3fn  # float8_utils.py:31
E5M2 = torch.float8_e5m2  # float8_utils.py:32


def tensor_to_amax(x: torch.Tensor) -> torch.Tensor:
    """float8_utils.py:102-112 (single process: no all-reduce).  0-dim, x's dtype."""
    return torch.max(torch.abs(x))


def amax_to_scale(amax: torch.Tensor, float8_dtype: torch.dtype, orig_dtype: torch.dtype) -> torch.Tensor:
    """float8_utils.py:35-57.  ``fmax / clamp(amax, EPS)`` is ``reciprocal() * fmax`` in amax's dtype."""
    res = torch.clamp(amax, min=EPS).reciprocal() * torch.finfo(float8_dtype).max
    if orig_dtype is torch.float16:
        res = torch.clamp(res, max=torch.finfo(torch.float16).max)
    return res.to(torch.float32)


def tensor_to_scale(x: torch.Tensor, float8_dtype: torch.dtype) -> torch.Tensor:
    """float8_utils.py:115-120."""
    return amax_to_scale(tensor_to_amax(x), float8_dtype, x.dtype)


def cast_to_fp8(x: torch.Tensor, scale: torch.Tensor, float8_dtype: torch.dtype) -> torch.Tensor:
    """float8_tensor.py:158-159 + float8_utils.py:123-139.

    The rank of ``scale`` matters: a 0-dim fp32 scale leaves a bf16 product
    (dynamic scaling), a ``[1]``-shaped one promotes the product to fp32
    (delayed-scaling buffers).
    """
    y = x * scale
    fmax = torch.finfo(float8_dtype).max
    return y.clamp(min=-fmax, max=fmax).to(float8_dtype)


def mm_emulated(a: torch.Tensor, sa: torch.Tensor, b: torch.Tensor, sb: torch.Tensor, out_dtype: torch.dtype):
    """float8_aten_api.py:16-28.  a: fp8 [m,k]; b: fp8 [k,n] (any strides)."""
    return torch.mm(a.float() / sa, b.float() / sb).to(out_dtype)


def linear_fwd_bwd_dynamic(x: torch.Tensor, w: torch.Tensor, dy: torch.Tensor) -> Dict[str, torch.Tensor]:
    """One Float8Linear fwd+bwd with dynamic scaling on all three tensors, emulated GEMMs.

    float8_linear.py:356-373 (forward), :64-95 (the two backward GEMMs),
    float8_scaling_utils.py:33-62 and :204-216 (the casts).
    x: [M,K], w: [N,K], dy: [M,N], all one dtype.  Returns every intermediate.
    """
    sx, sw = tensor_to_scale(x, E4M3), tensor_to_scale(w, E4M3)
    x8, w8 = cast_to_fp8(x, sx, E4M3), cast_to_fp8(w, sw, E4M3)
    y = mm_emulated(x8, sx, w8.t(), sw, x.dtype)
    sg = tensor_to_scale(dy, E5M2)
    g8 = cast_to_fp8(dy, sg, E5M2)
    dx = mm_emulated(g8, sg, w8, sw, dy.dtype)  # grad_output @ weight
    dw = mm_emulated(g8.t(), sg, x8, sx, dy.dtype)  # grad_output^T @ input
    return dict(sx=sx, sw=sw, sg=sg, x8=x8, w8=w8, g8=g8, y=y, dx=dx, dw=dw)


class DelayedTensorState:
    """The three buffers of one tensor of one layer (float8_linear.py:180-222)."""

    def __init__(self, float8_dtype: torch.dtype, history_len: int):
        default = torch.finfo(E4M3 if float8_dtype == E4M3 else E5M2).max
        self.float8_dtype = float8_dtype
        self.amax = torch.tensor([default], dtype=torch.float32)
        self.history = torch.zeros(history_len, dtype=torch.float32)
        self.scale = torch.tensor([1.0], dtype=torch.float32)

    def maybe_init(self, x: torch.Tensor, is_initialized: bool) -> None:
        """float8_scaling_utils.py:99-125."""
        if is_initialized:
            return
        new_amax = tensor_to_amax(x)
        self.amax.fill_(new_amax)
        self.history[0] = new_amax
        self.scale.copy_(amax_to_scale(torch.max(self.history), self.float8_dtype, x.dtype))

    def cast(self, x: torch.Tensor) -> torch.Tensor:
        """float8_scaling_utils.py:65-96: record this step's amax, cast with the EXISTING scale."""
        self.amax.fill_(tensor_to_amax(x))
        return cast_to_fp8(x, self.scale, self.float8_dtype)

    def sync(self, x_dtype: torch.dtype) -> None:
        """One row of sync_float8_amax_and_scale_history (float8_linear_utils.py:287-319).

        The reference rolls a ``torch.vstack`` copy of the histories and copies
        only the new scales back, so ``self.history`` stays as it is.
        """
        stack = self.history.clone().reshape(1, -1)
        rolled = torch.roll(stack, 1, dims=1)
        rolled[:, 0] = self.amax
        new_amax = torch.max(rolled, dim=1).values
        self.scale.copy_(amax_to_scale(new_amax, self.float8_dtype, x_dtype))


class LinearOracle:
    """Stateful restatement of one Float8Linear (no bias) for any scaling mix.

    ``scaling`` is a 3-tuple of "dyn"/"del" for (input, weight, grad_output).
    Flags follow float8_linear.py:156-177 and :335-354.
    """

    def __init__(self, w: torch.Tensor, scaling=("dyn", "dyn", "dyn"), history_len: int = 16):
        self.w = w
        self.scaling = scaling
        self.any_delayed = "del" in scaling
        self.st = {
            "input": DelayedTensorState(E4M3, history_len),
            "weight": DelayedTensorState(E4M3, history_len),
            "grad_output": DelayedTensorState(E5M2, history_len),
        }
        self.is_amax_initialized = False
        self.last_seen_input_dtype = None

    def _cast(self, kind: str, idx: int, t: torch.Tensor, is_init: bool):
        f8 = self.st[kind].float8_dtype
        if self.scaling[idx] == "del":
            self.st[kind].maybe_init(t, is_init)
            return self.st[kind].cast(t), self.st[kind].scale
        s = tensor_to_scale(t, f8)
        return cast_to_fp8(t, s, f8), s

    def sync(self) -> None:
        for kind in ("input", "weight", "grad_output"):
            self.st[kind].sync(self.last_seen_input_dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.any_delayed:
            self.last_seen_input_dtype = x.dtype
        # the flag value seen by all three casts of this iteration is the one from
        # before the forward (float8_linear.py:318-333 passes it into the backward)
        self._is_init = self.is_amax_initialized
        self._x_shape = x.shape
        x2 = x.reshape(-1, x.shape[-1])
        self.x8, self.sx = self._cast("input", 0, x2, self._is_init)
        self.w8, self.sw = self._cast("weight", 1, self.w, self._is_init)
        self.sx, self.sw = self.sx.clone(), self.sw.clone()
        y = mm_emulated(self.x8, self.sx, self.w8.t(), self.sw, x.dtype)
        if self.any_delayed:
            self.is_amax_initialized = True
        return y.reshape(*x.shape[:-1], -1)

    def backward(self, dy: torch.Tensor):
        dy2 = dy.reshape(-1, dy.shape[-1])
        self.g8, sg = self._cast("grad_output", 2, dy2, self._is_init)
        self.sg = sg.clone()
        dx = mm_emulated(self.g8, self.sg, self.w8, self.sw, dy.dtype)
        dw = mm_emulated(self.g8.t(), self.sg, self.x8, self.sx, dy.dtype)
        return dx.reshape(self._x_shape), dw

    def fwd_bwd(self, x: torch.Tensor, dy: torch.Tensor) -> Dict[str, torch.Tensor]:
        y = self.forward(x)
        dx, dw = self.backward(dy)
        return dict(x8=self.x8, w8=self.w8, g8=self.g8, sx=self.sx, sw=self.sw, sg=self.sg, y=y, dx=dx, dw=dw)


def sqnr(x: torch.Tensor, y: torch.Tensor) -> float:
    """float8_utils.py:142-154 (signal-to-quantisation-noise ratio in dB)."""
    return (20 * torch.log10(torch.norm(x.double()) / torch.norm(x.double() - y.double()))).item()
