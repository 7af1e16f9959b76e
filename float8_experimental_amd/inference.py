"""fp8 inference linear: the weight is cast once, activations per call (or never).

Same names and behaviour as the reference's ``float8_experimental/inference.py``
(``ActivationCasting``, ``QuantConfig``, ``Float8InferenceLinear``, ``cast_to_float8_e4m3_inference``,
``quantize_to_float8``); forward-only reuse of the training path's kernels: the activation's
amax + scale (K1), its saturated cast (K2) and the scaled fp8 GEMM (K3, with the bias added in
its epilogue).  The weight stays a ``Float8Tensor`` parameter with row-major bytes, as the
reference keeps it (``inference.py:119-141``), so state dicts interchange; next to it the module
caches the same bytes in the k-blocked placement the GEMM reads fastest.
"""
import weakref
from dataclasses import dataclass
from enum import Enum, auto
from typing import Callable, Optional

import torch
import torch.nn as nn

from . import _custom_ops  # noqa: F401  (registers torch.ops.f8mi.*)
from . import _native
from .float8_linear_utils import swap_linear_layers
from .float8_tensor import (
    Float8Tensor,
    GemmInputRole,
    LinearMMConfig,
    ScaledMMConfig,
    _product_dtype,
    hp_tensor_and_scale_to_float8,
    tensor_already_casted_to_fp8,
)
from .float8_utils import e4m3_dtype, tensor_to_scale


class ActivationCasting(Enum):
    """What happens to the activations (``inference.py:30-42`` of the reference).

    WEIGHT_ONLY: nothing; the fp8 weight is dequantised in the forward pass and the matmul runs in high precision
    DYNAMIC: cast per call with a scale computed from the activation
    STATIC: cast per call with the scale given at conversion time
    """

    WEIGHT_ONLY = auto()
    DYNAMIC = auto()
    STATIC = auto()


@dataclass(frozen=True)
class QuantConfig:
    """``activation_casting`` and, for STATIC, the activation's scale (``inference.py:45-67``)."""

    activation_casting: ActivationCasting
    static_quantization_scale: Optional[torch.Tensor] = None

    # kept for source compatibility; the GEMM here takes any inner dimension, nothing is padded
    pad_inner_dim = False

    def __post_init__(self):
        if self.activation_casting == ActivationCasting.STATIC:
            assert isinstance(
                self.static_quantization_scale, torch.Tensor
            ), "When activation_casting is 'static', activation_scale must be a tensor."


def _to_kblock(rowmajor_fp8: torch.Tensor) -> torch.Tensor:
    """[rows, k] fp8 bytes -> [k/64, rows, 64]: the placement f8mi_gemm_nt_kb reads (bytes moved, not changed); a k that
    is no multiple of 64 is extended with zero bytes to a multiple of 128 first (F8MI_LAYOUT_KBLOCK64_PAD128)."""
    rows, k = rowmajor_fp8.shape
    kb = _native.KB
    data = rowmajor_fp8.view(torch.uint8)
    if k % kb != 0:
        data = torch.nn.functional.pad(data, (0, _native.padded_k(k) - k))
    return data.view(rows, data.shape[1] // kb, kb).permute(1, 0, 2).contiguous().view(rowmajor_fp8.dtype)


# k-blocked copies of quantised weights, by the address of the row-major bytes; refreshed when those bytes change
# (version counter) and dropped with the weight.  Module-level so that the custom op, which sees plain tensors, finds it.
_KB_WEIGHTS = {}


def _kblocked_weight(w_data: torch.Tensor) -> torch.Tensor:
    """The k-blocked copy of a quantised weight.  An in-place update of the weight (``copy_``, ``load_state_dict``)
    refreshes the copy IN PLACE: its address stays what a captured graph (``torch.compile(mode="reduce-overhead")``, a
    HIP graph) recorded, so replays read the new bytes once any eager call has come by; only a weight of another shape
    or dtype at the same address gets a new copy."""
    key = w_data.data_ptr()
    tag = (tuple(w_data.shape), w_data.dtype)
    hit = _KB_WEIGHTS.get(key)
    if hit is None or hit[0] != tag:
        if hit is None:
            weakref.finalize(w_data, _KB_WEIGHTS.pop, key, None)
        hit = _KB_WEIGHTS[key] = [tag, _to_kblock(w_data), w_data._version]
    elif hit[2] != w_data._version:
        hit[1].view(torch.uint8).copy_(_to_kblock(w_data).view(torch.uint8))
        hit[2] = w_data._version
    return hit[1]


def _fp8_linear(x2: torch.Tensor, w_data: torch.Tensor, w_scale: torch.Tensor, static_scale: Optional[torch.Tensor],
                bias: Optional[torch.Tensor]) -> torch.Tensor:
    """x2 [m, k] high precision, w_data [n, k] fp8 row-major -> [m, n] in x2's dtype: activation cast (static scale if
    given, else dynamic) and the scaled GEMM with the bias in its epilogue."""
    k = x2.shape[1]
    use_kb = _native.kblock_layout(k)  # row-major for a short contraction, else k-blocked (zero-padded when ragged)
    if static_scale is not None:
        scale = static_scale
        x8, _ = _native.cast(x2, scale, e4m3_dtype, product_dtype=_product_dtype(x2, scale), out_kblock=use_kb)
    else:
        x8, _, scale = _native.cast_dynamic(x2, e4m3_dtype, out_kblock=use_kb)
    if use_kb:
        return _native.gemm_nt_kb(x8, scale, _kblocked_weight(w_data), w_scale, x2.dtype, bias=bias)
    return _native.gemm_nt(x8, scale, w_data, w_scale, x2.dtype, bias=bias)


@torch.library.custom_op("f8mi::inference_linear", mutates_args=())
def _inference_linear_op(x2: torch.Tensor, w_data: torch.Tensor, w_scale: torch.Tensor, static_scale: Optional[torch.Tensor],
                         bias: Optional[torch.Tensor]) -> torch.Tensor:
    """``_fp8_linear`` as one opaque node for ``torch.compile`` (workspaces are temporaries inside a compiled graph)."""
    with _native.transient_workspaces():
        return _fp8_linear(x2, w_data, w_scale, static_scale, bias)


@_inference_linear_op.register_fake
def _(x2, w_data, w_scale, static_scale, bias):
    return torch.empty((x2.shape[0], w_data.shape[0]), dtype=x2.dtype, device=x2.device)


@torch._dynamo.allow_in_graph
def _inference_linear_traced(x2: torch.Tensor, weight: "Float8Tensor", static_scale: Optional[torch.Tensor],
                             bias: Optional[torch.Tensor]) -> torch.Tensor:
    # taken apart here, below dynamo: the compiler's tracer sees the Float8Tensor's payload and scale as plain tensors
    return torch.ops.f8mi.inference_linear(x2, weight._data, weight._scale, static_scale, bias)


class Float8InferenceLinear(torch.nn.Linear):
    """``nn.Linear`` whose weight is an fp8 ``Float8Tensor`` (``inference.py:70-172`` of the reference)."""

    def __init__(self, quant_config: QuantConfig, linear_mm_config: LinearMMConfig, in_features: int, out_features: int,
                 bias: bool = True, device: Optional[torch.device] = None, dtype: Optional[torch.dtype] = None) -> None:
        super().__init__(in_features, out_features, bias, device, dtype)
        self.linear_mm_config = linear_mm_config
        self.activation_casting = quant_config.activation_casting
        if self.activation_casting == ActivationCasting.STATIC:
            self.register_buffer("static_quantization_scale", quant_config.static_quantization_scale)
        else:
            self.static_quantization_scale = None

    # ---- forward
    def _weight_kblocked(self) -> torch.Tensor:
        return _kblocked_weight(self.weight._data)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if self.activation_casting == ActivationCasting.WEIGHT_ONLY:
            # the reference does not pass the bias on this branch either (inference.py:104-107)
            return torch.nn.functional.linear(input, self.weight.to_original_precision())
        w = self.weight
        assert isinstance(w, Float8Tensor), "quantize_weight() has not been called"
        if tensor_already_casted_to_fp8(input) or self.linear_mm_config.output.emulate or not input.is_cuda:
            # composed route: Float8Tensor ops (and the loud error for CPU tensors)
            x_fp8 = cast_to_float8_e4m3_inference(input, self.linear_mm_config,
                                                  static_quantization_scale=self.static_quantization_scale)
            return torch.nn.functional.linear(x_fp8, w, self.bias)
        x2 = input.reshape(-1, input.shape[-1])
        bias = self.bias
        if bias is not None and bias.dtype != input.dtype:
            bias = bias.to(input.dtype)
        if torch.compiler.is_compiling():  # one opaque node: the ctypes calls cannot be traced
            y = _inference_linear_traced(x2, w, self.static_quantization_scale, bias)
        else:
            y = _fp8_linear(x2, w._data, w._scale, self.static_quantization_scale, bias)
        return y.reshape(*input.shape[:-1], self.out_features)

    # ---- builders (inference.py:119-172)
    def quantize_weight(self, dtype: torch.dtype = e4m3_dtype) -> None:
        """Casts the weight once (dynamic scale) into a non-trainable ``Float8Tensor`` parameter."""
        assert not isinstance(self.weight, Float8Tensor), "Weight has already been quantized, cannot quantize again."
        scale = tensor_to_scale(self.weight, dtype)
        quantized_weight = hp_tensor_and_scale_to_float8(self.weight, scale, dtype, self.linear_mm_config,
                                                         GemmInputRole.WEIGHT)
        self.weight = nn.Parameter(quantized_weight)
        self.weight.requires_grad = False
        if quantized_weight._data.is_cuda and _native.kblock_layout(self.in_features) != _native.ROWMAJOR:
            self._weight_kblocked()  # now, not inside the first forward (which may be a node of a compiled graph)

    def set_weight_and_bias(self, weight: torch.nn.Parameter, bias: Optional[torch.nn.Parameter]):
        self.weight = weight
        self.bias = bias

    @classmethod
    def from_float(cls, module: nn.Module, quant_config: QuantConfig, use_fast_accum: bool) -> "Float8InferenceLinear":
        """An fp8-compute linear from an ``nn.Linear`` (or a ``Float8Linear``), sharing its parameters."""
        forward_config = ScaledMMConfig(False, use_fast_accum, pad_inner_dim=quant_config.pad_inner_dim)
        linear_mm_config = LinearMMConfig(forward_config, forward_config, forward_config)
        linear = cls(quant_config, linear_mm_config, module.in_features, module.out_features, False,
                     device=torch.device("meta"))
        linear.set_weight_and_bias(module.weight, module.bias)
        linear.quantize_weight()
        return linear


def cast_to_float8_e4m3_inference(inpt_tensor: torch.Tensor, linear_mm_config: LinearMMConfig, reduce_amax: bool = False,
                                  static_quantization_scale: Optional[torch.Tensor] = None) -> Float8Tensor:
    """e4m3 ``Float8Tensor`` of an activation: static scale if given, else dynamic (``inference.py:175-208``).

    A tensor that already is a ``Float8Tensor`` is returned as it is."""
    if tensor_already_casted_to_fp8(inpt_tensor):
        return inpt_tensor
    scale = (static_quantization_scale if static_quantization_scale is not None
             else tensor_to_scale(inpt_tensor, e4m3_dtype, reduce_amax))
    return hp_tensor_and_scale_to_float8(inpt_tensor, scale, e4m3_dtype, linear_mm_config, GemmInputRole.INPUT)


def quantize_to_float8(module: nn.Module, quant_config: QuantConfig, *,
                       module_filter_fn: Optional[Callable[[nn.Module, str], bool]] = None,
                       use_fast_accum: bool = True) -> nn.Module:
    """Swaps every (filtered) ``nn.Linear`` of ``module`` for a ``Float8InferenceLinear`` (``inference.py:211-244``).

    A root-level ``nn.Linear`` is not modified in place but returned converted; one with children raises."""
    return swap_linear_layers(module, lambda m: Float8InferenceLinear.from_float(m, quant_config, use_fast_accum),
                              module_filter_fn=module_filter_fn)
