"""``Float8Linear``: ``nn.Linear`` whose three matmuls run in float8 on MI355X
(mirror of the reference's ``float8_linear.py``).

The reference strings the layer together from four autograd functions and a tensor
subclass (cast x, cast W, matmul, cast dY in backward).  Here the whole layer is ONE
autograd function around five kernel launches per direction: amax+scale and
cast per tensor, and one matrix-core GEMM per product.  Where the sizes allow it each
tensor has ONE fp8 copy and the backward GEMMs read it transposed; otherwise the
transposed fp8 copies are written by the cast kernels while the data is in registers,
and only those are kept for backward.
The pieces of the reference's composition (``cast_input_to_float8`` ...,
``manual_float8_matmul``) are still here and give the same numbers.
"""
from typing import Optional

import torch

from . import _native
from .config import Float8LinearConfig, ScalingType
from . import float8_aten_api  # noqa: F401  (registers torch.ops.aten.mm_float8_emulated)
from .float8_scaling_utils import (
    _maybe_initialize_amaxes_scales_for_float8_cast,
    hp_tensor_to_float8_delayed,
    hp_tensor_to_float8_dynamic,
    NoopFwToFloat8E5M2BwDelayed,
    NoopFwToFloat8E5M2BwDynamic,
)
from .float8_tensor import (
    Float8Tensor,
    GemmInputRole,
    LinearMMConfig,
    ScaledMMConfig,
    hp_tensor_and_scale_to_float8,
)
from .float8_utils import e4m3_dtype, e5m2_dtype

_KINDS = ("input", "weight", "grad_output")


@torch._dynamo.allow_in_graph
class manual_float8_matmul(torch.autograd.Function):
    """``input_fp8 @ weight_fp8_t`` on Float8Tensors with both backward products
    (reference float8_linear.py:43-95)."""

    @staticmethod
    def forward(ctx, input_fp8, weight_fp8_t):
        ctx.save_for_backward(input_fp8, weight_fp8_t)
        flat = input_fp8.reshape(-1, input_fp8.shape[-1])
        out = torch.mm(flat, weight_fp8_t)
        return out.reshape(*input_fp8.shape[:-1], out.shape[-1])

    @staticmethod
    def backward(ctx, grad_output_fp8):
        input_fp8, weight_fp8_t = ctx.saved_tensors
        go = grad_output_fp8.reshape(-1, grad_output_fp8.shape[-1])
        grad_input = torch.mm(go, weight_fp8_t.t())
        grad_input = grad_input.reshape(*grad_output_fp8.shape[:-1], grad_input.shape[-1])
        flat = input_fp8.reshape(-1, input_fp8.shape[-1])
        grad_weight = torch.mm(go.t(), flat)
        return grad_input, grad_weight.t()


class _DelayedBuffers:
    """amax / history / scale of one tensor of one layer, plus the flag captured at forward."""

    __slots__ = ("amax", "history", "scale")

    def __init__(self, amax, history, scale):
        self.amax, self.history, self.scale = amax, history, scale


def _cast_for_gemm(t2d: torch.Tensor, float8_dtype, delayed: Optional[_DelayedBuffers], is_initialized: bool,
                   want_row: bool, want_t: bool, row_kb: int = 0, t_kb: int = 0,
                   known_scale: Optional[torch.Tensor] = None):
    """fp8 copies of a 2-D tensor for the GEMMs: (as is, transposed, scale).

    dynamic: amax+scale, then the cast, in one library call (float8_utils.py:115-120 +
    float8_tensor.py:158-159 of the reference; one launch for a small tensor); delayed: first-iteration init if needed,
    then ONE launch that casts with the existing scale and records this step's amax
    (float8_scaling_utils.py:65-125).  ``row_kb`` / ``t_kb`` ask for the k-blocked layout
    of the respective copy (same bytes, placed [k/64][rows][64] for the GEMM that contracts it;
    ``_native.KBLOCK_PAD``: with the contraction zero-padded to a multiple of 128).
    ``known_scale`` (dynamic scaling only): a scale computed beforehand for exactly this tensor
    (``precompute_float8_dynamic_scale_for_fsdp``); the amax pass is skipped.
    """
    if delayed is None:
        if known_scale is None:
            return _native.cast_dynamic(t2d, float8_dtype, want_out=want_row, want_out_t=want_t, out_kblock=row_kb,
                                        out_t_kblock=t_kb)
        row, tr = _native.cast(t2d, known_scale, float8_dtype, product_dtype=t2d.dtype, want_out=want_row, want_out_t=want_t,
                               out_kblock=row_kb, out_t_kblock=t_kb)
        return row, tr, known_scale
    if not is_initialized:
        _native.amax_scale(t2d, float8_dtype, want_scale=False, amax_out=delayed.amax)
        _native.delayed_init(delayed.amax, delayed.history, delayed.scale, float8_dtype, t2d.dtype == torch.float16)
    row, tr = _native.cast(t2d, delayed.scale, float8_dtype, product_dtype=torch.float32, want_out=want_row,
                           want_out_t=want_t, amax_out=delayed.amax, out_kblock=row_kb, out_t_kblock=t_kb)
    return row, tr, delayed.scale


def _gemm(a8, sa, b8, sb, out_dtype, kb: bool):
    return _native.gemm_nt_kb(a8, sa, b8, sb, out_dtype) if kb else _native.gemm_nt(a8, sa, b8, sb, out_dtype)


class _float8_linear_fn(torch.autograd.Function):
    """y = x W^T with every matmul of forward and backward in fp8 (no bias).

    Each of the three GEMMs contracts a different dimension (in_features, out_features, tokens).
    When all three are multiples of 128 (and at least 384) each tensor is cast ONCE, k-blocked over
    its own last dimension, and the two GEMMs that use it read that one copy -- as it is where its last
    dimension is contracted, through LDS transpose loads where it is not (``f8mi_gemm_kb_ex``): no
    transposed fp8 copies exist.  Otherwise the cast writes the tensor and its transpose, each k-blocked
    for its GEMM's contraction -- as it is when that is a multiple of 64, zero-padded to a multiple of 128
    when it is not (ragged layers: the reference pads the inner dimension for torch._scaled_mm the same way,
    float8_utils.py:206-247) -- and row-major only where the contraction is short.
    """

    @staticmethod
    def forward(ctx, x, weight, mod, is_amax_initialized):
        k = x.shape[-1]
        x2 = x.reshape(-1, k)
        m, n = x2.shape[0], weight.shape[0]
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        emulate = mod.linear_mm_config.output.emulate
        emulate_bw = mod.linear_mm_config.grad_input.emulate or mod.linear_mm_config.grad_weight.emulate
        dl = mod._delayed_buffers
        tn = not emulate and not emulate_bw and _native.tn_ok(m, k, n)
        if tn:
            x8, _, sx = _cast_for_gemm(x2, e4m3_dtype, dl("input"), is_amax_initialized, True, False, True, False)
            w8, _, sw = _cast_for_gemm(weight, e4m3_dtype, dl("weight"), is_amax_initialized, True, False, True, False,
                                        known_scale=mod._precomputed_weight_scale)
            y = _native.gemm_nt_kb(x8, sx, w8, sw, x.dtype)
            ctx.kb = None
            ctx.save_for_backward(x8, w8, sx, sw)
        else:
            kb_fwd = 0 if emulate else _native.kblock_layout(k)      # y = x W^T contracts in_features
            kb_dx = 0 if emulate_bw else _native.kblock_layout(n)    # dx = dy W contracts out_features
            kb_dw = 0 if emulate_bw else _native.kblock_layout(m)    # dw = dy^T x contracts tokens
            x8, x8t, sx = _cast_for_gemm(x2, e4m3_dtype, dl("input"), is_amax_initialized, True, need_dw, kb_fwd, kb_dw)
            w8, w8t, sw = _cast_for_gemm(weight, e4m3_dtype, dl("weight"), is_amax_initialized, True, need_dx, kb_fwd, kb_dx,
                                          known_scale=mod._precomputed_weight_scale)
            if emulate:
                y = torch.ops.aten.mm_float8_emulated(x8, sx, w8.t(), sw, x.dtype)
            else:
                y = _gemm(x8, sx, w8, sw, x.dtype, kb_fwd)
            ctx.kb = (kb_dx, kb_dw)
            ctx.save_for_backward(x8t, w8t, sx, sw)
        ctx.mod = mod
        ctx.is_amax_initialized = is_amax_initialized
        ctx.x_shape = x.shape
        return y.reshape(*x.shape[:-1], n)

    @staticmethod
    def backward(ctx, dy):
        mod = ctx.mod
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        dy2 = dy.reshape(-1, dy.shape[-1])
        dlg = mod._delayed_buffers("grad_output")
        dx = dw = None
        if ctx.kb is None:  # one copy per tensor: x8 [K/64, M, 64], w8 [K/64, N, 64], g8 [N/64, M, 64]
            x8, w8, sx, sw = ctx.saved_tensors
            g8, _, sg = _cast_for_gemm(dy2, e5m2_dtype, dlg, ctx.is_amax_initialized, True, False, True, False)
            if need_dx:  # grad_input = dY @ W: dY as it is, W read transposed
                dx = _native.gemm_kb_ex(g8, False, sg, w8, True, sw, dy.dtype).reshape(ctx.x_shape)
            if need_dw:  # grad_weight = dY^T @ x: both read transposed
                dw = _native.gemm_kb_ex(g8, True, sg, x8, True, sx, dy.dtype)
            return dx, dw, None, None
        x8t, w8t, sx, sw = ctx.saved_tensors
        kb_dx, kb_dw = ctx.kb
        g8, g8t, sg = _cast_for_gemm(dy2, e5m2_dtype, dlg, ctx.is_amax_initialized, need_dx, need_dw, kb_dx, kb_dw)
        emulate = mod.linear_mm_config.grad_input.emulate
        if need_dx:  # grad_input = dY @ W          [M,N] x [N,K]
            if emulate:
                dx = torch.ops.aten.mm_float8_emulated(g8, sg, w8t.t(), sw, dy.dtype)
            else:
                dx = _gemm(g8, sg, w8t, sw, dy.dtype, kb_dx)
            dx = dx.reshape(ctx.x_shape)
        if need_dw:  # grad_weight = dY^T @ x       [N,M] x [M,K]
            if emulate:
                dw = torch.ops.aten.mm_float8_emulated(g8t, sg, x8t.t(), sx, dy.dtype)
            else:
                dw = _gemm(g8t, sg, x8t, sx, dy.dtype, kb_dw)
        return dx, dw, None, None


class Float8Linear(torch.nn.Linear):
    """``nn.Linear`` with float8 compute and per-tensor dynamic or delayed scaling
    (reference float8_linear.py:98-438).  Construct through ``from_float`` /
    ``convert_to_float8_training``; ``config`` is a required keyword."""

    def __init__(self, *args, **kwargs):
        self.always_float32_buffers = set()  # before nn.Module.__init__: _apply may run early
        # counts replacements of the delayed-scaling buffers (creation, .to(), ...): what caches of their addresses key on
        self._buffer_gen = 0
        self._static_marked_gen = -1
        config = kwargs.pop("config")
        super().__init__(*args, **kwargs)
        self.config = config
        # enable_fsdp_float8_all_gather: the one-GPU share of that flow is kept -- the weight's scale may be
        # computed ahead of the forward pass, for all layers in one launch
        # (precompute_float8_dynamic_scale_for_fsdp), and the forward then casts the weight with it.  The
        # reference wraps the weight in a tensor subclass for FSDP2's all-gather hooks; with one GPU there is
        # nothing to gather and the parameter stays a plain tensor.
        self._precomputed_weight_scale = None

        self.scaling_type_input = config.cast_config_input.scaling_type
        self.scaling_type_weight = config.cast_config_weight.scaling_type
        self.scaling_type_grad_output = config.cast_config_grad_output.scaling_type
        self.has_any_delayed_scaling = ScalingType.DELAYED in (
            self.scaling_type_input, self.scaling_type_weight, self.scaling_type_grad_output)

        self.create_buffers()

        mm = lambda g: ScaledMMConfig(config.emulate, g.use_fast_accum, False, config.pad_inner_dim)
        self.linear_mm_config = LinearMMConfig(mm(config.gemm_config_output), mm(config.gemm_config_grad_input),
                                               mm(config.gemm_config_grad_weight))

        # plain attributes, not buffers (not serialised; reference float8_linear.py:156-169)
        self.is_amax_initialized = not config.enable_amax_init
        self.amax_and_scale_synced = not config.enable_amax_init
        self.last_seen_input_dtype = None
        self.enable_pre_and_post_forward = config.enable_pre_and_post_forward

    # ---- buffers -------------------------------------------------------------------------

    def create_buffers(self):
        """amax (default: the fp8 format's max), zero history, scale 1 for each of the three
        tensors -- all nine as soon as any tensor is delayed (reference :180-222)."""
        if not self.has_any_delayed_scaling:
            return
        history_len = self.config.delayed_scaling_config.history_len
        device = self.weight.device
        defaults = {"input": torch.finfo(torch.float8_e4m3fn).max, "weight": torch.finfo(torch.float8_e4m3fn).max,
                    "grad_output": torch.finfo(torch.float8_e5m2).max}
        for kind in _KINDS:
            self.register_always_float32_buffer(f"fp8_amax_{kind}", torch.tensor([defaults[kind]], device=device))
            self.register_always_float32_buffer(f"fp8_amax_history_{kind}", torch.zeros(history_len, device=device))
            self.register_always_float32_buffer(f"fp8_scale_{kind}", torch.tensor([1.0], device=device))

    def register_always_float32_buffer(self, name: str, tensor: Optional[torch.Tensor], persistent: bool = True) -> None:
        self.register_buffer(name=name, tensor=tensor, persistent=persistent)
        self.always_float32_buffers.add(name)
        self._buffer_gen += 1

    def _apply(self, fn, recurse=True):
        ret = super()._apply(fn, recurse)
        self.convert_amax_buffer_to_float32()
        self._buffer_gen += 1
        return ret

    def __setattr__(self, name, value):
        if name in self.__dict__.get("always_float32_buffers", ()):  # a buffer assigned anew: addresses may have changed
            self.__dict__["_buffer_gen"] = self.__dict__.get("_buffer_gen", 0) + 1
        super().__setattr__(name, value)

    def _load_from_state_dict(self, *args, **kwargs):
        super()._load_from_state_dict(*args, **kwargs)  # load_state_dict(assign=True) swaps the buffer tensors
        self._buffer_gen += 1

    def convert_amax_buffer_to_float32(self):
        """``module.to(bf16)`` must not touch the bookkeeping precision (reference :224-238)."""
        for key in self.always_float32_buffers:
            if self._buffers[key] is not None:
                self._buffers[key] = self._buffers[key].to(torch.float32)

    def _delayed_buffers(self, kind: str) -> Optional[_DelayedBuffers]:
        if getattr(self, f"scaling_type_{kind}") is not ScalingType.DELAYED:
            return None
        return _DelayedBuffers(getattr(self, f"fp8_amax_{kind}"), getattr(self, f"fp8_amax_history_{kind}"),
                               getattr(self, f"fp8_scale_{kind}"))

    # ---- the reference's building blocks (same numbers as the fused path) -----------------

    def cast_input_to_float8(self, input: torch.Tensor, is_amax_initialized: bool) -> torch.Tensor:
        """reference :240-276"""
        input = self._autocast_input(input)
        if self.scaling_type_input is ScalingType.DELAYED:
            _maybe_initialize_amaxes_scales_for_float8_cast(
                input, self.fp8_amax_input, self.fp8_amax_history_input, self.fp8_scale_input,
                self.config.delayed_scaling_config.scale_fn_name, e4m3_dtype, is_amax_initialized, reduce_amax=True)
            return hp_tensor_to_float8_delayed(input, self.fp8_scale_input, e4m3_dtype, self.fp8_amax_input,
                                               linear_mm_config=self.linear_mm_config,
                                               gemm_input_role=GemmInputRole.INPUT)
        assert self.scaling_type_input is ScalingType.DYNAMIC
        return hp_tensor_to_float8_dynamic(input, e4m3_dtype, self.linear_mm_config)

    def cast_weight_to_float8(self, weight: torch.Tensor, is_amax_initialized: bool) -> torch.Tensor:
        """reference :278-316"""
        if isinstance(self.weight, Float8Tensor):  # already cast by a wrapper
            return self.weight
        if self.scaling_type_weight is ScalingType.DELAYED:
            _maybe_initialize_amaxes_scales_for_float8_cast(
                weight, self.fp8_amax_weight, self.fp8_amax_history_weight, self.fp8_scale_weight,
                self.config.delayed_scaling_config.scale_fn_name, e4m3_dtype, is_amax_initialized, reduce_amax=False)
            return hp_tensor_to_float8_delayed(weight, self.fp8_scale_weight, e4m3_dtype, self.fp8_amax_weight,
                                               linear_mm_config=self.linear_mm_config,
                                               gemm_input_role=GemmInputRole.WEIGHT)
        assert self.scaling_type_weight is ScalingType.DYNAMIC
        if self._precomputed_weight_scale is not None:  # what fsdp_pre_all_gather does (fsdp_utils.py:166-174)
            return hp_tensor_and_scale_to_float8(self.weight, self._precomputed_weight_scale, e4m3_dtype,
                                                 self.linear_mm_config, GemmInputRole.WEIGHT)
        return hp_tensor_to_float8_dynamic(self.weight, e4m3_dtype, self.linear_mm_config,
                                           gemm_input_role=GemmInputRole.WEIGHT)

    def cast_output_to_float8_in_bw(self, output: torch.Tensor) -> torch.Tensor:
        """reference :318-333"""
        if self.scaling_type_grad_output is ScalingType.DELAYED:
            return NoopFwToFloat8E5M2BwDelayed.apply(
                output, self.fp8_amax_grad_output, self.fp8_amax_history_grad_output, self.fp8_scale_grad_output,
                self.config.delayed_scaling_config.scale_fn_name, self.is_amax_initialized, self.linear_mm_config)
        assert self.scaling_type_grad_output is ScalingType.DYNAMIC
        return NoopFwToFloat8E5M2BwDynamic.apply(output, self.linear_mm_config)

    def forward_composed(self, input: torch.Tensor) -> torch.Tensor:
        """The reference's op-by-op composition (reference :356-373); same results as ``forward``."""
        if self.has_any_delayed_scaling:
            self.float8_pre_forward(input)
        return self._forward_composed_body(input)

    # ---- bookkeeping -----------------------------------------------------------------------

    def _autocast_input(self, input: torch.Tensor) -> torch.Tensor:
        # what F.linear's autocast rule would do to the activation (reference :245-249)
        if torch.is_autocast_enabled():
            input = input.to(torch.get_autocast_dtype('cuda'))
        return input

    def float8_pre_forward(self, input):
        if not self.enable_pre_and_post_forward:
            return
        if self.is_amax_initialized and (not self.amax_and_scale_synced) and torch.is_grad_enabled():
            raise AssertionError(
                "amaxes and scales not synced, please call `sync_float8_amax_and_scale_history` before forward")
        self.last_seen_input_dtype = input.dtype

    def float8_post_forward(self):
        if not self.enable_pre_and_post_forward:
            return
        # the next forward must be preceded by a sync
        self.is_amax_initialized = True
        self.amax_and_scale_synced = False

    # ---- forward ---------------------------------------------------------------------------

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if torch.compiler.is_compiling():
            return self._forward_under_compile(input)
        return self._forward_eager(input)

    def _forward_under_compile(self, input: torch.Tensor) -> torch.Tensor:
        """What ``torch.compile`` traces: one custom-op node per direction (plus the bias add), with the delayed-scaling
        buffers as arguments the node writes -- or, for ``emulate=True`` and pre-cast operands, the reference's op-by-op
        composition.  Anything that keeps Python state -- the first-iteration amax initialisation, the pre/post-forward
        flags (``enable_amax_init`` / ``enable_pre_and_post_forward``: switch both off for a graph without breaks, as
        with the reference) -- runs outside the graph."""
        stateless = (not self.has_any_delayed_scaling
                     or (self.is_amax_initialized and not self.enable_pre_and_post_forward))
        if not stateless:
            return self._forward_outside_graph(input)
        plain = (not self.config.emulate and self._precomputed_weight_scale is None
                 and not isinstance(self.weight, Float8Tensor) and not isinstance(input, Float8Tensor))
        if not plain:
            # emulate=True, a precomputed weight scale, operands that are Float8Tensors already: the reference's own
            # composition, whose pieces (casts, the matmul of two Float8Tensors, the emulated aten op) are opaque nodes
            return self._forward_composed_body(input)
        from ._custom_ops import linear

        def bufs(kind):
            if getattr(self, f"scaling_type_{kind}") is not ScalingType.DELAYED:
                return None
            return getattr(self, f"fp8_amax_{kind}"), getattr(self, f"fp8_scale_{kind}")

        output = linear(self._autocast_input(input), self.weight, bufs("input"), bufs("weight"), bufs("grad_output"))
        if self.bias is not None:
            output = output + self.bias.to(output.dtype)
        return output

    @torch._dynamo.disable
    def _forward_outside_graph(self, input: torch.Tensor) -> torch.Tensor:
        return self._forward_eager(input)

    def _forward_eager(self, input: torch.Tensor) -> torch.Tensor:
        if self.has_any_delayed_scaling:
            self.float8_pre_forward(input)
        if isinstance(self.weight, Float8Tensor) or isinstance(input, Float8Tensor):
            # pre-cast operands: only the composed path knows how to pass them through
            return self._forward_composed_body(input)
        x = self._autocast_input(input)
        output = _float8_linear_fn.apply(x, self.weight, self, self.is_amax_initialized)
        if self.bias is not None:
            output = output + self.bias.to(output.dtype)
        if self.has_any_delayed_scaling:
            self.float8_post_forward()
        return output

    def _forward_composed_body(self, input):
        input_fp8 = self.cast_input_to_float8(input, self.is_amax_initialized)
        weight_fp8 = self.cast_weight_to_float8(self.weight, self.is_amax_initialized)
        output = manual_float8_matmul.apply(input_fp8, weight_fp8.t())
        output = self.cast_output_to_float8_in_bw(output)
        if self.bias is not None:
            output = output + self.bias.to(output.dtype)
        if self.has_any_delayed_scaling:
            self.float8_post_forward()
        return output

    def scaling_repr(self):
        """e.g. ``i:del,w:dyn,go:dyn``"""
        return (f"i:{self.scaling_type_input.short_str()},w:{self.scaling_type_weight.short_str()},"
                f"go:{self.scaling_type_grad_output.short_str()}")

    def extra_repr(self):
        return f'{super().extra_repr()}, scaling="{self.scaling_repr()}"'

    @classmethod
    def from_float(cls, mod, config: Optional[Float8LinearConfig] = None):
        """A Float8Linear sharing ``mod``'s parameters (reference :384-438)."""
        if config is None:
            config = Float8LinearConfig()
        with torch.device("meta"):
            new_mod = cls(mod.in_features, mod.out_features, bias=False, config=config)
        new_mod.weight = mod.weight
        new_mod.bias = mod.bias
        new_mod.create_buffers()  # again, now on the weight's real device
        return new_mod
