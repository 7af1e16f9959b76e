"""Module swap and delayed-scaling bookkeeping (mirror of the reference's ``float8_linear_utils.py``)."""
import logging
import weakref
from typing import Callable, List, Optional

import torch
import torch.nn as nn

from . import _native
from .config import Float8LinearConfig, ScalingType
from .float8_linear import Float8Linear
from .float8_utils import e4m3_dtype, e5m2_dtype

log = logging.getLogger(__name__)
log.addHandler(logging.NullHandler())

_KINDS = (("input", e4m3_dtype), ("weight", e4m3_dtype), ("grad_output", e5m2_dtype))


def linear_requires_sync(config: Float8LinearConfig) -> bool:
    """True when any of the three tensors uses delayed scaling (reference :26-34)."""
    return ScalingType.DELAYED in (config.cast_config_input.scaling_type, config.cast_config_weight.scaling_type,
                                   config.cast_config_grad_output.scaling_type)


def _update_history_stack(new_amax: torch.Tensor, amax_history_stack: torch.Tensor) -> torch.Tensor:
    """Shifts every row of ``amax_history_stack`` [n, H] right by one and puts ``new_amax`` [n, 1]
    in column 0, in place (reference :37-56)."""
    assert amax_history_stack.dim() == 2, f"Expected amat_history_stack to be 2D, got {amax_history_stack.shape}"
    assert new_amax.size(0) == amax_history_stack.size(0), (
        f"Expected new_amax to have the same size as the first dimension of amax_history_stack, got "
        f"{new_amax.size(0)} and {amax_history_stack.size(0)}")
    shifted = torch.roll(amax_history_stack, 1, dims=1)
    shifted[:, 0] = new_amax.squeeze(-1)
    amax_history_stack.copy_(shifted)


def swap_linear_layers(module: nn.Module, from_float_func: Callable[[nn.Linear], nn.Linear], *,
                       module_filter_fn: Optional[Callable[[nn.Module, str], bool]] = None) -> nn.Module:
    """Replaces every ``nn.Linear`` that passes ``module_filter_fn(module, fqn)`` by
    ``from_float_func(module)`` (reference :59-122).  A root-level ``nn.Linear`` cannot be replaced
    in place and is returned converted instead; children are visited before their parents."""
    wanted = lambda m, fqn: isinstance(m, nn.Linear) and (module_filter_fn is None or module_filter_fn(m, fqn))
    if wanted(module, ""):
        if len(list(module.children())) > 0:
            raise AssertionError(f"Does not support a root nn.Linear with children: {module}")
        return from_float_func(module)

    def visit(mod: nn.Module, fqn: str, parent: Optional[nn.Module], name: str):
        for child_name, child in list(mod.named_children()):
            visit(child, child_name if fqn == "" else f"{fqn}.{child_name}", mod, child_name)
        if wanted(mod, fqn):
            assert parent is not None, f"Linear root module should return early: {mod}"
            setattr(parent, name, from_float_func(mod))

    visit(module, "", None, "")
    return module


def convert_to_float8_training(module: nn.Module, *, module_filter_fn: Optional[Callable[[nn.Module, str], bool]] = None,
                               config: Float8LinearConfig = None) -> nn.Module:
    """Swaps ``nn.Linear`` modules for ``Float8Linear`` (reference :125-154)."""
    if config is None:
        config = Float8LinearConfig()
    return swap_linear_layers(module, lambda m: Float8Linear.from_float(m, config=config),
                              module_filter_fn=module_filter_fn)


def get_float8_layers(model: torch.nn.Module) -> List[Float8Linear]:
    """All Float8Linear modules of ``model``; outside a compiled region their buffers are marked as living at
    fixed addresses, so that a compiled sync or step treats them as static inputs (reference :157-169)."""
    fp8_layers = [m for m in model.modules() if isinstance(m, Float8Linear)]
    if not torch.compiler.is_compiling():
        for layer in fp8_layers:
            if layer._static_marked_gen != layer._buffer_gen:  # once per set of buffers, not on every call
                for buf in layer.buffers():
                    torch._dynamo.mark_static_address(buf, guard=True)
                layer._static_marked_gen = layer._buffer_gen
    return fp8_layers


_tables = {}


def _sync_table(fp8_layers) -> torch.Tensor:
    """Device table of (amax, history, scale, format) pointers for all 3L buffers.  Cached per list of layers for as
    long as none of them has had its buffers replaced (``Float8Linear._buffer_gen`` counts that): a sync of 80 layers
    then costs the host a tuple of 80 pairs and 80 weak-reference checks instead of 720 pointer look-ups.

    ``id()`` of a layer that has been freed can come back for a new layer with the same generation count, so an
    entry also keeps a weak reference to each layer and counts as a hit only while all of them are the layers asked
    for; and it holds the buffer tensors themselves, so the addresses in the table stay allocated for as long as
    the entry lives."""
    key = tuple((id(child), child._buffer_gen) for child in fp8_layers)
    hit = _tables.get(key)
    if hit is not None and all(ref() is child for ref, child in zip(hit[1], fp8_layers)):
        return hit[0]
    if len(_tables) > 16:
        _tables.clear()
    entries = [(getattr(child, f"fp8_amax_{kind}"), getattr(child, f"fp8_amax_history_{kind}"), getattr(child, f"fp8_scale_{kind}"), f8)
               for child in fp8_layers for kind, f8 in _KINDS]
    table = _native.sync_table_cached(entries)
    _tables[key] = (table, [weakref.ref(child) for child in fp8_layers], entries)
    return table


@torch.no_grad()
def sync_float8_amax_and_scale_history(model: torch.nn.Module, fp8_layers=None) -> None:
    """Turns the amaxes recorded during the last iteration into the scales of the next one and marks
    the layers synced (reference :172-327).

    For every layer and each of input / weight / grad_output:
    ``S = roll(history, 1); S[0] = amax; scale = fmax / max(S)`` (fp32, two roundings).  Like the
    reference -- which rolls a stacked copy and copies only the scales back (:287-319) -- the
    layers' history buffers themselves are left as they are.  All of it is one kernel launch.
    The MAX all-reduce of the amaxes over ranks (:261-284) needs more than one GPU.
    """
    if fp8_layers is None:
        fp8_layers = get_float8_layers(model)
    if len(fp8_layers) == 0:
        log.warning("Calling sync_float8_amax_and_scale_history on a module with no Float8Linear layers")
        return

    x_dtypes = {child.last_seen_input_dtype for child in fp8_layers}
    if len(x_dtypes) != 1:
        raise ValueError(f"All layers must have the same last seen input_dtype, got {x_dtypes}")
    recipes = {child.config.delayed_scaling_config.scale_fn_name for child in fp8_layers}
    if len(recipes) != 1:
        raise ValueError(f"All layers must have the same scale_fn recipe, got {recipes}")
    hist_lens = {child.config.delayed_scaling_config.history_len for child in fp8_layers}
    if len(hist_lens) != 1:
        raise ValueError(f"All layers must have the same history_len, got {hist_lens}")
    if torch.distributed.is_available() and torch.distributed.is_initialized() and torch.distributed.get_world_size() > 1:
        raise NotImplementedError("amax all-reduce across ranks: this build drives a single GPU")

    orig_is_fp16 = next(iter(x_dtypes)) is torch.float16
    if torch.compiler.is_compiling():
        # the same launch as one opaque node that writes the scale buffers (reference: test_compile.py:257-274
        # compiles this function into a single frame)
        from ._custom_ops import sync

        rows = [(child, kind, f8) for child in fp8_layers for kind, f8 in _KINDS]
        sync([getattr(c, f"fp8_amax_{kind}") for c, kind, _ in rows],
             [getattr(c, f"fp8_amax_history_{kind}") for c, kind, _ in rows],
             [getattr(c, f"fp8_scale_{kind}") for c, kind, _ in rows],
             [f8 is e5m2_dtype for _, _, f8 in rows], orig_is_fp16)
    else:
        _native.sync(_sync_table(fp8_layers), next(iter(hist_lens)), orig_is_fp16, writeback_history=False)

    for child in fp8_layers:
        child.amax_and_scale_synced = True
