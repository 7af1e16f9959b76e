"""The one-GPU share of the reference's FSDP2 float8 all-gather flow (``fsdp_utils.py``).

In the reference every rank (1) computes max|w| of all its weight shards with one
``torch._foreach_norm``, all-reduces the stacked result and turns it into scales
(``precompute_float8_dynamic_scale_for_fsdp``, ``fsdp_utils.py:29-66``), (2) casts its shard to fp8 with
that scale just before the all-gather (``fsdp_pre_all_gather``, ``:163-182``) and (3) wraps the gathered
bytes as a ``Float8Tensor`` that the forward uses as it is (``fsdp_post_all_gather``).  This build drives one
GPU: there is nothing to reduce or gather, and what is left of (1)-(3) is kept -- the scales of all weights
in ONE pass of three launches (``f8mi_amax_scale_multi``), stored on the modules, and a forward that casts
the weight with the stored scale instead of reading the weight twice.  Weights that are ``DTensor``s
(a model that really went through ``fully_shard``) are refused.
"""
import torch
import torch.nn as nn

from . import _native
from .float8_utils import e4m3_dtype


@torch.no_grad()
def precompute_float8_dynamic_scale_for_fsdp(module: nn.Module) -> None:
    """Computes the fp8 scale of every dynamically scaled ``Float8Linear`` weight created with
    ``enable_fsdp_float8_all_gather=True``; call it after the optimizer step, as in the reference:

        model(input).sum().backward()
        optim.step()
        precompute_float8_dynamic_scale_for_fsdp(model)

    The next forward of each such layer casts its weight with this scale.  A scale stays in use until the
    next call replaces it, so the call belongs after EVERY optimizer step (the reference has the same contract).
    Same values as the per-tensor path: scale = fmax / clamp(max|w|, 1e-12) in the weight's dtype.
    """
    from .config import ScalingType
    from .float8_linear import Float8Linear
    from .float8_tensor import Float8Tensor

    if any(isinstance(m, Float8Linear) and m.scaling_type_weight is ScalingType.DELAYED for m in module.modules()):
        raise NotImplementedError("Only supports dynamic scaling")
    layers = [m for m in module.modules()
              if isinstance(m, Float8Linear) and m.config.enable_fsdp_float8_all_gather
              and not isinstance(m.weight, Float8Tensor)]
    if not layers:
        return
    if any(type(m.weight.data).__name__ == "DTensor" for m in layers):
        raise NotImplementedError("sharded (DTensor) weights need the FSDP2 all-gather flow over several GPUs; "
                                  "this build drives a single MI355X")
    groups = {}
    for m in layers:
        w = m.weight.detach()
        if w.is_contiguous() and w.data_ptr() % 16 == 0:
            groups.setdefault((w.device, w.dtype), []).append((m, w))
        else:  # a weight the multi-tensor kernel does not take: its own pass
            _, m._precomputed_weight_scale = _native.amax_scale(w, e4m3_dtype, want_amax=False)
    for members in groups.values():
        _, scales = _native.amax_scale_multi([w for _, w in members], e4m3_dtype)
        for i, (m, _) in enumerate(members):
            m._precomputed_weight_scale = scales[i]
