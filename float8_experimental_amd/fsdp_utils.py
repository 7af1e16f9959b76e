"""FSDP2 float8 all-gather hooks live here in the reference; they need several GPUs and are not
part of this single-GPU build.  The one name the reference exports from here is kept so that
``from float8_experimental import *``-style imports keep working."""


def precompute_float8_dynamic_scale_for_fsdp(module) -> None:
    raise NotImplementedError(
        "precompute_float8_dynamic_scale_for_fsdp belongs to the FSDP2 float8 all-gather flow, which needs "
        "more than one GPU; this build drives a single MI355X")
