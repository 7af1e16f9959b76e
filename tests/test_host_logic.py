"""Host-side behaviour of the API mirror: configs, module swap, flags, error paths.  No GPU, no compute."""
import copy
import logging

import pytest
import torch
import torch.nn as nn

import float8_experimental_amd as f8
from float8_experimental_amd import _native
from float8_experimental_amd.config import CastConfig, DelayedScalingConfig, Float8GemmConfig, Float8LinearConfig, ScalingType
from float8_experimental_amd.float8_linear import Float8Linear
from float8_experimental_amd.float8_linear_utils import (
    convert_to_float8_training,
    get_float8_layers,
    linear_requires_sync,
    swap_linear_layers,
    sync_float8_amax_and_scale_history,
)
from float8_experimental_amd.float8_tensor import (
    choose_scaled_mm_config,
    Float8Tensor,
    GemmInputRole,
    LinearMMConfig,
    ScaledMMConfig,
)
from float8_experimental_amd.float8_utils import _get_min_alignment, is_row_major, pad_tensor_for_matmul

DEL, DYN = ScalingType.DELAYED, ScalingType.DYNAMIC


def cfg(i=DYN, w=DYN, g=DYN, **kw):
    return Float8LinearConfig(cast_config_input=CastConfig(i), cast_config_weight=CastConfig(w),
                              cast_config_grad_output=CastConfig(g), **kw)


def test_public_names_match_the_reference():
    assert sorted(f8.__all__) == sorted([
        "DelayedScalingConfig", "ScalingType", "Float8GemmConfig", "Float8LinearConfig", "CastConfig",
        "convert_to_float8_training", "linear_requires_sync", "sync_float8_amax_and_scale_history",
        "precompute_float8_dynamic_scale_for_fsdp"])
    for name in f8.__all__ + ["Float8Tensor", "Float8Linear", "GemmInputRole", "LinearMMConfig", "ScaledMMConfig"]:
        assert hasattr(f8, name)


def test_config_defaults_and_enums():
    c = Float8LinearConfig()
    assert c.cast_config_input.scaling_type is DYN and c.cast_config_weight.scaling_type is DYN
    assert c.cast_config_grad_output.scaling_type is DYN
    assert c.gemm_config_output.use_fast_accum is True and c.gemm_config_grad_input.use_fast_accum is False
    assert (c.enable_amax_init, c.enable_pre_and_post_forward, c.enable_fsdp_float8_all_gather, c.pad_inner_dim,
            c.emulate) == (True, True, False, False, False)
    assert c.delayed_scaling_config == DelayedScalingConfig(history_len=16, scale_fn_name="max")
    assert ScalingType.DELAYED.value == "delayed" and ScalingType.DYNAMIC.value == "dynamic"
    assert DEL.short_str() == "del" and DYN.short_str() == "dyn"
    with pytest.raises(AssertionError):
        DelayedScalingConfig(scale_fn_name="mean")
    with pytest.raises(Exception):  # frozen
        c.emulate = True
    assert linear_requires_sync(cfg()) is False
    for combo in [(DEL, DYN, DYN), (DYN, DEL, DYN), (DYN, DYN, DEL)]:
        assert linear_requires_sync(cfg(*combo)) is True


def test_mm_config_selection():
    a = LinearMMConfig()
    assert a.output == ScaledMMConfig(False, True, False, False)
    R = GemmInputRole
    assert choose_scaled_mm_config(R.INPUT, a, R.WEIGHT, a) is a.output
    assert choose_scaled_mm_config(R.GRAD_OUTPUT, a, R.WEIGHT, a) is a.grad_input
    assert choose_scaled_mm_config(R.GRAD_OUTPUT, a, R.INPUT, a) is a.grad_weight
    b = LinearMMConfig(ScaledMMConfig(True, False, False, False), a.grad_input, ScaledMMConfig(True, False, False, False))
    with pytest.raises(AssertionError, match="linear_mm_config.output mismatch"):
        choose_scaled_mm_config(R.INPUT, a, R.WEIGHT, b)
    with pytest.raises(AssertionError, match="linear_mm_config.grad_weight mismatch"):
        choose_scaled_mm_config(R.GRAD_OUTPUT, a, R.INPUT, b)
    with pytest.raises(AssertionError, match="unexpected a_role"):
        choose_scaled_mm_config(R.WEIGHT, a, R.INPUT, a)


def test_swap_root_linear_and_children():
    lin = nn.Linear(16, 32)
    out = convert_to_float8_training(lin)
    assert isinstance(out, Float8Linear) and out.weight is lin.weight and out.bias is lin.bias
    assert type(lin) is nn.Linear  # a root linear is not modified in place

    class Odd(nn.Linear):
        def __init__(self):
            super().__init__(4, 4)
            self.child = nn.Linear(4, 4)

    with pytest.raises(AssertionError, match="Does not support a root nn.Linear with children"):
        convert_to_float8_training(Odd())


def test_swap_nested_and_filters():
    def build():
        return nn.Sequential(nn.Linear(8, 16), nn.ReLU(), nn.Sequential(nn.Linear(16, 32), nn.Linear(32, 40)),
                             nn.ModuleList([nn.Linear(40, 8)]))

    m = convert_to_float8_training(build())
    assert [type(x).__name__ for x in m.modules() if isinstance(x, nn.Linear)] == ["Float8Linear"] * 4
    assert len(get_float8_layers(m)) == 4
    # filter by shape: only dims divisible by 16 (the reference's example filter)
    m = convert_to_float8_training(build(), module_filter_fn=lambda mod, fqn: mod.in_features % 16 == 0 and mod.out_features % 16 == 0)
    kinds = {fqn: type(mod).__name__ for fqn, mod in m.named_modules() if isinstance(mod, nn.Linear)}
    assert kinds == {"0": "Linear", "2.0": "Float8Linear", "2.1": "Linear", "3.0": "Linear"}
    # filter by fully qualified name
    seen = []
    m = convert_to_float8_training(build(), module_filter_fn=lambda mod, fqn: seen.append(fqn) or fqn in ("2.1", "3.0"))
    assert sorted(seen) == ["0", "2.0", "2.1", "3.0"]
    kinds = {fqn: type(mod).__name__ for fqn, mod in m.named_modules() if isinstance(mod, nn.Linear)}
    assert kinds == {"0": "Linear", "2.0": "Linear", "2.1": "Float8Linear", "3.0": "Float8Linear"}
    # a custom from_float function goes through swap_linear_layers
    m = swap_linear_layers(build(), lambda lin: nn.Identity())
    assert not any(isinstance(x, nn.Linear) for x in m.modules())


def test_buffers_defaults_repr_and_dtype_moves():
    m = Float8Linear.from_float(nn.Linear(16, 32), config=cfg(DYN, DEL, DYN, delayed_scaling_config=DelayedScalingConfig(history_len=4)))
    assert m.scaling_repr() == "i:dyn,w:del,go:dyn"
    assert 'scaling="i:dyn,w:del,go:dyn"' in repr(m)
    names = sorted(n for n, _ in m.named_buffers())
    assert names == sorted(f"fp8_{a}_{k}" for a in ("amax", "amax_history", "scale") for k in ("input", "weight", "grad_output"))
    assert m.fp8_amax_input.item() == 448.0 and m.fp8_amax_weight.item() == 448.0 and m.fp8_amax_grad_output.item() == 57344.0
    assert m.fp8_amax_history_weight.shape == (4,) and bool((m.fp8_amax_history_weight == 0).all())
    assert m.fp8_scale_grad_output.item() == 1.0 and m.fp8_scale_input.shape == (1,)
    assert set(m.state_dict().keys()) == set(names) | {"weight", "bias"}  # persistent: checkpoints carry them
    m = m.to(torch.bfloat16)
    assert m.weight.dtype == torch.bfloat16
    assert all(b.dtype == torch.float32 for b in m.buffers())  # bookkeeping stays fp32
    m = m.half().float().double()
    assert all(b.dtype == torch.float32 for b in m.buffers())
    # all-dynamic layers carry no buffers at all
    assert len(list(Float8Linear.from_float(nn.Linear(4, 4)).buffers())) == 0
    # flags
    assert m.is_amax_initialized is False and m.amax_and_scale_synced is False
    m2 = Float8Linear.from_float(nn.Linear(4, 4), config=cfg(DEL, DEL, DEL, enable_amax_init=False))
    assert m2.is_amax_initialized is True and m2.amax_and_scale_synced is True
    assert copy.deepcopy(m2).scaling_repr() == "i:del,w:del,go:del"


def test_unsynced_forward_is_refused_before_any_compute():
    m = Float8Linear.from_float(nn.Linear(16, 32), config=cfg(DEL, DEL, DEL))
    m.is_amax_initialized = True  # as after a first forward
    m.amax_and_scale_synced = False
    with pytest.raises(AssertionError, match="amaxes and scales not synced"):
        m(torch.randn(2, 16))
    with torch.no_grad():  # the guard only applies when grad is enabled; then compute starts -> needs a GPU
        with pytest.raises(_native.Float8NativeError, match="no CPU fallback"):
            m(torch.randn(2, 16))


def test_cpu_tensors_fail_loudly_everywhere():
    m = convert_to_float8_training(nn.Sequential(nn.Linear(16, 32)))
    with pytest.raises(_native.Float8NativeError):
        m(torch.randn(4, 16))
    from float8_experimental_amd.float8_utils import amax_to_scale, tensor_to_amax, tensor_to_scale, to_fp8_saturated

    x = torch.randn(4, 4)
    for fn in (lambda: tensor_to_amax(x), lambda: tensor_to_scale(x, torch.float8_e4m3fn),
               lambda: to_fp8_saturated(x, torch.float8_e5m2), lambda: amax_to_scale(x.max(), torch.float8_e4m3fn, x.dtype)):
        with pytest.raises(_native.Float8NativeError):
            fn()
    with pytest.raises(ValueError, match="Unsupported float8_dtype"):
        tensor_to_scale(x, torch.float16)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", str(tmp_path / "libf8mi.so"))
    with pytest.raises(_native.Float8NativeError, match="no fallback"):
        _native.lib()


def test_sync_host_checks(caplog):
    with caplog.at_level(logging.WARNING):
        sync_float8_amax_and_scale_history(nn.Sequential(nn.Linear(4, 4)))
    assert "no Float8Linear layers" in caplog.text
    m = convert_to_float8_training(nn.Sequential(nn.Linear(8, 8), nn.Linear(8, 8)), config=cfg(DEL, DEL, DEL))
    m[0].last_seen_input_dtype, m[1].last_seen_input_dtype = torch.bfloat16, torch.float32
    with pytest.raises(ValueError, match="same last seen input_dtype"):
        sync_float8_amax_and_scale_history(m)
    # a model mixing all-dynamic and delayed layers has no buffers to read on the dynamic layer
    mixed = nn.Sequential(Float8Linear.from_float(nn.Linear(4, 4)), Float8Linear.from_float(nn.Linear(4, 4), config=cfg(DEL, DEL, DEL)))
    with pytest.raises(AttributeError):
        sync_float8_amax_and_scale_history(mixed)


def test_fsdp_flag_and_precompute_on_the_host():
    """enable_fsdp_float8_all_gather keeps its one-GPU meaning (scales of all weights computed ahead, in one pass);
    the host-side rules follow the reference (fsdp_utils.py:29-66)."""
    from float8_experimental_amd._native import Float8NativeError

    lin = Float8Linear.from_float(nn.Linear(4, 4), config=Float8LinearConfig(enable_fsdp_float8_all_gather=True))
    assert lin._precomputed_weight_scale is None
    # nothing to do: no layer was created with the flag (the reference returns silently as well)
    assert f8.precompute_float8_dynamic_scale_for_fsdp(nn.Linear(4, 4)) is None
    assert f8.precompute_float8_dynamic_scale_for_fsdp(nn.Sequential(Float8Linear.from_float(nn.Linear(4, 4)))) is None
    # delayed weight scaling anywhere in the model is refused
    with pytest.raises(NotImplementedError):
        f8.precompute_float8_dynamic_scale_for_fsdp(nn.Sequential(Float8Linear.from_float(nn.Linear(4, 4), config=cfg(DYN, DEL, DYN))))
    # and the computation itself needs the GPU: no CPU fallback
    with pytest.raises(Float8NativeError):
        f8.precompute_float8_dynamic_scale_for_fsdp(nn.Sequential(lin))


def test_tensor_parallel_styles_say_that_they_need_several_gpus():
    from float8_experimental_amd.float8_tensor_parallel import (Float8ColwiseParallel, Float8RowwiseParallel,
                                                                PrepareFloat8ModuleInput)

    for style in (Float8ColwiseParallel, Float8RowwiseParallel, PrepareFloat8ModuleInput):
        with pytest.raises(NotImplementedError, match="single MI355X"):
            style()


def test_float8_tensor_metadata_on_cpu():
    data = torch.zeros(4, 8, dtype=torch.float8_e4m3fn)
    t = Float8Tensor(data, torch.tensor(2.0), torch.bfloat16, None)
    assert t.dtype == torch.bfloat16 and t.shape == (4, 8) and t._linear_mm_config == LinearMMConfig()
    assert t._gemm_input_role is GemmInputRole.INPUT
    with pytest.raises(AssertionError, match="Scale should contain a single value"):
        Float8Tensor(data, torch.ones(2), torch.bfloat16, None)
    inner, meta = t.__tensor_flatten__()
    back = Float8Tensor.__tensor_unflatten__({"_data": t._data, "_scale": t._scale}, meta, None, None)
    assert back._orig_dtype == torch.bfloat16 and inner == ["_data", "_scale"]
    # view-type ops keep the metadata; unknown ops are refused
    tt = t.t()
    assert isinstance(tt, Float8Tensor) and tt.shape == (8, 4) and tt._scale is t._scale
    assert isinstance(t.view(2, 16), Float8Tensor) and isinstance(t[1:3], Float8Tensor)
    with pytest.raises(NotImplementedError, match="not supported"):
        torch.sin(t)


def test_padding_helpers():
    assert _get_min_alignment(10, 8) == 16 and _get_min_alignment(16, 16) == 16 and _get_min_alignment(0, 16) == 0
    assert pad_tensor_for_matmul(torch.randn(10, 10), dims=0).shape == (16, 10)
    assert pad_tensor_for_matmul(torch.randn(10, 10), dims=1).shape == (10, 16)
    assert pad_tensor_for_matmul(torch.randn(10, 10), dims=(0, 1)).shape == (16, 16)
    x = torch.randn(16, 32)
    assert pad_tensor_for_matmul(x, dims=(0, 1)) is x
    p = pad_tensor_for_matmul(torch.ones(3, 41).to(torch.float8_e4m3fn), dims=1)
    assert p.shape == (3, 48) and p.dtype == torch.float8_e4m3fn and bool((p.view(torch.uint8)[:, 41:] == 0).all())
    assert is_row_major((8, 1)) and not is_row_major((1, 8))


def test_emulated_mm_is_registered_as_an_aten_op():
    """Schema and Meta implementation of torch.ops.aten.mm_float8_emulated (reference float8_aten_api.py:37-49);
    no CPU kernel is registered: this package computes on the GPU only."""
    import float8_experimental_amd  # noqa: F401

    op = torch.ops.aten.mm_float8_emulated.default
    assert str(op._schema) == "aten::mm_float8_emulated(Tensor m1, Tensor s1, Tensor m2, Tensor s2, ScalarType dtype3) -> Tensor"
    m1 = torch.empty(5, 7, dtype=torch.float8_e4m3fn, device="meta")
    m2 = torch.empty(7, 3, dtype=torch.float8_e5m2, device="meta")
    s = torch.empty((), device="meta")
    out = op(m1, s, m2, s, torch.bfloat16)
    assert out.shape == (5, 3) and out.dtype == torch.bfloat16 and out.device.type == "meta"
    with pytest.raises(NotImplementedError):
        op(torch.zeros(2, 2).to(torch.float8_e4m3fn), torch.ones(()), torch.zeros(2, 2).to(torch.float8_e4m3fn), torch.ones(()), torch.float32)


def test_primitive_custom_ops_have_fake_implementations():
    """f8mi::amax_scale / cast / gemm_nt trace with fake tensors (shapes and dtypes only, no GPU)."""
    import float8_experimental_amd  # noqa: F401
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        x = torch.empty(6, 10, 32, dtype=torch.bfloat16, device="cuda")
        amax, scale = torch.ops.f8mi.amax_scale(x, torch.float8_e4m3fn, torch.bfloat16, False)
        assert amax.shape == () and scale.shape == () and scale.dtype == torch.float32
        bits, a = torch.ops.f8mi.cast(x, scale, torch.float8_e5m2, torch.bfloat16, True)
        assert bits.shape == x.shape and bits.dtype == torch.float8_e5m2 and a.shape == (1,)
        bits, a = torch.ops.f8mi.cast(x, scale, torch.float8_e4m3fn, torch.float32, False)
        assert a.numel() == 0
        a8 = torch.empty(12, 64, dtype=torch.float8_e4m3fn, device="cuda")
        b8 = torch.empty(20, 64, dtype=torch.float8_e4m3fn, device="cuda")
        y = torch.ops.f8mi.gemm_nt(a8, scale, b8, scale, torch.float16, None)
        assert y.shape == (12, 20) and y.dtype == torch.float16


def test_get_float8_layers_marks_buffers_static():
    """Reference float8_linear_utils.py:157-169: buffers of the delayed-scaling layers are marked as static addresses."""
    import float8_experimental_amd as f8

    cfg = f8.Float8LinearConfig(cast_config_input=f8.CastConfig(f8.ScalingType.DELAYED))
    model = torch.nn.Sequential(torch.nn.Linear(8, 8), torch.nn.ReLU(), torch.nn.Linear(8, 8))
    f8.convert_to_float8_training(model, config=cfg)
    layers = f8.float8_linear_utils.get_float8_layers(model)
    assert len(layers) == 2
    for layer in layers:
        bufs = list(layer.buffers())
        assert len(bufs) == 9
        for buf in bufs:
            assert getattr(buf, "_dynamo_static_input_type", None) == "guarded"


def test_sync_table_cache_does_not_trust_a_recycled_object_id(monkeypatch):
    """The pointer table of sync_float8_amax_and_scale_history is cached per (id(layer), buffer generation).  A layer
    that has been freed can hand its id() to a new layer with the same generation count: an entry left by the dead
    layer must not be served for the new one (it holds the dead layer's addresses)."""
    import gc
    import weakref

    from float8_experimental_amd import float8_linear_utils as flu

    cfg = f8.Float8LinearConfig(cast_config_input=f8.CastConfig(f8.ScalingType.DELAYED))
    layer = Float8Linear.from_float(nn.Linear(8, 8), config=cfg)
    built = []
    monkeypatch.setattr(_native, "sync_table_cached", lambda entries: built.append(list(entries)) or ("table", len(built)))
    monkeypatch.setattr(flu, "_tables", {})

    first = flu._sync_table([layer])
    assert flu._sync_table([layer]) is first and len(built) == 1  # same live layer, same buffers: a hit
    assert [t for row in flu._tables[next(iter(flu._tables))][2] for t in row[:3]] == [
        getattr(layer, f"fp8_{what}_{kind}") for kind in ("input", "weight", "grad_output") for what in ("amax", "amax_history", "scale")]

    # what a dead layer of the same id and generation leaves behind
    ghost = Float8Linear.from_float(nn.Linear(8, 8), config=cfg)
    dead = weakref.ref(ghost)
    del ghost
    gc.collect()
    assert dead() is None
    key = ((id(layer), layer._buffer_gen),)
    flu._tables[key] = ("stale", [dead], [])
    fresh = flu._sync_table([layer])
    assert fresh != "stale" and len(built) == 2
    assert flu._sync_table([layer]) is fresh and len(built) == 2

    # replaced buffers: the generation moves and the table is rebuilt from the new tensors
    layer.fp8_amax_input = torch.zeros(())
    assert flu._sync_table([layer]) is not fresh and len(built) == 3
    assert built[-1][0][0] is layer.fp8_amax_input
