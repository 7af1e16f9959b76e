"""torch.compile over the modules (reference: test/test_compile.py).  The kernels are opaque custom ops
to the compiler; what is checked is that compiled and eager runs give the same bits, forward and backward."""
import copy

import pytest
import torch
import torch.nn as nn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def f8():
    if not torch.cuda.is_available():
        pytest.fail("these tests need a GPU (run with -m gpu on an MI355X box)")
    import float8_experimental_amd as pkg
    from float8_experimental_amd import _native

    _native.lib()
    return pkg


def _run(mod, x, dy):
    x = x.clone().requires_grad_()
    for p in mod.parameters():
        p.grad = None
    y = mod(x)
    y.backward(dy)
    return [y.detach(), x.grad] + [p.grad for p in mod.parameters()]


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("shape,n", [((4, 96, 512), 448), ((130, 200), 448), ((3, 768, 2048), 2432)])
def test_dynamic_scaling_compiles_as_one_graph(f8, backend, bias, shape, n):
    # the last case's first layer is large enough for one fp8 copy per tensor, read transposed in backward
    torch.manual_seed(0)
    k = shape[-1]
    model = nn.Sequential(nn.Linear(k, n, bias=bias), nn.ReLU(), nn.Linear(n, 384, bias=bias)).to(DEV, dtype=torch.bfloat16)
    f8.convert_to_float8_training(model)
    x = torch.randn(shape, device=DEV, dtype=torch.bfloat16)
    dy = torch.randn(*shape[:-1], 384, device=DEV, dtype=torch.bfloat16)
    want = _run(model, x, dy)
    torch._dynamo.reset()
    compiled = torch.compile(model, backend=backend, fullgraph=True)
    got = _run(compiled, x, dy)
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    got = _run(compiled, x * 2, dy)  # a second call reuses the graph
    want = _run(model, x * 2, dy)
    for a, b in zip(got, want):
        assert torch.equal(a, b)


def test_frozen_weight_and_no_grad_under_compile(f8):
    torch.manual_seed(1)
    lin = nn.Linear(512, 384, bias=False).to(DEV, dtype=torch.bfloat16)
    mod = f8.Float8Linear.from_float(lin)
    mod.weight.requires_grad_(False)
    x = torch.randn(64, 512, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    torch._dynamo.reset()
    cm = torch.compile(mod, backend="aot_eager", fullgraph=True)
    y = cm(x)
    y.sum().backward()
    x2 = x.detach().clone().requires_grad_()
    y2 = mod(x2)
    y2.sum().backward()
    assert torch.equal(y, y2) and torch.equal(x.grad, x2.grad) and mod.weight.grad is None
    with torch.no_grad():
        assert torch.equal(cm(x), y2)


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
@pytest.mark.parametrize("kinds", ["DDD", "DyD", "yDy"])  # input, weight, grad_output: D delayed, y dynamic
@pytest.mark.parametrize("shape,n", [((32, 512), 448), ((3, 768, 2048), 2432)])
def test_delayed_scaling_compiles_as_one_graph(f8, backend, kinds, shape, n):
    """Reference: test_compile.py runs delayed scaling with enable_amax_init=False, enable_pre_and_post_forward=False
    under fullgraph=True.  Here the amax buffers are written by the graph; the sync stays an eager call between steps."""
    torch.manual_seed(4)
    st = lambda c: f8.CastConfig(f8.ScalingType.DELAYED if c == "D" else f8.ScalingType.DYNAMIC)
    cfg = f8.Float8LinearConfig(cast_config_input=st(kinds[0]), cast_config_weight=st(kinds[1]),
                                cast_config_grad_output=st(kinds[2]), enable_amax_init=False,
                                enable_pre_and_post_forward=False)
    k = shape[-1]
    base = nn.Sequential(nn.Linear(k, n, bias=True), nn.GELU(), nn.Linear(n, 384, bias=False)).to(DEV, dtype=torch.bfloat16)
    a, b = copy.deepcopy(base), copy.deepcopy(base)
    f8.convert_to_float8_training(a, config=cfg)
    f8.convert_to_float8_training(b, config=cfg)
    torch._dynamo.reset()
    cb = torch.compile(b, backend=backend, fullgraph=True)
    for it in range(4):
        x = torch.randn(shape, device=DEV, dtype=torch.bfloat16) * 1.5 ** it
        dy = torch.randn(*shape[:-1], 384, device=DEV, dtype=torch.bfloat16) * 10.0 ** (it - 2)
        f8.sync_float8_amax_and_scale_history(a)
        f8.sync_float8_amax_and_scale_history(b)
        for u, v in zip(_run(cb, x, dy), _run(a, x, dy)):
            assert torch.equal(u, v), it
        for (name, b1), (_, b2) in zip(a.named_buffers(), b.named_buffers()):
            assert torch.equal(b1, b2), (it, name)


@pytest.mark.parametrize("backend", ["eager", "aot_eager", "inductor"])
def test_sync_compiles_into_one_frame(f8, backend):
    """Reference: test_compile.py:257-274 (one frame) and :294-320 (fullgraph): the sync of all layers is one node."""
    from torch._dynamo.testing import CompileCounterWithBackend

    torch.manual_seed(5)
    D = f8.CastConfig(f8.ScalingType.DELAYED)
    cfg = f8.Float8LinearConfig(cast_config_input=D, cast_config_weight=D, cast_config_grad_output=D)
    base = nn.Sequential(nn.Linear(256, 320, bias=True), nn.ReLU(), nn.Linear(320, 128, bias=True)).to(DEV, dtype=torch.bfloat16)
    a, b = copy.deepcopy(base), copy.deepcopy(base)
    f8.convert_to_float8_training(a, config=cfg)
    f8.convert_to_float8_training(b, config=cfg)
    torch._dynamo.reset()
    cnts = CompileCounterWithBackend(backend)
    csync = torch.compile(f8.sync_float8_amax_and_scale_history, backend=cnts, fullgraph=True)
    for it in range(3):
        x = torch.randn(48, 256, device=DEV, dtype=torch.bfloat16) * 3.0 ** it
        dy = torch.randn(48, 128, device=DEV, dtype=torch.bfloat16)
        f8.sync_float8_amax_and_scale_history(a)
        try:
            csync(b)
        except Exception as e:
            if backend == "inductor" and it == 0:
                pytest.skip(f"inductor cannot generate code here: {type(e).__name__}")
            raise
        if it == 0:
            assert cnts.frame_count == 1
        for (name, b1), (_, b2) in zip(a.named_buffers(), b.named_buffers()):
            assert torch.equal(b1, b2), (it, name)
        for u, v in zip(_run(b, x, dy), _run(a, x, dy)):
            assert torch.equal(u, v), it
    # one more specialisation once the layers have seen an input (their recorded input dtype goes from None to bf16)
    assert cnts.frame_count == 2
    assert all(m.amax_and_scale_synced is False for m in f8.float8_linear_utils.get_float8_layers(b))  # post-forward ran


def test_whole_delayed_scaling_step_as_one_graph(f8):
    """sync + forward in one compiled function: the scales the sync node writes are the ones the casts read."""
    torch.manual_seed(6)
    D = f8.CastConfig(f8.ScalingType.DELAYED)
    cfg = f8.Float8LinearConfig(cast_config_input=D, cast_config_weight=D, cast_config_grad_output=D,
                                enable_amax_init=False, enable_pre_and_post_forward=False)
    base = nn.Sequential(nn.Linear(512, 640, bias=False), nn.GELU(), nn.Linear(640, 384, bias=True)).to(DEV, dtype=torch.bfloat16)
    a, b = copy.deepcopy(base), copy.deepcopy(base)
    f8.convert_to_float8_training(a, config=cfg)
    f8.convert_to_float8_training(b, config=cfg)

    def step(mod, x):
        f8.sync_float8_amax_and_scale_history(mod)
        return mod(x)

    torch._dynamo.reset()
    cstep = torch.compile(step, backend="aot_eager", fullgraph=True)
    for it in range(4):
        x = torch.randn(96, 512, device=DEV, dtype=torch.bfloat16) * 2.0 ** it
        dy = torch.randn(96, 384, device=DEV, dtype=torch.bfloat16) * 0.1 ** it
        xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
        ya, yb = step(a, xa), cstep(b, xb)
        ya.backward(dy)
        yb.backward(dy)
        assert torch.equal(ya, yb) and torch.equal(xa.grad, xb.grad), it
        for pa, pb in zip(a.parameters(), b.parameters()):
            assert torch.equal(pa.grad, pb.grad), it
        for (name, b1), (_, b2) in zip(a.named_buffers(), b.named_buffers()):
            assert torch.equal(b1, b2), (it, name)


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
def test_delayed_scaling_and_inference_modules_run_outside_the_graph(f8, backend):
    """State-carrying modules are not traced (graph break); compiled and eager runs still agree exactly."""
    from float8_experimental_amd.inference import ActivationCasting, QuantConfig, quantize_to_float8

    torch.manual_seed(2)
    cfg = f8.Float8LinearConfig(cast_config_input=f8.CastConfig(f8.ScalingType.DELAYED),
                                cast_config_weight=f8.CastConfig(f8.ScalingType.DELAYED),
                                cast_config_grad_output=f8.CastConfig(f8.ScalingType.DELAYED))
    base = nn.Sequential(nn.Linear(512, 448, bias=True), nn.GELU(), nn.Linear(448, 384, bias=True)).to(DEV, dtype=torch.bfloat16)
    a, b = copy.deepcopy(base), copy.deepcopy(base)
    f8.convert_to_float8_training(a, config=cfg)
    f8.convert_to_float8_training(b, config=cfg)
    torch._dynamo.reset()
    cb = torch.compile(b, backend=backend)
    for it in range(3):
        x = torch.randn(32, 512, device=DEV, dtype=torch.bfloat16) * (it + 1)
        dy = torch.randn(32, 384, device=DEV, dtype=torch.bfloat16)
        f8.sync_float8_amax_and_scale_history(a)
        f8.sync_float8_amax_and_scale_history(b)
        for u, v in zip(_run(cb, x, dy), _run(a, x, dy)):
            assert torch.equal(u, v)
    q = quantize_to_float8(copy.deepcopy(base), QuantConfig(ActivationCasting.DYNAMIC))
    torch._dynamo.reset()
    cq = torch.compile(q, backend=backend)
    x = torch.randn(32, 512, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        assert torch.equal(cq(x), q(x))


def test_inductor_backend_if_it_is_usable_here(f8):
    """The default backend compiles the user's own pointwise ops around the opaque float8 nodes."""
    torch.manual_seed(3)
    model = nn.Sequential(nn.Linear(512, 448, bias=True), nn.SiLU(), nn.Linear(448, 384, bias=False)).to(DEV, dtype=torch.bfloat16)
    f8.convert_to_float8_training(model)
    x = torch.randn(64, 512, device=DEV, dtype=torch.bfloat16)
    dy = torch.randn(64, 384, device=DEV, dtype=torch.bfloat16)
    want = _run(model, x, dy)
    torch._dynamo.reset()
    compiled = torch.compile(model, backend="inductor", fullgraph=True)
    try:
        got = _run(compiled, x, dy)
    except Exception as e:  # no code generator for this GPU in the installed torch: nothing of ours to test
        pytest.skip(f"inductor cannot generate code here: {type(e).__name__}")
    # the float8 nodes are the same kernels, but the compiler fuses its own pointwise code (SiLU in fp32, one
    # rounding), so the second layer sees inputs that differ in the last bf16 bit and a few of them fall on
    # the other side of an fp8 rounding boundary: agreement is statistical, far above the float8 noise floor
    for a, b in zip(got, want):
        assert f8.float8_utils.compute_error(b.float(), a.float()).item() > 25


def test_inductor_backend_with_delayed_scaling(f8):
    """The amax buffers are graph inputs that the compiled code mutates; the sync stays an eager call between steps."""
    torch.manual_seed(7)
    D = f8.CastConfig(f8.ScalingType.DELAYED)
    cfg = f8.Float8LinearConfig(cast_config_input=D, cast_config_weight=D, cast_config_grad_output=D,
                                enable_amax_init=False, enable_pre_and_post_forward=False)
    base = nn.Sequential(nn.Linear(512, 448, bias=True), nn.SiLU(), nn.Linear(448, 384, bias=False)).to(DEV, dtype=torch.bfloat16)
    a, b = copy.deepcopy(base), copy.deepcopy(base)
    f8.convert_to_float8_training(a, config=cfg)
    f8.convert_to_float8_training(b, config=cfg)
    torch._dynamo.reset()
    cb = torch.compile(b, backend="inductor", fullgraph=True)
    for it in range(3):
        x = torch.randn(64, 512, device=DEV, dtype=torch.bfloat16) * 1.5 ** it
        dy = torch.randn(64, 384, device=DEV, dtype=torch.bfloat16)
        f8.sync_float8_amax_and_scale_history(a)
        f8.sync_float8_amax_and_scale_history(b)
        want = _run(a, x, dy)
        try:
            got = _run(cb, x, dy)
        except Exception as e:
            if it == 0:
                pytest.skip(f"inductor cannot generate code here: {type(e).__name__}")
            raise
        # the first layer sees identical inputs: its recorded amaxes agree exactly; behind the compiler's own SiLU the
        # values differ in the last bf16 bit (see the dynamic-scaling inductor test), so the rest agrees statistically
        assert torch.equal(a[0].fp8_amax_input, b[0].fp8_amax_input) and torch.equal(a[0].fp8_amax_weight, b[0].fp8_amax_weight)
        for (name, b1), (_, b2) in zip(a.named_buffers(), b.named_buffers()):
            torch.testing.assert_close(b1, b2, rtol=0.02, atol=0)
        if it > 0:  # iteration 0 runs on the default scale 1.0: small values underflow in fp8 and there is little signal
            for u, v in zip(got, want):
                assert f8.float8_utils.compute_error(v.float(), u.float()).item() > 20
