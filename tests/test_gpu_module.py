"""Float8Linear / Float8Tensor / sync on the GPU against the golden fixtures and the CPU oracle.

Mirrors the reference's own test strategy (test/test_base.py, test/test_numerics_integration.py):
every scaling combination, 2-D/3-D/4-D inputs, bias on/off, bf16/fp32, SQNR against nn.Linear,
buffers moving off their defaults -- plus bit-level checks the reference cannot make.
"""
import copy
import io
import itertools

import numpy as np
import pytest
import torch
import torch.nn as nn

from tests.helpers import F8, TORCH_DT, fp8_bytes, from_bits, load

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


def _cfg(f8, i, w, g, hist=16, **kw):
    m = {"dyn": f8.ScalingType.DYNAMIC, "del": f8.ScalingType.DELAYED}
    return f8.Float8LinearConfig(cast_config_input=f8.CastConfig(m[i]), cast_config_weight=f8.CastConfig(m[w]),
                                 cast_config_grad_output=f8.CastConfig(m[g]),
                                 delayed_scaling_config=f8.DelayedScalingConfig(history_len=hist), **kw)


def _gemm_close(got, want, tol=1e-2, what=""):
    """north-star bar: max error <= 1e-2 relative to the output's scale (bf16 outputs)."""
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    denom = want.abs().max().item() or 1.0
    err = (got - want).abs().max().item() / denom
    assert err <= tol, (what, err)


# ----------------------------------------------------- golden trajectories

TRAJ = [
    ("traj_del_bf16", ("del", "del", "del"), 4, 7, "bf16"),
    ("traj_del_fp32", ("del", "del", "del"), 16, 5, "fp32"),
    ("traj_mix1_bf16", ("dyn", "del", "dyn"), 16, 4, "bf16"),
    ("traj_mix2_bf16", ("del", "dyn", "del"), 2, 5, "bf16"),
    ("traj_dyn_bf16", ("dyn", "dyn", "dyn"), 16, 2, "bf16"),
    ("traj_del_h1_bf16", ("del", "del", "del"), 1, 4, "bf16"),
]


@pytest.mark.parametrize("emulate", [False, True])
@pytest.mark.parametrize("name,scaling,hist,steps,dt", TRAJ)
def test_golden_trajectory(f8, name, scaling, hist, steps, dt, emulate):
    """The same 2-layer model, inputs and step sequence the reference ran when the fixture was written:
    every amax / history / scale buffer after each sync and each step must be bit-identical."""
    g = load(name)
    tdt = TORCH_DT[dt]
    model = nn.Sequential(nn.Linear(16, 32, bias=True), nn.Linear(32, 16, bias=False)).to(tdt)
    with torch.no_grad():
        model[0].weight.copy_(from_bits(g["w0"], dt))
        model[0].bias.copy_(from_bits(g["b0"], dt))
        model[1].weight.copy_(from_bits(g["w1"], dt))
    config = _cfg(f8, *scaling, hist=hist, emulate=emulate)
    model = f8.convert_to_float8_training(model, config=config).to(DEV)
    delayed = f8.linear_requires_sync(config)

    # Buffers fed by tensors that are GEMM outputs (layer 1's input = layer 0's output, layer 0's
    # grad_output = layer 1's grad_input) inherit the GEMM's summation-order noise; the rest of the
    # bookkeeping sees the fixture's exact bits and must reproduce it exactly.
    downstream = {(1, "input"), (0, "grad_output")}

    def check_buffers(tag):
        for li, lay in enumerate(model):
            for kind in ("input", "weight", "grad_output"):
                for field, attr in (("amax", "fp8_amax_"), ("hist", "fp8_amax_history_"), ("scale", "fp8_scale_")):
                    got = getattr(lay, attr + kind).cpu().numpy()
                    want = g[f"{tag}.L{li}.{field}_{kind}"]
                    if (li, kind) in downstream:  # one bf16 ulp of the tensor the amax was taken of
                        np.testing.assert_allclose(got, want, rtol=2.0**-7, err_msg=str((name, tag, li, field, kind)))
                    else:
                        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (name, tag, li, field, kind, got, want)

    for t in range(steps):
        x = from_bits(g[f"t{t}.x"], dt).to(DEV).requires_grad_()
        gy = from_bits(g[f"t{t}.gy"], dt).to(DEV)
        for p in model.parameters():
            p.grad = None
        if delayed:
            f8.sync_float8_amax_and_scale_history(model)
            check_buffers(f"t{t}.synced")
        y = model(x)
        y.backward(gy)
        if delayed:
            check_buffers(f"t{t}.after")
        for key, val in (("y", y), ("dx", x.grad), ("dw0", model[0].weight.grad), ("db0", model[0].bias.grad),
                         ("dw1", model[1].weight.grad)):
            _gemm_close(val, from_bits(g[f"t{t}.{key}"], dt), 1e-2, (name, t, key))


# ------------------------------------------------- all combos vs the oracle


@pytest.mark.parametrize("x_shape", [(16, 16), (2, 16, 16), (3, 2, 16, 16)])
@pytest.mark.parametrize("scaling", list(itertools.product(["dyn", "del"], repeat=3)))
@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("bias", [True, False])
def test_linear_all_combos_vs_oracle_and_nn_linear(f8, x_shape, scaling, dt, bias):
    """Reference test_base.py:150-266: two iterations, sync before each forward when delayed."""
    from oracle import torch_oracle as to

    torch.manual_seed(sum(map(ord, "".join(scaling))) + len(x_shape))
    tdt = TORCH_DT[dt]
    ref_lin = nn.Linear(16, 32, bias=bias).to(tdt)
    mod = f8.Float8Linear.from_float(copy.deepcopy(ref_lin), config=_cfg(f8, *scaling)).to(DEV)
    orc = to.LinearOracle(ref_lin.weight.detach().clone(), scaling, 16)
    delayed = "del" in scaling
    for it in range(2):
        x = torch.randn(*x_shape).to(tdt)  # same distribution each step: delayed scales stay valid
        dy = torch.randn(*x_shape[:-1], 32).to(tdt)
        xd = x.to(DEV).requires_grad_()
        mod.weight.grad = None
        if bias:
            mod.bias.grad = None
        if delayed:
            f8.sync_float8_amax_and_scale_history(mod)
            orc.sync()
        y = mod(xd)
        y.backward(dy.to(DEV))
        # oracle, same sequence
        want_y = orc.forward(x)
        if bias:
            want_y = want_y + ref_lin.bias.detach().to(want_y.dtype)
        want_dx, want_dw = orc.backward(dy)
        _gemm_close(y, want_y, 1e-2, ("y", scaling, it))
        _gemm_close(xd.grad, want_dx, 1e-2, ("dx", scaling, it))
        _gemm_close(mod.weight.grad, want_dw, 1e-2, ("dw", scaling, it))
        # bookkeeping: bit-exact
        if delayed:
            for kind in ("input", "weight", "grad_output"):
                for attr, val in (("fp8_amax_", orc.st[kind].amax), ("fp8_amax_history_", orc.st[kind].history),
                                  ("fp8_scale_", orc.st[kind].scale)):
                    got = getattr(mod, attr + kind).cpu()
                    assert torch.equal(got.view(torch.int32), val.view(torch.int32)), (scaling, it, attr, kind)
        # against nn.Linear in high precision (reference thresholds: 18 dB / 17 dB)
        xr = x.clone().requires_grad_()
        ref_lin.weight.grad = None
        if bias:
            ref_lin.bias.grad = None
        yr = ref_lin(xr)
        yr.backward(dy)
        assert to.sqnr(yr, y.cpu()) >= 18.0
        assert to.sqnr(ref_lin.weight.grad, mod.weight.grad.cpu()) >= 17.0
        assert to.sqnr(xr.grad, xd.grad.cpu()) >= 12.0
        if bias:
            torch.testing.assert_close(ref_lin.bias.grad, mod.bias.grad.cpu())
    if delayed:  # buffers moved off their defaults (reference test_base.py:196-218)
        idx = {"input": 0, "weight": 1, "grad_output": 2}
        for kind, default in (("input", 448.0), ("weight", 448.0), ("grad_output", 57344.0)):
            if scaling[idx[kind]] == "del":
                assert getattr(mod, f"fp8_amax_{kind}").item() != default
                assert getattr(mod, f"fp8_amax_history_{kind}").abs().sum().item() > 0
                assert getattr(mod, f"fp8_scale_{kind}").item() != 1.0
        assert mod.is_amax_initialized and not mod.amax_and_scale_synced
        with pytest.raises(AssertionError, match="not synced"):
            mod(torch.randn(4, 16, device=DEV, dtype=tdt))


@pytest.mark.parametrize("scaling", [("dyn", "dyn", "dyn"), ("del", "del", "del"), ("dyn", "del", "dyn")])
def test_fused_forward_equals_the_composed_reference_pipeline(f8, scaling):
    """`forward` (one autograd function, fused kernels) and `forward_composed` (the reference's
    cast -> Float8Tensor mm -> cast-in-backward chain) produce identical bits."""
    torch.manual_seed(1)
    lin = nn.Linear(64, 96, bias=True).to(torch.bfloat16)
    a = f8.Float8Linear.from_float(copy.deepcopy(lin), config=_cfg(f8, *scaling)).to(DEV)
    b = f8.Float8Linear.from_float(copy.deepcopy(lin), config=_cfg(f8, *scaling)).to(DEV)
    for it in range(3):
        x = (torch.randn(5, 40, 64) * (it + 1)).to(torch.bfloat16).to(DEV)
        dy = torch.randn(5, 40, 96).to(torch.bfloat16).to(DEV)
        outs = []
        for mod, fwd in ((a, a.forward), (b, b.forward_composed)):
            if "del" in scaling:
                f8.sync_float8_amax_and_scale_history(mod)
            xi = x.clone().requires_grad_()
            mod.weight.grad = None
            y = fwd(xi)
            y.backward(dy)
            outs.append((y, xi.grad, mod.weight.grad, mod.bias.grad))
        for u, v in zip(*outs):
            assert torch.equal(u, v)
        if "del" in scaling:
            for (n1, b1), (n2, b2) in zip(a.named_buffers(), b.named_buffers()):
                assert torch.equal(b1, b2), n1


@pytest.mark.parametrize("scaling", [("dyn", "dyn", "dyn"), ("del", "del", "del")])
@pytest.mark.parametrize("m,k,n", [(512, 384, 448), (384, 512, 200), (100, 448, 384), (448, 200, 640),
                                   (512, 384, 640), (384, 768, 512), (2304, 2048, 2304), (4352, 4096, 4224)])
def test_fused_path_with_k_blocked_operands_equals_the_composed_pipeline(f8, scaling, m, k, n):
    """Sizes at which some or all of the three GEMMs take k-blocked operands (contraction a multiple
    of 64 and >= 384), and sizes at which every tensor is cast once and read transposed by the GEMM that
    contracts its other dimension (the last two: all three multiples of 128 and every product of more than 64
    tiles of 256 x 256), against the composed, row-major pipeline: identical bits everywhere."""
    from float8_experimental_amd import _native

    assert _native.tn_ok(m, k, n) == (m >= 2304)
    torch.manual_seed(2)
    lin = nn.Linear(k, n, bias=False).to(torch.bfloat16)
    a = f8.Float8Linear.from_float(copy.deepcopy(lin), config=_cfg(f8, *scaling)).to(DEV)
    b = f8.Float8Linear.from_float(copy.deepcopy(lin), config=_cfg(f8, *scaling)).to(DEV)
    for it in range(2):
        x = (torch.randn(m, k) * (it + 1)).to(torch.bfloat16).to(DEV)
        dy = torch.randn(m, n).to(torch.bfloat16).to(DEV)
        outs = []
        for mod, fwd in ((a, a.forward), (b, b.forward_composed)):
            if "del" in scaling:
                f8.sync_float8_amax_and_scale_history(mod)
            xi = x.clone().requires_grad_()
            mod.weight.grad = None
            y = fwd(xi)
            y.backward(dy)
            outs.append((y, xi.grad, mod.weight.grad))
        for u, v in zip(*outs):
            assert torch.equal(u, v)


@pytest.mark.parametrize("scaling", [("dyn", "dyn", "dyn"), ("del", "del", "del")])
def test_fp16_layer_fused_equals_composed_and_scales_stay_finite(f8, scaling):
    """fp16 weights and activations: scales are computed in fp16 and clamped to 65504 (reference float8_utils.py:54-55,
    test_base.py:566-586), also when the tensor is tiny; fused and composed routes agree bit for bit."""
    from oracle import torch_oracle as to

    torch.manual_seed(12)
    m, k, n = 200, 448, 384
    lin = nn.Linear(k, n, bias=True).to(torch.float16)
    a = f8.Float8Linear.from_float(copy.deepcopy(lin), config=_cfg(f8, *scaling)).to(DEV)
    b = f8.Float8Linear.from_float(copy.deepcopy(lin), config=_cfg(f8, *scaling)).to(DEV)
    ref = copy.deepcopy(lin).to(DEV)
    for it, mag in enumerate((1.0, 1e-6, 1.0)):   # the middle batch is tiny: 448 / amax would overflow fp16
        x = (torch.randn(m, k) * mag).to(torch.float16).to(DEV)
        dy = torch.randn(m, n).to(torch.float16).to(DEV)
        outs = []
        for mod, fwd in ((a, a.forward), (b, b.forward_composed)):
            if "del" in scaling:
                f8.sync_float8_amax_and_scale_history(mod)
            xi = x.clone().requires_grad_()
            mod.weight.grad = mod.bias.grad = None
            y = fwd(xi)
            y.backward(dy)
            outs.append((y, xi.grad, mod.weight.grad))
        for u, v in zip(*outs):
            assert u.dtype == torch.float16 and torch.isfinite(u).all()
            assert torch.equal(u, v), it
        if scaling[0] == "dyn" and mag == 1.0:
            assert to.sqnr(ref(x).detach().cpu(), outs[0][0].detach().cpu()) > 18.0
    from float8_experimental_amd import _native

    _, s = _native.amax_scale(torch.full((8, 8), 1e-7, dtype=torch.float16, device=DEV), torch.float8_e4m3fn)
    assert s.item() == 65504.0


def test_fused_equals_composed_over_a_random_sweep_of_sizes(f8):
    """Whatever operand layouts and GEMM kernels the sizes select on the two routes (k-blocked or row-major; few-row,
    128-row-tile, large-tile kernels; one fp8 copy or two), forward and both gradients are the same bits."""
    rng = np.random.default_rng(7)
    dims = [64, 100, 128, 200, 256, 320, 384, 448, 512, 640, 1024, 1152, 2048, 2304]
    torch.manual_seed(13)
    for case in range(24):
        m, k, n = (int(rng.choice(dims)) for _ in range(3))
        lin = nn.Linear(k, n, bias=False).to(torch.bfloat16)
        a = f8.Float8Linear.from_float(copy.deepcopy(lin)).to(DEV)
        b = f8.Float8Linear.from_float(copy.deepcopy(lin)).to(DEV)
        x = torch.randn(m, k).to(torch.bfloat16).to(DEV)
        dy = torch.randn(m, n).to(torch.bfloat16).to(DEV)
        outs = []
        for mod, fwd in ((a, a.forward), (b, b.forward_composed)):
            xi = x.clone().requires_grad_()
            y = fwd(xi)
            y.backward(dy)
            outs.append((y, xi.grad, mod.weight.grad))
        for name, u, v in zip(("y", "dx", "dw"), *outs):
            assert torch.equal(u, v), (case, m, k, n, name)


@pytest.mark.parametrize("frozen", ["weight", "input"])
def test_single_copy_path_with_one_gradient_not_needed(f8, frozen):
    torch.manual_seed(4)
    m, k, n = 2304, 2048, 2432  # one fp8 copy per tensor, read transposed in backward
    lin = nn.Linear(k, n, bias=False).to(torch.bfloat16)
    a = f8.Float8Linear.from_float(copy.deepcopy(lin)).to(DEV)
    b = f8.Float8Linear.from_float(copy.deepcopy(lin)).to(DEV)
    x = torch.randn(m, k).to(torch.bfloat16).to(DEV)
    dy = torch.randn(m, n).to(torch.bfloat16).to(DEV)
    outs = []
    for mod, fwd in ((a, a.forward), (b, b.forward_composed)):
        mod.weight.requires_grad_(frozen != "weight")
        xi = x.clone().requires_grad_(frozen != "input")
        y = fwd(xi)
        y.backward(dy)
        outs.append((y, xi.grad, mod.weight.grad))
    for u, v in zip(*outs):
        assert (u is None and v is None) or torch.equal(u, v)
    assert outs[0][1 if frozen == "input" else 2] is None


@pytest.mark.parametrize("scaling", [("dyn", "dyn", "dyn"), ("del", "del", "del")])
@pytest.mark.parametrize("k,n", [(384, 512), (100, 36)])
def test_empty_batch(f8, scaling, k, n):
    """No tokens: empty outputs, zero weight gradient, nothing launched on null pointers.  (The reference raises
    inside torch.max on an empty tensor; an empty amax is defined as 0 here.)"""
    torch.manual_seed(8)
    lin = nn.Linear(k, n, bias=True).to(torch.bfloat16)
    mod = f8.Float8Linear.from_float(lin, config=_cfg(f8, *scaling)).to(DEV)
    for shape, fwd in (((0, k), mod.forward), ((2, 0, k), mod.forward), ((0, k), mod.forward_composed)):
        if "del" in scaling:
            f8.sync_float8_amax_and_scale_history(mod)
        x = torch.randn(shape, device=DEV, dtype=torch.bfloat16, requires_grad=True)
        mod.weight.grad = mod.bias.grad = None
        y = fwd(x)
        assert y.shape == (*shape[:-1], n) and y.dtype == torch.bfloat16
        y.backward(torch.randn(y.shape, device=DEV, dtype=torch.bfloat16))
        assert x.grad.shape == x.shape
        assert mod.weight.grad.shape == (n, k) and not mod.weight.grad.any()
    # and the layer still works afterwards (delayed scaling: one batch later, once a real amax is in the history --
    # the scales after empty batches come from amax = 0 and saturate everything, as delayed scaling will)
    from oracle import torch_oracle as to

    x = torch.randn(8, k, device=DEV, dtype=torch.bfloat16)
    want = torch.nn.functional.linear(x, mod.weight, mod.bias)
    for _ in range(2 if "del" in scaling else 1):
        if "del" in scaling:
            f8.sync_float8_amax_and_scale_history(mod)
        got = mod(x)
    assert to.sqnr(want.detach().cpu(), got.detach().cpu()) > 18.0


def test_two_host_threads_on_their_own_streams(f8):
    """The library keeps no mutable state between calls except what the caller hands it (workspace per stream):
    two threads stepping their own layers on their own streams get the results of running alone."""
    import threading

    torch.manual_seed(9)
    shapes = [(384, 512, 640), (200, 448, 96)]
    mods, xs, dys, want = [], [], [], []
    for m, k, n in shapes:
        lin = nn.Linear(k, n, bias=False).to(torch.bfloat16)
        mods.append(f8.Float8Linear.from_float(lin).to(DEV))
        xs.append(torch.randn(m, k, device=DEV, dtype=torch.bfloat16))
        dys.append(torch.randn(m, n, device=DEV, dtype=torch.bfloat16))

    def run(i, out):
        x = xs[i].clone().requires_grad_()
        y = mods[i](x)
        gx, gw = torch.autograd.grad(y, [x, mods[i].weight], dys[i])
        out.append((y.detach(), gx, gw))

    for i in range(2):
        run(i, want)
    torch.cuda.synchronize()
    got = [[], []]
    errors = []

    def worker(i):
        try:
            with torch.cuda.stream(torch.cuda.Stream()):
                for _ in range(25):
                    run(i, got[i])
                torch.cuda.current_stream().synchronize()
        except Exception as e:  # surfaced below: an exception in a thread would otherwise pass silently
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(2):
        assert len(got[i]) == 25
        for trio in got[i]:
            for a, b in zip(trio, want[i]):
                assert torch.equal(a, b)


# --------------------------------------------------------------- scales computed ahead of the forward


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
def test_precomputed_weight_scales_give_the_same_step(f8, dt):
    """precompute_float8_dynamic_scale_for_fsdp on one GPU: all weight scales in one pass; the forward that
    uses them equals the forward that computes each scale itself, fused and composed, bit for bit."""
    from float8_experimental_amd import _native

    torch.manual_seed(6)
    dims = [(384, 512), (512, 200), (200, 384)]
    base = nn.Sequential(*[nn.Linear(k, n, bias=(i == 1)) for i, (k, n) in enumerate(dims)]).to(dt)
    cfg = f8.Float8LinearConfig(enable_fsdp_float8_all_gather=True)
    a = f8.convert_to_float8_training(copy.deepcopy(base), config=cfg).to(DEV)
    b = f8.convert_to_float8_training(copy.deepcopy(base)).to(DEV)
    opt_a = torch.optim.SGD(a.parameters(), lr=0.1)
    opt_b = torch.optim.SGD(b.parameters(), lr=0.1)
    for it in range(3):
        x = torch.randn(384, 384).to(dt).to(DEV)
        dy = torch.randn(384, 384).to(dt).to(DEV)
        f8.precompute_float8_dynamic_scale_for_fsdp(a)
        for lay_a, lay_b in zip(a, b):
            _, s = _native.amax_scale(lay_b.weight.detach(), torch.float8_e4m3fn)
            assert lay_a._precomputed_weight_scale.item() == s.item()
        outs = []
        for mod, opt, composed in ((a, opt_a, it == 2), (b, opt_b, False)):
            opt.zero_grad(set_to_none=True)
            xi = x.clone().requires_grad_()
            h = xi
            for lay in mod:
                h = lay.forward_composed(h) if composed else lay(h)
            h.backward(dy)
            outs.append([h.detach(), xi.grad] + [p.grad.clone() for p in mod.parameters()])
            opt.step()
        for u, v in zip(*outs):
            assert torch.equal(u, v), it
    assert f8.precompute_float8_dynamic_scale_for_fsdp(b) is None  # no layer of b carries the flag
    assert all(lay._precomputed_weight_scale is None for lay in b)


# --------------------------------------------------------------- config 1


def test_cfg1_against_the_reference_fixture(f8):
    """Benchmark configuration 1 (the reference's CPU-runnable case): x[2048,4096] ~N(0,1), Linear(4096,4096) default init, seed 0, y.sum().backward()."""
    import hashlib

    g = load("cfg1")
    sha = lambda a: np.frombuffer(hashlib.sha256(np.ascontiguousarray(a).tobytes()).digest(), np.uint8)
    torch.manual_seed(0)
    lin = nn.Linear(4096, 4096, bias=False).to(torch.bfloat16)
    x = torch.randn(2048, 4096).to(torch.bfloat16)
    assert np.array_equal(sha(x.view(torch.int16).numpy()), g["x_sha"])
    from float8_experimental_amd.float8_scaling_utils import hp_tensor_to_float8_dynamic
    from float8_experimental_amd.float8_tensor import LinearMMConfig

    xd, wd = x.to(DEV), lin.weight.detach().to(DEV)
    x8 = hp_tensor_to_float8_dynamic(xd, torch.float8_e4m3fn, LinearMMConfig())
    w8 = hp_tensor_to_float8_dynamic(wd, torch.float8_e4m3fn, LinearMMConfig())
    assert x8._scale.cpu().numpy().view(np.uint32) == g["sx"].view(np.uint32)
    assert w8._scale.cpu().numpy().view(np.uint32) == g["sw"].view(np.uint32)
    assert np.array_equal(sha(fp8_bytes(x8._data)), g["x_fp8_sha"])
    assert np.array_equal(sha(fp8_bytes(w8._data)), g["w_fp8_sha"])
    mod = f8.convert_to_float8_training(nn.Sequential(lin)).to(DEV)
    xg = xd.clone().requires_grad_()
    y = mod(xg)
    y.sum().backward()  # dY is an expanded (stride-0) tensor of ones
    dy8 = hp_tensor_to_float8_dynamic(torch.ones_like(y), torch.float8_e5m2, LinearMMConfig())
    assert dy8._scale.item() == 57344.0 == g["sg"]
    assert np.array_equal(sha(fp8_bytes(dy8._data)), g["dy_fp8_sha"])
    _gemm_close(y[:16, :32], from_bits(g["y_slice"], "bf16"), 1e-2, "y")
    _gemm_close(xg.grad[:16, :32], from_bits(g["dx_slice"], "bf16"), 1e-2, "dx")
    _gemm_close(mod[0].weight.grad[:16, :32], from_bits(g["dw_slice"], "bf16"), 1e-2, "dw")
    for key, val in (("y_norm", y), ("dx_norm", xg.grad), ("dw_norm", mod[0].weight.grad)):
        assert abs(val.double().norm().item() / float(g[key]) - 1) < 1e-3, key


def test_sync_follows_buffers_that_are_replaced(f8):
    """sync keeps a table of buffer addresses per list of layers; every way of replacing a buffer tensor -- assignment,
    .to(), load_state_dict(assign=True) -- makes it rebuild the table, so the scales always come from the buffers the
    modules hold now."""
    cfg = _cfg(f8, "del", "del", "del", hist=4)
    model = nn.Sequential(*[f8.Float8Linear.from_float(nn.Linear(64, 64, bias=False), config=cfg) for _ in range(3)]).to(DEV)
    for mod in model:
        mod.last_seen_input_dtype = torch.bfloat16

    def scales():
        return [getattr(mod, f"fp8_scale_{kind}").item() for mod in model for kind in ("input", "weight", "grad_output")]

    f8.sync_float8_amax_and_scale_history(model)
    assert scales() == [1.0] * 9                     # default amax = fmax of the format
    model[1].fp8_amax_weight = torch.tensor([7.0], device=DEV)          # a new tensor under the same name
    f8.sync_float8_amax_and_scale_history(model)
    assert scales()[4] == 448.0 * np.float32(1.0 / 7.0) and scales()[:4] == [1.0] * 4
    model.to("cpu")
    model.to(DEV)                                                       # every buffer moved
    model[2].fp8_amax_grad_output.fill_(2.0)
    f8.sync_float8_amax_and_scale_history(model)
    assert scales()[8] == 57344.0 / 2.0 and scales()[4] == 448.0 * np.float32(1.0 / 7.0)
    sd = {k: v.clone() for k, v in model.state_dict().items()}
    sd["0.fp8_amax_input"] = torch.tensor([14.0], device=DEV)
    model.load_state_dict(sd, assign=True)                              # every buffer swapped for the dict's tensor
    f8.sync_float8_amax_and_scale_history(model)
    assert scales()[0] == 448.0 * np.float32(1.0 / 14.0) and scales()[8] == 57344.0 / 2.0
    assert model[0].fp8_scale_input.data_ptr() == sd["0.fp8_scale_input"].data_ptr()


# --------------------------------------------------------------- config 5


@pytest.mark.parametrize("m,k,n", [(4099, 1000, 3000), (4099, 4097, 11007)])
def test_cfg5_ragged_heavy_tailed(f8, m, k, n):
    """Non-multiple-of-16 shapes, Student-t(3) data with 0.1 % outliers x1000: saturation, amax extremes,
    ragged MFMA tiles.  Bytes and scales bit-exact, GEMMs within 1e-2 of the emulated oracle."""
    from oracle import torch_oracle as to

    torch.manual_seed(5)

    def heavy(shape):
        t = torch.distributions.StudentT(3.0).sample(shape)
        return torch.where(torch.rand(shape) < 0.001, t * 1000, t).to(torch.bfloat16)

    x, w, dy = heavy((m, k)), heavy((n, k)), heavy((m, n))
    ref = to.linear_fwd_bwd_dynamic(x, w, dy)
    lin = nn.Linear(k, n, bias=False).to(torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
    mod = f8.Float8Linear.from_float(lin).to(DEV)
    xd = x.to(DEV).requires_grad_()
    y = mod(xd)
    y.backward(dy.to(DEV))
    from float8_experimental_amd import _native

    for t_cpu, key8, keys, fmt in ((x, "x8", "sx", torch.float8_e4m3fn), (w, "w8", "sw", torch.float8_e4m3fn),
                                   (dy, "g8", "sg", torch.float8_e5m2)):
        td = t_cpu.to(DEV)
        _, s = _native.amax_scale(td, fmt)
        assert s.item() == ref[keys].item()
        b, bt = _native.cast(td, s, fmt, want_out_t=True)
        want = ref[key8].view(torch.uint8)
        assert torch.equal(b.view(torch.uint8).cpu(), want)
        assert torch.equal(bt.view(torch.uint8).cpu(), want.t().contiguous())
    _gemm_close(y, ref["y"], 1e-2, "y")
    _gemm_close(xd.grad, ref["dx"], 1e-2, "dx")
    _gemm_close(mod.weight.grad, ref["dw"], 1e-2, "dw")


def test_ragged_layers_random_sweep_against_the_oracle(f8):
    """Thirty layers with sizes that are multiples of nothing (and a few that are), dynamic and delayed scaling: every
    contraction that reaches 384 once padded runs on zero-padded k-blocked copies.  Scales and amax buffers bit-exact,
    y / dx / dw within 1e-2 of the emulated oracle."""
    from oracle import torch_oracle as to

    g = torch.Generator().manual_seed(2024)
    pick = lambda lo, hi: int(torch.randint(lo, hi, (1,), generator=g))
    for case in range(30):
        m, k, n = pick(1, 1400), pick(1, 1400), pick(1, 1400)
        if case % 5 == 0:
            m, k, n = 64 * pick(1, 12), 64 * pick(1, 12), 64 * pick(1, 12)
        delayed = case % 3 == 2
        x = (torch.randn(m, k, generator=g) * 3).to(torch.bfloat16)
        w = (torch.randn(n, k, generator=g) * 0.2).to(torch.bfloat16)
        dy = (torch.randn(m, n, generator=g) * 0.05).to(torch.bfloat16)
        lin = nn.Linear(k, n, bias=False).to(torch.bfloat16)
        with torch.no_grad():
            lin.weight.copy_(w)
        mod = f8.Float8Linear.from_float(lin, config=_cfg(f8, *(("del",) * 3 if delayed else ("dyn",) * 3))).to(DEV)
        xd = x.to(DEV).requires_grad_()
        y = mod(xd)
        y.backward(dy.to(DEV))
        if delayed:
            # first iteration: the scales come from this step's amaxes (amax init), in fp32
            amax = lambda t: t.abs().max().float()
            for kind, t, fmax in (("input", x, 448.0), ("weight", w, 448.0), ("grad_output", dy, 57344.0)):
                assert getattr(mod, f"fp8_amax_{kind}").item() == amax(t).item(), (case, kind)
                want = np.float32(fmax) * (np.float32(1.0) / np.float32(max(amax(t).item(), 1e-12)))
                assert getattr(mod, f"fp8_scale_{kind}").item() == want, (case, kind)
            sx, sw, sg = (getattr(mod, f"fp8_scale_{kind}").cpu() for kind in ("input", "weight", "grad_output"))
            x8, w8, g8 = to.cast_to_fp8(x, sx, torch.float8_e4m3fn), to.cast_to_fp8(w, sw, torch.float8_e4m3fn), to.cast_to_fp8(dy, sg, torch.float8_e5m2)
            ref = {"y": to.mm_emulated(x8, sx, w8.t(), sw, torch.bfloat16), "dx": to.mm_emulated(g8, sg, w8, sw, torch.bfloat16),
                   "dw": to.mm_emulated(g8.t(), sg, x8, sx, torch.bfloat16)}
        else:
            ref = to.linear_fwd_bwd_dynamic(x, w, dy)
        _gemm_close(y, ref["y"], 1e-2, ("y", case, m, k, n))
        _gemm_close(xd.grad, ref["dx"], 1e-2, ("dx", case, m, k, n))
        _gemm_close(mod.weight.grad, ref["dw"], 1e-2, ("dw", case, m, k, n))


# ------------------------------------------------- LLaMa FFN integration


@pytest.mark.parametrize("scaling", [("dyn", "dyn", "dyn"), ("del", "del", "del"), ("del", "dyn", "del")])
def test_llama_ffn_sqnr(f8, scaling):
    """Reference test_numerics_integration.py:76-165: SwiGLU FFN 4096 -> 14336 -> 4096, two different
    inputs, SQNR > 20 dB on the output and on every parameter gradient."""
    from oracle import torch_oracle as to

    class FFN(nn.Module):
        def __init__(self, dim, hidden):
            super().__init__()
            self.w1 = nn.Linear(dim, hidden, bias=False)
            self.w2 = nn.Linear(hidden, dim, bias=False)
            self.w3 = nn.Linear(dim, hidden, bias=False)

        def forward(self, x):
            return self.w2(nn.functional.silu(self.w1(x)) * self.w3(x))

    torch.manual_seed(0)
    ref = FFN(4096, 14336).to(torch.bfloat16).to(DEV)
    fp8 = f8.convert_to_float8_training(copy.deepcopy(ref), config=_cfg(f8, *scaling))
    for it in range(2):
        x = torch.randn(1, 8192, 4096, device=DEV, dtype=torch.bfloat16)
        for model in (ref, fp8):
            for p in model.parameters():
                p.grad = None
        if "del" in scaling:
            f8.sync_float8_amax_and_scale_history(fp8)
        y_ref = ref(x)
        y_ref.sum().backward()
        y = fp8(x)
        y.sum().backward()
        assert to.sqnr(y_ref.float().cpu(), y.float().cpu()) > 20.0
        for (n1, p1), (n2, p2) in zip(ref.named_parameters(), fp8.named_parameters()):
            assert to.sqnr(p1.grad.float().cpu(), p2.grad.float().cpu()) > 20.0, n1


# ---------------------------------------------------------- Float8Tensor ops


def test_float8_tensor_ops(f8):
    """Reference test_base.py:60-144."""
    from float8_experimental_amd.float8_tensor import Float8Tensor, hp_tensor_and_scale_to_float8
    from float8_experimental_amd.float8_utils import e4m3_dtype, e5m2_dtype, fp8_tensor_statistics, tensor_to_scale

    # dtype is preserved through a round trip
    for hp, lp in itertools.product((torch.float32, torch.float16, torch.bfloat16), (e4m3_dtype, e5m2_dtype)):
        x = torch.randn(4, 4, dtype=hp, device=DEV)
        s = tensor_to_scale(x, lp)
        x8 = hp_tensor_and_scale_to_float8(x, s, lp)
        assert x8.to_original_precision().dtype == hp and x8._data.dtype == lp
    # the gradient passes unchanged through both casts
    for lp in (e4m3_dtype, e5m2_dtype):
        x = torch.randn(1, device=DEV).requires_grad_()
        grad = torch.randn(1, device=DEV)
        x8 = hp_tensor_and_scale_to_float8(x, tensor_to_scale(x, lp), lp)
        x8.to_original_precision().backward(grad)
        torch.testing.assert_close(grad, x.grad, rtol=0, atol=0)
    # split / cat are bitwise
    a = torch.rand(16, 16, dtype=torch.bfloat16, device=DEV)
    sa = tensor_to_scale(a, e4m3_dtype)
    a8 = hp_tensor_and_scale_to_float8(a, sa, e4m3_dtype)
    back = torch.cat(torch.split(a8, 16), dim=0)
    assert isinstance(back, Float8Tensor) and torch.equal(back._data.view(torch.uint8), a8._data.view(torch.uint8))
    # index_put_ needs equal scales
    v = torch.rand(16, dtype=torch.bfloat16, device=DEV)
    sv = tensor_to_scale(v, e4m3_dtype)
    v8 = hp_tensor_and_scale_to_float8(v, sv, e4m3_dtype)
    index = torch.randint(0, 15, (16,), dtype=torch.long, device=DEV)
    b = torch.rand(16, 16, dtype=torch.bfloat16, device=DEV)
    b8 = hp_tensor_and_scale_to_float8(b, sv, e4m3_dtype)
    b8_bad = hp_tensor_and_scale_to_float8(b, tensor_to_scale(b, e4m3_dtype) * 2, e4m3_dtype)
    with pytest.raises(AssertionError):
        b8_bad[index] = v8
    b8[index] = v8
    # copy_: hp <- fp8 dequantises, fp8 <- hp is refused
    dst = torch.empty(16, dtype=torch.bfloat16, device=DEV)
    dst.copy_(v8)
    torch.testing.assert_close(dst, v8.to_original_precision())
    with pytest.raises(RuntimeError):
        v8.copy_(dst)
    other = hp_tensor_and_scale_to_float8(v * 0.5, sv, e4m3_dtype)
    v8.copy_(other)
    assert torch.equal(v8._data.view(torch.uint8), other._data.view(torch.uint8))
    # weights_only serialisation round trip
    buf = io.BytesIO()
    torch.save({"t": a8}, buf)
    buf.seek(0)
    got = torch.load(buf, weights_only=True)["t"]
    assert isinstance(got, Float8Tensor) and torch.equal(got._data.view(torch.uint8), a8._data.view(torch.uint8))
    assert got._scale.item() == a8._scale.item()
    # saturation / underflow counts (reference test_base.py:688-713)
    ones = torch.ones(4, 4, dtype=torch.bfloat16, device=DEV)
    s = tensor_to_scale(ones, e4m3_dtype)
    big = hp_tensor_and_scale_to_float8(ones * 1e9, s, e4m3_dtype)
    assert fp8_tensor_statistics(big, e4m3_dtype) == (0, 16)
    tiny = hp_tensor_and_scale_to_float8(ones * 1e-9, s, e4m3_dtype)
    assert fp8_tensor_statistics(tiny, e4m3_dtype) == (16, 0)
    # fp16 with a tiny amax: the scale stays finite (reference test_base.py:566-586)
    z = torch.zeros(8, dtype=torch.float16, device=DEV)
    assert tensor_to_scale(z, e4m3_dtype).item() == 65504.0


def test_scaled_mm_through_float8_tensors(f8):
    """Reference test_base.py:388-552: a @ b on Float8Tensors, real vs emulated configs, bias, padding."""
    from float8_experimental_amd.float8_python_api import addmm_float8_unwrapped
    from float8_experimental_amd.float8_tensor import (GemmInputRole, hp_tensor_and_scale_to_float8, LinearMMConfig,
                                                       ScaledMMConfig)
    from float8_experimental_amd.float8_utils import e4m3_dtype, tensor_to_scale

    torch.manual_seed(42)
    for out_dt in (torch.bfloat16, torch.float16, torch.float32):
        for use_bias in (False, True):
            a = torch.randn(16, 41 if use_bias else 48, device=DEV, dtype=out_dt)
            b = torch.randn(a.shape[1], 128, device=DEV, dtype=out_dt)
            sa, sb = tensor_to_scale(a, e4m3_dtype), tensor_to_scale(b, e4m3_dtype)
            real = LinearMMConfig()
            emu = LinearMMConfig(ScaledMMConfig(True, False, False, False), ScaledMMConfig(True, False, False, False),
                                 ScaledMMConfig(True, False, False, False))
            pad = LinearMMConfig(ScaledMMConfig(False, True, False, True), ScaledMMConfig(False, False, False, True),
                                 ScaledMMConfig(False, False, False, True))
            outs = {}
            for name, c in (("real", real), ("emu", emu), ("pad", pad)):
                a8 = hp_tensor_and_scale_to_float8(a, sa, e4m3_dtype, c, GemmInputRole.INPUT)
                b8 = hp_tensor_and_scale_to_float8(b, sb, e4m3_dtype, c, GemmInputRole.WEIGHT)
                if use_bias:
                    outs[name] = torch.addmm(torch.linspace(-2, 2, 128, device=DEV).to(out_dt), a8, b8)
                else:
                    outs[name] = torch.mm(a8, b8)
                assert outs[name].dtype == out_dt
            tol = 7e-2 if out_dt != torch.float32 else 2e-3  # the reference's own bars (test_base.py:428-432)
            torch.testing.assert_close(outs["real"], outs["emu"], atol=tol, rtol=tol)
            assert torch.equal(outs["real"], outs["pad"])  # zero padding of k changes nothing
            # mismatched configs are refused
            a8 = hp_tensor_and_scale_to_float8(a, sa, e4m3_dtype, real, GemmInputRole.INPUT)
            b8 = hp_tensor_and_scale_to_float8(b, sb, e4m3_dtype, emu, GemmInputRole.WEIGHT)
            with pytest.raises(AssertionError, match="linear_mm_config.output mismatch"):
                torch.mm(a8, b8)
    # the unwrapped entry point with a column-major b, as preprocess_addmm hands it over
    a = torch.randn(64, 96, device=DEV).to(e4m3_dtype)
    b = torch.randn(80, 96, device=DEV).to(e4m3_dtype).t()
    one = torch.ones((), device=DEV)
    y = addmm_float8_unwrapped(a, one, b, one, torch.float32)
    bound = a.float().abs() @ b.float().abs()
    assert bool(((y - a.float() @ b.float()).abs() <= 2.0**-13 * bound).all())


def test_autocast_and_dtype_moves(f8):
    """Reference test_base.py:268-372."""
    lin = nn.Linear(32, 16, device=DEV, dtype=torch.float32)
    mod = f8.Float8Linear.from_float(copy.deepcopy(lin), config=_cfg(f8, "del", "del", "del"))
    x = torch.randn(16, 32, device=DEV)
    for ac in (torch.bfloat16, torch.float16):
        f8.sync_float8_amax_and_scale_history(mod)
        with torch.autocast("cuda", dtype=ac):
            y = mod(x)
        assert y.dtype == ac
        y.sum().backward()
        assert mod.weight.grad.dtype == torch.float32
        assert mod.last_seen_input_dtype == torch.float32  # recorded before the autocast conversion, as in the reference
    f8.sync_float8_amax_and_scale_history(mod)
    y = mod(x)
    assert y.dtype == torch.float32
    for dt in (torch.bfloat16, torch.float16):
        m2 = f8.Float8Linear.from_float(copy.deepcopy(lin), config=_cfg(f8, "del", "dyn", "del")).to(dt)
        assert all(b.dtype == torch.float32 for b in m2.buffers())
        f8.sync_float8_amax_and_scale_history(m2)
        y = m2(x.to(dt))
        assert y.dtype == dt
        y.sum().backward()
        assert all(b.dtype == torch.float32 for b in m2.buffers())


def test_frozen_weight_and_no_grad(f8):
    lin = nn.Linear(64, 32, bias=False, device=DEV, dtype=torch.bfloat16)
    mod = f8.Float8Linear.from_float(lin)
    x = torch.randn(8, 64, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        y0 = mod(x)
    lin.weight.requires_grad_(False)
    xg = x.clone().requires_grad_()
    y1 = mod(xg)
    y1.sum().backward()
    assert torch.equal(y0, y1) and xg.grad is not None and lin.weight.grad is None
    lin.weight.requires_grad_(True)
    y2 = mod(x)  # input without grad
    y2.sum().backward()
    assert lin.weight.grad is not None
