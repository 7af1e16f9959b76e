"""Float8InferenceLinear on the GPU: the reference's inference flows (test/test_inference_flows.py) plus
bit-level checks against the oracle and against the training module."""
import copy
import io

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from tests.helpers import fp8_bytes

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


class FeedForward(nn.Module):
    def __init__(self, d=4096, ffn=14336, bias=False):
        super().__init__()
        self.w1 = nn.Linear(d, ffn, bias=bias)
        self.w3 = nn.Linear(d, ffn, bias=bias)
        self.w2 = nn.Linear(ffn, d, bias=bias)

    def forward(self, x):
        return self.w2(F.silu(self.w1(x)) * self.w3(x))


def _sqnr(f8, a, b):
    return f8.float8_utils.compute_error(a, b).item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", ["dynamic", "static", "weight_only"])
def test_mlp_flows_sqnr(f8, dtype, mode):
    """test_inference_flows.py:62-168: SQNR > 20 dB against the high-precision MLP."""
    from float8_experimental_amd.inference import ActivationCasting, Float8InferenceLinear, QuantConfig, quantize_to_float8

    torch.manual_seed(0)
    base = FeedForward().to(DEV, dtype=dtype)
    q = copy.deepcopy(base)
    cfg = {"dynamic": QuantConfig(ActivationCasting.DYNAMIC),
           "static": QuantConfig(ActivationCasting.STATIC, static_quantization_scale=torch.tensor([1.0], device=DEV)),
           "weight_only": QuantConfig(ActivationCasting.WEIGHT_ONLY)}[mode]
    quantize_to_float8(q, cfg)
    n = 0
    for m in q.modules():
        if isinstance(m, Float8InferenceLinear):
            assert isinstance(m.weight, f8.Float8Tensor) and m.weight.requires_grad is False
            n += 1
    assert n == 3
    x = torch.randn(4, 1024, 4096, device=DEV, dtype=dtype)
    with torch.no_grad():
        want, got = base(x), q(x)
    assert got.dtype == dtype and got.shape == want.shape
    assert _sqnr(f8, want, got) > 20


@pytest.mark.parametrize("backend", ["eager", "aot_eager", "inductor"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", ["dynamic", "static", "weight_only"])
def test_mlp_flows_compile_fullgraph(f8, backend, dtype, mode):
    """test_inference_flows.py:60-168 compiles both MLPs with fullgraph=True: the quantised MLP must trace without a
    break (each fp8 linear is one opaque node) and keep SQNR > 20 dB against the high-precision one; with the eager and
    aot_eager backends, where the compiler changes no arithmetic of its own, the bits of the uncompiled module."""
    from float8_experimental_amd.inference import ActivationCasting, QuantConfig, quantize_to_float8

    if backend == "inductor":
        from tests.test_gpu_compile import _need_inductor

        _need_inductor()
    torch.manual_seed(1)
    base = FeedForward(d=1024, ffn=2816, bias=(mode != "weight_only")).to(DEV, dtype=dtype)
    q = copy.deepcopy(base)
    cfg = {"dynamic": QuantConfig(ActivationCasting.DYNAMIC),
           "static": QuantConfig(ActivationCasting.STATIC, static_quantization_scale=torch.tensor([1.0], device=DEV)),
           "weight_only": QuantConfig(ActivationCasting.WEIGHT_ONLY)}[mode]
    quantize_to_float8(q, cfg)
    x = torch.randn(4, 256, 1024, device=DEV, dtype=dtype)
    torch._dynamo.reset()
    cq = torch.compile(q, backend=backend, fullgraph=True)
    with torch.no_grad():
        want, eager, got = base(x), q(x), cq(x)
        got2 = cq(x * 0.5)  # a second call reuses the graph
        eager2 = q(x * 0.5)
    assert got.dtype == dtype and got.shape == want.shape
    assert _sqnr(f8, want, got) > 20
    if backend != "inductor":
        assert torch.equal(got, eager) and torch.equal(got2, eager2)
    else:  # the compiler fuses SiLU and the product in fp32: last-bit differences in what the second linear sees
        assert _sqnr(f8, eager, got) > 25 and _sqnr(f8, eager2, got2) > 25


@pytest.mark.parametrize("shape,bias", [((3, 40, 512), True), ((130, 448), False), ((7, 200), True), ((64, 4096), True),
                                        ((300, 1000), True), ((20, 4097), False)])
@pytest.mark.parametrize("static", [False, True])
def test_fast_path_equals_the_composed_float8tensor_route_and_the_oracle(f8, shape, bias, static):
    """The module's own route (cast in the GEMM's layout, bias in the epilogue) against the reference's
    composition F.linear(Float8Tensor, Float8Tensor, bias), bit for bit, and against the CPU oracle."""
    from float8_experimental_amd.inference import (ActivationCasting, Float8InferenceLinear, QuantConfig,
                                                   cast_to_float8_e4m3_inference)
    from oracle import torch_oracle as to

    torch.manual_seed(1)
    k, n = shape[-1], 320
    lin = nn.Linear(k, n, bias=bias).to(torch.bfloat16)
    sq = torch.tensor([37.0]) if static else None
    cfg = QuantConfig(ActivationCasting.STATIC, static_quantization_scale=sq.to(DEV)) if static else QuantConfig(ActivationCasting.DYNAMIC)
    mod = Float8InferenceLinear.from_float(copy.deepcopy(lin).to(DEV), cfg, use_fast_accum=True)
    x = (torch.randn(shape) * 3).to(torch.bfloat16)
    with torch.no_grad():
        got = mod(x.to(DEV))
        x8 = cast_to_float8_e4m3_inference(x.to(DEV), mod.linear_mm_config, static_quantization_scale=mod.static_quantization_scale)
        composed = F.linear(x8, mod.weight, mod.bias)
    assert torch.equal(got, composed)
    # oracle: weight and activation bytes exact, output within the GEMM tolerance of the emulated product
    sw = to.tensor_to_scale(lin.weight.detach(), torch.float8_e4m3fn)
    w8 = to.cast_to_fp8(lin.weight.detach(), sw, torch.float8_e4m3fn)
    assert np.array_equal(fp8_bytes(mod.weight._data), fp8_bytes(w8)) and mod.weight._scale.item() == sw.item()
    x2 = x.reshape(-1, k)
    sx = sq if static else to.tensor_to_scale(x2, torch.float8_e4m3fn)
    xo = to.cast_to_fp8(x2, sx, torch.float8_e4m3fn)
    assert np.array_equal(fp8_bytes(x8._data).reshape(-1, k), fp8_bytes(xo))
    want = to.mm_emulated(xo, sx, w8.t(), sw, torch.bfloat16).float()
    if bias:
        want = want + lin.bias.detach().float()
    err = (got.float().cpu().reshape(-1, n) - want).abs().max().item() / want.abs().max().item()
    assert err <= 1e-2, err


def test_in_place_weight_update_reaches_eager_and_captured_calls(f8):
    """The module keeps a k-blocked copy of the quantised weight for the GEMM.  Overwriting the weight's bytes in place
    (what load_state_dict does) must show in the next eager call AND in replays of a HIP graph captured before the
    update: the copy is refreshed in place, at the address the graph recorded, by the first eager call after it."""
    from float8_experimental_amd.inference import ActivationCasting, Float8InferenceLinear, QuantConfig

    torch.manual_seed(3)
    k, n = 1024, 768
    lin_a, lin_b = nn.Linear(k, n, bias=False).to(torch.bfloat16).to(DEV), nn.Linear(k, n, bias=False).to(torch.bfloat16).to(DEV)
    cfg = QuantConfig(ActivationCasting.DYNAMIC)
    mod = Float8InferenceLinear.from_float(copy.deepcopy(lin_a), cfg, use_fast_accum=True)
    other = Float8InferenceLinear.from_float(copy.deepcopy(lin_b), cfg, use_fast_accum=True)
    x = (torch.randn(256, k, device=DEV) * 2).to(torch.bfloat16)
    y_static = torch.empty(256, n, dtype=torch.bfloat16, device=DEV)
    with torch.no_grad():
        want_a, want_b = mod(x), other(x)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            mod(x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_static.copy_(mod(x))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_static, want_a)
        before = mod._weight_kblocked().data_ptr()
        mod.weight._data.view(torch.uint8).copy_(other.weight._data.view(torch.uint8))   # in place: same storage, new version
        mod.weight._scale.copy_(other.weight._scale)
        assert torch.equal(mod(x), want_b)                     # eager sees the new bytes
        assert mod._weight_kblocked().data_ptr() == before     # ... in the same k-blocked buffer
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_static, want_b)                   # and so does the graph captured before the update


def test_weight_only_dequantises_and_ignores_the_bias_like_the_reference(f8):
    from float8_experimental_amd.inference import ActivationCasting, Float8InferenceLinear, QuantConfig

    torch.manual_seed(2)
    lin = nn.Linear(256, 128, bias=True).to(DEV, dtype=torch.bfloat16)
    mod = Float8InferenceLinear.from_float(copy.deepcopy(lin), QuantConfig(ActivationCasting.WEIGHT_ONLY), use_fast_accum=True)
    x = torch.randn(9, 256, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        got = mod(x)
        want = F.linear(x, mod.weight.to_original_precision())  # inference.py:104-107: no bias on this branch
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fp8_training_then_save_load_then_inference_is_bit_identical(f8, dtype):
    """test_inference_flows.py:190-240, at a reduced width: Float8Linear training, state dict round trip
    through torch.save / torch.load(weights_only=True) into meta-device modules, conversion to inference
    modules: outputs equal the training modules' eval outputs exactly."""
    from float8_experimental_amd.inference import ActivationCasting, Float8InferenceLinear, QuantConfig, quantize_to_float8

    torch.manual_seed(3)
    d, ffn = 512, 1408
    mlp = FeedForward(d, ffn).to(DEV, dtype=torch.float32)
    f8.convert_to_float8_training(mlp)
    opt = torch.optim.SGD(mlp.parameters(), lr=1e-3)
    target = torch.randn(4, 256, d, device=DEV, dtype=dtype)
    for _ in range(5):
        opt.zero_grad()
        with torch.autocast("cuda", dtype=dtype, enabled=dtype != torch.float32):
            out = mlp(torch.randn(4, 256, d, device=DEV, dtype=dtype))
        F.mse_loss(out.float(), target.float()).backward()
        opt.step()
    mlp.eval()
    mlp = mlp.to(dtype)
    x = torch.randn(4, 256, d, device=DEV, dtype=dtype)
    with torch.no_grad():
        og_out = mlp(x)
    buf = io.BytesIO()
    torch.save(mlp.state_dict(), buf)
    buf.seek(0)
    with torch.device("meta"):
        new = FeedForward(d, ffn).to(dtype=dtype)
        f8.convert_to_float8_training(new)
    new.load_state_dict(torch.load(buf, weights_only=True), strict=True, assign=True)
    quantize_to_float8(new, QuantConfig(ActivationCasting.DYNAMIC))
    assert sum(isinstance(m, Float8InferenceLinear) for m in new.modules()) == 3
    with torch.no_grad():
        new_out = new(x)
    assert torch.equal(og_out, new_out)
    # and the quantised module's own state dict survives a weights_only round trip
    buf = io.BytesIO()
    torch.save(new.state_dict(), buf)
    buf.seek(0)
    sd = torch.load(buf, weights_only=True)
    assert isinstance(sd["w1.weight"], f8.Float8Tensor)
    assert torch.equal(sd["w1.weight"]._data.view(torch.uint8), new.w1.weight._data.view(torch.uint8))
