"""Pins the CPU oracle (oracle/) before anything is compared against it.

Three independent sources are played against each other:
  * the golden fixtures written by the reference itself (tests/golden/*.npz),
  * torch's own operators on CPU (the arithmetic the reference is made of),
  * closed forms / known answers from the fp8 format definitions.
All of it runs without a GPU.
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import torch_oracle as to
from tests.helpers import CODE_DT, F8, TORCH_DT, fp8_bytes, from_bits, load, np_for_c, same_bytes_mod_nan_sign


# ----------------------------------------------------------------- fp8 codec


def _all_bf16_as_f32():
    bits = np.arange(65536, dtype=np.uint32) << 16
    return bits.view(np.float32)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_codec_matches_torch_on_every_bf16_pattern(fmt):
    code, tdt = F8[fmt]
    x = _all_bf16_as_f32()
    ours = co.f32_to_fp8(x, code)
    theirs = fp8_bytes(torch.from_numpy(x.copy()).to(tdt))
    assert same_bytes_mod_nan_sign(ours, theirs)
    # finite inputs must agree exactly, sign of zero included
    fin = np.isfinite(x)
    assert np.array_equal(ours[fin], theirs[fin])


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_codec_matches_torch_on_fp32_sweep(fmt):
    code, tdt = F8[fmt]
    rng = np.random.default_rng(7)
    bits = np.concatenate([
        np.arange(0, 2**32, 4099, dtype=np.uint64).astype(np.uint32),  # strided sweep of all fp32
        rng.integers(0, 2**32, size=1 << 20, dtype=np.uint64).astype(np.uint32),
    ])
    x = bits.view(np.float32)
    ours = co.f32_to_fp8(x, code)
    theirs = fp8_bytes(torch.from_numpy(x.copy()).to(tdt))
    assert same_bytes_mod_nan_sign(ours, theirs)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_every_fp8_code_is_a_fixed_point(fmt):
    code, tdt = F8[fmt]
    codes = np.arange(256, dtype=np.uint8)
    vals = co.fp8_to_f32(codes, code)
    ref = torch.from_numpy(codes.copy()).view(tdt).float().numpy()
    ok = ~np.isnan(ref)
    assert np.array_equal(vals[ok], ref[ok]) and np.array_equal(np.isnan(vals), np.isnan(ref))
    back = co.f32_to_fp8(vals, code)
    assert np.array_equal(back[ok], codes[ok])


def test_codec_known_answers():
    e4, e5 = F8["e4m3"][0], F8["e5m2"][0]
    f = lambda v, fmt: int(co.f32_to_fp8(np.array([v], np.float32), fmt)[0])
    assert f(448.0, e4) == 0x7E and f(-448.0, e4) == 0xFE
    assert f(1.0, e4) == 0x38 and f(1.0, e5) == 0x3C
    # ties to even: 17 is halfway between 16 and 18 (mantissa 000 vs 001), 19 between 18 and 20
    assert co.fp8_to_f32(np.array([f(17.0, e4)], np.uint8), e4)[0] == 16.0
    assert co.fp8_to_f32(np.array([f(19.0, e4)], np.uint8), e4)[0] == 20.0
    # smallest subnormals: 2^-9 (e4m3fn), 2^-16 (e5m2); half of them ties to zero (even)
    assert f(2.0**-9, e4) == 0x01 and f(2.0**-10, e4) == 0x00 and f(2.0**-10 * 1.01, e4) == 0x01
    assert f(2.0**-16, e5) == 0x01 and f(2.0**-17, e5) == 0x00
    assert f(57344.0, e5) == 0x7B and f(np.inf, e5) == 0x7C and f(np.inf, e4) == 0x7F
    assert f(np.nan, e4) & 0x7F == 0x7F and f(np.nan, e5) & 0x7F == 0x7F
    assert f(-0.0, e4) == 0x80


@pytest.mark.parametrize("dt", ["bf16", "fp16"])
def test_half_roundings_match_torch(dt):
    rng = np.random.default_rng(3)
    bits = np.concatenate([np.arange(0, 2**32, 65521, dtype=np.uint64).astype(np.uint32),
                           rng.integers(0, 2**32, size=1 << 16, dtype=np.uint64).astype(np.uint32)])
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    ref = torch.from_numpy(x.copy()).to(TORCH_DT[dt]).view(torch.int16).numpy().view(np.uint16)
    L = co.lib()
    fn = L.f8o_f32_to_bf16 if dt == "bf16" else L.f8o_f32_to_fp16
    ours = np.array([fn(float(v)) for v in x[:20000]], np.uint16)
    assert np.array_equal(ours, ref[:20000])
    # and back: all 65536 patterns widen exactly
    allb = np.arange(65536, dtype=np.uint16)
    wide = torch.from_numpy(allb.view(np.int16).copy()).view(TORCH_DT[dt]).float().numpy()
    back = L.f8o_bf16_to_f32 if dt == "bf16" else L.f8o_fp16_to_f32
    mine = np.array([back(int(b)) for b in allb], np.float32)
    ok = ~np.isnan(wide)
    assert np.array_equal(mine[ok], wide[ok])


# --------------------------------------------------------------------- scale


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
@pytest.mark.parametrize("dt", ["bf16", "fp16"])
def test_scale_matches_torch_for_every_16bit_amax(dt, fmt):
    code, tdt = F8[fmt]
    allb = np.arange(0, 0x7C00 if dt == "fp16" else 0x7F80, dtype=np.uint16)  # all non-negative finite
    amax = torch.from_numpy(allb.view(np.int16).copy()).view(TORCH_DT[dt])
    ref = to.amax_to_scale(amax, tdt, TORCH_DT[dt]).numpy()
    wide = amax.float().numpy()
    ours = np.array([co.amax_to_scale(a, CODE_DT[dt], code, dt == "fp16") for a in wide], np.float32)
    assert np.array_equal(ours.view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
@pytest.mark.parametrize("orig", ["bf16", "fp16", "fp32"])
def test_scale_fp32_math_matches_torch(orig, fmt):
    code, tdt = F8[fmt]
    rng = np.random.default_rng(11)
    amax = np.abs(rng.standard_normal(20000).astype(np.float32)) * 10.0 ** rng.integers(-14, 6, 20000).astype(np.float32)
    amax[:4] = [0.0, 1e-13, 1.0, 3.4e38]
    ref = to.amax_to_scale(torch.from_numpy(amax.copy()), tdt, TORCH_DT[orig]).numpy()
    ours = np.array([co.amax_to_scale(a, co.FP32, code, orig == "fp16") for a in amax], np.float32)
    assert np.array_equal(ours.view(np.uint32), ref.view(np.uint32))


def test_scale_known_answers():
    # amax = 1 -> scale = fmax exactly; powers of two are exact in every dtype
    for dt in (co.BF16, co.FP16, co.FP32):
        assert co.amax_to_scale(1.0, dt, co.E4M3FN) == 448.0
        assert co.amax_to_scale(1.0, dt, co.E5M2) == 57344.0
        assert co.amax_to_scale(4.0, dt, co.E4M3FN) == 112.0
        assert co.amax_to_scale(0.5, dt, co.E5M2, dt == co.FP16) == (65504.0 if dt == co.FP16 else 114688.0)
    # all-zero tensor: EPS is rounded to the tensor dtype first
    assert co.amax_to_scale(0.0, co.BF16, co.E4M3FN) == np.float32(446401720877056.0)
    assert co.amax_to_scale(0.0, co.FP32, co.E4M3FN) == np.float32(448.0) * (np.float32(1.0) / np.float32(1e-12))
    # fp16: EPS rounds to 0, 1/0 = inf, clamp to 65504 (reference test_base.py:566-586)
    assert co.amax_to_scale(0.0, co.FP16, co.E4M3FN, True) == 65504.0
    assert np.isnan(co.amax_to_scale(np.nan, co.BF16, co.E4M3FN))
    # dY = ones (benchmark configuration 1): scale 57344, every byte 0x7B
    assert co.cast(np.full((2, 4), 0x3F80, np.uint16), co.BF16, 57344.0, co.BF16, co.E5M2)[0].tolist() == [[0x7B] * 4] * 2


# ------------------------------------------------- golden: casts and scales


def _cases(g):
    return sorted({k[: -len(".x")] for k in g.files if k.endswith(".x")})


def test_golden_scales_and_casts_both_oracles():
    g = load("casts")
    n = 0
    for case in _cases(g):
        dt = case.split(".")[0]
        x = from_bits(g[case + ".x"], dt)
        xc = np_for_c(x)
        for fmt, (code, tdt) in F8.items():
            s_gold = g[f"{case}.{fmt}.scale"]
            # amax + scale
            a = co.amax(xc, CODE_DT[dt])
            assert a == to.tensor_to_amax(x).float().item()
            s_c = co.amax_to_scale(a, CODE_DT[dt], code, dt == "fp16")
            s_t = to.tensor_to_scale(x, tdt).numpy()
            assert np.float32(s_c).view(np.uint32) == s_gold.view(np.uint32), (case, fmt)
            assert s_t.view(np.uint32) == s_gold.view(np.uint32), (case, fmt)
            # dynamic-style cast (0-dim scale: product in x's dtype)
            want = g[f"{case}.{fmt}.dyn"]
            got_c, got_ct = co.cast(xc, CODE_DT[dt], s_gold, CODE_DT[dt], code, transpose=True)
            got_t = fp8_bytes(to.cast_to_fp8(x, torch.tensor(float(s_gold)), tdt))
            assert np.array_equal(got_c, want), (case, fmt, "c dyn")
            assert np.array_equal(got_ct, want.T), (case, fmt, "c dyn transposed")
            assert np.array_equal(got_t, want), (case, fmt, "torch dyn")
            # delayed-style cast ([1] scale: product in fp32), partly saturating
            s1 = g[f"{case}.{fmt}.scale1"]
            want = g[f"{case}.{fmt}.del"]
            got_c, _ = co.cast(xc, CODE_DT[dt], s1[0], co.FP32, code)
            got_t = fp8_bytes(to.cast_to_fp8(x, torch.from_numpy(s1.copy()), tdt))
            assert np.array_equal(got_c, want), (case, fmt, "c del")
            assert np.array_equal(got_t, want), (case, fmt, "torch del")
            n += 1
    assert n == 36


def test_golden_history_to_scale():
    g = load("casts")
    hist = g["hist"]
    for fmt, (code, tdt) in F8.items():
        for dt in ("bf16", "fp16", "fp32"):
            want = g[f"hist.{fmt}.{dt}"]
            got = np.array([co.amax_to_scale(row.max(), co.FP32, code, dt == "fp16") for row in hist], np.float32)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (fmt, dt)


def test_casts_random_c_vs_torch():
    """Beyond the fixtures: the two restatements agree on fresh heavy-tailed data."""
    torch.manual_seed(5)
    for dt in ("bf16", "fp16", "fp32"):
        x = (torch.distributions.StudentT(3.0).sample((257, 131)) * 3).to(TORCH_DT[dt])
        x[3, 5] = 1000.0
        for fmt, (code, tdt) in F8.items():
            s = to.tensor_to_scale(x, tdt)
            for prod, sc in ((CODE_DT[dt], s), (co.FP32, s.reshape(1) * 1.3)):
                want = fp8_bytes(to.cast_to_fp8(x, sc, tdt))
                got, _ = co.cast(np_for_c(x), CODE_DT[dt], sc.reshape(-1)[0].item(), prod, code)
                assert np.array_equal(got, want), (dt, fmt, prod)


# ------------------------------------------------------------------- sync


def test_sync_entry_closed_forms():
    h = np.array([3.0, 0.0, 9.0, 100.0], np.float32)
    # roll drops the LAST slot (100) and puts amax in front: max(5, 3, 0, 9) = 9
    s = co.sync_entry(5.0, h, co.E4M3FN)
    assert s == np.float32(448.0) * (np.float32(1.0) / np.float32(9.0))
    assert h.tolist() == [3.0, 0.0, 9.0, 100.0]  # reference behaviour: history untouched
    s = co.sync_entry(5.0, h, co.E4M3FN, writeback=True)
    assert h.tolist() == [5.0, 3.0, 0.0, 9.0]
    # fresh module: amax = fmax default, zero history -> scale 1
    assert co.sync_entry(448.0, np.zeros(16, np.float32), co.E4M3FN) == 1.0
    assert co.sync_entry(57344.0, np.zeros(16, np.float32), co.E5M2) == 1.0
    # history of length one holds nothing but the current amax
    assert co.sync_entry(2.0, np.array([64.0], np.float32), co.E4M3FN) == 224.0
    # init: history[0] <- amax, scale from max(history)
    h = np.array([0.0, 0.0, 7.0], np.float32)
    s = co.delayed_init(2.0, h, co.E5M2)
    assert h.tolist() == [2.0, 0.0, 7.0] and s == np.float32(57344.0) * (np.float32(1.0) / np.float32(7.0))


# -------------------------------------------------------------------- gemm


def test_gemm_closed_forms_and_brute_force():
    e4, e5 = co.E4M3FN, co.E5M2
    one4, one5 = 0x38, 0x3C
    # identity: A * I = A
    a = np.random.default_rng(0).integers(0, 0x7E, size=(5, 6), dtype=np.uint8)
    eye = np.zeros((6, 6), np.uint8)
    np.fill_diagonal(eye, one4)
    out = co.gemm_emulated(a, e4, 1.0, eye, e4, 1.0, co.FP32)
    assert np.array_equal(out, co.fp8_to_f32(a, e4).reshape(5, 6))
    # all ones: every entry = k / (sa*sb)
    out = co.gemm_emulated(np.full((3, 40), one5, np.uint8), e5, 2.0, np.full((4, 40), one4, np.uint8), e4, 4.0, co.BF16)
    assert np.all(out == 5.0)
    # brute force in float64 on random codes, against both restatements
    rng = np.random.default_rng(1)
    a = rng.integers(0, 256, size=(7, 33), dtype=np.uint8)
    b = rng.integers(0, 256, size=(9, 33), dtype=np.uint8)
    a[(a & 0x7C) == 0x7C] = 0x10  # keep e5m2 inf/NaN out
    b[(b & 0x7F) == 0x7F] = 0x10  # keep e4m3fn NaN out
    sa, sb = 3.5, 0.25
    av = co.fp8_to_f32(a, e5).reshape(a.shape).astype(np.float64)
    bv = co.fp8_to_f32(b, e4).reshape(b.shape).astype(np.float64)
    exact = (av / sa) @ (bv / sb).T
    out = co.gemm_emulated(a, e5, sa, b, e4, sb, co.FP32)
    np.testing.assert_allclose(out, exact, rtol=1e-6, atol=1e-6 * np.abs(exact).max())
    t = to.mm_emulated(torch.from_numpy(a).view(torch.float8_e5m2), torch.tensor(sa),
                       torch.from_numpy(b).view(torch.float8_e4m3fn).t(), torch.tensor(sb), torch.float32).numpy()
    np.testing.assert_allclose(t, exact, rtol=1e-5, atol=1e-5 * np.abs(exact).max())
    # a transposed operand would fail this: non-square, asymmetric
    assert out.shape == (7, 9)


# ---------------------------------------------------- golden: trajectories

TRAJ = [
    ("traj_del_bf16", ("del", "del", "del"), 4, 7, "bf16"),
    ("traj_del_fp32", ("del", "del", "del"), 16, 5, "fp32"),
    ("traj_mix1_bf16", ("dyn", "del", "dyn"), 16, 4, "bf16"),
    ("traj_mix2_bf16", ("del", "dyn", "del"), 2, 5, "bf16"),
    ("traj_dyn_bf16", ("dyn", "dyn", "dyn"), 16, 2, "bf16"),
    ("traj_del_h1_bf16", ("del", "del", "del"), 1, 4, "bf16"),
]


def _check_buffers(g, tag, layers, name):
    for li, lay in enumerate(layers):
        for kind in ("input", "weight", "grad_output"):
            st = lay.st[kind]
            for field, val in (("amax", st.amax), ("hist", st.history), ("scale", st.scale)):
                want = g[f"{tag}.L{li}.{field}_{kind}"]
                assert np.array_equal(val.numpy().view(np.uint32), want.view(np.uint32)), (name, tag, li, field, kind)


@pytest.mark.parametrize("name,scaling,hist,steps,dt", TRAJ)
def test_golden_trajectory_torch_oracle(name, scaling, hist, steps, dt):
    """Multi-step sync -> forward -> backward of a 2-layer model, against what the reference produced."""
    g = load(name)
    w0, b0, w1 = from_bits(g["w0"], dt), from_bits(g["b0"], dt), from_bits(g["w1"], dt)
    l0 = to.LinearOracle(w0, scaling, hist)
    l1 = to.LinearOracle(w1, scaling, hist)
    delayed = "del" in scaling
    for t in range(steps):
        x, gy = from_bits(g[f"t{t}.x"], dt), from_bits(g[f"t{t}.gy"], dt)
        if delayed:
            l0.sync()
            l1.sync()
            _check_buffers(g, f"t{t}.synced", (l0, l1), name)
        h = l0.forward(x) + b0
        y = l1.forward(h)
        dh, dw1 = l1.backward(gy)
        dx, dw0 = l0.backward(dh)
        db0 = dh.reshape(-1, dh.shape[-1]).sum(0)
        if delayed:
            _check_buffers(g, f"t{t}.after", (l0, l1), name)
        # GEMM outputs: the fp32 summation order of the CPU BLAS is not part of the contract, so the bar is one ulp of
        # the output dtype (bf16: 2^-7 relative) plus half an ulp of the largest output for sums that cancel.  (On the
        # CPU the fixtures were written on, the oracle reproduces them bit for bit.)
        for key, val in (("y", y), ("dx", dx), ("dw0", dw0), ("dw1", dw1), ("db0", db0)):
            want = from_bits(g[f"t{t}.{key}"], dt).float()
            torch.testing.assert_close(val.float(), want, rtol=2.0**-7, atol=2.0**-9 * want.abs().max().item())


def test_golden_trajectory_c_oracle_scales():
    """The scalar C restatement of init + sync reproduces every scale of the all-delayed run."""
    g = load("traj_del_bf16")
    hist_len, steps = 4, 7
    for li in range(2):
        for kind, fmt in (("input", co.E4M3FN), ("weight", co.E4M3FN), ("grad_output", co.E5M2)):
            hist = np.zeros(hist_len, np.float32)
            amax = np.float32(448.0 if fmt == co.E4M3FN else 57344.0)
            for t in range(steps):
                s = co.sync_entry(amax, hist, fmt)
                assert np.float32(s).view(np.uint32) == g[f"t{t}.synced.L{li}.scale_{kind}"].view(np.uint32)[0]
                assert np.array_equal(hist, g[f"t{t}.synced.L{li}.hist_{kind}"])
                amax = g[f"t{t}.after.L{li}.amax_{kind}"][0]  # this step's tensor amax (from the fixture)
                if t == 0:
                    s = co.delayed_init(amax, hist, fmt)
                    assert np.float32(s).view(np.uint32) == g[f"t0.after.L{li}.scale_{kind}"].view(np.uint32)[0]
                assert np.array_equal(hist, g[f"t{t}.after.L{li}.hist_{kind}"])


# ------------------------------------------------------- golden: config 1


def test_golden_cfg1_bytes_and_scales():
    import hashlib

    g = load("cfg1")
    sha = lambda a: np.frombuffer(hashlib.sha256(np.ascontiguousarray(a).tobytes()).digest(), np.uint8)
    torch.manual_seed(0)
    lin = torch.nn.Linear(4096, 4096, bias=False).to(torch.bfloat16)
    x = torch.randn(2048, 4096).to(torch.bfloat16)
    w = lin.weight.detach()
    assert np.array_equal(sha(x.view(torch.int16).numpy()), g["x_sha"]), "seeded input differs from the fixture's"
    assert np.array_equal(sha(w.view(torch.int16).numpy()), g["w_sha"])
    sx, sw = to.tensor_to_scale(x, to.E4M3), to.tensor_to_scale(w, to.E4M3)
    assert sx.numpy().view(np.uint32) == g["sx"].view(np.uint32)
    assert sw.numpy().view(np.uint32) == g["sw"].view(np.uint32)
    assert np.array_equal(sha(fp8_bytes(to.cast_to_fp8(x, sx, to.E4M3))), g["x_fp8_sha"])
    assert np.array_equal(sha(fp8_bytes(to.cast_to_fp8(w, sw, to.E4M3))), g["w_fp8_sha"])
    # the scalar C restatement on the same tensors
    xc = np_for_c(x)
    a = co.amax(xc, co.BF16)
    assert co.amax_to_scale(a, co.BF16, co.E4M3FN) == g["sx"]
    assert np.array_equal(sha(co.cast(xc, co.BF16, g["sx"], co.BF16, co.E4M3FN)[0]), g["x_fp8_sha"])
    # dY = ones: scale 57344, every byte 0x7B
    assert g["sg"] == 57344.0 and g["dy_fp8_first"].tolist() == [0x7B] * 8
    dy = torch.ones(2048, 4096, dtype=torch.bfloat16)
    sg = to.tensor_to_scale(dy, to.E5M2)
    assert sg.item() == 57344.0
    assert np.array_equal(sha(fp8_bytes(to.cast_to_fp8(dy, sg, to.E5M2))), g["dy_fp8_sha"])
