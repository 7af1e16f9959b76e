"""Parity of the HIP kernels (through the C ABI) with the CPU oracle.  Needs an MI355X.

Bars: amax, scales and fp8 bytes bit-exact (NaN codes may differ in the sign
bit); GEMM within a stated tolerance of the emulated fp32 product.
"""
import math

import numpy as np
import pytest
import torch

from tests.helpers import CODE_DT, F8, TORCH_DT, fp8_bytes, np_for_c, same_bytes_mod_nan_sign

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def nat():
    if not torch.cuda.is_available():
        pytest.fail("these tests need a GPU (run with -m gpu on an MI355X box)")
    from float8_experimental_amd import _native

    _native.lib()
    return _native


def _oracles():
    from oracle import c_oracle as co
    from oracle import torch_oracle as to

    return co, to


def heavy(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    t = torch.distributions.StudentT(3.0).sample(shape)
    mask = torch.rand(shape, generator=g) < 0.001
    return torch.where(mask, t * 1000, t).to(dtype)


# ------------------------------------------------------------------ K1 amax


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", [(1,), (7,), (4, 8), (33, 47), (257, 1031), (1024, 4096), (3, 5, 64)])
def test_amax_scale_matches_oracle(nat, dt, shape):
    co, to = _oracles()
    torch.manual_seed(hash((dt, shape)) % 1000)
    x = heavy(shape, TORCH_DT[dt], 1)
    xd = x.to(DEV)
    for fmt, (code, tdt) in F8.items():
        amax, scale = nat.amax_scale(xd, tdt)
        want_a = to.tensor_to_amax(x).float()
        want_s = to.tensor_to_scale(x, tdt)
        assert amax.cpu().view(torch.int32).item() == want_a.view(torch.int32).item()
        assert scale.cpu().view(torch.int32).item() == want_s.view(torch.int32).item(), (dt, fmt, shape)
        # fp32 math (delayed-scaling buffers)
        _, s32 = nat.amax_scale(xd, tdt, math_dtype=torch.float32)
        want = to.amax_to_scale(want_a, tdt, TORCH_DT[dt])
        assert s32.cpu().view(torch.int32).item() == want.view(torch.int32).item()


def test_amax_strided_rows_and_unaligned_views(nat):
    co, to = _oracles()
    torch.manual_seed(3)
    base = torch.randn(64, 300).to(torch.bfloat16)
    based = base.to(DEV)
    for view in (lambda t: t[:, 3:259], lambda t: t[5:40, 1:2], lambda t: t[:, ::2], lambda t: t.t()):
        x, xd = view(base), view(based)
        amax, scale = nat.amax_scale(xd, torch.float8_e4m3fn)
        assert amax.item() == to.tensor_to_amax(x).float().item()
        assert scale.item() == to.tensor_to_scale(x, torch.float8_e4m3fn).item()


def test_amax_specials(nat):
    co, to = _oracles()
    for dt in (torch.bfloat16, torch.float16, torch.float32):
        z = torch.zeros(1000, dtype=dt, device=DEV)
        for f8 in (torch.float8_e4m3fn, torch.float8_e5m2):
            a, s = nat.amax_scale(z, f8)
            assert a.item() == 0.0
            assert s.item() == to.tensor_to_scale(torch.zeros(4, dtype=dt), f8).item()
        z[77] = float("nan")
        a, s = nat.amax_scale(z, torch.float8_e4m3fn)
        assert torch.isnan(a).item() and torch.isnan(s).item()
        z[77] = float("-inf")
        a, s = nat.amax_scale(z, torch.float8_e4m3fn)
        assert a.item() == float("inf") and s.item() == 0.0
    # the workspace is left clean: a later call on other data is unaffected
    a, _ = nat.amax_scale(torch.full((10,), 0.5, dtype=torch.bfloat16, device=DEV), torch.float8_e4m3fn)
    assert a.item() == 0.5


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
def test_amax_of_many_tensors_in_one_pass_matches_oracle(nat, dt):
    """f8mi_amax_scale_multi: sizes around the tile (32 KB) and vector (16 B) boundaries, an empty tensor,
    a NaN and an inf, against the oracle and against the one-tensor entry point, bit for bit."""
    co, to = _oracles()
    tdt = TORCH_DT[dt]
    tile = nat.lib().f8mi_amax_tile_elems(nat._DT[tdt])
    sizes = [1, 7, 8, 9, 0, tile - 1, tile, tile + 1, 3 * tile, 3 * tile + 5, 1000003, 5 * tile - 8, 2, 20 * tile + 3]
    hosts = [heavy((n,), tdt, 10 + i) * (0.01 * (i + 1)) for i, n in enumerate(sizes)]
    hosts[5][-1] = float("nan")          # in the partial last tile
    hosts[8][tile + 17] = float("-inf")  # in a whole tile
    hosts[9][-1] = 3.0e4                 # the maximum sits in the < 16-byte tail
    devs = [h.to(DEV) for h in hosts]
    for fmt, (code, f8dt) in F8.items():
        amaxes, scales = nat.amax_scale_multi(devs, f8dt)
        assert amaxes.shape == scales.shape == (len(sizes),)
        for i, (h, d) in enumerate(zip(hosts, devs)):
            a1, s1 = nat.amax_scale(d, f8dt)
            assert amaxes[i].view(torch.int32).item() == a1.view(torch.int32).item(), (dt, fmt, sizes[i])
            assert scales[i].view(torch.int32).item() == s1.view(torch.int32).item(), (dt, fmt, sizes[i])
            if h.numel() and not torch.isnan(h).any():
                assert amaxes[i].item() == to.tensor_to_amax(h).float().item()
                assert scales[i].cpu().view(torch.int32).item() == to.tensor_to_scale(h, f8dt).view(torch.int32).item()
        assert torch.isnan(amaxes[5]).item() and torch.isnan(scales[5]).item()
        assert amaxes[8].item() == float("inf") and scales[8].item() == 0.0
    # the same list again (cached table) after the data changed
    devs[0].fill_(5.0)
    amaxes, _ = nat.amax_scale_multi(devs, torch.float8_e4m3fn)
    assert amaxes[0].item() == 5.0


def test_amax_of_more_tensors_than_one_call_takes(nat):
    n = nat.lib().f8mi_workspace_bytes() // 4 + 300
    torch.manual_seed(5)
    big = torch.randn(n, 24, device=DEV).to(torch.bfloat16)  # rows of 48 bytes: 16-byte aligned
    rows = [big[i] for i in range(n)]
    amaxes, scales = nat.amax_scale_multi(rows, torch.float8_e5m2)
    want = big.abs().amax(dim=1).float()
    assert torch.equal(amaxes, want)
    _, s = nat.amax_scale(rows[n - 1], torch.float8_e5m2)
    assert scales[n - 1].item() == s.item()


@pytest.mark.parametrize("dt", ["bf16", "fp16"])
def test_scale_math_sweep_16bit(nat, dt):
    """Scale arithmetic in the tensor's own dtype over a sweep of amax bit patterns."""
    co, to = _oracles()
    top = 0x7C00 if dt == "fp16" else 0x7F80
    pats = np.unique(np.concatenate([np.arange(0, top, 37), np.array([0, 1, 2, top - 1, 0x3F80, 0x3C00])])).astype(np.uint16)
    for fmt, (code, tdt) in F8.items():
        for p in pats[:: 1 if dt == "bf16" else 2]:
            x = torch.from_numpy(np.array([0, p, 0], np.uint16).view(np.int16)).view(TORCH_DT[dt]).to(DEV)
            a, s = nat.amax_scale(x, tdt)
            want = co.amax_to_scale(a.item(), CODE_DT[dt], code, dt == "fp16")
            assert np.float32(s.item()).view(np.uint32) == np.float32(want).view(np.uint32), (dt, fmt, hex(int(p)))


# ------------------------------------------------------------------ K2 cast


def _ref_cast(x_cpu, scale_cpu, tdt, delayed):
    _, to = _oracles()
    s = scale_cpu.reshape(1) if delayed else scale_cpu.reshape(())
    return fp8_bytes(to.cast_to_fp8(x_cpu, s, tdt))


@pytest.mark.parametrize("dt", ["bf16", "fp16"])
@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_cast_every_16bit_pattern(nat, dt, fmt):
    code, tdt = F8[fmt]
    allb = np.arange(65536, dtype=np.uint16)
    x = torch.from_numpy(allb.view(np.int16).copy()).view(TORCH_DT[dt]).reshape(256, 256)
    xd = x.to(DEV)
    scales = [1.0, 448.0 / 3.0, 0.0123, 57344.0 / 0.011, 1e-6, 3.3e4, 2.0**-20, 1.7]
    for s in scales:
        for delayed in (False, True):
            sc = torch.tensor(s, dtype=torch.float32)
            if dt == "fp16" and not delayed and s > 65504:
                continue
            want = _ref_cast(x, sc, tdt, delayed)
            out, out_t = nat.cast(xd, sc.to(DEV), tdt, product_dtype=torch.float32 if delayed else TORCH_DT[dt],
                                  want_out_t=True)
            got = fp8_bytes(out)
            assert same_bytes_mod_nan_sign(got, want), (dt, fmt, s, delayed, int((got != want).sum()))
            assert np.array_equal(fp8_bytes(out_t), got.T)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_cast_fp32_bit_patterns(nat, fmt):
    code, tdt = F8[fmt]
    rng = np.random.default_rng(5)
    bits = np.concatenate([np.arange(0, 2**32, 8191, dtype=np.uint64).astype(np.uint32)[: 512 * 1024],
                           rng.integers(0, 2**32, size=512 * 1024, dtype=np.uint64).astype(np.uint32)])
    x = torch.from_numpy(bits.view(np.float32).copy()).reshape(1024, 1024)
    xd = x.to(DEV)
    for s in (1.0, 0.37, 1234.5):
        sc = torch.tensor(s, dtype=torch.float32)
        want = _ref_cast(x, sc, tdt, True)
        out, out_t = nat.cast(xd, sc.to(DEV), tdt, want_out_t=True)
        assert same_bytes_mod_nan_sign(fp8_bytes(out), want)
        assert np.array_equal(fp8_bytes(out_t), fp8_bytes(out).T)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", [(1, 1), (1, 129), (129, 1), (16, 16), (33, 47), (128, 128), (257, 131), (130, 1000),
                                   (1000, 136), (4099, 1000), (2, 3, 40)])
def test_cast_shapes_dynamic_and_delayed(nat, dt, shape):
    co, to = _oracles()
    x = heavy(shape, TORCH_DT[dt], 2)
    xd = x.to(DEV)
    x2 = x.reshape(-1, shape[-1])
    for fmt, (code, tdt) in F8.items():
        s = to.tensor_to_scale(x, tdt)
        # dynamic: product in the tensor's dtype
        out, out_t = nat.cast(xd, s.to(DEV), tdt, want_out_t=True)
        want = fp8_bytes(to.cast_to_fp8(x, s, tdt))
        assert out.shape == x.shape and out_t.shape == (x2.shape[1], x2.shape[0])
        assert np.array_equal(fp8_bytes(out), want), (dt, fmt, shape)
        assert np.array_equal(fp8_bytes(out_t), want.reshape(x2.shape).T)
        # delayed: [1]-shaped scale that saturates part of the tensor, amax fused
        s1 = (s * 2.5).reshape(1)
        amax = torch.full((1,), -1.0, dtype=torch.float32, device=DEV)
        out, out_t = nat.cast(xd, s1.to(DEV), tdt, product_dtype=torch.float32, want_out_t=True, amax_out=amax)
        want = fp8_bytes(to.cast_to_fp8(x, s1, tdt))
        assert np.array_equal(fp8_bytes(out), want), (dt, fmt, shape, "delayed")
        assert np.array_equal(fp8_bytes(out_t), want.reshape(x2.shape).T)
        assert amax.item() == to.tensor_to_amax(x).float().item()
        # only the transposed copy
        _, only_t = nat.cast(xd, s1.to(DEV), tdt, product_dtype=torch.float32, want_out=False, want_out_t=True)
        assert np.array_equal(fp8_bytes(only_t), want.reshape(x2.shape).T)


@pytest.mark.parametrize("dt", ["bf16", "fp32"])
@pytest.mark.parametrize("shape", [(64, 64), (128, 192), (448, 384), (320, 1024), (1000, 128), (192, 1000), (4, 96, 256)])
def test_cast_kblocked_layout_is_a_permutation_of_the_row_major_bytes(nat, dt, shape):
    """k-blocked outputs ([k/64][rows][64]) hold exactly the row-major result's bytes, re-placed; where a
    dimension is not a multiple of 64 the request is refused."""
    co, to = _oracles()
    x = heavy(shape, TORCH_DT[dt], 5)
    xd = x.to(DEV)
    rows, cols = x.numel() // shape[-1], shape[-1]
    tdt = torch.float8_e4m3fn
    s = to.tensor_to_scale(x, tdt).to(DEV)
    ref, ref_t = nat.cast(xd, s, tdt, want_out_t=True)
    ref_b, ref_tb = fp8_bytes(ref).reshape(rows, cols), fp8_bytes(ref_t)
    row_ok, t_ok = cols % 64 == 0, rows % 64 == 0
    amax = torch.zeros(1, dtype=torch.float32, device=DEV)
    out, out_t = nat.cast(xd, s, tdt, want_out=row_ok, want_out_t=t_ok, out_kblock=row_ok, out_t_kblock=t_ok,
                          amax_out=amax if (row_ok or t_ok) else None) if (row_ok or t_ok) else (None, None)
    if row_ok:
        assert out.shape == (cols // 64, rows, 64)
        assert np.array_equal(fp8_bytes(out), ref_b.reshape(rows, cols // 64, 64).transpose(1, 0, 2))
        # mixed: k-blocked out with a row-major transpose
        o2, t2 = nat.cast(xd, s, tdt, want_out_t=True, out_kblock=True)
        assert np.array_equal(fp8_bytes(o2), fp8_bytes(out)) and np.array_equal(fp8_bytes(t2), ref_tb)
    else:
        with pytest.raises(AssertionError):
            nat.cast(xd, s, tdt, out_kblock=True)
    if t_ok:
        assert out_t.shape == (rows // 64, cols, 64)
        assert np.array_equal(fp8_bytes(out_t), ref_tb.reshape(cols, rows // 64, 64).transpose(1, 0, 2))
    else:
        with pytest.raises(AssertionError):
            nat.cast(xd, s, tdt, want_out=False, want_out_t=True, out_t_kblock=True)
    if row_ok or t_ok:
        assert amax.item() == to.tensor_to_amax(x).float().item()


def test_cast_kblocked_refused_by_the_library_when_not_a_multiple_of_64(nat):
    x = torch.ones(100, 96, dtype=torch.bfloat16, device=DEV)
    s = torch.ones((), device=DEV)
    out = torch.empty(100 * 96, dtype=torch.uint8, device=DEV)
    L = nat.lib()
    rc = L.f8mi_cast_layout(x.data_ptr(), 100, 96, 96, 0, s.data_ptr(), 0, 0, out.data_ptr(), 1, None, 0, None, None)
    assert rc != 0 and b"64" in L.f8mi_last_error()
    rc = L.f8mi_cast_layout(x.data_ptr(), 100, 96, 96, 0, s.data_ptr(), 0, 0, None, 0, out.data_ptr(), 1, None, None)
    assert rc != 0
    rc = L.f8mi_cast_layout(x.data_ptr(), 100, 96, 96, 0, s.data_ptr(), 0, 0, out.data_ptr(), 7, None, 0, None, None)
    assert rc != 0


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
def test_delayed_cast_with_workspace_equals_the_cast_without(nat, dt):
    """f8mi_cast_delayed folds the amax into the 1024 words of its workspace and a second launch reduces them: same bytes
    and the same amax as f8mi_cast_layout with amax_dev, the oracle's amax (NaN, inf, all-zero and all-negative-zero
    tensors included), and the workspace is all zero again after every call -- also on the next, smaller call."""
    co, to = _oracles()
    L = nat.lib()
    assert L.f8mi_delayed_workspace_bytes() == 4096
    tdt = torch.float8_e4m3fn
    cases = [heavy((777, 1031), TORCH_DT[dt], 3), heavy((4, 8), TORCH_DT[dt], 4), heavy((2048, 4096), TORCH_DT[dt], 5),
             torch.zeros(300, 200, dtype=TORCH_DT[dt]), -torch.zeros(130, 70, dtype=TORCH_DT[dt])]
    nan = heavy((257, 513), TORCH_DT[dt], 6)
    nan[100, 17] = float("nan")
    inf = heavy((129, 257), TORCH_DT[dt], 7)
    inf[5, 5] = float("-inf")
    cases += [nan, inf]
    ws = nat.delayed_workspace(torch.device(DEV))
    for x in cases:
        xd = x.to(DEV)
        s1 = torch.tensor([1.7], device=DEV)
        a_new = torch.full((1,), -1.0, device=DEV)
        a_old = torch.full((1,), -1.0, device=DEV)
        out, out_t = nat.cast(xd, s1, tdt, product_dtype=torch.float32, want_out_t=True, amax_out=a_new)   # f8mi_cast_delayed
        o2 = torch.empty_like(out)
        t2 = torch.empty_like(out_t)
        rc = L.f8mi_cast_layout(xd.data_ptr(), x.shape[0], x.shape[1], x.shape[1], CODE_DT[dt], s1.data_ptr(), 2, 0, o2.data_ptr(), 0,
                                t2.data_ptr(), 0, a_old.data_ptr(), None)
        assert rc == 0
        assert torch.equal(out.view(torch.uint8), o2.view(torch.uint8)) and torch.equal(out_t.view(torch.uint8), t2.view(torch.uint8))
        want = to.tensor_to_amax(x).float()
        for a in (a_new, a_old):
            assert (math.isnan(a.item()) and math.isnan(want.item())) or a.item() == want.item(), (dt, tuple(x.shape), a.item(), want.item())
        assert not ws.any().item(), "the workspace must be all zero after a call"


def _unblock(t_kb):
    """[kc/64, rows, 64] k-blocked bytes -> [rows, kc] row-major (numpy)."""
    b = fp8_bytes(t_kb)
    return b.transpose(1, 0, 2).reshape(b.shape[1], b.shape[0] * 64)


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", [(1, 1), (33, 47), (128, 128), (257, 131), (130, 1000), (1000, 136), (4099, 1000), (200, 4097),
                                   (3, 50, 70)])
def test_cast_zero_padded_kblocked_layout(nat, dt, shape):
    """F8MI_LAYOUT_KBLOCK64_PAD128 takes any shape: the output holds the row-major result's bytes, k-blocked after the
    contraction has been extended to a multiple of 128, and every byte of the extension is zero -- with a dynamic
    scale, a delayed one (amax fused), for both fp8 formats, for rows at an unaligned pitch, and under a NaN scale."""
    co, to = _oracles()
    x = heavy(shape, TORCH_DT[dt], 11)
    rows, cols = x.numel() // shape[-1], shape[-1]
    rp, cp = nat.padded_k(rows), nat.padded_k(cols)
    xd = x.to(DEV)

    def check(out, out_t, want, what):
        assert out.shape == (cp // 64, rows, 64) and out_t.shape == (rp // 64, cols, 64), what
        o, t = _unblock(out), _unblock(out_t)
        assert np.array_equal(o[:, :cols], want) and not o[:, cols:].any(), what
        assert np.array_equal(t[:, :rows], want.T) and not t[:, rows:].any(), what

    for fmt, (code, tdt) in F8.items():
        s = to.tensor_to_scale(x, tdt)
        want = fp8_bytes(to.cast_to_fp8(x, s, tdt)).reshape(rows, cols)
        out, out_t, sc = nat.cast_dynamic(xd, tdt, want_out_t=True, out_kblock=nat.KBLOCK_PAD, out_t_kblock=nat.KBLOCK_PAD)
        assert sc.item() == s.item()
        check(out, out_t, want, (dt, fmt, shape, "dynamic"))
        s1 = (s * 2.5).reshape(1)
        amax = torch.full((1,), -1.0, dtype=torch.float32, device=DEV)
        out, out_t = nat.cast(xd, s1.to(DEV), tdt, product_dtype=torch.float32, want_out_t=True, amax_out=amax,
                              out_kblock=nat.KBLOCK_PAD, out_t_kblock=nat.KBLOCK_PAD)
        check(out, out_t, fp8_bytes(to.cast_to_fp8(x, s1, tdt)).reshape(rows, cols), (dt, fmt, shape, "delayed"))
        assert amax.item() == to.tensor_to_amax(x).float().item()
    # one padded and one row-major output in the same call
    tdt = torch.float8_e4m3fn
    s = to.tensor_to_scale(x, tdt)
    want = fp8_bytes(to.cast_to_fp8(x, s, tdt)).reshape(rows, cols)
    out, out_t = nat.cast(xd, s.to(DEV), tdt, want_out_t=True, out_kblock=nat.KBLOCK_PAD)
    assert np.array_equal(_unblock(out)[:, :cols], want) and np.array_equal(fp8_bytes(out_t), want.T)
    out, out_t = nat.cast(xd, s.to(DEV), tdt, want_out_t=True, out_t_kblock=nat.KBLOCK_PAD)
    assert np.array_equal(fp8_bytes(out).reshape(rows, cols), want) and np.array_equal(_unblock(out_t)[:, :rows], want.T)
    # a NaN scale turns every element into a NaN code and leaves the padding zero
    out, out_t = nat.cast(xd, torch.full((), float("nan"), device=DEV), tdt, want_out_t=True, out_kblock=nat.KBLOCK_PAD,
                          out_t_kblock=nat.KBLOCK_PAD)
    o, t = _unblock(out), _unblock(out_t)
    assert ((o[:, :cols] & 0x7f) == 0x7f).all() and not o[:, cols:].any()
    assert ((t[:, :rows] & 0x7f) == 0x7f).all() and not t[:, rows:].any()
    # rows at a pitch that is no multiple of 16 bytes (a column slice of a wider tensor)
    if x.dim() == 2 and cols > 9:
        v, vd = x[:, 3:cols - 2], xd[:, 3:cols - 2]
        s = to.tensor_to_scale(v, tdt)
        want = fp8_bytes(to.cast_to_fp8(v, s, tdt)).reshape(rows, cols - 5)
        out, out_t, sc = nat.cast_dynamic(vd, tdt, want_out_t=True, out_kblock=nat.KBLOCK_PAD, out_t_kblock=nat.KBLOCK_PAD)
        o, t = _unblock(out), _unblock(out_t)
        assert sc.item() == s.item() and np.array_equal(o[:, :cols - 5], want) and not o[:, cols - 5:].any()
        assert np.array_equal(t[:, :rows], want.T) and not t[:, rows:].any()


def test_cast_row_strided_and_c_oracle(nat):
    co, to = _oracles()
    base = heavy((70, 400), torch.bfloat16, 4)
    x, xd = base[:, 8:264], base.to(DEV)[:, 8:264]     # 16-byte aligned rows, ld != cols
    y, yd = base[3:, 5:206], base.to(DEV)[3:, 5:206]   # unaligned
    for t, td in ((x, xd), (y, yd)):
        s = to.tensor_to_scale(t, torch.float8_e4m3fn)
        out, out_t = nat.cast(td, s.to(DEV), torch.float8_e4m3fn, want_out_t=True)
        want_c, want_ct = co.cast(np_for_c(t), co.BF16, s.item(), co.BF16, co.E4M3FN, transpose=True)
        assert np.array_equal(fp8_bytes(out), want_c) and np.array_equal(fp8_bytes(out_t), want_ct)


def test_cfg1_dy_ones(nat):
    """Benchmark configuration 1: dY = ones -> scale 57344, every e5m2 byte 0x7B."""
    dy = torch.ones(2048, 4096, dtype=torch.bfloat16, device=DEV)
    a, s = nat.amax_scale(dy, torch.float8_e5m2)
    assert a.item() == 1.0 and s.item() == 57344.0
    out, out_t = nat.cast(dy, s, torch.float8_e5m2, want_out_t=True)
    assert bool((out.view(torch.uint8) == 0x7B).all()) and bool((out_t.view(torch.uint8) == 0x7B).all())


@pytest.mark.parametrize("shape,strides", [((2048, 4096), (0, 0)), ((2048, 4096), (0, 1)), ((4, 300, 1000), (0, 0, 1)),
                                           ((40, 512), (0, 1))])
def test_expanded_gradient_is_cast_without_being_materialised(nat, shape, strides):
    """dY of ``y.sum().backward()`` is an expanded tensor (reference float8_scaling_utils.py:204-216 casts it like any
    other): amax, scale and bytes equal those of the materialised tensor, and the binding passes one row with row
    stride 0 instead of copying rows x cols elements."""
    torch.manual_seed(9)
    cols = shape[-1]
    base = (torch.ones(1, device=DEV) if strides[-1] == 0 else torch.randn(cols, device=DEV) * 0.3).to(torch.bfloat16)
    dy = torch.as_strided(base, shape, strides)
    full = dy.contiguous()
    read, rows, c, ld = nat._as_2d(dy)
    assert ld == 0 and read.numel() == cols and rows * c == full.numel()
    for f8, kb in ((torch.float8_e5m2, False), (torch.float8_e4m3fn, True)):
        kb = kb and cols % 64 == 0 and rows % 64 == 0
        a0, s0 = nat.amax_scale(full, f8)
        a1, s1 = nat.amax_scale(dy, f8)
        assert a0.item() == a1.item() and s0.item() == s1.item()
        o0, t0 = nat.cast(full.reshape(rows, cols), s0, f8, want_out_t=True, out_kblock=kb, out_t_kblock=kb)
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        before = torch.cuda.memory_allocated()
        o1, t1 = nat.cast(dy.reshape(rows, cols) if dy.dim() > 2 else dy, s1, f8, want_out_t=True, out_kblock=kb, out_t_kblock=kb)
        torch.cuda.synchronize()
        assert torch.cuda.max_memory_allocated() - before < 2 * full.numel() + (1 << 20)  # the two fp8 outputs, no bf16 copy
        assert torch.equal(o0.view(torch.uint8), o1.view(torch.uint8)) and torch.equal(t0.view(torch.uint8), t1.view(torch.uint8))
        o2, _, s2 = nat.cast_dynamic(dy.reshape(rows, cols) if dy.dim() > 2 else dy, f8, out_kblock=kb)
        assert s2.item() == s0.item() and torch.equal(o2.view(torch.uint8), o0.view(torch.uint8))
        amax = torch.zeros(1, device=DEV)
        one = torch.ones(1, device=DEV)
        nat.cast(dy, one, f8, product_dtype=torch.float32, amax_out=amax)  # the delayed-scaling cast records the amax
        assert amax.item() == a0.item()
    if strides[-1] == 0:  # dY = ones: scale 57344, every e5m2 byte 0x7B
        o, _, s = nat.cast_dynamic(dy, torch.float8_e5m2)
        assert s.item() == 57344.0 and bool((o.view(torch.uint8) == 0x7B).all())


def test_golden_cast_fixtures_on_gpu(nat):
    from tests.helpers import from_bits, load

    g = load("casts")
    for case in sorted({k[:-2] for k in g.files if k.endswith(".x")}):
        dt = case.split(".")[0]
        x = from_bits(g[case + ".x"], dt).to(DEV)
        for fmt, (code, tdt) in F8.items():
            a, s = nat.amax_scale(x, tdt)
            assert np.float32(s.item()).view(np.uint32) == g[f"{case}.{fmt}.scale"].view(np.uint32), (case, fmt)
            out, _ = nat.cast(x, s, tdt)
            assert np.array_equal(fp8_bytes(out), g[f"{case}.{fmt}.dyn"]), (case, fmt)
            s1 = torch.from_numpy(g[f"{case}.{fmt}.scale1"].copy()).to(DEV)
            out, _ = nat.cast(x, s1, tdt, product_dtype=torch.float32)
            assert np.array_equal(fp8_bytes(out), g[f"{case}.{fmt}.del"]), (case, fmt)


# ------------------------------------------------------------------ K3 gemm


@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", [(1, 8), (1, 8192), (3, 1000), (4, 8192), (16, 8192), (64, 512), (37, 129), (128, 1024),
                                   (200, 700), (5, 7, 64), (4096, 1), (4097, 3), (512, 4096)])
def test_cast_dynamic_equals_amax_scale_then_cast(nat, dt, shape):
    """f8mi_cast_dynamic (one workgroup up to 32 K elements, the two kernels beyond): scale and bytes of every output layout
    equal those of f8mi_amax_scale followed by f8mi_cast, bit for bit; NaN and all-zero tensors included."""
    tdt = TORCH_DT[dt]
    x = heavy(shape, tdt, 21).to(DEV)
    variants = [x]
    if len(shape) == 2 and shape[1] >= 64:
        variants.append(x[:, 3:shape[1] - 2])          # unaligned, strided rows
        z = torch.zeros_like(x)
        variants.append(z)
        n = x.clone()
        n[-1, -1] = float("nan")
        variants.append(n)
    for v in variants:
        rows, cols = v.reshape(-1, v.shape[-1]).shape
        for fmt, (code, f8dt) in F8.items():
            _, s_want = nat.amax_scale(v, f8dt, want_amax=False)
            kb, tkb = cols % 64 == 0, rows % 64 == 0
            for okb, otkb in {(False, False), (kb, tkb)}:
                o_want, t_want = nat.cast(v, s_want, f8dt, want_out_t=True, out_kblock=okb, out_t_kblock=otkb)
                o, t, s = nat.cast_dynamic(v, f8dt, want_out_t=True, out_kblock=okb, out_t_kblock=otkb)
                assert s.view(torch.int32).item() == s_want.view(torch.int32).item() or (torch.isnan(s) and torch.isnan(s_want))
                assert same_bytes_mod_nan_sign(fp8_bytes(o), fp8_bytes(o_want)), (dt, shape, fmt, okb)
                assert same_bytes_mod_nan_sign(fp8_bytes(t), fp8_bytes(t_want)), (dt, shape, fmt, otkb)
    o, t, s = nat.cast_dynamic(torch.empty(0, 64, device=DEV, dtype=tdt), torch.float8_e4m3fn, want_out_t=True)
    assert o.shape == (0, 64) and t.shape == (64, 0)
    _, s_want = nat.amax_scale(torch.empty(0, 64, device=DEV, dtype=tdt), torch.float8_e4m3fn)
    assert s.item() == s_want.item()


def _rand_fp8(shape, tdt, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    v = torch.randn(shape, generator=g) * scale
    fmax = torch.finfo(tdt).max
    return v.clamp(-fmax, fmax).to(tdt)


def _gemm_check(nat, m, n, k, a_fmt, b_fmt, out_dt, seed=0, bias=False, sa=3.0, sb=0.5):
    co, to = _oracles()
    ta, tb = F8[a_fmt][1], F8[b_fmt][1]
    a = _rand_fp8((m, k), ta, seed, 4.0)
    bt = _rand_fp8((n, k), tb, seed + 1, 4.0)
    sa_t, sb_t = torch.tensor(sa), torch.tensor(sb)
    bias_t = (torch.randn(n, generator=torch.Generator().manual_seed(seed + 2)) * 3).to(out_dt) if bias else None
    got = nat.gemm_nt(a.to(DEV), sa_t.to(DEV), bt.to(DEV), sb_t.to(DEV), out_dt,
                      bias=bias_t.to(DEV) if bias else None).cpu().double()
    ad, bd = a.double() / sa, bt.double() / sb
    exact = ad @ bd.T
    if bias:
        exact = exact + bias_t.double()
    bound = ad.abs() @ bd.abs().T + (bias_t.double().abs() if bias else 0)  # elementwise magnitude of the sum
    eps_out = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11, torch.float32: 2.0**-23}[out_dt]
    # stated tolerance: one output rounding + the matrix core's accumulation error.  The gfx950 fp8
    # MFMA aligns the products of a 64-deep block to the largest one and truncates below ~2^-14 of
    # it (measured; the vendor BLAS shows the same figures), so the error is bounded by 2^-13 of the
    # summed magnitudes of the terms.
    tol = eps_out * exact.abs() + 2.0**-13 * bound + 1e-30
    err = (got - exact).abs()
    worst = (err / tol).max().item()
    assert worst <= 1.0, (m, n, k, a_fmt, b_fmt, out_dt, worst)
    # and against the reference's emulated op itself (fp32 mm on CPU), north-star bar 1e-2
    emu = to.mm_emulated(a, sa_t, bt.t(), sb_t, out_dt)
    if bias:
        emu = emu + bias_t
    # (with a bias the emulated route rounds twice in the output dtype, product then sum: two output ulps of slack)
    allow = 1e-2 * (emu.double().abs() + 1e-2 * bound.max()) + (2 * eps_out * (emu.double().abs() + bias_t.double().abs()) if bias else 0)
    rel = ((got - emu.double()).abs() / allow).max().item()
    assert rel <= 1.0, (m, n, k, rel)


@pytest.mark.parametrize("m,n,k", [(256, 256, 128), (256, 256, 256), (512, 768, 384), (16, 32, 16), (1, 1, 1),
                                   (300, 520, 200), (257, 255, 129), (64, 4096, 1024), (1000, 3000, 4099 // 4 * 4),
                                   (129, 77, 4097), (40, 50, 1000), (2048, 512, 2048)])
def test_gemm_shapes(nat, m, n, k):
    _gemm_check(nat, m, n, k, "e4m3", "e4m3", torch.bfloat16, seed=m + n + k)


# The library has two GEMM kernels: 16-byte aligned operands with k % 64 == 0 and k >= 384 take the
# LDS-DMA kernel (compiled separately for an odd and an even count of 64-deep units), everything
# else the register-staged one.  k = 384 .. 704 walks the shortest pipelines of both parities,
# ragged m / n exercise the clamped edge rows, 8192 a long steady state.
@pytest.mark.parametrize("m,n,k", [(256, 256, 384), (256, 256, 448), (300, 200, 512), (257, 511, 576), (64, 96, 640),
                                   (512, 256, 704), (1, 1, 384), (520, 264, 8192), (256, 512, 8256)])
@pytest.mark.parametrize("out_dt", [torch.bfloat16, torch.float32])
def test_gemm_dma_kernel_shapes(nat, m, n, k, out_dt):
    _gemm_check(nat, m, n, k, "e5m2", "e4m3", out_dt, seed=m + n + k, bias=(m % 2 == 0))


# Few rows (m <= 256, k % 128 == 0, aligned): the kernel that streams Bt straight into the matrix cores and splits k
# over the eight waves of a workgroup.  m around the 16-row tile edges, n ragged against the 32-column
# workgroups, k from one step (seven idle waves) over nine (uneven split) to a long one.
@pytest.mark.parametrize("m", [1, 5, 16, 17, 32, 33, 64, 65, 100, 128, 129, 200, 256])
@pytest.mark.parametrize("n,k", [(7, 128), (32, 256), (200, 1152), (1000, 1024), (96, 8192)])
def test_gemm_few_rows_shapes(nat, m, n, k):
    fm = [("e4m3", "e4m3"), ("e5m2", "e4m3"), ("e4m3", "e5m2"), ("e5m2", "e5m2")][(m + n) % 4]
    out_dt = [torch.bfloat16, torch.float32, torch.float16][(m + k // 128) % 3]
    _gemm_check(nat, m, n, k, fm[0], fm[1], out_dt, seed=m + n + k, bias=(m % 2 == 1))


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (16, 520, 2048), (48, 1000, 640), (64, 264, 8192), (120, 264, 1024), (250, 520, 2048)])
def test_gemm_few_rows_kblocked_equals_row_major_bitwise(nat, m, n, k):
    a = _rand_fp8((m, k), torch.float8_e4m3fn, m + k, 4.0).to(DEV)
    bt = _rand_fp8((n, k), torch.float8_e4m3fn, n + k, 4.0).to(DEV)
    sa, sb = torch.tensor(2.0, device=DEV), torch.tensor(0.25, device=DEV)
    bias = torch.randn(n, device=DEV).to(torch.bfloat16)
    want = nat.gemm_nt(a, sa, bt, sb, torch.bfloat16, bias=bias)
    got = nat.gemm_nt_kb(_to_kb(a), sa, _to_kb(bt), sb, torch.bfloat16, bias=bias)
    assert torch.equal(got, want)
    # rows are independent: any subset of A's rows gives the same rows of C, whichever tile count it lands in
    sub = nat.gemm_nt(a[: max(1, m // 3)].contiguous(), sa, bt, sb, torch.bfloat16, bias=bias)
    assert torch.equal(sub, want[: max(1, m // 3)])


# Outputs that at most 256 tiles of 128 x 128 or of 128 x 256 cover (k % 128 == 0), unless the few-row kernel is
# estimated to be faster, take those tiles.
@pytest.mark.parametrize("m,n,k", [(257, 128, 128), (300, 520, 1024), (512, 1000, 256), (1024, 2048, 640), (384, 8192, 2048),
                                   (4099, 500, 1152), (1024, 8192, 1024), (1000, 5000, 384), (2049, 3000, 128),
                                   (64, 28672, 512), (20, 16384, 256)])  # few rows, wide Bt: one partial row of tiles
@pytest.mark.parametrize("out_dt", [torch.bfloat16, torch.float32])
def test_gemm_mid_tile_kernel_shapes(nat, m, n, k, out_dt):
    fm = [("e4m3", "e4m3"), ("e5m2", "e4m3"), ("e4m3", "e5m2"), ("e5m2", "e5m2")][(m + n + k // 128) % 4]
    _gemm_check(nat, m, n, k, fm[0], fm[1], out_dt, seed=m + n + k, bias=(n % 2 == 0))


# Few 128-row tiles and a long contraction: with the stream's scratch buffer k is split over workgroups and a second
# kernel adds the parts in a fixed order.
@pytest.mark.parametrize("m,n,k", [(256, 2048, 16384), (512, 1024, 8192), (100, 4096, 16384)])
def test_gemm_split_over_k(nat, m, n, k):
    a = _rand_fp8((m, k), torch.float8_e4m3fn, m + k, 4.0).to(DEV)
    bt = _rand_fp8((n, k), torch.float8_e5m2, n + k, 4.0).to(DEV)
    sa, sb = torch.tensor(0.5, device=DEV), torch.tensor(4.0, device=DEV)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 3).to(torch.bfloat16).to(DEV)
    split32 = nat.gemm_nt(a, sa, bt, sb, torch.float32)
    whole32 = nat.gemm_nt(a, sa, bt, sb, torch.float32, split_k=False)
    # another summation order (else the split did not run) but the same sums to fp32 accuracy, every time the same bits,
    # whichever layout the operands come in
    assert not torch.equal(split32, whole32)
    scale = whole32.abs().max()
    assert ((split32 - whole32).abs().max() / scale).item() < 1e-5
    assert torch.equal(nat.gemm_nt(a, sa, bt, sb, torch.float32), split32)
    assert torch.equal(nat.gemm_nt_kb(_to_kb(a), sa, _to_kb(bt), sb, torch.float32), split32)
    got = nat.gemm_nt_kb(_to_kb(a), sa, _to_kb(bt), sb, torch.bfloat16, bias=bias)
    assert torch.equal(got, nat.gemm_nt(a, sa, bt, sb, torch.bfloat16, bias=bias))
    want = (split32 + bias.float()).to(torch.bfloat16)  # one rounding of the scaled sum plus bias
    assert ((got.float() - want.float()).abs() <= 2 * torch.finfo(torch.bfloat16).eps * want.float().abs() + 1e-6).all()
    _gemm_check(nat, m, n, k, "e4m3", "e5m2", torch.bfloat16, seed=m + n, bias=True)


def test_gemm_split_over_k_random_shapes(nat):
    """Seeded shapes around the limits of the split (rows, ragged n, parts of k): whatever the plan, the result with
    the scratch buffer agrees with the one without to fp32 accuracy, and some of the shapes do get split."""
    import random

    rng = random.Random(1234)
    sa, sb = torch.tensor(2.0, device=DEV), torch.tensor(0.25, device=DEV)
    split = 0
    for case in range(14):
        m = rng.choice([17, 33, 64, 100, 128, 129, 200, 256, 257, 384, 512, 640])
        n = 4 * rng.randint(64, 768)
        k = 128 * rng.choice([32, 40, 64, 96, 112, 128, 192])
        name, parts, _ = nat.gemm_plan(m, n, k)
        split += name == "tiles128_split_k"
        a = _rand_fp8((m, k), torch.float8_e4m3fn, case, 4.0).to(DEV)
        bt = _rand_fp8((n, k), torch.float8_e4m3fn, case + 100, 4.0).to(DEV)
        with_ws = nat.gemm_nt(a, sa, bt, sb, torch.float32)
        without = nat.gemm_nt(a, sa, bt, sb, torch.float32, split_k=False)
        tol = 1e-5 if nat.gemm_plan(m, n, k, split_k=False)[0] != "few_rows" or name == "tiles128_split_k" else 0.0
        err = ((with_ws - without).abs().max() / without.abs().max()).item()
        assert err <= max(tol, 1e-5), (m, n, k, name, parts, err)
        if name != "tiles128_split_k":
            assert torch.equal(with_ws, without), (m, n, k, name)
        assert torch.equal(nat.gemm_nt_kb(_to_kb(a), sa, _to_kb(bt), sb, torch.float32), with_ws), (m, n, k, name)
    assert split >= 3, split


# More than one round of 256 x 256 tiles with few tiles in the last one: the last tile rows go to a 128-row-tile kernel.
@pytest.mark.parametrize("m,n,k,m_pad", [(4352, 4096, 512, 8192),      # 272 tiles: 16 of them as 128 x 128 tiles
                                         (8500, 2048, 384, 16384),     # ragged last tile row
                                         (6144, 4096, 640, 8192),      # 384 tiles: 128 of them as 128 x 256 tiles
                                         (16640, 4000, 384, 20480)])   # four full rounds, then 16 tiles; ragged columns
def test_gemm_split_of_a_sparse_last_round_changes_no_bit(nat, m, n, k, m_pad):
    """Reference: the same rows inside a matrix padded with zero rows to whole rounds, which the large-tile kernel
    computes alone."""
    a = _rand_fp8((m, k), torch.float8_e4m3fn, m + k, 4.0).to(DEV)
    bt = _rand_fp8((n, k), torch.float8_e5m2, n + k, 4.0).to(DEV)
    sa, sb = torch.tensor(0.5, device=DEV), torch.tensor(4.0, device=DEV)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 3).to(torch.bfloat16).to(DEV)
    assert (m_pad // 256) * ((n + 255) // 256) % 256 == 0
    a_pad = torch.cat([a.view(torch.uint8), torch.zeros(m_pad - m, k, dtype=torch.uint8, device=DEV)]).view(a.dtype)
    for out_dt, b in ((torch.bfloat16, bias), (torch.float32, None)):
        want = nat.gemm_nt(a_pad, sa, bt, sb, out_dt, bias=b)[:m]
        assert torch.equal(nat.gemm_nt(a, sa, bt, sb, out_dt, bias=b), want)
        assert torch.equal(nat.gemm_nt_kb(_to_kb(a), sa, _to_kb(bt), sb, out_dt, bias=b), want)
    _gemm_check(nat, m, n, k, "e4m3", "e5m2", torch.bfloat16, seed=m + n, bias=True)


@pytest.mark.parametrize("m,n,k", [(300, 520, 1024), (1000, 264, 2048), (512, 1024, 384), (1100, 4500, 640),
                                   (200, 8192, 512),     # 129 - 256 rows and a wide Bt: the 128-row tiles, not the few-row kernel
                                   (100, 16384, 384)])   # so do 17 - 128 rows when Bt is wide enough
def test_gemm_mid_tile_kernel_equals_the_large_tile_kernel_bitwise(nat, m, n, k):
    """The same rows of A inside a matrix tall enough for the 256 x 256-tile kernel: identical bits (same accumulation
    order), row-major and k-blocked."""
    a = _rand_fp8((m, k), torch.float8_e5m2, m + k, 4.0).to(DEV)
    bt = _rand_fp8((n, k), torch.float8_e4m3fn, n + k, 4.0).to(DEV)
    sa, sb = torch.tensor(2.0, device=DEV), torch.tensor(0.25, device=DEV)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 3).to(torch.bfloat16).to(DEV)
    tall = 256 * (128 // ((n + 255) // 256) + 2)
    a_tall = torch.cat([a.view(torch.uint8), torch.zeros(tall - m, k, dtype=torch.uint8, device=DEV)]).view(a.dtype)
    for out_dt, b in ((torch.bfloat16, bias), (torch.float32, None)):
        want = nat.gemm_nt(a_tall, sa, bt, sb, out_dt, bias=b)[:m]
        assert torch.equal(nat.gemm_nt(a, sa, bt, sb, out_dt, bias=b), want)
        if k >= 384:
            assert torch.equal(nat.gemm_nt_kb(_to_kb(a), sa, _to_kb(bt), sb, out_dt, bias=b), want)


def test_gemm_random_sweep_over_all_dispatch_paths(nat):
    """Seeded random (m, n, k), formats, output types, bias, row strides and 16-byte misalignment: whichever kernel
    the library picks (few-row, 16x16x128 or 32x32x64 LDS-DMA, register-staged) the result is within the stated
    tolerance of the exact product, and equal bit for bit to the same call on a dense, aligned copy when both take
    the same kernel family."""
    rng = np.random.default_rng(2024)
    fmts = ["e4m3", "e5m2"]
    outs = [torch.bfloat16, torch.float32, torch.float16]
    one = None
    for case in range(48):
        kind = case % 6
        m = int(rng.choice([1, 3, 16, 40, 64, 100, 128, 129, 255, 256, 300, 513]))
        n = int(rng.choice([1, 8, 31, 64, 200, 256, 257, 520]))
        k = int(rng.choice([[16, 48, 100, 129, 250], [128, 256, 1152], [384, 640, 1024, 2048], [448, 576, 704],
                            [392, 1000, 4097], [128, 384, 512]][kind]))
        a_fmt, b_fmt = fmts[int(rng.integers(2))], fmts[int(rng.integers(2))]
        out_dt = outs[int(rng.integers(3))]
        _gemm_check(nat, m, n, k, a_fmt, b_fmt, out_dt, seed=1000 + case, bias=bool(rng.integers(2)))
        # the same product from operands with a padded row stride, and from operands shifted off 16-byte alignment
        ta, tb = F8[a_fmt][1], F8[b_fmt][1]
        a = _rand_fp8((m, k), ta, 2000 + case, 4.0).to(DEV)
        bt = _rand_fp8((n, k), tb, 3000 + case, 4.0).to(DEV)
        if one is None:
            one = torch.ones((), device=DEV)
        want = nat.gemm_nt(a, one, bt, one, torch.float32)
        pad = 16 * int(rng.integers(1, 5))
        a_p = torch.zeros(m, k + pad, dtype=torch.uint8, device=DEV).view(ta)
        b_p = torch.zeros(n, k + pad, dtype=torch.uint8, device=DEV).view(tb)
        a_p[:, :k].view(torch.uint8).copy_(a.view(torch.uint8))
        b_p[:, :k].view(torch.uint8).copy_(bt.view(torch.uint8))
        got = nat.gemm_nt(a_p[:, :k], one, b_p[:, :k], one, torch.float32)
        if k % 16 == 0:
            assert torch.equal(got, want), (case, m, n, k, "padded rows")  # same kernel: strides only
        else:
            torch.testing.assert_close(got, want, rtol=1e-3, atol=1e-2)
        a_o = torch.empty(m * k + 3, dtype=torch.uint8, device=DEV)[3:].view(ta).view(m, k)
        a_o.view(torch.uint8).copy_(a.view(torch.uint8))
        got = nat.gemm_nt(a_o, one, bt, one, torch.float32)   # unaligned: the register-staged kernel
        torch.testing.assert_close(got, want, rtol=1e-3, atol=1e-2 * max(1.0, k / 256))


def test_gemm_kernels_agree_bitwise(nat):
    """Same operands through the LDS-DMA kernel (aligned view) and the register-staged kernel (the same
    values at a 1-byte offset, which forces the unaligned path): identical accumulation order, identical bits."""
    m, n, k = 300, 520, 1024
    a = _rand_fp8((m, k), torch.float8_e4m3fn, 31, 4.0).to(DEV)
    bt = _rand_fp8((n, k), torch.float8_e4m3fn, 32, 4.0).to(DEV)
    s1 = torch.ones((), device=DEV)
    fast = nat.gemm_nt(a, s1, bt, s1, torch.float32)
    a_off = torch.empty(m * k + 1, dtype=torch.uint8, device=DEV)[1:].view(torch.float8_e4m3fn).view(m, k)
    b_off = torch.empty(n * k + 1, dtype=torch.uint8, device=DEV)[1:].view(torch.float8_e4m3fn).view(n, k)
    a_off.copy_(a)
    b_off.copy_(bt)
    assert a_off.data_ptr() % 16 != 0
    slow = nat.gemm_nt(a_off, s1, b_off, s1, torch.float32)
    assert torch.equal(fast, slow)


def _to_kb(t):
    """[rows, k] fp8 -> k-blocked [k/64, rows, 64] (byte permutation on the device)."""
    rows, k = t.shape
    return t.view(torch.uint8).view(rows, k // 64, 64).permute(1, 0, 2).contiguous().view(t.dtype)


@pytest.mark.parametrize("m,n,k", [(256, 256, 384), (300, 200, 448), (257, 511, 576), (1, 7, 640), (520, 264, 8192), (1024, 768, 2048)])
def test_gemm_kblocked_equals_row_major_bitwise(nat, m, n, k):
    a = _rand_fp8((m, k), torch.float8_e5m2, m + k, 4.0).to(DEV)
    bt = _rand_fp8((n, k), torch.float8_e4m3fn, n + k, 4.0).to(DEV)
    sa, sb = torch.tensor(3.0, device=DEV), torch.tensor(0.5, device=DEV)
    bias = (torch.randn(n) * 3).to(torch.bfloat16).to(DEV)
    for out_dt, b in ((torch.bfloat16, bias), (torch.float32, None), (torch.float16, None)):
        want = nat.gemm_nt(a, sa, bt, sb, out_dt, bias=b)
        got = nat.gemm_nt_kb(_to_kb(a), sa, _to_kb(bt), sb, out_dt, bias=b)
        assert torch.equal(got, want), (m, n, k, out_dt)


@pytest.mark.parametrize("m,n,k", [(256, 256, 384), (320, 192, 512), (64, 128, 640), (704, 448, 1024), (512, 256, 8192),
                                   (16384 // 8, 1024, 2048)])
def test_gemm_with_transposed_operands_equals_row_major_bitwise(nat, m, n, k):
    """f8mi_gemm_kb_ex: Bt, or A and Bt, given as the k-blocked copy of the transposed matrix (what the other
    GEMMs of a linear layer hold), read with LDS transpose loads: identical bits to the row-major GEMM."""
    a = _rand_fp8((m, k), torch.float8_e5m2, m + k + 5, 4.0).to(DEV)
    bt = _rand_fp8((n, k), torch.float8_e4m3fn, n + k + 6, 4.0).to(DEV)
    sa, sb = torch.tensor(3.0, device=DEV), torch.tensor(0.5, device=DEV)
    a_tr = _to_kb(a.view(torch.uint8).t().contiguous().view(a.dtype))    # [m/64, k, 64]
    bt_tr = _to_kb(bt.view(torch.uint8).t().contiguous().view(bt.dtype))  # [n/64, k, 64]
    bias = (torch.randn(n) * 3).to(torch.bfloat16).to(DEV)
    # the row-major product from the tile kernels (up to 256 rows f8mi_gemm_nt takes the few-row kernel, which sums in
    # another order: pad A with zero rows past that limit and cut the result)
    a_ref = a if m > 256 else torch.cat([a.view(torch.uint8), torch.zeros(320 - m, k, dtype=torch.uint8, device=DEV)]).view(a.dtype)
    for out_dt, b in ((torch.bfloat16, bias), (torch.float32, None)):
        want = nat.gemm_nt(a_ref, sa, bt, sb, out_dt, bias=b, split_k=False)[:m]  # transposed operands are never split over k
        got = nat.gemm_kb_ex(_to_kb(a), False, sa, bt_tr, True, sb, out_dt, bias=b)
        assert torch.equal(got, want), (m, n, k, out_dt, "bt transposed")
        got = nat.gemm_kb_ex(a_tr, True, sa, bt_tr, True, sb, out_dt, bias=b)
        assert torch.equal(got, want), (m, n, k, out_dt, "both transposed")
        got = nat.gemm_kb_ex(_to_kb(a), False, sa, _to_kb(bt), False, sb, out_dt, bias=b)
        if m > 256:
            assert torch.equal(got, want)
        else:
            torch.testing.assert_close(got.float(), want.float(), rtol=2.0**-7, atol=1e-2)
    with pytest.raises(nat.Float8NativeError):
        nat.gemm_kb_ex(a_tr, True, sa, _to_kb(bt), False, sb, torch.bfloat16)


def _to_kb_padded(t):
    """[rows, k] fp8 -> zero-padded k-blocked [padded_k/64, rows, 64] and the row-major padded matrix (device)."""
    rows, k = t.shape
    kp = -(-k // 128) * 128
    padded = torch.zeros(rows, kp, dtype=torch.uint8, device=t.device)
    padded[:, :k] = t.view(torch.uint8)
    return padded.view(rows, kp // 64, 64).permute(1, 0, 2).contiguous().view(t.dtype), padded.view(t.dtype)


@pytest.mark.parametrize("m,n,k", [(300, 200, 385), (257, 511, 1000), (129, 77, 4097), (4099, 1000, 3000), (1000, 3000, 4099),
                                   (64, 8190, 2047), (20, 515, 8191)])
def test_gemm_on_zero_padded_kblocked_operands(nat, m, n, k):
    """A ragged contraction on the LDS-DMA kernels: operands k-blocked with the contraction zero-padded to a multiple of
    128 (what the cast writes with F8MI_LAYOUT_KBLOCK64_PAD128) give the bits of the row-major product over the padded
    length, and the value of the unpadded product (register-staged kernel) within the accumulation tolerance.  n and
    the row pitch of C are odd in most cases: C leaves in 16-byte stores at 2-byte alignment."""
    a = _rand_fp8((m, k), torch.float8_e5m2, m + k, 4.0).to(DEV)
    bt = _rand_fp8((n, k), torch.float8_e4m3fn, n + k, 4.0).to(DEV)
    sa, sb = torch.tensor(3.0, device=DEV), torch.tensor(0.5, device=DEV)
    a_kb, a_pad = _to_kb_padded(a)
    b_kb, b_pad = _to_kb_padded(bt)
    bias = (torch.randn(n) * 3).to(torch.bfloat16).to(DEV)
    for out_dt, b in ((torch.bfloat16, bias), (torch.float32, None), (torch.float16, None)):
        got = nat.gemm_nt_kb(a_kb, sa, b_kb, sb, out_dt, bias=b, split_k=False)
        want = nat.gemm_nt(a_pad, sa, b_pad, sb, out_dt, bias=b, split_k=False)
        assert torch.equal(got, want), (m, n, k, out_dt)
        ragged = nat.gemm_nt(a, sa, bt, sb, out_dt, bias=b, split_k=False).double()
        bound = (a.float().abs() @ bt.float().abs().t()).double() / 1.5
        eps_out = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11, torch.float32: 2.0**-23}[out_dt]
        tol = 2 * eps_out * ragged.abs() + 2.0**-12 * bound + 1e-30
        assert ((got.double() - ragged).abs() <= tol).all(), (m, n, k, out_dt)
    _gemm_check(nat, m, n, k, "e5m2", "e4m3", torch.bfloat16, seed=m + n + k)


@pytest.mark.parametrize("m,n,k", [(16, 128, 48), (16, 128, 41), (2048, 4096, 2048), (4096, 2048, 384), (2112, 2176, 640),
                                   (2050, 4096, 1024), (4096, 2100, 1024), (16384, 8192, 8192)])
def test_scaled_mm_on_row_major_operands_equals_the_copy_route_bitwise(nat, m, n, k):
    """f8mi_gemm_ex / scaled_mm: a @ b with b row-major (the grad_input product) and with a column-major as well (the
    grad_weight product) gives the bits of gemm_nt on the copies preprocess_addmm would have made -- read transposed by
    the kernel where the product is large and aligned (checked through the return code), copied where it is not."""
    a = _rand_fp8((m, k), torch.float8_e5m2, m + k, 4.0).to(DEV)
    b = _rand_fp8((k, n), torch.float8_e4m3fn, n + k, 4.0).to(DEV)            # row-major [k, n]
    a_cm = a.view(torch.uint8).t().contiguous().view(a.dtype).t()               # the same matrix, column-major
    bt = b.view(torch.uint8).t().contiguous().view(b.dtype)                     # [n, k]: what gemm_nt takes
    sa, sb = torch.tensor(3.0, device=DEV), torch.tensor(0.5, device=DEV)
    bias = (torch.randn(n) * 3).to(torch.bfloat16).to(DEV)
    for out_dt, bi in ((torch.bfloat16, bias), (torch.float32, None)):
        want = nat.gemm_nt(a, sa, bt, sb, out_dt, bias=bi, split_k=False)
        assert torch.equal(nat.scaled_mm(a, sa, b, sb, out_dt, bias=bi), want), (m, n, k, out_dt, "b row-major")
        assert torch.equal(nat.scaled_mm(a_cm, sa, b, sb, out_dt, bias=bi), want), (m, n, k, out_dt, "a column-major, b row-major")
        assert torch.equal(nat.scaled_mm(a, sa, bt.t(), sb, out_dt, bias=bi), want)
        assert torch.equal(nat.scaled_mm(a_cm, sa, bt.t(), sb, out_dt, bias=bi), want)   # (1, 0): a is copied
    # which of them the kernel took without a copy
    L = nat.lib()
    out = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    fast_b = k % 128 == 0 and k >= 384 and n % 64 == 0 and -(-m // 128) * -(-n // 128) > 256
    rc = L.f8mi_gemm_ex(a.data_ptr(), 1, 0, k, b.data_ptr(), 0, 1, n, m, n, k, sa.data_ptr(), sb.data_ptr(), out.data_ptr(), 0, n, None, None)
    assert rc == (0 if fast_b else nat.ERR_UNSUPPORTED), (m, n, k, rc)
    rc = L.f8mi_gemm_ex(a_cm.data_ptr(), 1, 1, m, b.data_ptr(), 0, 1, n, m, n, k, sa.data_ptr(), sb.data_ptr(), out.data_ptr(), 0, n, None, None)
    assert rc == (0 if fast_b and m % 64 == 0 else nat.ERR_UNSUPPORTED), (m, n, k, rc)
    rc = L.f8mi_gemm_ex(a_cm.data_ptr(), 1, 1, m, bt.data_ptr(), 0, 0, k, m, n, k, sa.data_ptr(), sb.data_ptr(), out.data_ptr(), 0, n, None, None)
    assert rc == nat.ERR_UNSUPPORTED


def test_gemm_kblocked_refuses_short_or_ragged_k(nat):
    s1 = torch.ones((), device=DEV)
    for k in (64, 320):
        a = torch.zeros(k // 64, 8, 64, dtype=torch.float8_e4m3fn, device=DEV)
        with pytest.raises(nat.Float8NativeError):
            nat.gemm_nt_kb(a, s1, a, s1, torch.bfloat16)


@pytest.mark.parametrize("a_fmt,b_fmt", [("e4m3", "e4m3"), ("e5m2", "e4m3"), ("e4m3", "e5m2"), ("e5m2", "e5m2")])
@pytest.mark.parametrize("out_dt", [torch.bfloat16, torch.float16, torch.float32])
def test_gemm_formats_and_output_dtypes(nat, a_fmt, b_fmt, out_dt):
    _gemm_check(nat, 384, 320, 448, a_fmt, b_fmt, out_dt, seed=7, bias=(out_dt != torch.float16))


def test_gemm_closed_forms(nat):
    one4 = torch.tensor([1.0]).to(torch.float8_e4m3fn)
    # identity: A @ I = A exactly (every fp8 value is a bf16 value)
    a = _rand_fp8((300, 256), torch.float8_e4m3fn, 3, 50.0)
    eye = torch.eye(256).to(torch.float8_e4m3fn)
    s1 = torch.ones((), device=DEV)
    out = nat.gemm_nt(a.to(DEV), s1, eye.to(DEV), s1, torch.bfloat16)
    assert torch.equal(out.cpu().float(), a.float())
    # all ones: k / (sa * sb)
    a = torch.ones(70, 1000).to(torch.float8_e5m2)
    b = torch.ones(90, 1000).to(torch.float8_e4m3fn)
    out = nat.gemm_nt(a.to(DEV), torch.tensor(2.0, device=DEV), b.to(DEV), torch.tensor(4.0, device=DEV), torch.float32)
    assert bool((out == 125.0).all())
    # one-hot rows pick single columns (catches a transposed or permuted operand)
    a = torch.zeros(64, 512)
    idx = torch.arange(64) * 7 % 512
    a[torch.arange(64), idx] = 2.0
    bt = _rand_fp8((96, 512), torch.float8_e4m3fn, 9, 8.0)
    out = nat.gemm_nt(a.to(torch.float8_e4m3fn).to(DEV), s1, bt.to(DEV), s1, torch.float32).cpu()
    assert torch.equal(out, 2.0 * bt.float()[:, idx].t())
    # zero-padding the reduction changes nothing (reference test_base.py:477-552 pads to 16)
    a = _rand_fp8((50, 41), torch.float8_e4m3fn, 11)
    bt = _rand_fp8((128, 41), torch.float8_e4m3fn, 12)
    o1 = nat.gemm_nt(a.to(DEV), s1, bt.to(DEV), s1, torch.float32)
    ap = torch.nn.functional.pad(a.view(torch.uint8), (0, 7)).view(torch.float8_e4m3fn)
    bp = torch.nn.functional.pad(bt.view(torch.uint8), (0, 7)).view(torch.float8_e4m3fn)
    o2 = nat.gemm_nt(ap.to(DEV), s1, bp.to(DEV), s1, torch.float32)
    assert torch.equal(o1, o2)
    # k = 0: the empty sum
    o = nat.gemm_nt(torch.empty(5, 0, dtype=torch.float8_e4m3fn, device=DEV), s1,
                    torch.empty(6, 0, dtype=torch.float8_e4m3fn, device=DEV), s1, torch.bfloat16)
    assert o.shape == (5, 6) and bool((o == 0).all())


def test_gemm_strided_operands(nat):
    co, to = _oracles()
    a = _rand_fp8((200, 512), torch.float8_e4m3fn, 21)
    bt = _rand_fp8((300, 512), torch.float8_e4m3fn, 22)
    ad, bd = a.to(DEV), bt.to(DEV)
    s1 = torch.ones((), device=DEV)
    # row-strided views (ld > k), aligned and not
    for sl in (slice(0, 256), slice(16, 400), slice(3, 260)):
        out = nat.gemm_nt(ad[:, sl], s1, bd[:, sl], s1, torch.float32).cpu()
        want = a[:, sl].double() @ bt[:, sl].double().t()
        bound = a[:, sl].double().abs() @ bt[:, sl].double().abs().t()
        assert bool(((out.double() - want).abs() <= 2.0**-13 * bound).all())


@pytest.mark.parametrize("out_dt", [torch.bfloat16, torch.float16])
def test_gemm_epilogue_of_tiles_inside_c_equals_the_checked_one_bitwise(nat, out_dt):
    """A 256 x 256 tile that lies inside C is written without bounds checks, one on the edge of C with them.  Dropping
    the last 8 rows and columns of a product turns its last row and column of tiles from the first kind into the
    second; what both products share must not change by a bit."""
    m, n, k = 4096, 4096, 512
    assert nat.gemm_plan(m, n, k)[0] == "tiles256" and nat.gemm_plan(m - 8, n - 8, k)[0] == "tiles256"
    a = _rand_fp8((m, k), torch.float8_e5m2, 31).to(DEV)
    bt = _rand_fp8((n, k), torch.float8_e4m3fn, 32).to(DEV)
    sa, sb = torch.tensor(3.0, device=DEV), torch.tensor(0.37, device=DEV)
    bias = torch.linspace(-1, 1, n).to(out_dt).to(DEV)
    for b in (None, bias):
        whole = nat.gemm_nt(a, sa, bt, sb, out_dt, bias=b)
        part = nat.gemm_nt(a[:m - 8], sa, bt[:n - 8], sb, out_dt, bias=None if b is None else b[:n - 8].contiguous())
        assert torch.equal(whole[:m - 8, :n - 8], part)
        # and the tiles inside C against the exact product
        exact = (a[:512].cpu().double() @ bt[:512].cpu().double().t()) / (3.0 * 0.37) + (0 if b is None else b[:512].cpu().double())
        err = (whole[:512, :512].cpu().double() - exact).abs()
        assert bool((err <= {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}[out_dt] * exact.abs() + 2.0**-12 * (
            a[:512].cpu().double().abs() @ bt[:512].cpu().double().abs().t()) / (3.0 * 0.37)).all())


# ------------------------------------------------------------------ K4 sync


def test_sync_and_init_match_oracle(nat):
    co, to = _oracles()
    rng = np.random.default_rng(0)
    n, H = 999, 16
    amax = (np.abs(rng.standard_normal(n)) * 10.0 ** rng.integers(-14, 5, n)).astype(np.float32)
    hist = (np.abs(rng.standard_normal((n, H))) * 10.0 ** rng.integers(-14, 5, (n, 1))).astype(np.float32)
    hist[::7] = 0
    amax[:3] = [0.0, 448.0, np.nan]
    fmts = rng.integers(0, 2, n)
    for fp16 in (False, True):
        for wb in (False, True):
            a_d = torch.from_numpy(amax.copy()).to(DEV).reshape(n, 1)
            h_d = torch.from_numpy(hist.copy()).to(DEV)
            s_d = torch.zeros(n, 1, device=DEV)
            entries = [(a_d[i], h_d[i], s_d[i], (torch.float8_e4m3fn, torch.float8_e5m2)[fmts[i]]) for i in range(n)]
            nat.sync(nat.sync_table(entries, torch.device(DEV)), H, fp16, wb)
            got_s, got_h = s_d.cpu().numpy().reshape(-1), h_d.cpu().numpy()
            # the same through the entry point that takes the entries as kernel arguments (32 per launch: 999 = 31 * 32 + 7)
            h2_d = torch.from_numpy(hist.copy()).to(DEV)
            s2_d = torch.zeros(n, 1, device=DEV)
            nat.sync_host([(a_d[i], h2_d[i], s2_d[i], e[3]) for i, e in enumerate(entries)], H, fp16, wb)
            assert torch.equal(s2_d.view(torch.int32), s_d.view(torch.int32)) and torch.equal(h2_d.view(torch.int32), h_d.view(torch.int32))
            for i in range(n):
                h = hist[i].copy()
                want = co.sync_entry(amax[i], h, int(fmts[i]), fp16, wb)
                assert np.float32(got_s[i]).view(np.uint32) == np.float32(want).view(np.uint32) or (np.isnan(want) and np.isnan(got_s[i])), i
                assert np.array_equal(got_h[i], h, equal_nan=True), (i, wb)
    # init
    for i in range(0, 60):
        h = hist[i].copy()
        a_d = torch.tensor([amax[i]], device=DEV)
        h_d = torch.from_numpy(h.copy()).to(DEV)
        s_d = torch.zeros(1, device=DEV)
        nat.delayed_init(a_d, h_d, s_d, (torch.float8_e4m3fn, torch.float8_e5m2)[fmts[i]], False)
        want = co.delayed_init(amax[i], h, int(fmts[i]), False)
        assert np.array_equal(h_d.cpu().numpy(), h, equal_nan=True)
        assert np.float32(s_d.item()).view(np.uint32) == np.float32(want).view(np.uint32) or np.isnan(want)


# ------------------------------------------- full-size properties (config 2)


def test_full_size_properties_llama70b_wo(nat):
    """M=16384, K=N=8192: size-independent properties where the oracle is too slow."""
    torch.manual_seed(0)
    M, K, N = 16384, 8192, 8192
    x = torch.randn(M, K, device=DEV, dtype=torch.bfloat16)
    w = (torch.rand(N, K, device=DEV, dtype=torch.float32) * 2 - 1).mul_(K**-0.5).to(torch.bfloat16)
    ax, sx = nat.amax_scale(x, torch.float8_e4m3fn)
    aw, sw = nat.amax_scale(w, torch.float8_e4m3fn)
    assert ax.item() == x.abs().max().float().item() and aw.item() == w.abs().max().float().item()
    x8, x8t = nat.cast(x, sx, torch.float8_e4m3fn, want_out_t=True)
    w8, w8t = nat.cast(w, sw, torch.float8_e4m3fn, want_out_t=True)
    assert torch.equal(x8t.view(torch.uint8), x8.view(torch.uint8).t().contiguous())
    assert torch.equal(w8t.view(torch.uint8), w8.view(torch.uint8).t().contiguous())
    # the cast is the same function of (x, scale) everywhere: torch's own ops on the GPU agree byte for byte
    ref = (x * sx).clamp(-448, 448).to(torch.float8_e4m3fn)
    assert torch.equal(ref.view(torch.uint8), x8.view(torch.uint8))
    # idempotence: re-casting the dequantised tensor at scale 1 gives the same bytes
    one = torch.ones((), device=DEV)
    again, _ = nat.cast(x8.to(torch.bfloat16), one, torch.float8_e4m3fn)
    assert torch.equal(again.view(torch.uint8), x8.view(torch.uint8))
    # GEMM: checksum of checksums in fp64, and exact linearity in power-of-two scales
    y = nat.gemm_nt(x8, sx, w8, sw, torch.float32)
    col = (x8.double().sum(0) / sx.double()) @ (w8.double().t() / sw.double())
    torch.testing.assert_close(y.double().sum(0), col, rtol=1e-4, atol=1e-4 * col.abs().max().item())
    row = (x8.double() / sx.double()) @ (w8.double().sum(0) / sw.double())
    torch.testing.assert_close(y.double().sum(1), row, rtol=1e-4, atol=1e-4 * row.abs().max().item())
    y2 = nat.gemm_nt(x8, sx * 2, w8, sw * 4, torch.float32)
    assert torch.equal(y2 * 8, y)
    # a 64 x 64 corner against the emulated product computed in fp64
    sub = (x8[:64].double() / sx.double()) @ (w8[:64].double().t() / sw.double())
    torch.testing.assert_close(y[:64, :64].double(), sub, rtol=1e-4, atol=1e-4)
    # grad_weight-shaped product from the transposed copies: (x^T x)[i][j], symmetric by construction
    g = nat.gemm_nt(x8t[:512], sx, x8t[:768], sx, torch.float32)
    torch.testing.assert_close(g[:, :512], g[:, :512].t(), rtol=1e-5, atol=1e-3)


def test_tensors_of_more_than_2_31_elements(nat):
    """Index arithmetic past 32 bits: amax, cast (all layouts) and the GEMM's output addressing on a tensor of
    2.29e9 elements, checked on slices against torch's own ops on the GPU (the cast is the same function of
    (x, scale) everywhere, so slices pin it) and on planted maxima."""
    rows, cols = 70000, 32768
    assert rows * cols > 2**31
    g = torch.Generator(device=DEV).manual_seed(11)
    x = torch.empty(rows, cols, device=DEV, dtype=torch.bfloat16).normal_(generator=g)
    x[rows - 1, cols - 3] = 1000.0   # the maximum sits past element 2^31
    amax, scale = nat.amax_scale(x, torch.float8_e4m3fn)
    assert amax.item() == 1000.0
    x[rows - 1, cols - 3] = 0.5
    x[17, 5] = -2000.0
    amax, scale = nat.amax_scale(x, torch.float8_e4m3fn)
    assert amax.item() == 2000.0
    ams, _ = nat.amax_scale_multi([x[:3], x], torch.float8_e4m3fn)
    assert ams[1].item() == 2000.0
    ref_rows = [0, 1, 127, 128, 32767, 65535, 65536, rows - 129, rows - 2, rows - 1]
    want = (x[ref_rows] * scale).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    out, out_t = nat.cast(x, scale, torch.float8_e4m3fn, want_out_t=True)
    assert torch.equal(out[ref_rows].view(torch.uint8), want)
    assert torch.equal(out_t[:, ref_rows].view(torch.uint8), want.t())
    del out_t
    okb, _ = nat.cast(x, scale, torch.float8_e4m3fn, out_kblock=True)  # [cols/64, rows, 64]
    assert torch.equal(okb[:, ref_rows, :].view(torch.uint8).permute(1, 0, 2).reshape(len(ref_rows), cols), want)
    del okb
    # GEMM with more than 2^31 outputs: C = out[:, :384] (70000 x 384) times a 32768 x 384 matrix
    a8 = out[:, :384].contiguous()
    b8 = _rand_fp8((cols, 384), torch.float8_e4m3fn, 3, 2.0).to(DEV)
    one = torch.ones((), device=DEV)
    c = nat.gemm_nt(a8, one, b8, one, torch.bfloat16)
    assert c.numel() > 2**31
    for r0 in (0, 65536 - 128, rows - 256):
        ref = nat.gemm_nt(a8[r0:r0 + 256].contiguous(), one, b8, one, torch.bfloat16)
        assert torch.equal(c[r0:r0 + 256], ref), r0
    exact = a8[rows - 64:].double() @ b8.double().t()
    torch.testing.assert_close(c[rows - 64:].double(), exact, rtol=2.0**-7, atol=0.5)
