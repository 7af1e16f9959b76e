"""Writes the golden fixtures of this directory.

Run once, in the build container only, where the upstream float8_experimental
sources are mounted at /root/reference.  It imports the upstream package on CPU
(emulate=True) and records, for a handful of tiny seeded scenarios, what the
upstream code computes: scales, amax / history buffers over several
sync+forward+backward steps, fp8 payload bytes, outputs and gradients.  The
fixtures are plain ``.npz`` files (numbers only); bf16 tensors are stored as
their int16 bit patterns, fp8 payloads as uint8.

    python tests/golden/make_golden.py

Nothing in the test-suite imports this script or the upstream package: tests
only read the ``.npz`` files.
"""
import hashlib
import os
import sys

import numpy as np
import torch
import torch.nn as nn

REF = os.environ.get("F8_REFERENCE", "/root/reference")
sys.path.insert(0, REF)

from float8_experimental.config import (  # noqa: E402
    CastConfig,
    DelayedScalingConfig,
    Float8LinearConfig,
    ScalingType,
)
from float8_experimental.float8_linear_utils import (  # noqa: E402
    convert_to_float8_training,
    linear_requires_sync,
    sync_float8_amax_and_scale_history,
)
from float8_experimental.float8_tensor import (  # noqa: E402
    hp_tensor_and_scale_to_float8,
)
from float8_experimental.float8_utils import (  # noqa: E402
    amax_history_to_scale_stack,
    e4m3_dtype,
    e5m2_dtype,
    tensor_to_scale,
)

HERE = os.path.dirname(os.path.abspath(__file__))
KINDS = ("input", "weight", "grad_output")


def bits(t: torch.Tensor) -> np.ndarray:
    """Lossless numpy image of a tensor (bf16 -> int16 bits, fp8 -> uint8)."""
    t = t.detach().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().copy()
    if t.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        return t.view(torch.uint8).numpy().copy()
    return t.numpy().copy()


def cfg(i, w, g, hist=16):
    m = {"dyn": ScalingType.DYNAMIC, "del": ScalingType.DELAYED}
    return Float8LinearConfig(
        cast_config_input=CastConfig(scaling_type=m[i]),
        cast_config_weight=CastConfig(scaling_type=m[w]),
        cast_config_grad_output=CastConfig(scaling_type=m[g]),
        delayed_scaling_config=DelayedScalingConfig(history_len=hist),
        emulate=True,
    )


def buffers(model, out, tag):
    for li, mod in enumerate(m for m in model.modules() if hasattr(m, "fp8_amax_input")):
        for k in KINDS:
            out[f"{tag}.L{li}.amax_{k}"] = bits(getattr(mod, f"fp8_amax_{k}"))
            out[f"{tag}.L{li}.hist_{k}"] = bits(getattr(mod, f"fp8_amax_history_{k}"))
            out[f"{tag}.L{li}.scale_{k}"] = bits(getattr(mod, f"fp8_scale_{k}"))


def trajectory(name, i, w, g, hist, steps, dtype, xgrow, ggrow, x_shape=(8, 16)):
    """Multi-step sync -> forward -> backward run of a 2-layer model."""
    torch.manual_seed(1234)
    model = nn.Sequential(nn.Linear(16, 32, bias=True), nn.Linear(32, 16, bias=False)).to(dtype)
    out = {"w0": bits(model[0].weight), "b0": bits(model[0].bias), "w1": bits(model[1].weight)}
    config = cfg(i, w, g, hist)
    model = convert_to_float8_training(model, config=config)
    x0 = torch.randn(*x_shape, dtype=dtype)
    g0 = torch.randn(*x_shape[:-1], 16, dtype=dtype) * 0.01
    out["x0"], out["g0"] = bits(x0), bits(g0)
    out["xgrow"], out["ggrow"] = np.float32(xgrow), np.float32(ggrow)
    for t in range(steps):
        x = (x0.float() * (xgrow**t)).to(dtype).requires_grad_()
        gy = (g0.float() * (ggrow**t)).to(dtype)
        for p in model.parameters():
            p.grad = None
        if linear_requires_sync(config):
            sync_float8_amax_and_scale_history(model)
            buffers(model, out, f"t{t}.synced")
        y = model(x)
        y.backward(gy)
        out[f"t{t}.x"], out[f"t{t}.gy"] = bits(x), bits(gy)
        out[f"t{t}.y"] = bits(y)
        out[f"t{t}.dx"] = bits(x.grad)
        out[f"t{t}.dw0"] = bits(model[0].weight.grad)
        out[f"t{t}.db0"] = bits(model[0].bias.grad)
        out[f"t{t}.dw1"] = bits(model[1].weight.grad)
        if linear_requires_sync(config):
            buffers(model, out, f"t{t}.after")
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)
    print("wrote", name, len(out), "arrays")


def heavy(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    t = torch.distributions.StudentT(3.0).sample(shape)  # global RNG
    mask = torch.rand(shape, generator=g) < 0.01
    t = torch.where(mask, t * 1000, t)
    return t.to(dtype)


def casts():
    """tensor_to_scale + cast of assorted tensors, dynamic- and delayed-style."""
    torch.manual_seed(99)
    out = {}
    cases = {}
    for dn, dt in (("bf16", torch.bfloat16), ("fp16", torch.float16), ("fp32", torch.float32)):
        cases[f"{dn}.randn"] = torch.randn(33, 47).to(dt)
        cases[f"{dn}.heavy"] = heavy((29, 40), dt, 5)
        cases[f"{dn}.tiny"] = (torch.randn(17, 9) * 1e-6).to(dt)
        cases[f"{dn}.zeros"] = torch.zeros(4, 8, dtype=dt)
        cases[f"{dn}.ones"] = torch.ones(4, 8, dtype=dt)
        sp = torch.tensor(
            [0.0, -0.0, 1.0, -1.0, 0.5, 3.0, 17.0, 19.0, 448.0, -448.0, 1e-3, 2.0**-9, 2.0**-10, 6e-5, 240.0, 0.0625]
        )
        cases[f"{dn}.special"] = sp.reshape(2, 8).to(dt)
    for cn, x in cases.items():
        out[f"{cn}.x"] = bits(x)
        for fn, fdt in (("e4m3", e4m3_dtype), ("e5m2", e5m2_dtype)):
            s = tensor_to_scale(x, fdt)  # 0-dim fp32
            out[f"{cn}.{fn}.scale"] = bits(s)
            out[f"{cn}.{fn}.dyn"] = bits(hp_tensor_and_scale_to_float8(x, s, fdt)._data)
            # delayed-style: the module's scale buffer has shape [1]; use a scale that
            # saturates part of the tensor (1.7x too large) to pin the clamp as well
            s1 = (s * 1.7).reshape(1)
            out[f"{cn}.{fn}.scale1"] = bits(s1)
            out[f"{cn}.{fn}.del"] = bits(hp_tensor_and_scale_to_float8(x, s1, fdt)._data)
    # stacked history -> scale (sync's arithmetic), incl. fp16 clamp
    hist = torch.tensor(
        [[0.0, 0.0, 0.0, 0.0], [1.0, 0.5, 0.0, 3.0], [1e-13, 0.0, 0.0, 0.0], [3e-3, 7e-3, 1e-5, 0.0], [500.0, 1e4, 3.3, 0.1]]
    )
    out["hist"] = bits(hist)
    for fn, fdt in (("e4m3", e4m3_dtype), ("e5m2", e5m2_dtype)):
        for dn, dt in (("bf16", torch.bfloat16), ("fp16", torch.float16), ("fp32", torch.float32)):
            out[f"hist.{fn}.{dn}"] = bits(amax_history_to_scale_stack(hist, fdt, dt, "max"))
    np.savez_compressed(os.path.join(HERE, "casts.npz"), **out)
    print("wrote casts", len(out), "arrays")


def sha(t):
    return np.frombuffer(hashlib.sha256(bits(t).tobytes()).digest(), dtype=np.uint8).copy()


def cfg1():
    """Benchmark configuration 1: one dynamic fwd+bwd of Linear(4096,4096) on x[2048,4096], seed 0."""
    torch.manual_seed(0)
    lin = nn.Linear(4096, 4096, bias=False).to(torch.bfloat16)
    x = torch.randn(2048, 4096).to(torch.bfloat16).requires_grad_()
    out = {"x_sha": sha(x), "w_sha": sha(lin.weight)}
    w = lin.weight.detach().clone()
    sx = tensor_to_scale(x.detach(), e4m3_dtype)
    sw = tensor_to_scale(w, e4m3_dtype)
    out["sx"], out["sw"] = bits(sx), bits(sw)
    out["x_fp8_sha"] = sha(hp_tensor_and_scale_to_float8(x.detach(), sx, e4m3_dtype)._data)
    out["w_fp8_sha"] = sha(hp_tensor_and_scale_to_float8(w, sw, e4m3_dtype)._data)
    m = convert_to_float8_training(nn.Sequential(lin), config=cfg("dyn", "dyn", "dyn"))
    y = m(x)
    y.sum().backward()
    dy = torch.ones_like(y)
    sg = tensor_to_scale(dy, e5m2_dtype)
    out["sg"] = bits(sg)
    out["dy_fp8_sha"] = sha(hp_tensor_and_scale_to_float8(dy, sg, e5m2_dtype)._data)
    out["dy_fp8_first"] = bits(hp_tensor_and_scale_to_float8(dy, sg, e5m2_dtype)._data[0, :8])
    # GEMM results depend on the CPU BLAS summation order: keep small slices + norms
    out["y_slice"] = bits(y[:16, :32])
    out["dx_slice"] = bits(x.grad[:16, :32])
    out["dw_slice"] = bits(lin.weight.grad[:16, :32])
    out["y_norm"] = np.float64(y.double().norm().item())
    out["dx_norm"] = np.float64(x.grad.double().norm().item())
    out["dw_norm"] = np.float64(lin.weight.grad.double().norm().item())
    np.savez_compressed(os.path.join(HERE, "cfg1.npz"), **out)
    print("wrote cfg1")


if __name__ == "__main__":
    torch.set_num_threads(8)
    casts()
    trajectory("traj_del_bf16", "del", "del", "del", 4, 7, torch.bfloat16, 1.7, 1.3)
    trajectory("traj_del_fp32", "del", "del", "del", 16, 5, torch.float32, 1.1, 0.8, x_shape=(2, 3, 16))
    trajectory("traj_mix1_bf16", "dyn", "del", "dyn", 16, 4, torch.bfloat16, 1.5, 1.5)
    trajectory("traj_mix2_bf16", "del", "dyn", "del", 2, 5, torch.bfloat16, 0.6, 2.0)
    trajectory("traj_dyn_bf16", "dyn", "dyn", "dyn", 16, 2, torch.bfloat16, 3.0, 3.0, x_shape=(3, 2, 16))
    trajectory("traj_del_h1_bf16", "del", "del", "del", 1, 4, torch.bfloat16, 1.7, 1.3)
    cfg1()
