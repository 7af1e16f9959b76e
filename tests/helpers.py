"""Shared helpers of the test-suite (numpy <-> torch bit views, fixture loading)."""
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

TORCH_DT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}
CODE_DT = {"bf16": 0, "fp16": 1, "fp32": 2}
F8 = {"e4m3": (0, torch.float8_e4m3fn), "e5m2": (1, torch.float8_e5m2)}


def load(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"))


def from_bits(a: np.ndarray, dt: str) -> torch.Tensor:
    """Fixture array -> torch tensor (bf16 is stored as int16 bits)."""
    if dt == "bf16":
        return torch.from_numpy(np.ascontiguousarray(a).view(np.int16).copy()).view(torch.bfloat16)
    return torch.from_numpy(np.ascontiguousarray(a).copy())


def to_u16(t: torch.Tensor) -> np.ndarray:
    """bf16/fp16 tensor -> uint16 bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def np_for_c(t: torch.Tensor) -> np.ndarray:
    if t.dtype in (torch.bfloat16, torch.float16):
        return to_u16(t)
    return t.detach().cpu().contiguous().numpy().copy()


def fp8_bytes(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.uint8).numpy().copy()


def same_bytes_mod_nan_sign(a: np.ndarray, b: np.ndarray) -> bool:
    """fp8 payload equality; NaN codes (0x7F / 0xFF) may differ in the sign bit only."""
    a = np.asarray(a, np.uint8)
    b = np.asarray(b, np.uint8)
    if a.shape != b.shape:
        return False
    diff = a != b
    if not diff.any():
        return True
    return bool((((a[diff] & 0x7F) == 0x7F) & ((b[diff] & 0x7F) == 0x7F)).all())
