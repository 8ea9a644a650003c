"""Shared helpers of the test-suite: torch <-> numpy views of bf16 / e4m3fn data
and the error metrics the parity tests use."""
from __future__ import annotations

import numpy as np
import torch

FP8 = torch.float8_e4m3fn


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    """torch bf16 tensor -> numpy uint16 bit patterns (CPU)."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_from_bits(u: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(u).view(np.int16)).view(torch.bfloat16)


def fp8_bytes(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def fp8_from_bytes(u: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(u, dtype=np.uint8)).view(FP8)


def f32_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().to(torch.float32).numpy()


def u32_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int32).numpy().view(np.uint32)


def rel_err(c: np.ndarray, ref: np.ndarray) -> float:
    """max |c - ref| / max(|ref|, eps) with eps = one bf16 ulp at the row's RMS
    magnitude (2^-8 * rms): elements far below the row's scale are judged on an
    absolute footing instead of being divided by ~0."""
    c = np.asarray(c, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if c.size == 0:
        return 0.0
    rms = np.sqrt(np.mean(ref * ref, axis=-1, keepdims=True))
    eps = np.maximum(rms * 2.0 ** -8, 1e-30)
    return float(np.max(np.abs(c - ref) / np.maximum(np.abs(ref), eps)))


def assert_rel(c, ref, tol=1e-2, what=""):
    assert np.all(np.isfinite(np.asarray(c, dtype=np.float64))), f"{what}: non-finite output"
    e = rel_err(c, ref)
    assert e <= tol, f"{what}: max rel err {e:.3e} > {tol}"
