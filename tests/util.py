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


# Elements smaller than FLOOR * (rms of their row) are judged against FLOOR * rms
# instead of their own magnitude.  Why not a smaller floor: the matrix instruction the
# kernels are built on (v_mfma_f32_16x16x128_f8f6f4) aligns the 128 products of a dot
# product to the largest one and truncates what falls more than ~13 bits below it
# (tests/test_gpu_matmul.py::test_mfma_keeps_13_bits_below_the_largest_product), so a
# result carries an absolute error of a few 1e-4 of the row's rms whatever its own size.
# Measured against float64 on BASELINE's data: rms error 1.4e-5..3.2e-5 of the row rms,
# worst element 4.5e-4, no bias, no growth with K.
FLOOR = 2.0 ** -4
F32_BUDGET = 2e-3  # max |err| / rms(row) allowed for f32 outputs (measured: <= 4.5e-4)


def rel_err(c: np.ndarray, ref: np.ndarray, floor: float = FLOOR) -> float:
    """max |c - ref| / max(|ref|, floor * rms(row of ref))."""
    c = np.asarray(c, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if c.size == 0:
        return 0.0
    rms = np.sqrt(np.mean(ref * ref, axis=-1, keepdims=True))
    eps = np.maximum(rms * floor, 1e-30)
    return float(np.max(np.abs(c - ref) / np.maximum(np.abs(ref), eps)))


def err_over_rms(c: np.ndarray, ref: np.ndarray) -> float:
    """max |c - ref| / rms(row of ref): the absolute error in units of the row's scale."""
    c = np.asarray(c, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if c.size == 0:
        return 0.0
    rms = np.maximum(np.sqrt(np.mean(ref * ref, axis=-1, keepdims=True)), 1e-30)
    return float(np.max(np.abs(c - ref) / rms))


def assert_rel(c, ref, tol=1e-2, what="", abs_budget=None):
    """The parity bar of the MFMA matmuls: max rel err <= tol (1e-2, bf16 or f32 out), and
    where the caller passes abs_budget (f32 outputs: F32_BUDGET), no element further than
    abs_budget * rms(row) from the reference (bf16 rounding alone is 2^-9 of the element, so
    the budget is not applied to bf16 outputs)."""
    cf = np.asarray(c, dtype=np.float64)
    assert np.all(np.isfinite(cf)), f"{what}: non-finite output"
    e = rel_err(cf, ref)
    assert e <= tol, f"{what}: max rel err {e:.3e} > {tol}"
    if abs_budget is not None:
        a = err_over_rms(cf, ref)
        assert a <= abs_budget, f"{what}: max |err| / rms(row) = {a:.3e} > {abs_budget}"
