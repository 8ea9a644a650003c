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


STRICT_FLOOR = 2.0 ** -8  # "bf16 ulp at the row's rms": the floor the scalar-order kernels meet and the MFMA does not


def reference_style_excess(c: np.ndarray, ref: np.ndarray, atol: float = 1e-2, rtol: float = 1e-2, unit_rms: bool = False) -> float:
    """max (|c - ref| - rtol * |ref|) / atol: at most 1 when |c - ref| <= atol + rtol * |ref| everywhere, the bar of
    the reference's own test of its MFMA path (test_scaled_matmul.mojo:140-154 with atol = rtol = 1.5e-2; 1e-2
    here).  unit_rms: both arrays are first divided by the rms of their row of ref, for test data whose
    magnitude is arbitrary (the absolute term is meant for results of the order of one)."""
    c = np.asarray(c, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    if c.size == 0:
        return 0.0
    if unit_rms:
        rms = np.maximum(np.sqrt(np.mean(ref * ref, axis=-1, keepdims=True)), 1e-30)
        c, ref = c / rms, ref / rms
    return float(np.max((np.abs(c - ref) - rtol * np.abs(ref)) / atol))


def assert_rel(c, ref, tol=1e-2, what="", abs_budget=None, natural_scale=False):
    """The parity bar of the MFMA matmuls: max rel err <= tol (1e-2, bf16 or f32 out); the reference's own
    criterion |c - ref| <= 1e-2 + 1e-2 * |ref| on rows normalised to unit rms (natural_scale=True: on the values
    as they are -- for benchmark-shaped data, whose results are of the order of one); and where the caller
    passes abs_budget (f32 outputs: F32_BUDGET), no element further than abs_budget * rms(row) from the
    reference (bf16 rounding alone is 2^-9 of the element, so the budget is not applied to bf16 outputs).
    Returns the figures, among them the error under the strict floor 2^-8 * rms, which is reported, not asserted."""
    cf = np.asarray(c, dtype=np.float64)
    assert np.all(np.isfinite(cf)), f"{what}: non-finite output"
    e = rel_err(cf, ref)
    assert e <= tol, f"{what}: max rel err {e:.3e} > {tol}"
    # (on unit-rms rows this follows from the bound above; on natural-scale data it is a condition of its own)
    x = reference_style_excess(cf, ref, atol=tol, rtol=tol, unit_rms=not natural_scale)
    assert x <= 1.0, f"{what}: |c - ref| exceeds {tol} + {tol} |ref| by a factor {x:.3f} of the absolute term"
    figures = {"rel_err": e, "rel_err_strict_floor": rel_err(cf, ref, STRICT_FLOOR), "reference_style_excess": x,
               "err_over_rms": err_over_rms(cf, ref)}
    if abs_budget is not None:
        assert figures["err_over_rms"] <= abs_budget, f"{what}: max |err| / rms(row) = {figures['err_over_rms']:.3e} > {abs_budget}"
    return figures
