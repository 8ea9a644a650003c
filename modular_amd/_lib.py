"""ctypes binding of libmaxfp8.so (the C ABI declared in include/maxfp8.h).

The library is the only compute path of this package: if it is missing the
import of any operator fails loudly -- there is no CPU or PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmaxfp8.so")

# maxfp8_dtype
BF16, F16, F32, E4M3FN = 0, 1, 2, 3
# maxfp8_granularity
GRAN_TENSOR, GRAN_ROWWISE, GRAN_COLWISE, GRAN_BLOCK = 0, 1, 2, 3
# maxfp8_algo
ALGO_AUTO, ALGO_NAIVE, ALGO_TILED, ALGO_SKINNY = 0, 1, 2, 3
# maxfp8_status
OK, ERR_DTYPE, ERR_SHAPE, ERR_ALIGN, ERR_GRANULARITY, ERR_LAUNCH, ERR_NULL, ERR_WORKSPACE = 0, -1, -2, -3, -4, -5, -6, -7

EXPORTS = (
    "maxfp8_last_error",
    "maxfp8_version",
    "maxfp8_tuning_reload",
    "maxfp8_quantize_dynamic_scaled_fp8",
    "maxfp8_batched_quantize_dynamic_scaled_fp8",
    "maxfp8_quantize_dynamic_scaled_fp8_gather",
    "maxfp8_quantize_dynamic_scaled_fp8_scatter",
    "maxfp8_grouped_matmul_dynamic_scaled_fp8_scatter",
    "maxfp8_rms_norm_fused_quantize_dynamic_scaled_fp8",
    "maxfp8_matmul_dynamic_scaled_fp8",
    "maxfp8_matmul_dynamic_scaled_fp8_noalloc",
    "maxfp8_matmul_noalloc_max_scratch_bytes",
    "maxfp8_batched_matmul_dynamic_scaled_fp8",
    "maxfp8_matmul_workspace_bytes",
    "maxfp8_matmul_describe",
    "maxfp8_grouped_matmul_dynamic_scaled_fp8",
    "maxfp8_grouped_matmul_rowwise_dynamic_scaled_fp8",
    "maxfp8_fused_qkv_matmul_ragged_paged_scale",
    "maxfp8_quantize_static_scaled_fp8",
    "maxfp8_quantize_tensor_dynamic_scaled_fp8",
    "maxfp8_moe_create_indices",
    "maxfp8_fused_silu",
    "maxfp8_cast_f32_to_e4m3fn",
    "maxfp8_cast_e4m3fn_to_f32",
    "maxfp8_cast_f32_to_bf16",
    "maxfp8_copy_bytes",
    "maxfp8_decode_weight_read_probe",
    "maxfp8_mfma_issue_probe",
    "maxfp8_handovers_given_up",
)

_lib = None


class LibraryMissing(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """Loads the HIP library; raises LibraryMissing when it was not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LibraryMissing(
            f"{LIB_PATH} not found: build the gfx950 kernels with `python -m modular_amd.build` "
            "(there is no fallback path)")
    L = ctypes.CDLL(LIB_PATH)
    i64, vp, ci, cf = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    L.maxfp8_last_error.restype = ctypes.c_char_p
    L.maxfp8_last_error.argtypes = []
    L.maxfp8_version.restype = ctypes.c_char_p
    L.maxfp8_version.argtypes = []
    L.maxfp8_tuning_reload.restype = None
    L.maxfp8_tuning_reload.argtypes = []
    L.maxfp8_quantize_dynamic_scaled_fp8.restype = ci
    L.maxfp8_quantize_dynamic_scaled_fp8.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci, cf, vp]
    L.maxfp8_quantize_dynamic_scaled_fp8_gather.restype = ci
    L.maxfp8_quantize_dynamic_scaled_fp8_gather.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, ci, ci, cf, vp]
    L.maxfp8_quantize_dynamic_scaled_fp8_scatter.restype = ci
    L.maxfp8_quantize_dynamic_scaled_fp8_scatter.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64, ci, ci, cf, vp]
    L.maxfp8_grouped_matmul_dynamic_scaled_fp8_scatter.restype = ci
    L.maxfp8_grouped_matmul_dynamic_scaled_fp8_scatter.argtypes = [vp] * 8 + [i64] * 7 + [ci, ci, ci, vp]
    L.maxfp8_batched_quantize_dynamic_scaled_fp8.restype = ci
    L.maxfp8_batched_quantize_dynamic_scaled_fp8.argtypes = [vp, vp, vp] + [i64] * 10 + [ci, ci, cf, vp]
    L.maxfp8_rms_norm_fused_quantize_dynamic_scaled_fp8.restype = ci
    L.maxfp8_rms_norm_fused_quantize_dynamic_scaled_fp8.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, ci, ci, cf, cf, cf, vp]
    L.maxfp8_matmul_dynamic_scaled_fp8.restype = ci
    L.maxfp8_matmul_dynamic_scaled_fp8.argtypes = ([vp] * 5 + [i64] * 6 + [ci, ci] + [i64] * 5 +
                                                  [ci, ci, ci, vp, ctypes.c_size_t, vp])
    L.maxfp8_matmul_dynamic_scaled_fp8_noalloc.restype = ci
    L.maxfp8_matmul_dynamic_scaled_fp8_noalloc.argtypes = ([vp] * 5 + [i64] * 6 + [ci, ci] + [i64] * 5 + [ci, ci, ci, vp])
    L.maxfp8_matmul_noalloc_max_scratch_bytes.restype = ctypes.c_size_t
    L.maxfp8_matmul_noalloc_max_scratch_bytes.argtypes = []
    L.maxfp8_batched_matmul_dynamic_scaled_fp8.restype = ci
    L.maxfp8_batched_matmul_dynamic_scaled_fp8.argtypes = [vp] * 5 + [i64] * 17 + [ci, ci, ci, vp]
    L.maxfp8_matmul_describe.restype = ci
    L.maxfp8_matmul_describe.argtypes = [i64, i64, i64, ci, ci, ctypes.c_char_p, ctypes.c_size_t]
    L.maxfp8_matmul_workspace_bytes.restype = ctypes.c_size_t
    L.maxfp8_matmul_workspace_bytes.argtypes = [i64, i64, i64]
    L.maxfp8_grouped_matmul_dynamic_scaled_fp8.restype = ci
    L.maxfp8_grouped_matmul_dynamic_scaled_fp8.argtypes = [vp] * 7 + [i64] * 7 + [ci, ci, ci, vp]
    L.maxfp8_grouped_matmul_rowwise_dynamic_scaled_fp8.restype = ci
    L.maxfp8_grouped_matmul_rowwise_dynamic_scaled_fp8.argtypes = [vp] * 7 + [i64] * 6 + [ci, ci, vp]
    L.maxfp8_fused_qkv_matmul_ragged_paged_scale.restype = ci
    L.maxfp8_fused_qkv_matmul_ragged_paged_scale.argtypes = [vp] * 10 + [i64] * 18 + [ci, ci, vp]
    L.maxfp8_quantize_static_scaled_fp8.restype = ci
    L.maxfp8_quantize_static_scaled_fp8.argtypes = [vp, vp, i64, i64, i64, i64, ci, cf, vp]
    L.maxfp8_quantize_tensor_dynamic_scaled_fp8.restype = ci
    L.maxfp8_quantize_tensor_dynamic_scaled_fp8.argtypes = [vp, vp, vp, i64, i64, i64, i64, ci, ci, cf, vp]
    L.maxfp8_moe_create_indices.restype = ci
    L.maxfp8_moe_create_indices.argtypes = [vp] * 6 + [i64, i64, vp]
    L.maxfp8_fused_silu.restype = ci
    L.maxfp8_fused_silu.argtypes = [vp] * 4 + [i64] * 6 + [ci, ci, vp]
    L.maxfp8_cast_f32_to_e4m3fn.restype = ci
    L.maxfp8_cast_f32_to_e4m3fn.argtypes = [vp, vp, i64, vp]
    L.maxfp8_cast_f32_to_bf16.restype = ci
    L.maxfp8_cast_f32_to_bf16.argtypes = [vp, vp, i64, vp]
    L.maxfp8_cast_e4m3fn_to_f32.restype = ci
    L.maxfp8_cast_e4m3fn_to_f32.argtypes = [vp, vp, i64, vp]
    L.maxfp8_copy_bytes.restype = ci
    L.maxfp8_copy_bytes.argtypes = [vp, vp, i64, vp]
    L.maxfp8_decode_weight_read_probe.restype = ci
    L.maxfp8_decode_weight_read_probe.argtypes = [vp, i64, i64, i64, i64, vp]
    L.maxfp8_handovers_given_up.restype = ctypes.c_longlong
    L.maxfp8_handovers_given_up.argtypes = []
    L.maxfp8_mfma_issue_probe.restype = ci
    L.maxfp8_mfma_issue_probe.argtypes = [ci, ci, ci, i64, vp, vp, vp, vp, vp, vp, vp]
    _lib = L
    return L


def last_error() -> str:
    return lib().maxfp8_last_error().decode("utf-8", "replace")


def check(status: int) -> None:
    """Maps a negative maxfp8_status to the exception class the reference's
    Python wrappers raise for the same mistake."""
    if status == OK:
        return
    msg = last_error() or f"maxfp8 error {status}"
    if status == ERR_DTYPE:
        raise TypeError(msg)
    if status in (ERR_SHAPE, ERR_ALIGN, ERR_GRANULARITY, ERR_NULL, ERR_WORKSPACE):
        raise ValueError(msg)
    raise RuntimeError(msg)


def tuning_reload() -> None:
    """Re-reads the MAXFP8_* tuning switches from the environment (they are read once per process otherwise)."""
    lib().maxfp8_tuning_reload()


def matmul_describe(M: int, N: int, K: int, block_scaling: bool = True, with_workspace: bool = True) -> str:
    """The launches MAXFP8_ALGO_AUTO makes for a fast-layout matmul, as text (diagnostic)."""
    buf = ctypes.create_string_buffer(256)
    lib().maxfp8_matmul_describe(M, N, K, int(block_scaling), int(with_workspace), buf, 256)
    return buf.value.decode()
