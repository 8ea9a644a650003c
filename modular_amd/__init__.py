"""MI355X-native FP8 linear path: dynamic activation quantisation, scaled FP8
matmul and its grouped (MoE) variant, behind the op names of the reference.

All compute runs in hand-written gfx950 HIP kernels (modular_amd/csrc) loaded
through the C ABI of include/maxfp8.h; there is no CPU or PyTorch fallback.
"""
from .quant_config import (InputScaleSpec, QuantConfig, QuantFormat, ScaleGranularity, ScaleOrigin,
                           WeightScaleSpec, blockwise_fp8_config, rowwise_fp8_config)
from .kv_cache import KVCacheParams, PagedCacheValues
from .kernels import (grouped_matmul_rowwise_dynamic_scaled_fp8, fused_qkv_ragged_matmul_scaled_float8, matmul_k_cache_ragged_scaled_float8,
                      batched_dynamic_scaled_fp8_matmul, batched_quantize_dynamic_scaled_fp8, dynamic_scaled_matmul,
                      grouped_dynamic_scaled_fp8_matmul, matmul_static_scaled_float8,
                      quantize_static_scaled_float8, quantize_tensor_dynamic_scaled_float8,
                      quantize_dynamic_scaled_float8, rms_norm_fused_quantize_dynamic_scaled_fp8)
from .moe_kernels import fused_silu, fused_silu_quantized, moe_create_indices
from .moe import Fp8Strategy, expert_matmuls_fp8
from .quant_ops import matmul_float8, quantized_fused_qkv_matmul, quantized_grouped_matmul, quantized_matmul
from .linear import MLP, Linear
from .weights_quant import parse_quant_config

__all__ = [
    "InputScaleSpec", "QuantConfig", "QuantFormat", "ScaleGranularity", "ScaleOrigin", "WeightScaleSpec",
    "blockwise_fp8_config", "rowwise_fp8_config", "dynamic_scaled_matmul",
    "grouped_dynamic_scaled_fp8_matmul", "quantize_dynamic_scaled_float8", "matmul_float8",
    "quantized_matmul", "Linear", "MLP", "rms_norm_fused_quantize_dynamic_scaled_fp8",
    "moe_create_indices", "fused_silu", "fused_silu_quantized",
    "quantize_static_scaled_float8", "matmul_static_scaled_float8", "parse_quant_config",
    "batched_dynamic_scaled_fp8_matmul", "batched_quantize_dynamic_scaled_fp8",
    "quantize_tensor_dynamic_scaled_float8", "fused_qkv_ragged_matmul_scaled_float8",
    "matmul_k_cache_ragged_scaled_float8", "KVCacheParams", "PagedCacheValues", "quantized_fused_qkv_matmul", "grouped_matmul_rowwise_dynamic_scaled_fp8", "expert_matmuls_fp8",
    "Fp8Strategy", "quantized_grouped_matmul",
]
