"""FP8 dispatch of a quantised linear, mirroring `quantized_matmul` /
`_matmul_float8` (max/python/max/nn/quant_ops.py:516-592, 336-481): the static
per-tensor branch and the dynamic tensor / per-row / block branches; and of the
quantised grouped matmul of the MoE layers, `quantized_grouped_matmul`
(quant_ops.py:880-1007, FP8 formats).
"""
from __future__ import annotations

import weakref

import torch

from .kernels import (dynamic_scaled_matmul, fused_qkv_ragged_matmul_scaled_float8,
                      grouped_dynamic_scaled_fp8_matmul, grouped_matmul_rowwise_dynamic_scaled_fp8,
                      matmul_static_scaled_float8, quantize_dynamic_scaled_float8, quantize_static_scaled_float8,
                      quantize_tensor_dynamic_scaled_float8)
from .kv_cache import KVCacheParams, PagedCacheValues
from .quant_config import InputScaleSpec, QuantConfig, QuantFormat, ScaleGranularity, WeightScaleSpec


def matmul_float8(
    x: torch.Tensor,
    weight: torch.Tensor,
    weight_scale: torch.Tensor,
    input_scale: torch.Tensor | None,
    quant_config: QuantConfig,
) -> torch.Tensor:
    """x @ weight.T with float8 quantisation; x [M, K] bf16, weight [N, K] e4m3fn."""
    if input_scale is not None:
        # Static quantisation: the input scale was computed offline (quant_ops.py:384-417).
        xq = quantize_static_scaled_float8(x, input_scale, out_type=weight.dtype)
        if quant_config.weight_scale.is_tensor and weight_scale.dim() >= 2:
            # fused QKV: per-projection weight scales broadcast to rowwise [N, 1]; the scalar
            # input scale is broadcast to the per-token layout [1, M]
            weight_scale = weight_scale.to(x.device)
            a_scales = input_scale.reshape(1, 1).to(device=x.device, dtype=weight_scale.dtype).expand(1, xq.shape[0]).contiguous()
            in_spec = InputScaleSpec(ScaleGranularity.COLWISE, quant_config.input_scale.origin, weight_scale.dtype)
            w_spec = WeightScaleSpec(ScaleGranularity.ROWWISE, weight_scale.dtype)
            return dynamic_scaled_matmul(xq, weight, a_scales, weight_scale, in_spec, w_spec, out_type=torch.bfloat16)
        return matmul_static_scaled_float8(xq, weight, input_scale, weight_scale)

    if quant_config.input_scale.is_tensor and quant_config.weight_scale.is_tensor:
        # Dynamic tensor-wise FP8 is executed as per-token x per-channel with the
        # scalar weight scale broadcast to [N, 1] (quant_ops.py:418-461).
        n_out = weight.shape[0]
        if weight_scale.dim() < 2:
            weight_scale = weight_scale.reshape(1, 1).expand(n_out, 1).contiguous()
        weight_scale = weight_scale.to(x.device)
        in_spec = InputScaleSpec(ScaleGranularity.COLWISE, quant_config.input_scale.origin, weight_scale.dtype)
        w_spec = WeightScaleSpec(ScaleGranularity.ROWWISE, weight_scale.dtype)
        xq, x_scales = quantize_dynamic_scaled_float8(x, in_spec, w_spec, scales_type=weight_scale.dtype,
                                                      out_type=weight.dtype)
        return dynamic_scaled_matmul(xq, weight, x_scales, weight_scale, in_spec, w_spec,
                                     out_type=torch.bfloat16)

    # dynamic per-row / block scaling (quant_ops.py:462-481)
    xq, x_scale = quantize_dynamic_scaled_float8(
        x, quant_config.input_scale, quant_config.weight_scale,
        scales_type=weight_scale.dtype, out_type=weight.dtype)
    weight_scale = weight_scale.to(x.device)
    return dynamic_scaled_matmul(xq, weight, x_scale, weight_scale, quant_config.input_scale,
                                 quant_config.weight_scale, out_type=torch.bfloat16)


def quantized_matmul(
    x: torch.Tensor,
    weight: torch.Tensor,
    weight_scale: torch.Tensor,
    input_scale: torch.Tensor | None = None,
    quant_config: QuantConfig | None = None,
) -> torch.Tensor:
    """Entry point of the quantised linear (quant_ops.py:516-592): only the FP8
    formats are in this package."""
    if quant_config is None:
        raise ValueError("quant_config is required for a quantized matmul")
    if weight.dtype != torch.float8_e4m3fn:
        raise TypeError(f"weight dtype {weight.dtype} is not float8_e4m3fn")
    return matmul_float8(x, weight, weight_scale, input_scale, quant_config)


def quantized_fused_qkv_matmul(
    kv_params: KVCacheParams,
    x: torch.Tensor,
    wqkv: torch.Tensor,
    kv_collection: PagedCacheValues,
    layer_idx: int,
    input_row_offsets: torch.Tensor,
    n_heads: int,
    quant_config: QuantConfig,
    weight_scale: torch.Tensor,
    input_scale: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
    _output_dim: int | None = None,
) -> torch.Tensor:
    """Entry point of the quantised fused QKV projection (quant_ops.py:594-760), FP8 formats:
    quantise x the way the config says, then one matmul that returns Q and stores K and V in the
    paged cache.  (Scales in bfloat16 are widened to float32 for the kernel, which is exact.)"""
    if quant_config.format not in (QuantFormat.COMPRESSED_TENSORS_FP8, QuantFormat.FBGEMM_FP8, QuantFormat.BLOCKSCALED_FP8):
        raise NotImplementedError(f"{quant_config.format} is not an FP8 format of this package")
    common = dict(input_row_offsets=input_row_offsets, wqkv=wqkv, kv_collection=kv_collection, layer_idx=layer_idx,
                  n_heads=n_heads, bias=bias, _output_dim=_output_dim)
    if quant_config.is_static:
        assert input_scale is not None
        xq = quantize_static_scaled_float8(x, input_scale.cpu())
        x_scales = input_scale
    elif quant_config.input_scale.is_tensor and quant_config.weight_scale.is_tensor:
        # dynamic per-tensor input scale against the rowwise [N, 1] scales of the fused weight: the
        # kernel infers per-channel scaling from the [1, M] / [N, 1] shapes (quant_ops.py:707-738)
        xq, x_scales = quantize_tensor_dynamic_scaled_float8(x, quant_config.input_scale, quant_config.weight_scale,
                                                             out_type=wqkv.dtype, scales_type=weight_scale.dtype)
        return fused_qkv_ragged_matmul_scaled_float8(kv_params, input=xq, input_scale=x_scales.to(x.device).float(),
                                                     weight_scale=weight_scale.to(x.device).float(), quant_config=None,
                                                     **common)
    else:
        xq, x_scales = quantize_dynamic_scaled_float8(x, quant_config.input_scale, quant_config.weight_scale,
                                                      scales_type=weight_scale.dtype, out_type=wqkv.dtype)
    return fused_qkv_ragged_matmul_scaled_float8(kv_params, input=xq, input_scale=x_scales.to(x.device).float(),
                                                 weight_scale=weight_scale.to(x.device).float(), quant_config=quant_config,
                                                 **common)


# ---- grouped (MoE) entry point ---------------------------------------------------------------
# The reference keeps stacked FP8 expert weights in storage layout [E, in, out] = [E, K, N] and
# transposes them to [E, N, K] in the graph (quant_ops.py:941-944), where the transposition of a
# constant weight is folded away at compile time.  The eager equivalent: a storage tensor is
# transposed once and the K-innermost copy lives exactly as long as the storage tensor object does
# (one entry per live tensor, found through a weak reference and dropped with it; remade after an
# in-place write).  A model's every stacked weight and scale tensor keeps its copy, however many
# layers there are.  A caller that hands in a new view object on every call (`w.data`) would get a
# new copy every time: such callers transpose once themselves and pass k_innermost=True.
_K_INNERMOST: dict[int, tuple] = {}   # id(storage tensor) -> (weak reference to it, what it looked like, the copy)


def _k_innermost(t: torch.Tensor) -> torch.Tensor:
    """t.transpose(1, 2) as a contiguous tensor, made once per storage tensor."""
    looks = (t.data_ptr(), tuple(t.shape), tuple(t.stride()), t.dtype, t.device, t._version)
    key = id(t)
    hit = _K_INNERMOST.get(key)
    if hit is not None and hit[0]() is t and hit[1] == looks:
        return hit[2]
    # (fp8 has no copy kernel of its own in every torch build: move the bytes)
    tt = t.view(torch.uint8).transpose(1, 2).contiguous().view(t.dtype) if t.element_size() == 1 else t.transpose(1, 2).contiguous()
    _K_INNERMOST[key] = (weakref.ref(t, lambda _gone, key=key: _K_INNERMOST.pop(key, None)), looks, tt)
    return tt


def quantized_grouped_matmul(
    x: torch.Tensor,
    weight: torch.Tensor,
    weight_scale: torch.Tensor,
    expert_start_indices: torch.Tensor,
    expert_ids: torch.Tensor,
    usage_stats: torch.Tensor,
    quant_config: QuantConfig,
    *,
    k_innermost: bool = False,
) -> torch.Tensor:
    """Single entry point of the quantised grouped matmuls of a MoE layer (quant_ops.py:880-1007),
    FP8 formats: x [T, K] bf16 with its rows sorted by expert; weight in STORAGE layout [E, K, N]
    e4m3fn; weight_scale in storage layout -- [E, K/128, N/128] for block scaling, [E, N, 1] for
    per-channel scaling; usage_stats = [most rows on one expert, active experts] (device or CPU: the
    op takes them as host scalars, so a device tensor is copied, which waits for the GPU).

    Block scaling: both are transposed to the K-innermost orientation of the kernel, x is quantised
    in 1 x block groups with scales of the weight scales' dtype, then the grouped block-scaled matmul.
    Per-channel weight scales with per-token activation scales (no block size): the weight scales
    are used as they are, the [1, T] scales of the quantiser become the kernel's [T, 1].

    k_innermost=True (not in the reference, whose compiler folds the transposition of a constant away): weight and
    block scales are already in the kernel's orientation, [E, N, K] and [E, N/128, K/128] -- for callers that
    transpose once at load time."""
    if quant_config.format not in (QuantFormat.COMPRESSED_TENSORS_FP8, QuantFormat.FBGEMM_FP8, QuantFormat.BLOCKSCALED_FP8):
        raise ValueError(f"Unsupported quantization format for grouped matmul: {quant_config.format}")
    if weight.dim() != 3:
        raise ValueError(f"expected weight of rank 3 but got {weight.dim()}")
    weight_t = weight if k_innermost else _k_innermost(weight)
    stats_host = usage_stats.cpu()
    if quant_config.weight_scale.is_rowwise and quant_config.input_scale.block_size is None:
        x_fp8, x_scales = quantize_dynamic_scaled_float8(x, quant_config.input_scale, quant_config.weight_scale,
                                                         out_type=weight.dtype, scales_type=torch.float32)
        return grouped_matmul_rowwise_dynamic_scaled_fp8(x_fp8, weight_t, x_scales.transpose(0, 1), weight_scale,
                                                         expert_start_indices, expert_ids, stats_host)
    assert quant_config.input_scale.block_size is not None
    input_block_size = quant_config.input_scale.block_size[1]
    scale_t = weight_scale if k_innermost else _k_innermost(weight_scale)
    x_fp8, x_scales = quantize_dynamic_scaled_float8(x, quant_config.input_scale, quant_config.weight_scale,
                                                     group_size_or_per_token=input_block_size, out_type=weight.dtype,
                                                     scales_type=quant_config.weight_scale.dtype)
    return grouped_dynamic_scaled_fp8_matmul(x_fp8, weight_t, x_scales, scale_t, expert_start_indices, expert_ids,
                                             stats_host, quant_config.input_scale, quant_config.weight_scale)
