"""Scaled-quantisation configuration types, mirroring
max/python/max/nn/quant_config.py:26-66 (ScaleGranularity, ScaleOrigin),
:109-199 (WeightScaleSpec, InputScaleSpec) and :201-351 (QuantConfig) for the
FP8 formats this package executes.  dtypes are torch dtypes.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum

import torch


class ScaleGranularity(Enum):
    """Granularity of a quantisation scale; the string values are the ones the
    reference passes verbatim as op parameters."""

    TENSOR = "tensor"
    ROWWISE = "rowwise"
    COLWISE = "colwise"
    BLOCK = "block"

    def __str__(self) -> str:
        return self.value


class ScaleOrigin(Enum):
    STATIC = "static"
    DYNAMIC = "dynamic"

    @property
    def is_dynamic(self) -> bool:
        return self == ScaleOrigin.DYNAMIC

    @property
    def is_static(self) -> bool:
        return self == ScaleOrigin.STATIC


class QuantFormat(Enum):
    """Checkpoint formats that lead to the FP8 linear path."""

    COMPRESSED_TENSORS_FP8 = "compressed-tensors-fp8"
    FBGEMM_FP8 = "fbgemm-fp8"
    BLOCKSCALED_FP8 = "blockscaled-fp8"


def _is(kind: "ScaleGranularity"):
    return property(lambda self: self.granularity is kind)


class _GranularityProps:
    """is_tensor / is_rowwise / is_colwise / is_block of a spec."""
    granularity: ScaleGranularity
    is_tensor = _is(ScaleGranularity.TENSOR)
    is_rowwise = _is(ScaleGranularity.ROWWISE)
    is_colwise = _is(ScaleGranularity.COLWISE)
    is_block = _is(ScaleGranularity.BLOCK)


def _check_block(granularity: ScaleGranularity, block_size) -> None:
    if granularity == ScaleGranularity.BLOCK:
        if block_size is None:
            raise ValueError("block_size must be specified for block-wise scaling")
        if len(block_size) != 2:
            raise ValueError("block_size must be a tuple of two integers")


@dataclass
class WeightScaleSpec(_GranularityProps):
    granularity: ScaleGranularity
    dtype: torch.dtype
    block_size: tuple[int, int] | None = None

    def __post_init__(self) -> None:
        _check_block(self.granularity, self.block_size)


@dataclass
class InputScaleSpec(_GranularityProps):
    granularity: ScaleGranularity
    origin: ScaleOrigin
    dtype: torch.dtype
    activation_scale_ub: float | None = None
    block_size: tuple[int, int] | None = None

    def __post_init__(self) -> None:
        _check_block(self.granularity, self.block_size)


@dataclass
class QuantConfig:
    input_scale: InputScaleSpec
    weight_scale: WeightScaleSpec
    mlp_quantized_layers: set[int] = field(default_factory=set)
    attn_quantized_layers: set[int] = field(default_factory=set)
    format: QuantFormat = QuantFormat.BLOCKSCALED_FP8
    embedding_output_dtype: torch.dtype | None = None
    bias_dtype: torch.dtype | None = None

    @property
    def scales_granularity_mnk(self) -> tuple[int, int, int]:
        """(m, n, k) granularities; -1 = one scale along that axis
        (quant_config.py:313-351)."""
        def axes(spec, single, what):
            # (granularity along the spec's own axis, granularity along K); -1 = one scale for the axis
            if spec.is_block:
                assert spec.block_size is not None
                return tuple(spec.block_size)
            if getattr(spec, single):
                return (1, -1)
            if spec.is_tensor:
                return (-1, -1)
            raise ValueError(f"unsupported {what} scale granularity")

        m_g, k_in = axes(self.input_scale, "is_colwise", "input")
        n_g, k_w = axes(self.weight_scale, "is_rowwise", "weight")
        assert k_in == k_w, "k_input_granularity and k_weight_granularity must be the same"
        return (m_g, n_g, k_in)

    @property
    def is_static(self) -> bool:
        return self.input_scale.origin == ScaleOrigin.STATIC

    @property
    def is_dynamic(self) -> bool:
        return self.input_scale.origin == ScaleOrigin.DYNAMIC

    def quantized_scales_shape(self, quantized_shape: tuple[int, int]) -> tuple[int, int]:
        """Shape of the blockwise activation scales, transposed [ceil(K/128), M]
        (quant_config.py:452-472, 504-513)."""
        if self.input_scale.block_size is not None and tuple(self.input_scale.block_size) == (1, 128):
            return ((quantized_shape[1] + 127) // 128, quantized_shape[0])
        raise ValueError("Can not determine the quantized scales type")


def blockwise_fp8_config() -> QuantConfig:
    """DeepSeek-style: 1x128 dynamic activation groups, 128x128 weight blocks, f32 scales."""
    return QuantConfig(
        input_scale=InputScaleSpec(ScaleGranularity.BLOCK, ScaleOrigin.DYNAMIC, torch.float32, block_size=(1, 128)),
        weight_scale=WeightScaleSpec(ScaleGranularity.BLOCK, torch.float32, block_size=(128, 128)),
        format=QuantFormat.BLOCKSCALED_FP8,
    )


def rowwise_fp8_config() -> QuantConfig:
    """fbgemm-style: per-token dynamic activation scales, per-output-channel weight scales."""
    return QuantConfig(
        input_scale=InputScaleSpec(ScaleGranularity.COLWISE, ScaleOrigin.DYNAMIC, torch.float32),
        weight_scale=WeightScaleSpec(ScaleGranularity.ROWWISE, torch.float32),
        format=QuantFormat.FBGEMM_FP8,
    )
