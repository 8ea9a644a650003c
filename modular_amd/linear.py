"""FP8 `Linear`, mirroring max/python/max/nn/linear.py:103-250 (weights and scale
shapes) and :517-614 (`__call__` / `linear()`): weight [N, K] e4m3fn with K
innermost, inputs of any rank flattened to [M, K], bias added after the matmul.
"""
from __future__ import annotations

import torch

from .quant_config import QuantConfig, ScaleGranularity, ScaleOrigin
from .quant_ops import quantized_matmul


def infer_weight_scale_shape(out_dim: int, in_dim: int, quant_config: QuantConfig) -> tuple[int, ...]:
    """linear.py:217-250: rowwise (N, 1); tensor (); block (ceil(N/b0), ceil(K/b1))."""
    ws = quant_config.weight_scale
    if ws.is_rowwise:
        return (out_dim, 1)
    if ws.is_tensor:
        return ()
    if ws.is_block:
        assert ws.block_size is not None
        return (-(-out_dim // ws.block_size[0]), -(-in_dim // ws.block_size[1]))
    raise ValueError(f"only row-wise and tensor scaling are supported currently, but got {ws.granularity}")


class Linear(torch.nn.Module):
    """y = x @ W^T (+ bias) with W stored as e4m3fn and scales per `quant_config`."""

    def __init__(self, in_dim: int, out_dim: int, quant_config: QuantConfig, device=None,
                 has_bias: bool = False, bias_dtype: torch.dtype = torch.bfloat16) -> None:
        super().__init__()
        if quant_config.input_scale.granularity not in (ScaleGranularity.TENSOR, ScaleGranularity.COLWISE,
                                                        ScaleGranularity.BLOCK):
            raise ValueError(
                f"unsupported input scale granularity {quant_config.input_scale.granularity}. "
                "Only TENSOR, COLWISE and BLOCK granularities are supported, currently")
        self.in_dim, self.out_dim = in_dim, out_dim
        self.quant_config = quant_config
        self.register_buffer("weight", torch.zeros((out_dim, in_dim), dtype=torch.uint8, device=device)
                             .view(torch.float8_e4m3fn))
        shape = infer_weight_scale_shape(out_dim, in_dim, quant_config)
        self.register_buffer("weight_scale", torch.ones(shape, dtype=quant_config.weight_scale.dtype, device=device))
        # static quantisation: the pre-computed input scale is a scalar kept on the CPU (linear.py:176-184)
        self.input_scale = None
        if quant_config.input_scale.origin == ScaleOrigin.STATIC:
            self.input_scale = torch.ones((), dtype=quant_config.input_scale.dtype)
        if has_bias:
            self.register_buffer("bias", torch.zeros((out_dim,), dtype=quant_config.bias_dtype or bias_dtype,
                                                     device=device))
        else:
            self.bias = None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        y = quantized_matmul(x2, self.weight, self.weight_scale, self.input_scale, self.quant_config)
        if self.bias is not None:
            y = y + self.bias.to(y.dtype)
        return y.reshape(*lead, self.out_dim)
