"""Host wrappers of the MoE steps on either side of the grouped FP8 matmul, with the names,
arguments and output shapes of the reference's wrappers: `moe_create_indices`
(max/python/max/nn/kernels.py:4980-5060) and `fused_silu` / `fused_silu_quantized`
(max/python/max/nn/comm/ep/ep_kernels.py:1121-1165, 1168-1290; FP8 block-scaled flavour only)."""
from __future__ import annotations

import torch

from . import _lib
from .kernels import _DT, _FP8, _require_gpu, _stream
from .quant_config import QuantConfig


def moe_create_indices(topk_ids: torch.Tensor, num_local_experts: int, *, needs_scales_offset: bool = False,
                       scales_alignment: int = 128) -> tuple[torch.Tensor, ...]:
    """Returns (token_expert_order uint32 [n], expert_start_indices uint32 [E+1], restore_token_order
    uint32 [n], expert_ids int32 [E], expert_usage_stats uint32 [2]) for the 1-D expert assignments
    `topk_ids`.  Slot z is expert z; a slot's assignments keep their order."""
    if needs_scales_offset:
        raise NotImplementedError("scales offsets belong to the NVFP4 / MX formats")
    if topk_ids.dim() != 1:
        raise ValueError("topk_ids must be rank 1 (flattened token x top_k assignments)")
    if topk_ids.dtype not in (torch.int32, torch.uint32):
        raise TypeError("topk_ids must be int32 or uint32")
    _require_gpu(topk_ids)
    topk_ids = topk_ids.contiguous()
    n, dev = topk_ids.shape[0], topk_ids.device
    order = torch.empty((n,), dtype=torch.uint32, device=dev)
    start = torch.empty((num_local_experts + 1,), dtype=torch.uint32, device=dev)
    restore = torch.empty((n,), dtype=torch.uint32, device=dev)
    expert_ids = torch.empty((num_local_experts,), dtype=torch.int32, device=dev)
    stats = torch.empty((2,), dtype=torch.uint32, device=dev)
    st = _lib.lib().maxfp8_moe_create_indices(order.data_ptr(), start.data_ptr(), restore.data_ptr(), expert_ids.data_ptr(),
                                              stats.data_ptr(), topk_ids.data_ptr(), n, num_local_experts, _stream(topk_ids))
    _lib.check(st)
    return order, start, restore, expert_ids, stats


def _check_silu_input(input: torch.Tensor, row_offsets: torch.Tensor) -> None:
    if input.dim() != 2:
        raise ValueError("input must be rank 2 tensor")
    if row_offsets.dim() != 1 or row_offsets.dtype != torch.uint32:
        raise TypeError("row_offsets must be a rank 1 uint32 tensor")
    if input.dtype != torch.bfloat16:
        raise TypeError("input must be bfloat16")
    _require_gpu(input, row_offsets)


def fused_silu(input: torch.Tensor, row_offsets: torch.Tensor, *, round_activation: bool = False) -> torch.Tensor:
    """silu(input[:, :I]) * input[:, I:] for the rows below row_offsets[-1]; [max_rows, I].

    round_activation=True (not a parameter of the reference's kernel): silu's result is rounded to the input's dtype
    before the product, which is what the reference's dense MLP computes with its two separate bf16 operations
    (ops.silu(gate) * up, max/python/max/nn/linear.py:1072); the MoE kernel rounds once, after the product."""
    _check_silu_input(input, row_offsets)
    input = input.contiguous()
    rows, two_i = input.shape
    inter = two_i // 2
    out = torch.empty((rows, inter), dtype=input.dtype, device=input.device)
    st = _lib.lib().maxfp8_fused_silu(out.data_ptr(), None, input.data_ptr(), row_offsets.data_ptr(), row_offsets.shape[0],
                                      rows, inter, two_i, inter, 0, _DT[input.dtype], 2 if round_activation else 0,
                                      _stream(input))
    _lib.check(st)
    return out


def fused_silu_quantized(input: torch.Tensor, row_offsets: torch.Tensor, quant_config: QuantConfig,
                         out_type: torch.dtype = _FP8) -> tuple[torch.Tensor, torch.Tensor]:
    """The same, quantised to e4m3fn with one f32 scale per 128 outputs; scales transposed,
    [I / 128, max_rows] (the blockwise scales type of the reference, quant_config.py:504-513)."""
    _check_silu_input(input, row_offsets)
    if out_type != _FP8:
        raise ValueError("out_type must be float8_e4m3fn")
    if quant_config.input_scale.block_size != (1, 128):
        raise ValueError("Can not determine the quantized scales type")
    input = input.contiguous()
    rows, two_i = input.shape
    inter = two_i // 2
    out = torch.empty((rows, inter), dtype=_FP8, device=input.device)
    scales = torch.empty((-(-inter // 128), rows), dtype=torch.float32, device=input.device)
    st = _lib.lib().maxfp8_fused_silu(out.data_ptr(), scales.data_ptr(), input.data_ptr(), row_offsets.data_ptr(),
                                      row_offsets.shape[0], rows, inter, two_i, inter, rows, _DT[input.dtype], 1,
                                      _stream(input))
    _lib.check(st)
    return out, scales
