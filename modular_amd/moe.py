"""The expert matmuls of a block-scaled FP8 MoE layer, in the order of the reference's
`_expert_matmuls` (max/python/max/nn/moe/moe_fp8.py:487-616, FP8 block-scaled strategy):

    group the (token, expert) assignments by expert      moe_create_indices
    gather the tokens into that order and quantise       quantize_dynamic_scaled_float8(row_index=...)
    1 x 128 (the gather rides on the quantiser's loads)
    gate_up = grouped matmul                             grouped_dynamic_scaled_fp8_matmul
    silu(gate) * up on the rows in use                   fused_silu
    quantise 1 x 128, down = grouped matmul that stores  grouped_dynamic_scaled_fp8_matmul(out_row_index=...)
    its rows back in (token, k) order

Every step is one of this package's HIP kernels; the two row permutations cost no pass of their own."""
from __future__ import annotations

import torch

from .kernels import grouped_dynamic_scaled_fp8_matmul, quantize_dynamic_scaled_float8
from .moe_kernels import fused_silu, fused_silu_quantized, moe_create_indices
from .quant_config import QuantConfig


def expert_matmuls_fp8(
    x: torch.Tensor,
    router_idx: torch.Tensor,
    gate_up_proj: torch.Tensor,
    gate_up_proj_scales: torch.Tensor,
    down_proj: torch.Tensor,
    down_proj_scales: torch.Tensor,
    quant_config: QuantConfig,
    *,
    host_sync: bool = True,
    fuse_activation_quant: bool = False,
) -> torch.Tensor:
    """x [seq, hidden] bf16; router_idx [seq, k] expert ids; gate_up_proj [E, 2 * I, hidden] and
    down_proj [E, hidden, I] e4m3fn with 128 x 128 block scales.  Returns the experts' outputs
    [seq, k, hidden] (bf16), before the router weights are applied.

    The grouped matmul op takes two host scalars (most tokens on one expert, active experts), which
    the reference copies from the device between the grouping and the first matmul
    (max/python/max/nn/moe/quant_strategy.py:175).  This package's kernels read the offsets on the
    device and use the scalars only as upper bounds for their grids, so with `host_sync=False` the
    bounds (every row on one expert, every expert active) stand in and nothing waits for the GPU:
    same result, and the whole function can be captured in a HIP graph.

    `fuse_activation_quant=True` runs silu(gate) * up and the quantisation for the down projection as one kernel
    (`fused_silu_quantized`, the form the reference's expert-parallel path uses, ep_kernels.py:1168-1290) instead of
    `fused_silu` followed by the quantiser: one pass over gate_up instead of three passes over it and its
    activation; the product is quantised from f32 instead of from its bf16 rounding, so the fp8 codes can differ
    by one step from the two-kernel form."""
    if x.dim() != 2 or router_idx.dim() != 2 or router_idx.shape[0] != x.shape[0]:
        raise ValueError("expected x [seq, hidden] and router_idx [seq, k]")
    if not (quant_config.input_scale.is_block and quant_config.weight_scale.is_block):
        raise ValueError("the FP8 MoE path of this package is the block-scaled one")
    seq_len, top_k = router_idx.shape
    num_experts = gate_up_proj.shape[0]
    token_order, expert_start, restore_order, expert_ids, usage_stats = moe_create_indices(
        router_idx.reshape(-1).to(torch.int32), num_experts)
    if host_sync:
        stats_host = usage_stats.cpu()  # [most tokens on one expert, active experts]: the op's two host scalars
    else:
        stats_host = torch.tensor([seq_len * top_k, num_experts], dtype=torch.int64).to(torch.uint32)

    def quantise(t: torch.Tensor, **gather):
        return quantize_dynamic_scaled_float8(t, quant_config.input_scale, quant_config.weight_scale,
                                              scales_type=torch.float32, group_size_or_per_token=128, **gather)

    def grouped(t_q, t_s, weight, weight_scales, **scatter):
        return grouped_dynamic_scaled_fp8_matmul(t_q, weight, t_s, weight_scales, expert_start, expert_ids, stats_host,
                                                 quant_config.input_scale, quant_config.weight_scale, **scatter)

    # sorted row r is assignment token_order[r] = token * top_k + slot: it reads token token_order[r] // top_k
    gate_up = grouped(*quantise(x, row_index=token_order, index_div=top_k), gate_up_proj, gate_up_proj_scales)
    if fuse_activation_quant:
        act_q = fused_silu_quantized(gate_up, expert_start, quant_config)
    else:
        act_q = quantise(fused_silu(gate_up, expert_start))
    # ... and its result belongs in row token_order[r] of the [seq * top_k, hidden] output
    down = grouped(*act_q, down_proj, down_proj_scales, out_row_index=token_order)
    return down.reshape(seq_len, top_k, down.shape[-1])
