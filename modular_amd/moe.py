"""The expert matmuls of a block-scaled FP8 MoE layer, in the order of the reference's
`_expert_matmuls` (max/python/max/nn/moe/moe_fp8.py:487-616, FP8 block-scaled strategy):

    group the (token, expert) assignments by expert      moe_create_indices
    gather the tokens into that order and quantise       quantize_dynamic_scaled_float8(scatter_index=...)
    1 x 128 (a token is quantised once and stored to
    its top_k rows; other dtypes: row_index=..., the
    gather rides on the quantiser's loads)
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


class Fp8Strategy:
    """FP8 quantisation of a MoE layer: the reference's `Fp8Strategy`
    (max/python/max/nn/moe/quant_strategy.py:114-215), same methods and argument meaning.  The
    weights arrive in the kernel's orientation ([E, N, K], scales [E, N/128, K/128]), as the
    reference's MoE layer stacks them (moe/moe.py:616-650).

    Two keyword arguments go beyond the reference: `quantize(..., row_index=, index_div=)` and
    `grouped_matmul(..., out_row_index=)` hand the row gather in front of the first quantiser and
    the row scatter behind the last matmul to the kernels, where the reference's graph compiler
    fuses its `ops.gather` into the neighbouring ops."""

    def __init__(self, config: QuantConfig, dtype: torch.dtype = torch.float8_e4m3fn) -> None:
        self.config = config
        self.dtype = dtype

    def quantize(self, tensor: torch.Tensor, group_size: int, *, row_index: torch.Tensor | None = None,
                 index_div: int = 1, scatter_index: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        """Quantizes activations to FP8 and returns (quantized, scales)."""
        return quantize_dynamic_scaled_float8(tensor, self.config.input_scale, self.config.weight_scale,
                                              group_size_or_per_token=group_size, out_type=self.dtype,
                                              scales_type=self.config.weight_scale.dtype, row_index=row_index,
                                              index_div=index_div, scatter_index=scatter_index)

    def grouped_quantize(self, tensor: torch.Tensor, group_size: int, input_scale: torch.Tensor | None,
                         expert_start: torch.Tensor, scales_offset: torch.Tensor | None,
                         expert_ids: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """Falls back to ungrouped FP8 quantization (quant_strategy.py:140-151)."""
        return self.quantize(tensor, group_size)

    def grouped_matmul(self, weight: torch.Tensor, weight_scales: torch.Tensor, expert_scales: torch.Tensor | None = None,
                       expert_inputs: tuple[torch.Tensor, ...] = (), estimated_total_m: torch.Tensor | None = None,
                       a_scales_preshuffled: bool = False, a_scales_max_padded_m: int = 0, *,
                       out_row_index: torch.Tensor | None = None) -> torch.Tensor:
        """Runs the grouped FP8 matmul for the routed experts.  expert_inputs = (hidden, input_scales,
        expert_start, expert_ids, usage_stats); usage_stats become the op's host scalars, so a device
        tensor is copied to the CPU here (quant_strategy.py:175), which waits for the GPU.  The other
        arguments exist for conformance with the strategies of other formats and are ignored."""
        hidden, input_scales, expert_start, expert_ids, usage_stats = expert_inputs
        return grouped_dynamic_scaled_fp8_matmul(hidden, weight, input_scales, weight_scales, expert_start, expert_ids,
                                                 usage_stats.cpu(), self.config.input_scale, self.config.weight_scale,
                                                 out_row_index=out_row_index)

    def prepare_weight_scales(self, gate_up: torch.Tensor, down: torch.Tensor,
                              device: torch.device | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        """Passes FP8 weight scales through without reformatting."""
        return gate_up, down

    def fused_silu_quantize(self, gate_up_projs: torch.Tensor, input_scales: torch.Tensor | None = None,
                            expert_inputs: tuple[torch.Tensor, ...] = (), max_padded_M: int = 0,
                            clamp_activation: bool = False, swiglu_alpha: float = 0.0,
                            swiglu_limit: float = 0.0) -> tuple[torch.Tensor, torch.Tensor]:
        """Applies the fused SiLU gate and returns quantized activations (quant_strategy.py:193-215)."""
        assert not clamp_activation, "clamped SwiGLU-OAI activation is only supported on the MXFP4 EP path"
        _, _, expert_start_indices, _, _ = expert_inputs
        return fused_silu_quantized(gate_up_projs, expert_start_indices, self.config, self.dtype)


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
    strategy = Fp8Strategy(quant_config, gate_up_proj.dtype)
    group = quant_config.input_scale.block_size[1]
    seq_len, top_k = router_idx.shape
    num_experts = gate_up_proj.shape[0]
    token_order, expert_start, restore_order, expert_ids, usage_stats = moe_create_indices(
        router_idx.reshape(-1).to(torch.int32), num_experts)
    if not host_sync:
        # the bounds that need no look at the GPU: every row on one expert, every expert active
        usage_stats = torch.tensor([seq_len * top_k, num_experts], dtype=torch.int64).to(torch.uint32)

    # sorted row r is assignment token_order[r] = token * top_k + slot: it reads token token_order[r] // top_k.  Seen
    # from the token: it is quantised once and stored to its top_k sorted rows restore_order[token * top_k + slot] --
    # the same bytes, and what the kernel for bfloat16 activations, float32 scales and groups of 128 does
    if (x.dtype == torch.bfloat16 and group == 128 and quant_config.weight_scale.dtype == torch.float32 and
            x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0):
        permuted_quant, permuted_scales = strategy.quantize(x, group, scatter_index=restore_order)
    else:
        permuted_quant, permuted_scales = strategy.quantize(x, group, row_index=token_order, index_div=top_k)
    gate_up_scales, down_scales = strategy.prepare_weight_scales(gate_up_proj_scales, down_proj_scales, x.device)
    expert_inputs = (permuted_quant, permuted_scales, expert_start, expert_ids, usage_stats)
    gate_up = strategy.grouped_matmul(gate_up_proj, gate_up_scales, expert_inputs=expert_inputs)
    if fuse_activation_quant:
        gate_up_quant, gate_up_act_scales = strategy.fused_silu_quantize(gate_up, expert_inputs=expert_inputs)
    else:
        gate_up_quant, gate_up_act_scales = strategy.quantize(fused_silu(gate_up, expert_start), group)
    down_inputs = (gate_up_quant, gate_up_act_scales) + expert_inputs[2:]
    # ... and its result belongs in row token_order[r] of the [seq * top_k, hidden] output
    down = strategy.grouped_matmul(down_proj, down_scales, expert_inputs=down_inputs, out_row_index=token_order)
    return down.reshape(seq_len, top_k, down.shape[-1])
