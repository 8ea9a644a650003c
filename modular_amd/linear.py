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
        # Scalars that the static per-tensor ops take from the HOST stay on the CPU wherever the module goes: the
        # pre-computed input scale and, with it, a per-tensor weight scale (the reference keeps its scale weights
        # on the CPU, linear.py:176-205).  Both are entries of the state dict, so a checkpoint's `input_scale` /
        # `weight_scale` load like any other tensor.  Per-row and block scales live beside the weight on the GPU.
        static = quant_config.input_scale.origin == ScaleOrigin.STATIC
        self._host_scalars = (("input_scale",) if static else ()) + (("weight_scale",) if static and shape == () else ())
        scale_dev = "cpu" if "weight_scale" in self._host_scalars else device
        self.register_buffer("weight_scale", torch.ones(shape, dtype=quant_config.weight_scale.dtype, device=scale_dev))
        if static:
            self.register_buffer("input_scale", torch.ones((), dtype=quant_config.input_scale.dtype, device="cpu"))
        else:
            self.input_scale = None
        if has_bias:
            self.register_buffer("bias", torch.zeros((out_dim,), dtype=quant_config.bias_dtype or bias_dtype,
                                                     device=device))
        else:
            self.bias = None

    def _apply(self, fn, *args, **kwargs):
        # .to(device), .cuda(), .half() ... leave the host scalars where and what they are
        keep = {name: self._buffers[name] for name in self._host_scalars}
        out = super()._apply(fn, *args, **kwargs)
        self._buffers.update(keep)
        return out

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        y = quantized_matmul(x2, self.weight, self.weight_scale, self.input_scale, self.quant_config)
        if self.bias is not None:
            y = y + self.bias.to(y.dtype)
        return y.reshape(*lead, self.out_dim)


class MLP(torch.nn.Module):
    """Gated feed-forward block `down(act(gate(x)) * up(x))` with FP8 linears, mirroring
    max/python/max/nn/linear.py:865-1095.

    Like the reference, the gate and up projections run as ONE matmul over their concatenated
    weights when the quantisation allows it (`QuantConfig.can_use_fused_mlp`, linear.py:1029-1035);
    here the two weights ARE one buffer (`gate_up_weight`, with `gate_proj.weight` / `up_proj.weight`
    views of its halves), so nothing is concatenated per call.  With SiLU and no bias the activation
    and the product with `up` are one kernel (`fused_silu` with the activation rounded to bf16 before
    the product, as the reference's two bf16 operations `ops.silu(gate) * up` round it, linear.py:1072)
    whose bf16 result `down_proj` quantises like any other input: five launches for the whole block.

    `fuse_activation_quant=True` (dynamic block scaling only) also folds the quantisation for
    `down_proj` into that kernel (`fused_silu_quantized`: four launches, no bf16 intermediate).
    That kernel is the expert-parallel MoE quantiser (ep_comm.mojo:4505-4624), whose recipe is not
    the one `down_proj` applies -- scale = max(amax, 1e-4) / 448 without the upper bound of 1200,
    a division instead of a multiplication by the reciprocal, the f32 product instead of its bf16
    rounding -- so the fp8 codes it hands to the second matmul can differ by a step from the
    reference's: opt in where that is acceptable.  Every other case (bias, another activation, a
    clamp, static or per-tensor scales) takes the unfused route through the three `Linear`s.
    """

    _ACTIVATIONS = {
        "silu": torch.nn.functional.silu,
        "gelu": torch.nn.functional.gelu,
        "gelu_tanh": lambda t: torch.nn.functional.gelu(t, approximate="tanh"),
        "relu": torch.nn.functional.relu,
        "tanh": torch.tanh,
        "sigmoid": torch.sigmoid,
    }

    def __init__(self, hidden_dim: int, feed_forward_length: int, quant_config: QuantConfig, device=None,
                 has_bias: bool = False, activation_function: str = "silu", swiglu_limit: float = 0.0,
                 fuse_activation_quant: bool = False) -> None:
        super().__init__()
        if activation_function not in self._ACTIVATIONS:
            raise ValueError(f"Unsupported activation function: {activation_function}. "
                             f"Supported: {sorted(self._ACTIVATIONS)}")
        self.hidden_dim, self.feed_forward_length = hidden_dim, feed_forward_length
        self.quant_config = quant_config
        self.activation_function = activation_function
        self.swiglu_limit = swiglu_limit
        self.fuse_activation_quant = fuse_activation_quant
        self._row_offsets: dict[tuple, torch.Tensor] = {}  # [0, rows] per (rows, device): built once, on the device
        self.gate_proj = Linear(hidden_dim, feed_forward_length, quant_config, device=device, has_bias=has_bias)
        self.up_proj = Linear(hidden_dim, feed_forward_length, quant_config, device=device, has_bias=has_bias)
        self.down_proj = Linear(feed_forward_length, hidden_dim, quant_config, device=device, has_bias=has_bias)
        ws = quant_config.weight_scale
        block_ok = ws.is_block and ws.block_size is not None and feed_forward_length % ws.block_size[0] == 0
        self._one_matmul = (ws.is_rowwise or block_ok) and quant_config.input_scale.origin == ScaleOrigin.DYNAMIC
        if self._one_matmul:
            # one buffer for both weights (and one for their scales); the projections keep views of the halves
            f = feed_forward_length
            # (not part of the state dict: a checkpoint names gate_proj / up_proj, and loading those fills the halves)
            self.register_buffer("gate_up_weight", torch.zeros((2 * f, hidden_dim), dtype=torch.uint8, device=device)
                                 .view(torch.float8_e4m3fn), persistent=False)
            rows = self.gate_proj.weight_scale.shape[0]
            self.register_buffer("gate_up_weight_scale",
                                 torch.ones((2 * rows,) + tuple(self.gate_proj.weight_scale.shape[1:]),
                                            dtype=ws.dtype, device=device), persistent=False)
            self._tie_halves()

    def _tie_halves(self) -> None:
        f, rows = self.feed_forward_length, self.gate_up_weight_scale.shape[0] // 2
        self.gate_proj.weight, self.up_proj.weight = self.gate_up_weight[:f], self.gate_up_weight[f:]
        self.gate_proj.weight_scale, self.up_proj.weight_scale = (self.gate_up_weight_scale[:rows],
                                                                  self.gate_up_weight_scale[rows:])

    def _apply(self, fn, *args, **kwargs):
        # .to(device) and friends replace every buffer by a copy: afterwards the halves are views again
        out = super()._apply(fn, *args, **kwargs)
        if self._one_matmul:
            self._tie_halves()
        return out

    def _silu_kernel(self) -> bool:
        """silu(gate) * up as one kernel on the stacked [rows, 2 * F] result of the one matmul"""
        return (self._one_matmul and self.activation_function == "silu" and self.swiglu_limit == 0
                and self.gate_proj.bias is None and self.feed_forward_length % 8 == 0)

    def _fused(self) -> bool:
        cfg = self.quant_config
        return (self.fuse_activation_quant and self._silu_kernel() and cfg.input_scale.is_block and cfg.weight_scale.is_block
                and cfg.input_scale.block_size == (1, 128) and self.down_proj.bias is None
                and self.feed_forward_length % 128 == 0)

    def _all_rows(self, rows: int, device: torch.device) -> torch.Tensor:
        """The row_offsets operand of the silu kernels for a dense block: [0, rows] (uint32, on the device).  Kept
        per row count, so that a call neither copies from the host nor breaks a HIP graph capture."""
        key = (rows, device)
        t = self._row_offsets.get(key)
        if t is None:
            if len(self._row_offsets) >= 64:
                self._row_offsets.clear()
            t = torch.tensor([0, rows], dtype=torch.int64).to(torch.uint32).to(device)
            self._row_offsets[key] = t
        return t

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        from .kernels import dynamic_scaled_matmul, quantize_dynamic_scaled_float8
        from .moe_kernels import fused_silu, fused_silu_quantized

        cfg = self.quant_config
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        if self._fused():
            rows = x2.shape[0]
            xq, xs = quantize_dynamic_scaled_float8(x2, cfg.input_scale, cfg.weight_scale, scales_type=torch.float32)
            gate_up = dynamic_scaled_matmul(xq, self.gate_up_weight, xs, self.gate_up_weight_scale, cfg.input_scale,
                                            cfg.weight_scale, out_type=torch.bfloat16)
            hq, hs = fused_silu_quantized(gate_up, self._all_rows(rows, x2.device), cfg)
            y = dynamic_scaled_matmul(hq, self.down_proj.weight, hs, self.down_proj.weight_scale, cfg.input_scale,
                                      cfg.weight_scale, out_type=torch.bfloat16)
            return y.reshape(*lead, self.hidden_dim)
        if self._silu_kernel():
            both = quantized_matmul(x2, self.gate_up_weight, self.gate_up_weight_scale, None, cfg)
            hidden = fused_silu(both, self._all_rows(x2.shape[0], x2.device), round_activation=True)
            return self.down_proj(hidden).reshape(*lead, self.hidden_dim)
        act = self._ACTIVATIONS[self.activation_function]
        if self._one_matmul and self.gate_proj.bias is None:
            both = quantized_matmul(x2, self.gate_up_weight, self.gate_up_weight_scale, None, cfg)
            gate_out, up_out = act(both[:, :self.feed_forward_length]), both[:, self.feed_forward_length:]
        else:
            gate_out, up_out = act(self.gate_proj(x2)), self.up_proj(x2)
        if self.swiglu_limit > 0:
            gate_out = gate_out.clamp(max=self.swiglu_limit)
            up_out = up_out.clamp(min=-self.swiglu_limit, max=self.swiglu_limit)
        return self.down_proj(gate_out * up_out).reshape(*lead, self.hidden_dim)
