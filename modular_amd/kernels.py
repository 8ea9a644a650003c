"""Eager op wrappers with the names, argument order, shape rules and exceptions
of the reference's graph-op wrappers:

  quantize_dynamic_scaled_float8      max/python/max/nn/kernels.py:6876-6957
  dynamic_scaled_matmul               max/python/max/nn/kernels.py:6960-7078
  grouped_dynamic_scaled_fp8_matmul   max/python/max/nn/kernels.py:6327-6487
  batched_dynamic_scaled_fp8_matmul   max/python/max/nn/kernels.py:6642-6751
  fused_qkv_ragged_matmul_scaled_float8  max/python/max/nn/kernels.py:582-727
  matmul_k_cache_ragged_scaled_float8    max/python/max/nn/kernels.py:1475-1539
  grouped_matmul_rowwise_dynamic_scaled_fp8  max/python/max/nn/kernels.py:6490-6640

They take torch tensors that live on the MI355X and call the HIP kernels through
the C ABI on torch's current stream.  Nothing here computes on the CPU.
"""
from __future__ import annotations

import torch

from . import _lib
from .kv_cache import KVCacheParams, PagedCacheValues
from .quant_config import InputScaleSpec, QuantConfig, ScaleGranularity, ScaleOrigin, WeightScaleSpec

_FP8 = torch.float8_e4m3fn
_DT = {torch.bfloat16: _lib.BF16, torch.float16: _lib.F16, torch.float32: _lib.F32, _FP8: _lib.E4M3FN}
_ALGOS = {"auto": _lib.ALGO_AUTO, "naive": _lib.ALGO_NAIVE, "tiled": _lib.ALGO_TILED, "skinny": _lib.ALGO_SKINNY}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """The HIP stream torch currently launches on for t's device, as an integer handle.
    (torch.cuda.current_stream() builds a Stream object per call: 4 microseconds, as much as the launch itself.)"""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("maxfp8 kernels run on the GPU only: got a tensor on " + str(t.device))


def quantize_output_geometry(M: int, K: int, input_scale_spec: InputScaleSpec,
                             weight_scale_spec: WeightScaleSpec, group_size_or_per_token: int,
                             scales_type: torch.dtype) -> tuple[int, int]:
    """(group size, padded column count of the scales tensor), the rules of
    max/python/max/nn/kernels.py:6910-6931: the group is block_size[1] for block
    specs and K otherwise; block specs pad the token axis of the scales to 16 bytes."""
    if group_size_or_per_token == -1:
        if input_scale_spec.is_block or weight_scale_spec.is_block:
            assert input_scale_spec.block_size is not None
            group_size = input_scale_spec.block_size[1]
        else:
            group_size = int(K)
    else:
        group_size = group_size_or_per_token
    a_scales_dim1 = M
    if input_scale_spec.is_block or weight_scale_spec.is_block:
        if not (input_scale_spec.is_block and weight_scale_spec.is_block):
            raise ValueError("both input and weight must be blockwise scaled for blockwise scaling")
        padding_size = 16 // torch.empty((), dtype=scales_type).element_size()
        a_scales_dim1 = ((M + padding_size - 1) // padding_size) * padding_size
    return group_size, a_scales_dim1


def quantize_dynamic_scaled_float8(
    input: torch.Tensor,
    input_scale_spec: InputScaleSpec,
    weight_scale_spec: WeightScaleSpec,
    scale_ub: float = 1200.0,
    group_size_or_per_token: int = -1,
    out_type: torch.dtype = _FP8,
    scales_type: torch.dtype = torch.bfloat16,
    *,
    row_index: torch.Tensor | None = None,
    index_div: int = 1,
    scatter_index: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Dynamically quantize `input` [M, K] to fp8.

    Returns (quantized [M, K] e4m3fn, scales [K / group, M_pad]) where, for block
    specs, M_pad rounds M up to a multiple of 16 bytes / sizeof(scale); the padding
    columns are allocated but never written.

    With `row_index` (uint32 [R] on the device) the result has R rows and row r is
    quantised from `input[row_index[r] // index_div]`: the gather that the reference's
    graph compiler fuses into the op's input (builtin_kernels/quantization.mojo:1376-1390),
    e.g. `row_index=token_expert_order, index_div=top_k` in the MoE layer.

    With `scatter_index` (uint32 [M * copies] on the device) the result has M * copies rows
    and `input[r]` is quantised once and written to the rows `scatter_index[r * copies + j]`:
    the same bytes as the gather by the inverse permutation
    (`scatter_index=restore_token_order`), without quantising a token top_k times.  bfloat16
    input, float32 scales and groups of 128 only.
    """
    if input.dim() != 2:
        raise ValueError("input must be rank 2 tensor")
    if out_type != _FP8:
        # e4m3fnuz is only ever requested on gfx94x (kernels.py:8408-8417)
        raise ValueError("out_type must be float8_e4m3fn or float8_e4m3fnuz")
    M, K = input.shape
    if scatter_index is not None:
        if row_index is not None:
            raise ValueError("row_index and scatter_index exclude each other")
        if scatter_index.dtype != torch.uint32 or scatter_index.dim() != 1:
            raise TypeError("scatter_index must be a rank 1 uint32 tensor")
        if M == 0 or scatter_index.shape[0] % M != 0:
            raise ValueError(f"scatter_index must hold a whole number of destinations per input row ({M} rows)")
        src_rows, copies, M = M, scatter_index.shape[0] // M, scatter_index.shape[0]
    if row_index is not None:
        if row_index.dtype != torch.uint32 or row_index.dim() != 1:
            raise TypeError("row_index must be a rank 1 uint32 tensor")
        if index_div < 1:
            raise ValueError("index_div must be positive")
        src_rows, M = M, row_index.shape[0]

    group_size, a_scales_dim1 = quantize_output_geometry(
        M, K, input_scale_spec, weight_scale_spec, group_size_or_per_token, scales_type)

    if scales_type not in (torch.float32, torch.bfloat16):
        raise TypeError("scales dtype should be bfloat16 or float32")
    if input.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError(f"input dtype {input.dtype} is not bfloat16, float16 or float32")
    if group_size <= 0 or K % group_size != 0:
        raise ValueError(f"group size {group_size} must divide K = {K}")

    _require_gpu(input)
    if input.stride(1) != 1:
        input = input.contiguous()
    out = torch.empty((M, K), dtype=_FP8, device=input.device)
    scales = torch.empty((K // group_size, a_scales_dim1), dtype=scales_type, device=input.device)
    if scatter_index is not None:
        _require_gpu(scatter_index)
        st = _lib.lib().maxfp8_quantize_dynamic_scaled_fp8_scatter(
            out.data_ptr(), scales.data_ptr(), input.data_ptr(), scatter_index.data_ptr(), copies, src_rows, K, M,
            input.stride(0) if src_rows > 1 else K, K,
            group_size, a_scales_dim1, _DT[input.dtype], _DT[scales_type], float(scale_ub), _stream(input))
        _lib.check(st)
        return out, scales
    if row_index is not None:
        _require_gpu(row_index)
        st = _lib.lib().maxfp8_quantize_dynamic_scaled_fp8_gather(
            out.data_ptr(), scales.data_ptr(), input.data_ptr(), row_index.data_ptr(), index_div, M, K,
            input.stride(0) if src_rows > 1 else K, K,
            group_size, a_scales_dim1, _DT[input.dtype], _DT[scales_type], float(scale_ub), _stream(input))
        _lib.check(st)
        return out, scales
    st = _lib.lib().maxfp8_quantize_dynamic_scaled_fp8(
        out.data_ptr(), scales.data_ptr(), input.data_ptr(), M, K, input.stride(0) if M > 1 else K, K,
        group_size, a_scales_dim1, _DT[input.dtype], _DT[scales_type], float(scale_ub), _stream(input))
    _lib.check(st)
    return out, scales


def quantize_tensor_dynamic_scaled_float8(
    input: torch.Tensor,
    input_scale_spec: InputScaleSpec,
    weight_scale_spec: WeightScaleSpec,
    scale_ub: float = 1200.0,
    group_size_or_per_token: int = -1,
    out_type: torch.dtype = _FP8,
    scales_type: torch.dtype = torch.bfloat16,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Quantize `input` [M, K] to fp8 with one dynamic scale for the whole tensor
    (max/python/max/nn/kernels.py:6804-6873).  Returns (quantized [M, K], scales [1, M]);
    every element of scales holds the tensor's scale."""
    if input.dim() != 2:
        raise ValueError("input must be rank 2 tensor")
    if out_type != _FP8:
        raise ValueError("out_type must be float8_e4m3fn")
    if not (input_scale_spec.is_tensor and weight_scale_spec.is_tensor):
        raise ValueError("both input and weight must be tensor scaled for tensor scaling")
    if group_size_or_per_token != -1:
        raise ValueError("group_size_or_per_token should be -1 for dynamic tensor scaling so "
                         "group_size == num_cols == input.shape[1]")
    if scales_type not in (torch.float32, torch.bfloat16):
        raise TypeError("scales dtype should be bfloat16 or float32")
    if input.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError(f"input dtype {input.dtype} is not bfloat16, float16 or float32")
    _require_gpu(input)
    if input.stride(1) != 1:
        input = input.contiguous()
    M, K = input.shape
    out = torch.empty((M, K), dtype=_FP8, device=input.device)
    scales = torch.empty((1, M), dtype=scales_type, device=input.device)
    st = _lib.lib().maxfp8_quantize_tensor_dynamic_scaled_fp8(
        out.data_ptr(), scales.data_ptr(), input.data_ptr(), M, K, input.stride(0) if M > 1 else K, K,
        _DT[input.dtype], _DT[scales_type], float(scale_ub), _stream(input))
    _lib.check(st)
    return out, scales


def _host_scalar(t: torch.Tensor, what: str) -> float:
    if tuple(t.shape) not in ((), (1,)):
        raise ValueError(f"expected {what} to be a scalar, but got shape of {list(t.shape)}")
    if t.device.type != "cpu":
        raise ValueError(f"expected {what} to be on CPU, but got {t.device}")
    return float(t.reshape(()).to(torch.float32))


def quantize_static_scaled_float8(x: torch.Tensor, scale: torch.Tensor, scale_is_inverted: bool = True,
                                  out_type: torch.dtype = _FP8) -> torch.Tensor:
    """Quantizes a rank-2 tensor to float8 with a static per-tensor scale held on the CPU:
    clamp(x * (1 / scale)) (max/python/max/nn/kernels.py:6753-6801).  `scale_is_inverted` is accepted
    and, as in the reference's kernel, has no effect."""
    s = _host_scalar(scale, "scale")
    if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise ValueError(f"expected input dtype to be float16, bfloat16, or float32, but got {x.dtype}")
    if x.dim() != 2:
        raise ValueError(f"expected input rank to be 2, but got {x.dim()}")
    if out_type != _FP8:
        raise ValueError("out_type must be float8_e4m3fn")
    _require_gpu(x)
    if x.stride(1) != 1:
        x = x.contiguous()
    M, K = x.shape
    out = torch.empty((M, K), dtype=_FP8, device=x.device)
    st = _lib.lib().maxfp8_quantize_static_scaled_fp8(out.data_ptr(), x.data_ptr(), M, K, x.stride(0) if M > 1 else K, K,
                                                      _DT[x.dtype], s, _stream(x))
    _lib.check(st)
    return out


def matmul_static_scaled_float8(input: torch.Tensor, weight: torch.Tensor, input_scale: torch.Tensor,
                                weight_scale: torch.Tensor) -> torch.Tensor:
    """input @ weight.T for float8 operands with per-tensor CPU scalar scales, bfloat16 out:
    cast(acc * (input_scale * weight_scale)) (max/python/max/nn/kernels.py:8319-8405; epilogue
    builtin_kernels/linalg.mojo:1790-1802)."""
    a_s = _host_scalar(input_scale, "input_scale")
    b_s = _host_scalar(weight_scale, "weight_scale")
    if input.dtype != _FP8:
        raise ValueError(f"expected input dtype to be float8_e4m3fn or float8_e4m3fnuz, but got {input.dtype}")
    if weight.dtype != _FP8:
        raise ValueError(f"expected weight dtype to be float8_e4m3fn or float8_e4m3fnuz, but got {weight.dtype}")
    if input.dim() != 2:
        raise ValueError(f"expected input rank to be 2, but got {input.dim()}")
    if weight.dim() != 2:
        raise ValueError(f"expected weight rank to be 2, but got {weight.dim()}")
    if input.shape[1] != weight.shape[1]:
        raise ValueError("K dimension does not match for matmul")
    # the product of the two scales is formed first, in f32, and applied once
    prod = torch.tensor([[a_s]], dtype=torch.float32) * torch.tensor([[b_s]], dtype=torch.float32)
    one = torch.ones((1, 1), dtype=torch.float32)
    in_spec = InputScaleSpec(ScaleGranularity.TENSOR, ScaleOrigin.STATIC, torch.float32)
    w_spec = WeightScaleSpec(ScaleGranularity.TENSOR, torch.float32)
    return dynamic_scaled_matmul(input, weight, prod.to(input.device), one.to(input.device), in_spec, w_spec,
                                 out_type=torch.bfloat16)


def rms_norm_fused_quantize_dynamic_scaled_fp8(
    input: torch.Tensor,
    gamma: torch.Tensor,
    epsilon: float,
    weight_offset: float = 0.0,
    scale_ub: float = 1200.0,
    out_type: torch.dtype = _FP8,
    scales_type: torch.dtype = torch.float32,
) -> tuple[torch.Tensor, torch.Tensor]:
    """RMSNorm over the last axis fused with the per-row dynamic fp8 quantisation: the composite op
    `mo.composite.rms_norm_fused_quantize_dynamic_scaled_fp8` that the reference's graph compiler
    forms from rms_norm followed by quantize_dynamic_scaled_float8
    (builtin_kernels/quantization.mojo:112-237).

    Returns (quantized, same shape as input, e4m3fn; scales [1, rows] with rows = input.numel() / K)."""
    if input.dim() < 1:
        raise ValueError("input must have at least one axis")
    if gamma.dim() != 1:
        raise ValueError("gamma must be rank 1")
    if gamma.dtype != input.dtype:
        raise TypeError("gamma dtype must match input dtype")
    if out_type != _FP8:
        raise ValueError("output dtype should be float8_e4m3fn or float8_e4m3fnuz")
    if scales_type not in (torch.float32, torch.bfloat16):
        raise TypeError("scales dtype should be bfloat16 or float32")
    if input.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError(f"input dtype {input.dtype} is not bfloat16, float16 or float32")
    K = input.shape[-1]
    if gamma.shape[0] != K:
        raise ValueError(f"gamma has {gamma.shape[0]} elements, the normalised axis has {K}")
    _require_gpu(input)
    _require_gpu(gamma)
    x2 = input.reshape(-1, K)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    gamma = gamma.contiguous()
    out = torch.empty((rows, K), dtype=_FP8, device=input.device)
    scales = torch.empty((1, rows), dtype=scales_type, device=input.device)
    st = _lib.lib().maxfp8_rms_norm_fused_quantize_dynamic_scaled_fp8(
        out.data_ptr(), scales.data_ptr(), x2.data_ptr(), gamma.data_ptr(), rows, K,
        x2.stride(0) if rows > 1 else K, K, _DT[input.dtype], _DT[scales_type], float(epsilon),
        float(weight_offset), float(scale_ub), _stream(input))
    _lib.check(st)
    return out.reshape(input.shape), scales


def dynamic_scaled_matmul(
    a: torch.Tensor,
    b: torch.Tensor,
    a_scales: torch.Tensor,
    b_scales: torch.Tensor,
    input_scale_spec: InputScaleSpec,
    weight_scale_spec: WeightScaleSpec,
    out_type: torch.dtype = torch.bfloat16,
    *,
    algo: str = "auto",
) -> torch.Tensor:
    """C = A . B^T with scaling factors; `b` is [N, K] (already "transposed")."""
    if a.dim() != 2 or b.dim() != 2 or a_scales.dim() != 2 or b_scales.dim() != 2:
        raise ValueError("All arguments must be rank 2 tensors")
    if a.shape[1] != b.shape[1]:
        raise ValueError("The second dimension of b must match the second dimension of a")

    gm = gn = gk = -1
    if input_scale_spec.is_tensor and weight_scale_spec.is_tensor:
        if input_scale_spec.origin.is_dynamic:
            if not (b_scales.shape[0] == b_scales.shape[1] == 1):
                raise ValueError("scaler weight tensors must be of shape [1, 1] for dynamic tensor scaling")
        else:
            if not (a_scales.shape[0] == a_scales.shape[1] == b_scales.shape[0] == b_scales.shape[1] == 1):
                raise ValueError("scaler tensors must be of shape [1, 1] for tensor scaling")
        gin, gw = _lib.GRAN_TENSOR, _lib.GRAN_TENSOR
    elif input_scale_spec.is_colwise and weight_scale_spec.is_rowwise:
        if a_scales.shape[0] != 1:
            raise ValueError("only per-token scaling is supported for a")
        if b_scales.shape[1] != 1:
            raise ValueError("only channel-wise scaling is supported for b")
        gin, gw = _lib.GRAN_COLWISE, _lib.GRAN_ROWWISE
    elif input_scale_spec.is_block or weight_scale_spec.is_block:
        if input_scale_spec.block_size is None or weight_scale_spec.block_size is None:
            raise ValueError("both input and weight block size must be set for blockwise scaling")
        if not (input_scale_spec.is_block and weight_scale_spec.is_block):
            raise ValueError("both input and weight must be blockwise scaled for blockwise scaling")
        if a_scales.dtype != b_scales.dtype or a_scales.dtype != torch.float32:
            raise TypeError(
                f"a_scales and b_scales dtypes must be float32, but got {a_scales.dtype}, {b_scales.dtype}")
        if a_scales.shape[0] != b_scales.shape[1]:
            raise ValueError(
                "both a_scales and b_scales must have the same shape on the K dimension. got "
                f"a_scales.shape={tuple(a_scales.shape)} and b_scales.shape={tuple(b_scales.shape)}")
        gin, gw = _lib.GRAN_BLOCK, _lib.GRAN_BLOCK
        gm = input_scale_spec.block_size[0]
        gn, gk = weight_scale_spec.block_size
    else:
        raise ValueError("unsupported FP8 scaling granularity")

    if (a.dtype != b.dtype) or (a_scales.dtype != b_scales.dtype):
        raise TypeError(
            f"a and b dtypes {a.dtype}, {b.dtype} must match, as do a and b scales dtypes "
            f"{a_scales.dtype}, {b_scales.dtype}")
    if a.dtype != _FP8:
        raise TypeError(f"a and b must be float8_e4m3fn, got {a.dtype}")
    if a_scales.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise TypeError(f"scales dtype {a_scales.dtype} is not float32, bfloat16 or float16")
    if out_type not in (torch.bfloat16, torch.float32):
        raise TypeError(f"out_type {out_type} is not bfloat16 or float32")
    if gin == _lib.GRAN_COLWISE and a_scales.shape[1] < a.shape[0]:
        raise ValueError("a_scales must hold one scale per row of a")
    if gin == _lib.GRAN_COLWISE and b_scales.shape[0] != b.shape[0]:
        raise ValueError("b_scales must hold one scale per row of b")
    if gin == _lib.GRAN_BLOCK:
        if a_scales.shape[0] != -(-a.shape[1] // gk) or a_scales.shape[1] < -(-a.shape[0] // gm):
            raise ValueError(f"a_scales shape {tuple(a_scales.shape)} does not cover a {tuple(a.shape)}")
        if b_scales.shape[0] != -(-b.shape[0] // gn):
            raise ValueError(f"b_scales shape {tuple(b_scales.shape)} does not cover b {tuple(b.shape)}")

    _require_gpu(a, b, a_scales, b_scales)
    if a.stride(1) != 1:
        a = a.contiguous()
    if b.stride(1) != 1:
        b = b.contiguous()
    if a_scales.stride(1) != 1:
        a_scales = a_scales.contiguous()
    if b_scales.dim() == 2 and b_scales.shape[1] > 1 and b_scales.stride(1) != 1:
        b_scales = b_scales.contiguous()
    M, K = a.shape
    N = b.shape[0]
    c = torch.empty((M, N), dtype=out_type, device=a.device)
    lda = a.stride(0) if M > 1 else K
    ldb = b.stride(0) if N > 1 else K
    a_ld = a_scales.stride(0) if a_scales.shape[0] > 1 else a_scales.shape[1]
    b_ld = b_scales.stride(0) if b_scales.shape[0] > 1 else b_scales.shape[1]
    # split-K scratch for problems whose tiles would cover only part of the chip (0 bytes otherwise)
    ws_bytes = _lib.lib().maxfp8_matmul_workspace_bytes(M, N, K) if algo in ("auto", "tiled") else 0
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=a.device) if ws_bytes else None
    st = _lib.lib().maxfp8_matmul_dynamic_scaled_fp8(
        c.data_ptr(), a.data_ptr(), b.data_ptr(), a_scales.data_ptr(), b_scales.data_ptr(), M, N, K,
        lda, ldb, N, gin, gw, gm, gn, gk, a_ld, b_ld, _DT[out_type], _DT[a_scales.dtype], _ALGOS[algo],
        ws.data_ptr() if ws is not None else None, ws_bytes, _stream(a))
    _lib.check(st)
    return c


def batched_quantize_dynamic_scaled_fp8(
    input: torch.Tensor,
    group_size_or_per_token: int = 128,
    scale_ub: float = 1200.0,
    scales_type: torch.dtype = torch.float32,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Quantize every [M, K] slice of `input` [B, M, K] in one launch.

    The eager form of batched_quantize_dynamic_scaled_fp8
    (max/kernels/src/linalg/fp8_quantization.mojo:779-954).  `input` may be any view
    whose last axis is contiguous, e.g. the [row, batch, col] -> [batch, row, col]
    transpose the MLA graph quantizes (mla_graph.mojo:1010-1033): it is read in place.
    Returns (quantized [B, M, K] e4m3fn, scales [B, K / group, M_pad]); M_pad rounds
    M up to 16 bytes of scales, the shape batched_dynamic_scaled_fp8_matmul expects.
    """
    if input.dim() != 3:
        raise ValueError("input must be rank 3 tensor")
    if scales_type not in (torch.float32, torch.bfloat16):
        raise TypeError("scales dtype should be bfloat16 or float32")
    if input.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError(f"input dtype {input.dtype} is not bfloat16, float16 or float32")
    B, M, K = input.shape
    group_size = K if group_size_or_per_token == -1 else group_size_or_per_token
    if group_size <= 0 or K % group_size != 0:
        raise ValueError(f"group size {group_size} must divide K = {K}")
    _require_gpu(input)
    if input.stride(2) != 1 and K > 1:
        input = input.contiguous()
    pad = 16 // torch.empty((), dtype=scales_type).element_size()
    m_pad = -(-M // pad) * pad
    out = torch.empty((B, M, K), dtype=_FP8, device=input.device)
    scales = torch.empty((B, K // group_size, m_pad), dtype=scales_type, device=input.device)
    st = _lib.lib().maxfp8_batched_quantize_dynamic_scaled_fp8(
        out.data_ptr(), scales.data_ptr(), input.data_ptr(), B, M, K,
        input.stride(0) if B > 1 else M * K, input.stride(1) if M > 1 else K, M * K, K,
        group_size, (K // group_size) * m_pad, m_pad, _DT[input.dtype], _DT[scales_type], float(scale_ub),
        _stream(input))
    _lib.check(st)
    return out, scales


def batched_dynamic_scaled_fp8_matmul(
    a: torch.Tensor,
    b: torch.Tensor,
    a_scales: torch.Tensor,
    b_scales: torch.Tensor,
    input_scale_spec: InputScaleSpec,
    weight_scale_spec: WeightScaleSpec,
    out_type: torch.dtype = torch.bfloat16,
    *,
    algo: str = "auto",
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """C[i] = A[i] . B[i]^T with blockwise scaling factors; a [B, M, K], b [B, N, K],
    a_scales [B, ceil(K/128), M_pad], b_scales [B, ceil(N/128), ceil(K/128)].
    `out`, if given, is a [B, M, N] view with a contiguous last axis that receives the
    result in place (e.g. the [M, B, N] buffer the MLA graph writes, transposed)."""
    if a.dtype != b.dtype:
        raise TypeError(f"a and b dtypes must match, but got {a.dtype}, {b.dtype}")
    if a_scales.dtype != b_scales.dtype or a_scales.dtype != torch.float32:
        raise TypeError(f"a_scales and b_scales dtypes must be float32, but got {a_scales.dtype}, {b_scales.dtype}")
    if a.dim() != 3 or b.dim() != 3:
        raise ValueError("A and B must be rank 3 tensors")
    if a_scales.dim() != 3 or b_scales.dim() != 3:
        raise ValueError("A_scales and B_scales must be rank 3 tensors")
    if a.shape[0] != b.shape[0]:
        raise ValueError("The batch dimension of b must match the batch dimension of a")
    if a.shape[2] != b.shape[2]:
        raise ValueError("A and B K dimension does not match")
    if a.dtype != _FP8:
        raise TypeError(f"a and b dtypes must be float8_e4m3fn, but got {a.dtype}, {b.dtype}")
    if not (input_scale_spec.is_block and weight_scale_spec.is_block):
        raise ValueError("unsupported FP8 scaling granularity")
    if a_scales.shape[0] != b_scales.shape[0]:
        raise ValueError("both a_scales and b_scales must have the same shape on the batch dimension")
    if input_scale_spec.block_size is None or weight_scale_spec.block_size is None:
        raise ValueError("both input scale_granularity and weight scale_granularity must be set for batched "
                         "blockwise scaling")
    if tuple(input_scale_spec.block_size) != (1, 128):
        raise ValueError("batched blockwise scaling only supports (1,128) granularity for input")
    if tuple(weight_scale_spec.block_size) != (128, 128):
        raise ValueError("batched blockwise scaling only supports (128,128) granularity for weight")
    if out_type not in (torch.bfloat16, torch.float32):
        raise TypeError(f"out_type {out_type} is not bfloat16 or float32")
    B, M, K = a.shape
    N = b.shape[1]
    if a_scales.shape[0] != B or a_scales.shape[1] != -(-K // 128) or a_scales.shape[2] < M:
        raise ValueError(f"a_scales shape {tuple(a_scales.shape)} does not cover a {tuple(a.shape)}")
    if b_scales.shape[1] != -(-N // 128) or b_scales.shape[2] != -(-K // 128):
        raise ValueError(f"b_scales shape {tuple(b_scales.shape)} does not cover b {tuple(b.shape)}")

    _require_gpu(a, b, a_scales, b_scales)
    a, b, a_scales, b_scales = (t if t.stride(2) == 1 or t.shape[2] == 1 else t.contiguous()
                                for t in (a, b, a_scales, b_scales))
    if out is None:
        c = torch.empty((B, M, N), dtype=out_type, device=a.device)
    else:
        if tuple(out.shape) != (B, M, N) or out.dtype != out_type or (N > 1 and out.stride(2) != 1):
            raise ValueError(f"out must be a [{B}, {M}, {N}] {out_type} view with a contiguous last axis")
        _require_gpu(out)
        c = out

    def steps(t: torch.Tensor) -> tuple[int, int]:  # (batch, row) strides, well defined for extent-1 axes too
        rows, cols = t.shape[1], t.shape[2]
        row = t.stride(1) if rows > 1 else cols
        return (t.stride(0) if t.shape[0] > 1 else rows * row), row

    (a_bs, lda), (b_bs, ldb), (c_bs, ldc) = steps(a), steps(b), steps(c)
    (as_bs, a_ld), (bs_bs, b_ld) = steps(a_scales), steps(b_scales)
    st = _lib.lib().maxfp8_batched_matmul_dynamic_scaled_fp8(
        c.data_ptr(), a.data_ptr(), b.data_ptr(), a_scales.data_ptr(), b_scales.data_ptr(), B, M, N, K,
        a_bs, lda, b_bs, ldb, c_bs, ldc, 1, 128, 128, as_bs, a_ld, bs_bs, b_ld, _DT[out_type], _lib.F32,
        _ALGOS[algo], _stream(a))
    _lib.check(st)
    return c


def _u32(t: torch.Tensor, what: str) -> torch.Tensor:
    # torch has little support for uint32: int32 tensors with the same bits are accepted
    if t.dtype not in (torch.uint32, torch.int32):
        raise TypeError(f"expected {what} to have dtype uint32, but got {t.dtype}")
    return t.contiguous()


def _qkv_cache_matmul(kv_params: KVCacheParams, input: torch.Tensor, input_row_offsets: torch.Tensor,
                      weight: torch.Tensor, input_scale: torch.Tensor, weight_scale: torch.Tensor,
                      kv_collection: PagedCacheValues, layer_idx: int, q_dim: int,
                      scales_granularity_mnk: tuple[int, int, int], bias: torch.Tensor | None,
                      algo: str) -> torch.Tensor:
    if input.dtype != weight.dtype:
        raise ValueError(f"expected input and weight to have the same dtype, but got {input.dtype} and {weight.dtype}")
    if input.dtype != _FP8:
        raise TypeError(f"input and weight must be float8_e4m3fn, got {input.dtype}")
    if input.dim() != 2:
        raise ValueError(f"expected input to have rank 2, was {input.dim()}")
    tensors = [weight, input_row_offsets, input_scale, weight_scale] + ([] if bias is None else [bias])
    if not all(t.device == input.device for t in tensors):
        raise ValueError(f"expected all tensors to be on the same device as input ({input.device})")
    _require_gpu(input, kv_collection.kv_blocks, kv_collection.cache_lengths, kv_collection.lookup_table)
    if kv_params.dtype != torch.bfloat16 or kv_collection.kv_blocks.dtype != torch.bfloat16:
        raise TypeError("the paged cache must be bfloat16")
    blocks = kv_collection.kv_blocks
    if blocks.dim() != 6 or tuple(blocks.shape[1:]) != kv_params.blocks_shape(0)[1:] or not blocks.is_contiguous():
        raise ValueError(f"kv_blocks must be a contiguous {kv_params.blocks_shape(-1)} tensor, got {tuple(blocks.shape)}")
    row_offsets = _u32(input_row_offsets, "input_row_offsets")
    cache_lengths = _u32(kv_collection.cache_lengths, "cache_lengths")
    lut = _u32(kv_collection.lookup_table, "lookup_table")
    batch = row_offsets.shape[0] - 1
    if cache_lengths.shape[0] < batch or lut.dim() != 2 or lut.shape[0] < batch:
        raise ValueError("cache_lengths / lookup_table hold fewer sequences than input_row_offsets")
    if input_scale.dtype != torch.float32 or weight_scale.dtype != torch.float32:
        raise TypeError("input_scale and weight_scale must be float32")
    T, K = input.shape
    N = weight.shape[0]
    if weight.dim() != 2 or weight.shape[1] != K:
        raise ValueError("weight must be [N, K] with the K of input")
    input = input.contiguous()
    weight = weight.contiguous()
    input_scale = input_scale.contiguous()
    weight_scale = weight_scale.contiguous()
    if bias is not None:
        if bias.dtype != torch.bfloat16 or bias.numel() != N:
            raise ValueError("bias must be a bfloat16 vector of length N")
        bias = bias.contiguous()
    out = torch.empty((T, q_dim), dtype=torch.bfloat16, device=input.device)
    in_ld = input_scale.shape[1] if input_scale.dim() == 2 else 1
    w_ld = weight_scale.shape[1] if weight_scale.dim() == 2 else 1
    st = _lib.lib().maxfp8_fused_qkv_matmul_ragged_paged_scale(
        out.data_ptr() if q_dim else None, input.data_ptr(), row_offsets.data_ptr(), weight.data_ptr(),
        input_scale.data_ptr(), weight_scale.data_ptr(), blocks.data_ptr(), cache_lengths.data_ptr(), lut.data_ptr(),
        bias.data_ptr() if bias is not None else None, T, N, K, q_dim, batch, blocks.shape[0], kv_params.kv_dim,
        kv_params.num_layers, int(layer_idx), kv_params.page_size, kv_params.n_kv_heads, kv_params.head_dim,
        lut.shape[1], *scales_granularity_mnk, in_ld, w_ld, _lib.F32, _ALGOS[algo], _stream(input))
    _lib.check(st)
    return out


def fused_qkv_ragged_matmul_scaled_float8(
    kv_params: KVCacheParams,
    input: torch.Tensor,
    input_row_offsets: torch.Tensor,
    wqkv: torch.Tensor,
    kv_collection: PagedCacheValues,
    layer_idx: int,
    n_heads: int,
    input_scale: torch.Tensor,
    weight_scale: torch.Tensor,
    bias: torch.Tensor | None = None,
    quant_config: QuantConfig | None = None,
    _output_dim: int | None = None,
    *,
    algo: str = "auto",
) -> torch.Tensor:
    """Fused query, key and value projections of scaled float8 input and weights: returns
    Q [total_seq_len, n_heads * head_dim] (bf16) and writes K and V into the paged cache
    in place (max/python/max/nn/kernels.py:582-727)."""
    if input_scale.dim() < 2 and input_scale.numel() == 1:
        input_scale = input_scale.reshape(1, 1)
    if weight_scale.dim() < 2 and weight_scale.numel() == 1:
        weight_scale = weight_scale.reshape(1, 1)
    if quant_config is not None:
        mnk = quant_config.scales_granularity_mnk
    elif tuple(input_scale.shape) == (1, 1) and tuple(weight_scale.shape) == (1, 1):
        mnk = (-1, -1, -1)      # per-tensor quantization
    elif input_scale.shape[0] == 1 and weight_scale.shape[1] == 1:
        mnk = (1, 1, -1)        # per-channel quantization
    else:
        raise ValueError("Can not infer the quantization config from the input tensor shapes",
                         "Please provide a quant_config")
    output_dim = _output_dim if _output_dim is not None else n_heads * kv_params.head_dim
    return _qkv_cache_matmul(kv_params, input, input_row_offsets, wqkv, input_scale, weight_scale, kv_collection,
                             layer_idx, output_dim, tuple(mnk), bias, algo)


def matmul_k_cache_ragged_scaled_float8(
    kv_params: KVCacheParams,
    hidden_states: torch.Tensor,
    input_row_offsets: torch.Tensor,
    weight: torch.Tensor,
    input_scale: torch.Tensor,
    weight_scale: torch.Tensor,
    kv_collection: PagedCacheValues,
    scales_granularity_mnk: tuple[int, int, int],
    layer_idx: int,
    *,
    algo: str = "auto",
) -> None:
    """Block-scaled float8 matmul whose whole result is written to the key pages of the
    cache (max/python/max/nn/kernels.py:1475-1539)."""
    _qkv_cache_matmul(kv_params, hidden_states, input_row_offsets, weight, input_scale, weight_scale, kv_collection,
                      layer_idx, 0, tuple(scales_granularity_mnk), None, algo)


def grouped_dynamic_scaled_fp8_matmul(
    hidden_states: torch.Tensor,
    weight: torch.Tensor,
    a_scales: torch.Tensor,
    b_scales: torch.Tensor,
    expert_start_indices: torch.Tensor,
    expert_ids: torch.Tensor,
    expert_usage_stats_host: torch.Tensor,
    input_scale_spec: InputScaleSpec,
    weight_scale_spec: WeightScaleSpec,
    out_type: torch.dtype = torch.bfloat16,
    *,
    algo: str = "auto",
    out_row_index: torch.Tensor | None = None,
) -> torch.Tensor:
    """Grouped blockwise scaled matmul of the MoE layer: rows of `hidden_states`
    are sorted by expert, `expert_start_indices` delimits the groups,
    `expert_usage_stats_host` = [max tokens of any expert, number of active experts]
    on the CPU.

    With `out_row_index` (uint32 [T], a permutation) row m of the result lands in row
    `out_row_index[m]` of the returned tensor: the scatter that puts the down projection
    back into token order (max/python/max/nn/moe/moe_fp8.py:614-616) fused into the
    matmul's store, as the reference's compiler does with the op's output lambda."""
    if weight.dim() != 3:
        raise ValueError(f"expected weight of rank 3 but got {weight.dim()}")
    if hidden_states.dim() != 2:
        raise ValueError(f"expected hidden_states of rank 2 but got {hidden_states.dim()}")
    if weight.shape[2] != hidden_states.shape[1] or weight.shape[0] != expert_ids.shape[0]:
        raise ValueError(
            f"expected weight is of shape [num_experts, *, {hidden_states.shape[1]}] but got {tuple(weight.shape)}")
    if (hidden_states.dtype != weight.dtype) or (hidden_states.dtype != _FP8):
        raise TypeError(
            f"hidden_states and weight dtypes must be float8_e4m3fn, but got {hidden_states.dtype}, {weight.dtype}")
    if (a_scales.dtype != b_scales.dtype) or (a_scales.dtype not in (torch.float32, torch.bfloat16)):
        raise TypeError(
            f"a_scales and b_scales dtypes must be float32 or bfloat16 and match, but got {a_scales.dtype}, {b_scales.dtype}")
    if expert_ids.dtype != torch.int32:
        raise TypeError(f"expert_ids dtype must be int32, but got {expert_ids.dtype}")
    if expert_ids.dim() != 1:
        raise ValueError(f"expected expert_ids of rank 1 but got {expert_ids.dim()}")
    if expert_start_indices.dtype != torch.uint32:
        raise TypeError(f"expert_start_indices dtype must be uint32, but got {expert_start_indices.dtype}")
    if expert_start_indices.dim() != 1:
        raise ValueError(f"expected expert_start_indices of rank 1 but got {expert_start_indices.dim()}")
    if a_scales.dim() != 2 or b_scales.dim() != 3:
        raise ValueError(
            f"expected a_scales of rank 2 and b_scales of rank 3 but got {a_scales.dim()} and {b_scales.dim()}")

    if input_scale_spec.is_block and weight_scale_spec.is_block:
        if input_scale_spec.block_size is None or weight_scale_spec.block_size is None:
            raise ValueError("both input block_size and weight block_size must be set for grouped blockwise scaling")
        if input_scale_spec.block_size[0] != 1 or input_scale_spec.block_size[1] != 128:
            raise ValueError("grouped blockwise scaling only supports (1,128) granularity for input")
        if weight_scale_spec.block_size[0] != 128 or weight_scale_spec.block_size[1] != 128:
            raise ValueError("grouped blockwise scaling only supports (128,128) granularity for weight")
    else:
        raise ValueError("grouped FP8 matmul only supports blockwise scaling")
    if a_scales.dtype != torch.float32:
        raise TypeError("this build executes float32 scales only for the grouped matmul")

    T, K = hidden_states.shape
    E, N, _ = weight.shape
    kb, nb = -(-K // 128), -(-N // 128)
    if a_scales.shape[0] != kb or a_scales.shape[1] < T:
        raise ValueError(f"a_scales shape {tuple(a_scales.shape)} does not cover hidden_states {tuple(hidden_states.shape)}")
    if tuple(b_scales.shape) != (E, nb, kb):
        raise ValueError(f"b_scales shape {tuple(b_scales.shape)} is not {(E, nb, kb)}")
    stats = expert_usage_stats_host
    if stats.is_cuda:
        raise ValueError("expert_usage_stats_host must live on the CPU")
    max_tokens, num_active = int(stats[0]), int(stats[1])
    if expert_start_indices.shape[0] < num_active + 1:
        raise ValueError("expert_start_indices is shorter than num_active_experts + 1")

    _require_gpu(hidden_states, weight, a_scales, b_scales, expert_start_indices, expert_ids)
    hidden_states = hidden_states.contiguous()
    weight = weight.contiguous()
    a_scales = a_scales if a_scales.stride(1) == 1 else a_scales.contiguous()
    b_scales = b_scales.contiguous()
    c = torch.empty((T, N), dtype=out_type, device=hidden_states.device)
    a_ld = a_scales.stride(0) if a_scales.shape[0] > 1 else a_scales.shape[1]
    if out_row_index is not None:
        if out_row_index.dtype != torch.uint32 or tuple(out_row_index.shape) != (T,):
            raise TypeError(f"out_row_index must be a uint32 tensor of shape ({T},)")
        _require_gpu(out_row_index)
        st = _lib.lib().maxfp8_grouped_matmul_dynamic_scaled_fp8_scatter(
            c.data_ptr(), out_row_index.data_ptr(), hidden_states.data_ptr(), weight.data_ptr(), a_scales.data_ptr(),
            b_scales.data_ptr(), expert_start_indices.data_ptr(), expert_ids.data_ptr(), T, N, K, E, max_tokens,
            num_active, a_ld, _DT[out_type], _DT[a_scales.dtype], _ALGOS[algo], _stream(hidden_states))
        _lib.check(st)
        return c
    st = _lib.lib().maxfp8_grouped_matmul_dynamic_scaled_fp8(
        c.data_ptr(), hidden_states.data_ptr(), weight.data_ptr(), a_scales.data_ptr(), b_scales.data_ptr(),
        expert_start_indices.data_ptr(), expert_ids.data_ptr(), T, N, K, E, max_tokens, num_active, a_ld,
        _DT[out_type], _DT[a_scales.dtype], _ALGOS[algo], _stream(hidden_states))
    _lib.check(st)
    return c


def grouped_matmul_rowwise_dynamic_scaled_fp8(
    hidden_states: torch.Tensor,
    weight: torch.Tensor,
    a_scales: torch.Tensor,
    b_scales: torch.Tensor,
    expert_start_indices: torch.Tensor,
    expert_ids: torch.Tensor,
    expert_usage_stats_host: torch.Tensor,
    out_type: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """Grouped (ragged MoE) FP8 matmul with per-token activation scales [total_tokens, 1] and
    per-output-channel weight scales [num_experts, N, 1]:
    out[t, n] = (sum_k a[t, k] * b[expert_ids[g], n, k]) * a_scale[t] * b_scale[expert_ids[g], n]."""
    if hidden_states.dim() != 2:
        raise ValueError(f"expected hidden_states of rank 2 but got {hidden_states.dim()}")
    if weight.dim() != 3:
        raise ValueError(f"expected weight of rank 3 but got {weight.dim()}")
    if weight.shape[2] != hidden_states.shape[1] or weight.shape[0] != expert_ids.shape[0]:
        raise ValueError(f"expected weight of shape [num_experts, N, {hidden_states.shape[1]}] with num_experts = "
                         f"{expert_ids.shape[0]} but got {tuple(weight.shape)}")
    if (hidden_states.dtype != weight.dtype) or (hidden_states.dtype != _FP8):
        raise TypeError(
            f"hidden_states and weight dtypes must be float8_e4m3fn, but got {hidden_states.dtype}, {weight.dtype}")
    if a_scales.dim() != 2 or b_scales.dim() != 3:
        raise ValueError(
            f"expected a_scales of rank 2 and b_scales of rank 3 but got {a_scales.dim()} and {b_scales.dim()}")
    if a_scales.dtype != torch.float32 or b_scales.dtype != torch.float32:
        raise TypeError("a_scales and b_scales dtypes must both be float32 for rowwise / per-token granularity, "
                        f"but got {a_scales.dtype}, {b_scales.dtype}")
    T, K = hidden_states.shape
    E, N, _ = weight.shape
    if a_scales.shape[1] != 1 or a_scales.shape[0] < T:
        raise ValueError(f"expected per-token a_scales of shape [total_tokens, 1] but got {tuple(a_scales.shape)}")
    if tuple(b_scales.shape) != (E, N, 1):
        raise ValueError("expected per-channel b_scales of shape [num_experts, N, 1] matching weight [num_experts, N, K], "
                         f"but got b_scales {tuple(b_scales.shape)} and weight {tuple(weight.shape)}")
    if expert_ids.dtype != torch.int32:
        raise TypeError(f"expert_ids dtype must be int32, but got {expert_ids.dtype}")
    if expert_ids.dim() != 1:
        raise ValueError(f"expected expert_ids of rank 1 but got {expert_ids.dim()}")
    if expert_start_indices.dtype != torch.uint32:
        raise TypeError(f"expert_start_indices dtype must be uint32, but got {expert_start_indices.dtype}")
    if expert_start_indices.dim() != 1:
        raise ValueError(f"expected expert_start_indices of rank 1 but got {expert_start_indices.dim()}")
    if out_type not in (torch.bfloat16, torch.float32):
        raise TypeError(f"out_type {out_type} is not bfloat16 or float32")
    stats = expert_usage_stats_host
    if stats.is_cuda:
        raise ValueError("expert_usage_stats_host must live on the CPU")
    max_tokens, num_active = int(stats[0]), int(stats[1])
    if expert_start_indices.shape[0] < num_active + 1:
        raise ValueError("expert_start_indices is shorter than num_active_experts + 1")
    _require_gpu(hidden_states, weight, a_scales, b_scales, expert_start_indices, expert_ids)
    hidden_states, weight = hidden_states.contiguous(), weight.contiguous()
    a_scales, b_scales = a_scales.contiguous(), b_scales.contiguous()
    c = torch.empty((T, N), dtype=out_type, device=hidden_states.device)
    st = _lib.lib().maxfp8_grouped_matmul_rowwise_dynamic_scaled_fp8(
        c.data_ptr(), hidden_states.data_ptr(), weight.data_ptr(), a_scales.data_ptr(), b_scales.data_ptr(),
        expert_start_indices.data_ptr(), expert_ids.data_ptr(), T, N, K, E, max_tokens, num_active,
        _DT[out_type], _lib.F32, _stream(hidden_states))
    _lib.check(st)
    return c


# ---- utilities exposed for tests and calibration ------------------------------------

def cast_f32_to_e4m3fn(x: torch.Tensor) -> torch.Tensor:
    _require_gpu(x)
    x = x.contiguous().to(torch.float32)
    out = torch.empty(x.shape, dtype=_FP8, device=x.device)
    _lib.check(_lib.lib().maxfp8_cast_f32_to_e4m3fn(out.data_ptr(), x.data_ptr(), x.numel(), _stream(x)))
    return out


def cast_f32_to_bf16(x: torch.Tensor) -> torch.Tensor:
    _require_gpu(x)
    x = x.contiguous().to(torch.float32)
    out = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    _lib.check(_lib.lib().maxfp8_cast_f32_to_bf16(out.data_ptr(), x.data_ptr(), x.numel(), _stream(x)))
    return out


def cast_e4m3fn_to_f32(x: torch.Tensor) -> torch.Tensor:
    _require_gpu(x)
    x = x.contiguous()
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().maxfp8_cast_e4m3fn_to_f32(out.data_ptr(), x.data_ptr(), x.numel(), _stream(x)))
    return out


def copy_bytes(dst: torch.Tensor, src: torch.Tensor) -> None:
    _require_gpu(dst, src)
    n = src.numel() * src.element_size()
    _lib.check(_lib.lib().maxfp8_copy_bytes(dst.data_ptr(), src.data_ptr(), n, _stream(src)))
