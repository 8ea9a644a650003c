"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports every
symbol include/maxfp8.h declares, and the Python wrappers reproduce the reference
wrappers' shape rules and exceptions (max/python/max/nn/kernels.py:6327-6487, 6876-7078;
max/python/max/nn/quant_config.py:313-351; max/python/max/nn/linear.py:217-250)."""
import ctypes
import os
import re

import pytest
import torch

import modular_amd as mx
from modular_amd import _lib, kernels
from modular_amd.linear import infer_weight_scale_shape
from modular_amd.quant_config import (InputScaleSpec, QuantConfig, ScaleGranularity, ScaleOrigin,
                                      WeightScaleSpec)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FP8 = torch.float8_e4m3fn
BLK = mx.blockwise_fp8_config()
ROW = mx.rowwise_fp8_config()


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "maxfp8.h")).read()
    declared = set(re.findall(r"\b(maxfp8_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS)
    L = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(L, name), name
    assert b"gfx950" in _lib.lib().maxfp8_version()


def test_status_to_exception_mapping():
    with pytest.raises(TypeError):
        _lib.check(_lib.ERR_DTYPE)
    for code in (_lib.ERR_SHAPE, _lib.ERR_ALIGN, _lib.ERR_GRANULARITY, _lib.ERR_NULL):
        with pytest.raises(ValueError):
            _lib.check(code)
    with pytest.raises(RuntimeError):
        _lib.check(_lib.ERR_LAUNCH)
    _lib.check(_lib.OK)


def test_c_abi_argument_errors_need_no_gpu():
    L = _lib.lib()
    # zero-sized work is a silent no-op
    assert L.maxfp8_quantize_dynamic_scaled_fp8(None, None, None, 0, 128, 128, 128, 128, 0, 0, 2, 1200.0, None) == 0
    assert L.maxfp8_matmul_dynamic_scaled_fp8(None, None, None, None, None, 0, 8, 128, 128, 128, 8, 3, 3, 1, 128, 128,
                                              4, 1, 0, 2, 0, None, 0, None) == 0
    assert L.maxfp8_grouped_matmul_dynamic_scaled_fp8(None, None, None, None, None, None, None, 8, 128, 128, 2, 0, 2,
                                                      8, 0, 2, 0, None) == 0
    # bad arguments are reported before anything is launched
    assert L.maxfp8_quantize_dynamic_scaled_fp8(1, 1, 1, 4, 260, 260, 260, 128, 4, 0, 2, 1200.0, None) == _lib.ERR_SHAPE
    assert "must divide K" in _lib.last_error()
    assert L.maxfp8_quantize_dynamic_scaled_fp8(1, 1, 1, 4, 256, 256, 256, 128, 4, 3, 2, 1200.0, None) == _lib.ERR_DTYPE
    assert L.maxfp8_matmul_dynamic_scaled_fp8(1, 1, 1, 1, 1, 4, 8, 128, 128, 128, 8, 3, 1, 1, 128, 128,
                                              4, 1, 0, 2, 0, None, 0, None) == _lib.ERR_GRANULARITY
    assert "unsupported FP8 scaling granularity" in _lib.last_error()
    assert L.maxfp8_matmul_dynamic_scaled_fp8(1, 1, 1, 1, 1, 4, 8, 128, 128, 128, 8, 3, 3, 1, 128, 128,
                                              4, 1, 0, 0, 0, None, 0, None) == _lib.ERR_DTYPE


def test_row_strides_beyond_the_tile_offsets_are_refused():
    """The MFMA kernels address a tile through 32-bit offsets with the top bit as the out-of-range mark: a strided
    view whose 256 rows span 2^31 bytes must not reach them (it would read zeros for rows that exist)."""
    L = _lib.lib()
    big = (1 << 23) + 16          # 256 * big >= 2^31
    for algo in (_lib.ALGO_TILED, _lib.ALGO_SKINNY):
        for lda, ldb in ((big, 128), (128, big)):
            st = L.maxfp8_matmul_dynamic_scaled_fp8(16, 16, 16, 16, 16, 4, 8, 128, lda, ldb, 8, 2, 1, -1, -1, -1,
                                                    4, 1, 0, 2, algo, None, 0, None)
            assert st == _lib.ERR_ALIGN and "2^31" in _lib.last_error()
    # block scaling: the scales of all slabs of a tile, ceil(K / 128) * a_scales_ld floats, share one offset range
    st = L.maxfp8_matmul_dynamic_scaled_fp8(16, 16, 16, 16, 16, 4, 128, 128 * 1024, 128 * 1024, 128 * 1024, 128, 3, 3,
                                            1, 128, 128, 1 << 20, 1024, 0, 2, _lib.ALGO_TILED, None, 0, None)
    assert st == _lib.ERR_ALIGN
    st = L.maxfp8_grouped_matmul_rowwise_dynamic_scaled_fp8(16, 16, 16, 16, 16, 16, 16, 8, 128, 1 << 23, 2, 8, 2,
                                                            0, 2, None)
    assert st == _lib.ERR_SHAPE and "32-bit" in _lib.last_error()


def test_quantize_geometry_rules():
    g = kernels.quantize_output_geometry
    assert g(81, 2048, BLK.input_scale, BLK.weight_scale, -1, torch.float32) == (128, 84)   # pad to 16 bytes
    assert g(81, 2048, BLK.input_scale, BLK.weight_scale, -1, torch.bfloat16) == (128, 88)
    assert g(64, 4096, BLK.input_scale, BLK.weight_scale, -1, torch.float32) == (128, 64)
    assert g(5, 8192, ROW.input_scale, ROW.weight_scale, -1, torch.float32) == (8192, 5)    # per token, no padding
    assert g(5, 8192, ROW.input_scale, ROW.weight_scale, 256, torch.float32) == (256, 5)
    with pytest.raises(ValueError, match="both input and weight must be blockwise"):
        g(4, 256, BLK.input_scale, ROW.weight_scale, -1, torch.float32)


def test_quantize_wrapper_errors():
    x = torch.zeros((2, 3, 256), dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="rank 2"):
        mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale)
    with pytest.raises(ValueError, match="out_type"):
        mx.quantize_dynamic_scaled_float8(x[0], BLK.input_scale, BLK.weight_scale, out_type=torch.float8_e5m2)
    with pytest.raises(RuntimeError, match="GPU only"):
        mx.quantize_dynamic_scaled_float8(x[0], BLK.input_scale, BLK.weight_scale, scales_type=torch.float32)


def _mm_args(M=4, N=256, K=256, block=True):
    a = torch.zeros((M, K), dtype=torch.uint8).view(FP8)
    b = torch.zeros((N, K), dtype=torch.uint8).view(FP8)
    if block:
        return a, b, torch.ones((K // 128, M)), torch.ones((N // 128, K // 128))
    return a, b, torch.ones((1, M)), torch.ones((N, 1))


def test_matmul_wrapper_errors():
    a, b, sa, sb = _mm_args()
    with pytest.raises(ValueError, match="rank 2"):
        mx.dynamic_scaled_matmul(a[0], b, sa, sb, BLK.input_scale, BLK.weight_scale)
    with pytest.raises(ValueError, match="second dimension"):
        mx.dynamic_scaled_matmul(a[:, :128], b, sa, sb, BLK.input_scale, BLK.weight_scale)
    with pytest.raises(TypeError, match="must be float32"):
        mx.dynamic_scaled_matmul(a, b, sa.bfloat16(), sb.bfloat16(), BLK.input_scale, BLK.weight_scale)
    with pytest.raises(ValueError, match="same shape on the K dimension"):
        mx.dynamic_scaled_matmul(a, b, sa[:1], sb, BLK.input_scale, BLK.weight_scale)
    with pytest.raises(ValueError, match="block size must be set"):
        mx.dynamic_scaled_matmul(a, b, sa, sb, BLK.input_scale, ROW.weight_scale)
    with pytest.raises(ValueError, match="both input and weight must be blockwise"):
        mx.dynamic_scaled_matmul(a, b, sa, sb, BLK.input_scale,
                                 WeightScaleSpec(ScaleGranularity.ROWWISE, torch.float32, block_size=(128, 128)))
    with pytest.raises(ValueError, match="unsupported FP8 scaling granularity"):
        mx.dynamic_scaled_matmul(a, b, sa, sb, ROW.input_scale,
                                 WeightScaleSpec(ScaleGranularity.TENSOR, torch.float32))
    a, b, sa, sb = _mm_args(block=False)
    with pytest.raises(ValueError, match="per-token"):
        mx.dynamic_scaled_matmul(a, b, sa.t().contiguous(), sb, ROW.input_scale, ROW.weight_scale)
    with pytest.raises(ValueError, match="channel-wise"):
        mx.dynamic_scaled_matmul(a, b, sa, sb.t().contiguous(), ROW.input_scale, ROW.weight_scale)
    with pytest.raises(TypeError, match="must match"):
        mx.dynamic_scaled_matmul(a, b, sa, sb.bfloat16(), ROW.input_scale, ROW.weight_scale)
    with pytest.raises(RuntimeError, match="GPU only"):
        mx.dynamic_scaled_matmul(a, b, sa, sb, ROW.input_scale, ROW.weight_scale)


def test_grouped_wrapper_errors():
    T, E, N, K = 8, 2, 128, 256
    h = torch.zeros((T, K), dtype=torch.uint8).view(FP8)
    w = torch.zeros((E, N, K), dtype=torch.uint8).view(FP8)
    sa, sb = torch.ones((2, 8)), torch.ones((E, 1, 2))
    off = torch.tensor([0, 4, 8], dtype=torch.int64).to(torch.uint32)
    ids = torch.arange(E, dtype=torch.int32)
    stats = torch.tensor([4, 2], dtype=torch.int64).to(torch.uint32)
    call = lambda **kw: mx.grouped_dynamic_scaled_fp8_matmul(
        kw.get("h", h), kw.get("w", w), kw.get("sa", sa), kw.get("sb", sb), kw.get("off", off),
        kw.get("ids", ids), stats, kw.get("ispec", BLK.input_scale), kw.get("wspec", BLK.weight_scale))
    with pytest.raises(ValueError, match="weight of rank 3"):
        call(w=w[0])
    with pytest.raises(ValueError, match="hidden_states of rank 2"):
        call(h=h[0])
    with pytest.raises(ValueError, match="num_experts"):
        call(ids=torch.arange(3, dtype=torch.int32))
    with pytest.raises(TypeError, match="float8_e4m3fn"):
        call(h=h.view(torch.uint8))
    with pytest.raises(TypeError, match="float32 or bfloat16"):
        call(sa=sa.half(), sb=sb.half())
    with pytest.raises(TypeError, match="expert_ids dtype must be int32"):
        call(ids=ids.long())
    with pytest.raises(TypeError, match="expert_start_indices dtype must be uint32"):
        call(off=off.to(torch.int32))
    with pytest.raises(ValueError, match="a_scales of rank 2 and b_scales of rank 3"):
        call(sb=sb[0])
    with pytest.raises(ValueError, match=r"\(1,128\) granularity"):
        call(ispec=InputScaleSpec(ScaleGranularity.BLOCK, ScaleOrigin.DYNAMIC, torch.float32, block_size=(1, 64)))
    with pytest.raises(ValueError, match=r"\(128,128\) granularity"):
        call(wspec=WeightScaleSpec(ScaleGranularity.BLOCK, torch.float32, block_size=(64, 128)))
    with pytest.raises(ValueError, match="only supports blockwise"):
        call(ispec=ROW.input_scale, wspec=ROW.weight_scale)
    with pytest.raises(RuntimeError, match="GPU only"):
        call()


def test_quant_config_properties():
    assert BLK.scales_granularity_mnk == (1, 128, 128)
    assert ROW.scales_granularity_mnk == (1, 1, -1)
    t = QuantConfig(InputScaleSpec(ScaleGranularity.TENSOR, ScaleOrigin.DYNAMIC, torch.float32),
                    WeightScaleSpec(ScaleGranularity.TENSOR, torch.float32))
    assert t.scales_granularity_mnk == (-1, -1, -1)
    assert BLK.is_dynamic and not BLK.is_static
    assert BLK.quantized_scales_shape((81, 2048)) == (16, 81)
    with pytest.raises(ValueError):
        ROW.quantized_scales_shape((4, 256))
    with pytest.raises(ValueError, match="block_size must be specified"):
        WeightScaleSpec(ScaleGranularity.BLOCK, torch.float32)
    assert str(ScaleGranularity.COLWISE) == "colwise" and ScaleOrigin.DYNAMIC.is_dynamic


def test_linear_weight_scale_shapes():
    assert infer_weight_scale_shape(4096, 7168, ROW) == (4096, 1)
    assert infer_weight_scale_shape(576, 7168, BLK) == (5, 56)
    t = QuantConfig(InputScaleSpec(ScaleGranularity.TENSOR, ScaleOrigin.DYNAMIC, torch.float32),
                    WeightScaleSpec(ScaleGranularity.TENSOR, torch.float32))
    assert infer_weight_scale_shape(8, 8, t) == ()
    lin = mx.Linear(256, 384, BLK)
    assert lin.weight.shape == (384, 256) and lin.weight.dtype == FP8 and lin.weight_scale.shape == (3, 2)


def test_product_package_does_not_touch_the_oracle():
    pkg = os.path.join(ROOT, "modular_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in src and "from oracle" not in src and "maxfp8_oracle" not in src, f


def test_mlp_stacks_gate_and_up_in_one_buffer():
    """The gate / up weights of `MLP` are views of one stacked buffer (so the two projections run as one
    matmul without a per-call concatenation); checkpoints name the three projections only, and moving the
    module keeps the views tied."""
    import torch
    import modular_amd as mx

    m = mx.MLP(256, 512, mx.blockwise_fp8_config())
    # the one-kernel activation + quantisation is an opt-in: its recipe is not the one down_proj applies
    assert m._one_matmul and m._silu_kernel() and not m._fused()
    assert mx.MLP(256, 512, mx.blockwise_fp8_config(), fuse_activation_quant=True)._fused()
    assert sorted(m.state_dict()) == ["down_proj.weight", "down_proj.weight_scale", "gate_proj.weight",
                                      "gate_proj.weight_scale", "up_proj.weight", "up_proj.weight_scale"]
    new = {k: (torch.randint(0, 100, v.shape, dtype=torch.uint8).view(v.dtype) if v.dtype == torch.float8_e4m3fn
               else torch.rand(v.shape)) for k, v in m.state_dict().items()}
    m.load_state_dict(new)
    assert torch.equal(m.gate_up_weight[512:].view(torch.uint8), new["up_proj.weight"].view(torch.uint8))
    assert torch.equal(m.gate_up_weight_scale[:4], new["gate_proj.weight_scale"])
    m._apply(lambda t: t.clone())  # what .to(device) does to every buffer
    assert m.gate_proj.weight.data_ptr() == m.gate_up_weight.data_ptr()
    assert m.up_proj.weight_scale.data_ptr() == m.gate_up_weight_scale[4:].data_ptr()
    assert torch.equal(m.gate_up_weight[:512].view(torch.uint8), new["gate_proj.weight"].view(torch.uint8))
    # per-token scales stack as well; static or per-tensor scales, bias or another activation take the unfused route
    assert mx.MLP(256, 512, mx.rowwise_fp8_config())._one_matmul
    assert not mx.MLP(256, 512, mx.blockwise_fp8_config(), has_bias=True, fuse_activation_quant=True)._fused()
    assert not mx.MLP(256, 512, mx.blockwise_fp8_config(), activation_function="gelu", fuse_activation_quant=True)._fused()
    assert not mx.MLP(256, 512, mx.rowwise_fp8_config(), fuse_activation_quant=True)._fused()


def test_quantized_grouped_matmul_and_strategy_argument_rules():
    """The layer above the grouped op (quant_ops.py:880-1007, moe/quant_strategy.py:114-215): format and rank
    checks happen before anything touches the GPU, and the storage-layout transposition is made once per tensor."""
    import dataclasses

    from modular_amd import quant_ops

    x = torch.zeros((4, 256), dtype=torch.bfloat16)
    w = torch.zeros((2, 256, 128), dtype=torch.uint8).view(FP8)       # storage layout [E, K, N]
    ws = torch.ones((2, 2, 1))
    off = torch.tensor([0, 2, 4], dtype=torch.int64).to(torch.uint32)
    ids = torch.tensor([0, 1], dtype=torch.int32)
    stats = torch.tensor([2, 2], dtype=torch.int64).to(torch.uint32)
    bad = dataclasses.replace(BLK, format="mxfp4")
    with pytest.raises(ValueError, match="Unsupported quantization format for grouped matmul"):
        quant_ops.quantized_grouped_matmul(x, w, ws, off, ids, stats, bad)
    with pytest.raises(ValueError, match="rank 3"):
        quant_ops.quantized_grouped_matmul(x, w[0], ws, off, ids, stats, BLK)
    # [E, K, N] -> [E, N, K], contiguous, kept per storage tensor until it is written in place
    quant_ops._K_INNERMOST.clear()
    src = torch.arange(2 * 3 * 5, dtype=torch.uint8).reshape(2, 3, 5).view(FP8)
    t1 = quant_ops._k_innermost(src)
    assert tuple(t1.shape) == (2, 5, 3) and t1.is_contiguous()
    assert torch.equal(t1.view(torch.uint8), src.view(torch.uint8).transpose(1, 2))
    assert quant_ops._k_innermost(src) is t1
    src.view(torch.uint8).add_(1)
    t2 = quant_ops._k_innermost(src)
    assert t2 is not t1 and torch.equal(t2.view(torch.uint8), src.view(torch.uint8).transpose(1, 2))
    assert len(quant_ops._K_INNERMOST) == 1, "an in-place write replaces the tensor's entry"
    # every live storage tensor keeps its copy -- a model has more stacked weights than any fixed number of entries -- and
    # an entry goes when its tensor goes
    many = [torch.arange(2 * 3 * 5, dtype=torch.uint8).reshape(2, 3, 5) + i for i in range(40)]
    copies = [quant_ops._k_innermost(t) for t in many]
    for _ in range(3):
        assert all(quant_ops._k_innermost(t) is c for t, c in zip(many, copies)), "no tensor is transposed twice"
    assert len(quant_ops._K_INNERMOST) == 41
    del many, copies
    import gc
    gc.collect()
    assert len(quant_ops._K_INNERMOST) == 1
    del src
    gc.collect()
    assert len(quant_ops._K_INNERMOST) == 0
    # a CPU tensor never reaches a kernel
    with pytest.raises(RuntimeError, match="GPU only"):
        quant_ops.quantized_grouped_matmul(x, w, torch.ones((2, 2, 1)), off, ids, stats, BLK)
    st = mx.Fp8Strategy(BLK)
    assert st.dtype == FP8 and st.config is BLK
    a, b = st.prepare_weight_scales(ws, off, None)
    assert a is ws and b is off
    with pytest.raises(RuntimeError, match="GPU only"):
        st.quantize(x, 128)
