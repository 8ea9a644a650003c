"""GPU parity of the dynamic per-tensor quantiser: bytes and scales bit-exact with the oracle on
the reference test's shapes (test_scaled_fp8_quantization.mojo:670-705) and on BASELINE-sized
activations; every element of the [1, M] scales output carries the tensor's scale."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import synth
from modular_amd.quant_config import InputScaleSpec, ScaleGranularity, ScaleOrigin, WeightScaleSpec
from util import bf16_bits, f32_np, fp8_bytes

pytestmark = pytest.mark.gpu
NT = oracle.default_threads()
IN = InputScaleSpec(ScaleGranularity.TENSOR, ScaleOrigin.DYNAMIC, torch.float32)
WT = WeightScaleSpec(ScaleGranularity.TENSOR, torch.float32)
ODT = {torch.bfloat16: oracle.BF16, torch.float16: oracle.F16, torch.float32: oracle.F32}


def check(x, dev, scales_type, **kw):
    M, K = x.shape
    q, s = mx.quantize_tensor_dynamic_scaled_float8(x.to(dev), IN, WT, scales_type=scales_type, **kw)
    torch.cuda.synchronize()
    src = x.numpy() if x.dtype == torch.float32 else bf16_bits(x) if x.dtype == torch.bfloat16 else \
        x.view(torch.int16).numpy().view(np.uint16)
    q_ref, s_ref = oracle.quantize_tensor_dynamic(src, in_dtype=ODT[x.dtype], scales_dtype=ODT[scales_type], threads=NT,
                                                  scale_ub=kw.get("scale_ub", 1200.0))
    assert s.shape == (1, M)
    if scales_type == torch.bfloat16:
        assert np.array_equal(bf16_bits(s), s_ref), "scales differ"
    else:
        assert np.array_equal(f32_np(s).view(np.uint32), s_ref.view(np.uint32)), "scales differ"
    assert np.array_equal(fp8_bytes(q), q_ref), "quantized bytes differ"


@pytest.mark.parametrize("M,K,dtype", [(1, 1024, torch.bfloat16), (1, 16384, torch.bfloat16), (4, 16384, torch.bfloat16),
                                       (4, 576, torch.float32), (2, 260, torch.bfloat16), (2, 264, torch.bfloat16),
                                       (5000, 512, torch.bfloat16), (33, 1000, torch.float16)])
def test_reference_shapes(dev, M, K, dtype):
    g = torch.Generator().manual_seed(M * 131 + K)
    x = (torch.rand((M, K), generator=g) * 2 - 1).to(dtype)
    check(x, dev, torch.bfloat16 if dtype == torch.bfloat16 else torch.float32)
    check(x, dev, torch.float32)


def test_activation_sized_with_outliers(dev):
    x = synth.activations(4096, 7168, seed=3)
    check(x, dev, torch.float32)
    x[1234, 77] = 3000.0          # above scale_ub: the scale saturates at 1200 / 448, the element at 448
    check(x, dev, torch.float32)
    check(x, dev, torch.float32, scale_ub=5.0)


def test_strided_rows_zero_and_near_zero(dev):
    wide = torch.randn((16, 1024), generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    q, s = mx.quantize_tensor_dynamic_scaled_float8(wide.to(dev)[:, 256:768], IN, WT, scales_type=torch.float32)
    q_ref, s_ref = oracle.quantize_tensor_dynamic(bf16_bits(wide[:, 256:768].contiguous()))
    assert np.array_equal(fp8_bytes(q), q_ref) and np.array_equal(f32_np(s), s_ref)
    z = torch.zeros((3, 128), dtype=torch.float32)
    check(z, dev, torch.float32)
    z[1, 5] = 1e-38
    z[2, 7] = -1e-39
    check(z, dev, torch.float32)


def test_errors_and_empty(dev):
    x = torch.zeros((4, 128), dtype=torch.bfloat16, device=dev)
    blk = mx.blockwise_fp8_config()
    with pytest.raises(ValueError, match="tensor scaled"):
        mx.quantize_tensor_dynamic_scaled_float8(x, blk.input_scale, blk.weight_scale)
    with pytest.raises(ValueError, match="should be -1"):
        mx.quantize_tensor_dynamic_scaled_float8(x, IN, WT, group_size_or_per_token=128)
    with pytest.raises(ValueError, match="rank 2"):
        mx.quantize_tensor_dynamic_scaled_float8(x[0], IN, WT)
    q, s = mx.quantize_tensor_dynamic_scaled_float8(x[:0], IN, WT)
    assert q.shape == (0, 128) and s.shape == (1, 0)
