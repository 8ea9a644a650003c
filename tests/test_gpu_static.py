"""GPU parity of the static per-tensor FP8 flavour: quantize_static_scaled_float8 bit-exact with
the oracle, matmul_static_scaled_float8 against float64 (the product of the two scales is formed
first and applied once), and both static branches of matmul_float8."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import synth
from modular_amd.quant_config import InputScaleSpec, QuantConfig, QuantFormat, ScaleGranularity, ScaleOrigin, WeightScaleSpec
from util import fp8_bytes

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("M,K", [(64, 4096), (7, 1000), (1, 8), (300, 260), (2048, 4096)])
@pytest.mark.parametrize("scale", [0.02, 1.0, 3.7e-3])
def test_quantize_static_bit_exact(dev, M, K, scale):
    x = synth.activations(M, K, seed=M + K)
    q = mx.quantize_static_scaled_float8(x.to(dev), torch.tensor([scale]))
    s32 = float(np.float32(scale))
    assert np.array_equal(fp8_bytes(q), oracle.quantize_static(_bits(x), s32))


@pytest.mark.parametrize("dtype,odt", [(torch.float16, oracle.F16), (torch.float32, oracle.F32)])
def test_quantize_static_other_dtypes_and_strides(dev, dtype, odt):
    x = (torch.randn((33, 520), generator=torch.Generator().manual_seed(1)) * 4).to(dtype)
    xin = x.numpy() if dtype == torch.float32 else _bits(x)
    q = mx.quantize_static_scaled_float8(x.to(dev), torch.tensor(0.05))
    assert np.array_equal(fp8_bytes(q), oracle.quantize_static(xin, float(np.float32(0.05)), in_dtype=odt))
    wide = torch.randn((16, 1024)).to(torch.bfloat16)
    q = mx.quantize_static_scaled_float8(wide.to(dev)[:, 256:768], torch.tensor(0.1))
    assert np.array_equal(fp8_bytes(q), oracle.quantize_static(_bits(wide[:, 256:768].contiguous()), float(np.float32(0.1))))


def test_quantize_static_errors(dev):
    x = torch.zeros((4, 8), dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError, match="expected scale to be a scalar"):
        mx.quantize_static_scaled_float8(x, torch.ones(2))
    with pytest.raises(ValueError, match="expected scale to be on CPU"):
        mx.quantize_static_scaled_float8(x, torch.ones(1, device=dev))
    with pytest.raises(ValueError, match="expected input rank to be 2"):
        mx.quantize_static_scaled_float8(x[0], torch.ones(1))
    with pytest.raises(ValueError, match="expected input dtype"):
        mx.quantize_static_scaled_float8(x.to(torch.int32), torch.ones(1))


@pytest.mark.parametrize("M,N,K", [(5, 200, 512), (130, 264, 1024), (2048, 512, 256)])
def test_matmul_static(dev, M, N, K):
    rng = np.random.default_rng(M + N)
    ai, bi = rng.integers(-4, 5, (M, K)), rng.integers(-4, 5, (N, K))
    a = torch.from_numpy(oracle.e4m3fn_encode(ai.astype(np.float32))).view(torch.float8_e4m3fn)
    b = torch.from_numpy(oracle.e4m3fn_encode(bi.astype(np.float32))).view(torch.float8_e4m3fn)
    sa, sb = torch.tensor([0.013]), torch.tensor(0.0071)
    y = mx.matmul_static_scaled_float8(a.to(dev), b.to(dev), sa, sb)
    assert y.dtype == torch.bfloat16
    # integer operands: the accumulator is exact, so the result is exactly bf16(acc * (sa * sb))
    prod = np.float32(np.float32(0.013) * np.float32(0.0071))
    want = torch.from_numpy(((ai @ bi.T).astype(np.float32) * prod).astype(np.float32)).to(torch.bfloat16)
    assert torch.equal(y.cpu(), want)


def _static_cfg(weight_gran):
    return QuantConfig(InputScaleSpec(ScaleGranularity.TENSOR, ScaleOrigin.STATIC, torch.float32),
                       WeightScaleSpec(weight_gran, torch.float32))


def test_matmul_float8_static_branches(dev):
    M, K, N = 48, 1024, 384
    x = synth.activations(M, K, seed=3, outlier_frac=0.0)
    w = synth.weights_f32(N, K, seed=4)
    w_scale = float(w.abs().max()) / 448.0
    wq = (w / w_scale).clamp(-448, 448).to(torch.float8_e4m3fn)
    in_scale = float(x.float().abs().max()) / 448.0
    ref = x.float() @ w.T
    # scalar weight scale -> matmul_static_scaled_float8
    y = mx.matmul_float8(x.to(dev), wq.to(dev), torch.tensor(w_scale), torch.tensor(in_scale), _static_cfg(ScaleGranularity.TENSOR))
    assert float((y.float().cpu() - ref).abs().max()) <= 0.06 * float(ref.abs().max())
    # fused-QKV style: tensor granularity with the weight scale broadcast to [N, 1]
    y2 = mx.matmul_float8(x.to(dev), wq.to(dev), torch.full((N, 1), w_scale), torch.tensor(in_scale),
                          _static_cfg(ScaleGranularity.TENSOR))
    assert float((y2.float().cpu() - ref).abs().max()) <= 0.06 * float(ref.abs().max())
    # same quantised operands either way: the two results differ only by the order of the scale products
    assert float((y.float() - y2.float()).abs().max()) <= 2.0 ** -7 * float(y.float().abs().max())


def test_linear_with_static_input_scale(dev):
    M, K, N = 20, 512, 256
    lin = mx.Linear(K, N, _static_cfg(ScaleGranularity.TENSOR), device=dev)
    assert lin.input_scale is not None and lin.input_scale.device.type == "cpu" and tuple(lin.input_scale.shape) == ()
    x = synth.activations(M, K, seed=9, outlier_frac=0.0)
    w = synth.weights_f32(N, K, seed=10)
    w_scale = float(w.abs().max()) / 448.0
    lin.weight.copy_((w / w_scale).clamp(-448, 448).to(torch.float8_e4m3fn).to(dev))
    lin.weight_scale.fill_(w_scale)
    lin.input_scale.fill_(float(x.float().abs().max()) / 448.0)
    y = lin(x.to(dev).reshape(4, 5, K))
    ref = (x.float() @ w.T).reshape(4, 5, N)
    assert tuple(y.shape) == (4, 5, N)
    assert float((y.float().cpu() - ref).abs().max()) <= 0.06 * float(ref.abs().max())


def test_static_linear_loads_its_scales_from_a_state_dict(dev):
    """A checkpoint's `weight`, `weight_scale` and `input_scale` go in through load_state_dict and the layer runs:
    the two scalars stay on the CPU (the static ops take them from the host) wherever the module is moved."""
    M, K, N = 24, 512, 256
    x = synth.activations(M, K, seed=11, outlier_frac=0.0)
    w = synth.weights_f32(N, K, seed=12)
    w_scale = float(w.abs().max()) / 448.0
    in_scale = float(x.float().abs().max()) / 448.0
    state = {"weight": (w / w_scale).clamp(-448, 448).to(torch.float8_e4m3fn),
             "weight_scale": torch.tensor(w_scale), "input_scale": torch.tensor(in_scale)}
    lin = mx.Linear(K, N, _static_cfg(ScaleGranularity.TENSOR), device=dev)
    assert set(lin.state_dict()) == {"weight", "weight_scale", "input_scale"}
    lin.load_state_dict(state, strict=True)
    lin = lin.to(dev)
    assert lin.weight.is_cuda and lin.weight_scale.device.type == "cpu" and lin.input_scale.device.type == "cpu"
    assert float(lin.input_scale) == float(torch.tensor(in_scale)) and float(lin.weight_scale) == float(torch.tensor(w_scale))
    y = lin(x.to(dev))
    ref = x.float() @ w.T
    assert float((y.float().cpu() - ref).abs().max()) <= 0.06 * float(ref.abs().max())
    # the same numbers as the op called by hand
    want = mx.matmul_float8(x.to(dev), state["weight"].to(dev), state["weight_scale"], state["input_scale"],
                            _static_cfg(ScaleGranularity.TENSOR))
    assert torch.equal(y, want)
