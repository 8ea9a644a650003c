"""GPU parity of the fused RMSNorm + per-row FP8 quantisation.  On the reference test's data and
shapes the bytes must be equal (as test_rms_norm_fused_fp8.mojo:243-255 demands of the reference
kernel); on random data the sum of squares is reduced in an order of the kernel's own (the
reference does not fix one; the oracle uses the exactly rounded sum), so scales may differ in the
last bits and a byte may land on the neighbouring code: the bounds are stated in the tests."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from rmsnorm_cases import EPS, SHAPES, bits, pattern_input
from util import fp8_bytes

pytestmark = pytest.mark.gpu
NT = oracle.default_threads()


@pytest.mark.parametrize("shape", SHAPES + [(2, 2, 1024), (2, 3, 4, 256)])
@pytest.mark.parametrize("weight_offset,scale_ub", [(0.0, 448.0), (1.0, 448.0), (0.0, 1200.0)])
def test_reference_test_data(dev, shape, weight_offset, scale_ub):
    x, g = pattern_input(int(np.prod(shape[:-1])), shape[-1])
    want_q, want_s = oracle.rms_norm_fused_quantize(bits(x), bits(g), EPS, weight_offset, scale_ub=scale_ub, threads=NT)
    q, s = mx.rms_norm_fused_quantize_dynamic_scaled_fp8(x.reshape(shape).to(dev), g.to(dev), EPS, weight_offset, scale_ub)
    torch.cuda.synchronize()
    assert tuple(q.shape) == tuple(shape) and tuple(s.shape) == (1, x.shape[0])
    assert np.array_equal(fp8_bytes(q).reshape(want_q.shape), want_q)
    # (the reference test compares the bytes only; the scale carries the summation order of sum x^2)
    _check_scales(s.cpu().numpy(), want_s, x, g, EPS, weight_offset, scale_ub)


def _check_scales(got, oracle_scales, x, g, eps, weight_offset, scale_ub):
    """Within 4 ulp of the scale computed in float64 and of the oracle's."""
    idt = {torch.bfloat16: oracle.BF16, torch.float16: oracle.F16, torch.float32: oracle.F32}[x.dtype]
    xd = x.double().numpy()
    gd = g.double().numpy() + oracle.round_to_dtype(weight_offset, idt)
    inv = 1.0 / np.sqrt((xd * xd).mean(-1) + oracle.round_to_dtype(eps, idt))
    exact = np.minimum(np.abs(xd * gd).max(-1) * inv, scale_ub) / 448.0
    assert np.allclose(got[0], exact, rtol=4 * 2.0 ** -23, atol=0)
    assert np.allclose(got, oracle_scales, rtol=4 * 2.0 ** -23, atol=0)


def _compare_random(dev, x, g, eps, weight_offset, scales_type=torch.float32, scale_ub=1200.0):
    sd = oracle.F32 if scales_type == torch.float32 else oracle.BF16
    idt = {torch.bfloat16: oracle.BF16, torch.float16: oracle.F16, torch.float32: oracle.F32}[x.dtype]
    xin = x.numpy() if x.dtype == torch.float32 else bits(x)
    gin = g.numpy() if g.dtype == torch.float32 else bits(g)
    want_q, want_s = oracle.rms_norm_fused_quantize(xin, gin, eps, weight_offset, in_dtype=idt, scales_dtype=sd,
                                                    scale_ub=scale_ub, threads=NT)
    q, s = mx.rms_norm_fused_quantize_dynamic_scaled_fp8(x.to(dev), g.to(dev), eps, weight_offset, scale_ub,
                                                         scales_type=scales_type)
    torch.cuda.synchronize()
    got_q = fp8_bytes(q)
    if scales_type == torch.float32:
        _check_scales(s.cpu().numpy(), want_s, x, g, eps, weight_offset, scale_ub)
    else:
        gs = s.cpu().view(torch.int16).numpy().view(np.uint16).astype(np.int32)
        assert np.max(np.abs(gs - want_s.astype(np.int32))) <= 1
    dec = oracle.e4m3fn_decode_table()
    diff = got_q != want_q
    # a differing byte is the neighbouring code (a value within an ulp of a rounding boundary), and rare
    assert diff.mean() <= 2e-3, diff.mean()
    if diff.any():
        a, b = dec[got_q[diff]], dec[want_q[diff]]
        assert np.all(np.abs(a - b) <= np.maximum(np.abs(a), np.abs(b)) * 0.126 + 2.0 ** -9)


@pytest.mark.parametrize("rows,K", [(64, 4096), (33, 7168), (5, 1000), (3, 264), (4, 40000), (2048, 4096)])
def test_random_bf16(dev, rows, K):
    gen = torch.Generator().manual_seed(rows + K)
    x = (torch.randn((rows, K), generator=gen) * 1.7).to(torch.bfloat16)
    g = (1.0 + 0.2 * torch.randn(K, generator=gen)).to(torch.bfloat16)
    _compare_random(dev, x, g, 1e-6, 0.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("scales_type", [torch.float32, torch.bfloat16])
def test_other_dtypes(dev, dtype, scales_type):
    gen = torch.Generator().manual_seed(7)
    x = torch.randn((9, 1536), generator=gen).to(dtype)
    g = (0.5 + torch.rand(1536, generator=gen)).to(dtype)
    _compare_random(dev, x, g, 1e-5, 1.0, scales_type=scales_type)


def test_edges(dev):
    z = torch.zeros((3, 256), dtype=torch.bfloat16, device=dev)
    g = torch.ones(256, dtype=torch.bfloat16, device=dev)
    q, s = mx.rms_norm_fused_quantize_dynamic_scaled_fp8(z, g, EPS)
    assert not fp8_bytes(q).any() and not s.cpu().numpy().any()
    q, s = mx.rms_norm_fused_quantize_dynamic_scaled_fp8(z[:0], g, EPS)
    assert tuple(q.shape) == (0, 256) and tuple(s.shape) == (1, 0)
    with pytest.raises(TypeError):
        mx.rms_norm_fused_quantize_dynamic_scaled_fp8(z, g.float(), EPS)
    with pytest.raises(ValueError):
        mx.rms_norm_fused_quantize_dynamic_scaled_fp8(z, g[:128], EPS)


def test_feeds_the_rowwise_linear(dev):
    # fused op -> per-token x per-channel matmul: same result as normalising in f32 on the host
    gen = torch.Generator().manual_seed(3)
    M, K, N = 8, 2048, 512
    x = torch.randn((M, K), generator=gen).to(torch.bfloat16)
    g = (1.0 + 0.1 * torch.randn(K, generator=gen)).to(torch.bfloat16)
    cfg = mx.rowwise_fp8_config()
    from modular_amd import synth
    w, ws = synth.quantize_weight_rowwise(synth.weights_f32(N, K, seed=1))
    q, s = mx.rms_norm_fused_quantize_dynamic_scaled_fp8(x.to(dev), g.to(dev), EPS)
    y = mx.dynamic_scaled_matmul(q, w.to(dev), s, ws.to(dev), cfg.input_scale, cfg.weight_scale).float().cpu()
    xf = x.float()
    normed = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + EPS) * g.float()
    ref = normed @ (w.float() * ws).T
    assert float((y - ref).abs().max()) <= 0.06 * float(ref.abs().max())
