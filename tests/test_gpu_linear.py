"""End-to-end FP8 linear (quantise + matmul through `Linear`) against the CPU oracle on
BASELINE's first configuration: x bf16 [64, 4096] with outlier channels, W [4096, 4096]
block-quantised offline, bf16 out."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import synth
from util import assert_rel, bf16_bits, f32_np, fp8_bytes

pytestmark = pytest.mark.gpu
NT = oracle.default_threads()


def test_config0_single_linear(dev):
    M, K, N = 64, 4096, 4096
    cfg = mx.blockwise_fp8_config()
    x = synth.activations(M, K, seed=0)
    wq, ws = synth.quantize_weight_block(synth.weights_f32(N, K, seed=0))
    lin = mx.Linear(K, N, cfg, device=dev)
    lin.weight.copy_(wq.to(dev))
    lin.weight_scale.copy_(ws.to(dev))
    y = lin(x.to(dev).reshape(2, 32, K))
    torch.cuda.synchronize()
    assert tuple(y.shape) == (2, 32, N) and y.dtype == torch.bfloat16
    q, sa = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x), 128, threads=NT)
    ref = oracle.matmul_blockwise(q, fp8_bytes(wq), sa, ws.numpy(), threads=NT)
    assert_rel(f32_np(y.reshape(M, N)), ref, 1e-2, "config 0")
    # against the unquantised product the error is the quantisation noise, a few percent of the row rms
    full = x.float() @ synth.weights_f32(N, K, seed=0).t()
    err = (y.reshape(M, N).float().cpu() - full).norm() / full.norm()
    assert err < 0.08


def test_rowwise_linear_and_bias(dev):
    M, K, N = 5, 1024, 768
    cfg = mx.rowwise_fp8_config()
    x = synth.activations(M, K, seed=2, outlier_frac=0.0)
    wq, ws = synth.quantize_weight_rowwise(synth.weights_f32(N, K, seed=3))
    lin = mx.Linear(K, N, cfg, device=dev, has_bias=True)
    lin.weight.copy_(wq.to(dev))
    lin.weight_scale.copy_(ws.to(dev))
    lin.bias.copy_(torch.linspace(-1, 1, N).to(torch.bfloat16))
    y = lin(x.to(dev))
    torch.cuda.synchronize()
    q, sa = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x), K, threads=NT)
    ref = oracle.matmul_rowwise(q, fp8_bytes(wq), sa, ws.numpy(), threads=NT)
    bias = torch.linspace(-1, 1, N).to(torch.bfloat16)
    # the bias is added to the bf16 matmul result in bf16 (not fused, as in the reference's Linear):
    # two roundings of at most 2^-9 each, of the product and of the sum
    got = f32_np(y).astype(np.float64)
    want = ref.astype(np.float64) + bias.float().numpy().astype(np.float64)
    bound = 2.0 ** -8 * (np.abs(ref) + np.abs(want)) + 2e-3 * np.sqrt((ref.astype(np.float64) ** 2).mean(1, keepdims=True))
    assert np.all(np.abs(got - want) <= bound)
    y0 = mx.Linear(K, N, cfg, device=dev)
    y0.weight.copy_(wq.to(dev))
    y0.weight_scale.copy_(ws.to(dev))
    assert_rel(f32_np(y0(x.to(dev))), ref, 1e-2, "rowwise linear")


@pytest.mark.parametrize("M,K,N,w4", [(2048, 2048, 28672, None), (2048, 2048, 28672, "0"), (16, 512, 4096, None), (256, 1024, 1536, None)])
def test_linear_replays_from_a_graph(dev, tune, M, K, N, w4):
    """An FP8 linear (quantise + matmul) has no host synchronisation, so it records into a HIP graph: the four-wave
    persistent kernel, the eight-wave persistent kernel with a second region in another tile shape, the decode kernel,
    and the K-split shapes with their workspace.  Every replay, with eager work and synchronisations between them and
    new activations in the same buffer, must give the eager result."""
    from modular_amd import _lib
    tune(MAXFP8_W4=w4)
    cfg = mx.blockwise_fp8_config()
    wq, ws = synth.quantize_weight_block(synth.weights_f32(N, K, seed=3))
    lin = mx.Linear(K, N, cfg, device=dev)
    lin.weight.copy_(wq.to(dev))
    lin.weight_scale.copy_(ws.to(dev))
    x = synth.activations(M, K, seed=4).to(dev)
    if M == 2048:
        plan = _lib.matmul_describe(M, N, K)
        assert "persistent" in plan and ("four waves" in plan if w4 is None else " + " in plan), plan
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        lin(x)  # first call outside the capture: it sets the kernels' LDS attributes
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = lin(x)
    for i in range(3):
        x.copy_(synth.activations(M, K, seed=10 + i).to(dev))
        want = lin(x)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i}"
