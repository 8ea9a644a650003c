"""GPU parity of the batched (MLA) variants: every batch of the batched quantiser and of
the batched blockwise matmul must equal what the 2-D oracle gives for that slice --
bytes and scales bit for bit, naive matmul bit for bit, MFMA matmuls within 1e-2.
Shapes follow max/kernels/test/gpu/quantization/test_scaled_fp8_quantization.mojo:760-807
and max/kernels/test/gpu/linalg/test_batched_matmul_sm100_scaled.mojo:470-660."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import synth
from util import assert_rel, bf16_bits, f32_np, fp8_bytes

pytestmark = pytest.mark.gpu
BLK = mx.blockwise_fp8_config()
NT = oracle.default_threads()
TOL = 1e-2


def src_bits(x):
    if x.dtype == torch.bfloat16:
        return bf16_bits(x), oracle.BF16
    return x.numpy(), oracle.F32


def check_quant(x_view_gpu, x_cpu, group, scales_type):
    B, M, K = x_cpu.shape
    q, s = mx.batched_quantize_dynamic_scaled_fp8(x_view_gpu, group, scales_type=scales_type)
    torch.cuda.synchronize()
    G = K if group == -1 else group
    assert q.shape == (B, M, K) and s.shape[:2] == (B, K // G) and s.shape[2] >= M
    qb = fp8_bytes(q)
    for i in range(B):
        bits, dt = src_bits(x_cpu[i].contiguous())
        q_ref, s_ref = oracle.quantize_dynamic_scaled_fp8(
            bits, G, in_dtype=dt, threads=NT,
            scales_dtype=oracle.BF16 if scales_type == torch.bfloat16 else oracle.F32)
        assert np.array_equal(qb[i], q_ref), f"bytes differ in batch {i}"
        if scales_type == torch.bfloat16:
            assert np.array_equal(bf16_bits(s[i])[:, :M], s_ref), f"scales differ in batch {i}"
        else:
            assert np.array_equal(f32_np(s[i])[:, :M].view(np.uint32), s_ref.view(np.uint32)), f"scales differ in batch {i}"


@pytest.mark.parametrize("B,M,K,group,dtype", [
    (128, 400, 512, 128, torch.bfloat16), (128, 1024, 128, 128, torch.float32),
    (128, 400, 528, 132, torch.bfloat16), (128, 1024, 544, 136, torch.float32),
    (7, 1000, 576, -1, torch.float32), (3, 5, 7168, 128, torch.bfloat16), (1, 1, 128, 128, torch.bfloat16),
])
def test_batched_quantize_reference_shapes(dev, B, M, K, group, dtype):
    g = torch.Generator().manual_seed(B * 7919 + M * 31 + K)
    x = (torch.rand((B, M, K), generator=g) * 2 - 1).to(dtype)
    check_quant(x.to(dev), x, group, dtype if dtype == torch.bfloat16 else torch.float32)


def test_batched_quantize_reads_a_transposed_view_in_place(dev):
    # the MLA graph quantises q_nope [row, batch, col] as [batch, row, col] (mla_graph.mojo:1010-1033)
    g = torch.Generator().manual_seed(5)
    x = (torch.randn((37, 16, 512), generator=g) * 3).to(torch.bfloat16)   # [row, batch, col]
    xg = x.to(dev)
    check_quant(xg.transpose(0, 1), x.transpose(0, 1), 128, torch.float32)


def test_batched_quantize_empty(dev):
    for shape in [(0, 4, 128), (4, 0, 128)]:
        q, s = mx.batched_quantize_dynamic_scaled_fp8(torch.empty(shape, dtype=torch.bfloat16, device=dev), 128)
        assert q.shape == shape
    with pytest.raises(ValueError):
        mx.batched_quantize_dynamic_scaled_fp8(torch.empty((2, 128), dtype=torch.bfloat16, device=dev))
    with pytest.raises(ValueError):
        mx.batched_quantize_dynamic_scaled_fp8(torch.empty((2, 2, 192), dtype=torch.bfloat16, device=dev), 128)


# ---- batched blockwise matmul ---------------------------------------------------------------

def make(B, M, N, K, seed):
    a, b = synth.random_fp8((B, M, K), seed), synth.random_fp8((B, N, K), seed + 1)
    m_pad = -(-M // 4) * 4
    sa = synth.random_scales((B, -(-K // 128), m_pad), seed + 2)
    sb = synth.random_scales((B, -(-N // 128), -(-K // 128)), seed + 3)
    return a, b, sa, sb


def oracle_bmm(a, b, sa, sb, c_dtype=oracle.F32):
    return np.stack([oracle.matmul_blockwise(fp8_bytes(a[i]), fp8_bytes(b[i]), sa[i].numpy(), sb[i].numpy(),
                                             gmnk=(1, 128, 128), threads=NT, c_dtype=c_dtype)
                     for i in range(a.shape[0])])


def bmm(a, b, sa, sb, dev, out_type=torch.float32, algo="auto", out=None):
    c = mx.batched_dynamic_scaled_fp8_matmul(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev), BLK.input_scale,
                                             BLK.weight_scale, out_type=out_type, algo=algo, out=out)
    torch.cuda.synchronize()
    return c


@pytest.mark.parametrize("M,N,K,B", [(33, 70, 385, 3), (120, 128, 512, 5), (1, 256, 128, 2)])
def test_batched_naive_is_the_oracle(dev, M, N, K, B):
    a, b, sa, sb = make(B, M, N, K, seed=M + N + K + B)
    c = bmm(a, b, sa, sb, dev, algo="naive")
    assert np.array_equal(f32_np(c), oracle_bmm(a, b, sa, sb))
    cb = bmm(a, b, sa, sb, dev, out_type=torch.bfloat16, algo="naive")
    assert np.array_equal(bf16_bits(cb), oracle_bmm(a, b, sa, sb, c_dtype=oracle.BF16))


# test_batched_matmul_sm100_scaled.mojo:470-635 (M, N, K, B); the two largest are covered by
# test_batched_large_matches_the_naive_kernel
@pytest.mark.parametrize("M,N,K,B", [
    (208, 2048, 256, 3), (400, 128, 128, 4), (100, 512, 256, 7), (96, 1024, 1024, 2), (120, 1280, 512, 5),
    (120, 512, 128, 128), (120, 128, 512, 128), (120, 8192, 192, 3), (1000, 3072, 576, 3),
    (8, 512, 512, 16), (1, 7168, 512, 4), (17, 384, 2048, 6),
])
@pytest.mark.parametrize("out_type", [torch.bfloat16, torch.float32])
def test_batched_mfma_reference_shapes(dev, M, N, K, B, out_type):
    if out_type == torch.float32 and B * M * N * K > 3e9:
        pytest.skip("one output type is enough at this size")
    a, b, sa, sb = make(B, M, N, K, seed=M * 3 + N * 5 + K * 7 + B)
    c = bmm(a, b, sa, sb, dev, out_type=out_type)
    ref = oracle_bmm(a, b, sa, sb)
    for i in range(B):
        assert_rel(f32_np(c[i]), ref[i], TOL, f"batch {i}")


@pytest.mark.parametrize("algo", ["tiled", "skinny"])
def test_batched_equals_the_loop_over_batches(dev, algo):
    M = 8 if algo == "skinny" else 300
    a, b, sa, sb = make(5, M, 640, 1024, seed=11)
    c = bmm(a, b, sa, sb, dev, out_type=torch.bfloat16, algo=algo)
    ag, bg, sag, sbg = (t.to(dev) for t in (a, b, sa, sb))
    for i in range(5):
        ci = mx.dynamic_scaled_matmul(ag[i], bg[i], sag[i], sbg[i], BLK.input_scale, BLK.weight_scale, algo=algo)
        if algo == "skinny":
            assert torch.equal(c[i], ci), f"batch {i}"
        else:  # the 2-D call may split K or pick another tile: same sums in another order, one bf16 ulp apart at most
            assert_rel(f32_np(c[i]), f32_np(ci), 2.0 ** -7, f"batch {i}")


@pytest.mark.parametrize("M,N,K,B", [(1024, 2048, 2048, 5), (4096, 512, 128, 128)])
def test_batched_large_matches_the_naive_kernel(dev, M, N, K, B):
    # the naive kernel is the oracle bit for bit (test_batched_naive_is_the_oracle)
    a, b, sa, sb = make(B, M, N, K, seed=B)
    c = bmm(a, b, sa, sb, dev, out_type=torch.float32)
    ref = bmm(a, b, sa, sb, dev, out_type=torch.float32, algo="naive")
    for i in range(0, B, max(1, B // 8)):
        assert_rel(f32_np(c[i]), f32_np(ref[i]), TOL, f"batch {i}")


# the MLA graph's output is [M, B, N]: batch stride N, row stride B * N
# (test_batched_matmul_sm100_scaled.mojo:637-660, B=128 heads, 12 tokens)
@pytest.mark.parametrize("N,K", [(128, 512), (512, 128)])
def test_batched_non_row_major_c(dev, N, K):
    B, M = 128, 12
    a, b, sa, sb = make(B, M, N, K, seed=N)
    buf = torch.full((M, B, N), 7.0, dtype=torch.bfloat16, device=dev)
    bmm(a, b, sa, sb, dev, out_type=torch.bfloat16, out=buf.transpose(0, 1))
    ref = oracle_bmm(a, b, sa, sb)
    got = f32_np(buf).transpose(1, 0, 2)
    for i in range(B):
        assert_rel(got[i], ref[i], TOL, f"batch {i}")


def test_batched_matmul_errors_and_empty(dev):
    a, b, sa, sb = make(2, 4, 128, 128, seed=1)
    row = mx.rowwise_fp8_config()
    with pytest.raises(ValueError, match="unsupported FP8 scaling granularity"):
        mx.batched_dynamic_scaled_fp8_matmul(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev), row.input_scale, row.weight_scale)
    with pytest.raises(ValueError, match="rank 3"):
        mx.batched_dynamic_scaled_fp8_matmul(a[0].to(dev), b.to(dev), sa.to(dev), sb.to(dev), BLK.input_scale, BLK.weight_scale)
    with pytest.raises(ValueError, match="batch dimension"):
        mx.batched_dynamic_scaled_fp8_matmul(a[:1].to(dev), b.to(dev), sa.to(dev), sb.to(dev), BLK.input_scale, BLK.weight_scale)
    with pytest.raises(TypeError, match="float32"):
        mx.batched_dynamic_scaled_fp8_matmul(a.to(dev), b.to(dev), sa.to(dev).bfloat16(), sb.to(dev), BLK.input_scale,
                                             BLK.weight_scale)
    e = bmm(a[:, :0], b, sa[:, :, :0], sb, dev)
    assert e.shape == (2, 0, 128)
    e = bmm(a[:0], b[:0], sa[:0], sb[:0], dev)
    assert e.shape == (0, 4, 128)
