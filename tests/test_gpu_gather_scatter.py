"""The row gather in front of the dynamic quantiser and the row scatter behind the grouped
matmul: the MoE layer's two index_selects (max/python/max/nn/moe/moe_fp8.py:525-560, 614-616)
folded into the kernels, as the reference's compiler folds them into the ops' input and output
lambdas (builtin_kernels/quantization.mojo:1376-1390).  Moving rows changes no arithmetic, so
both are bit-exact against the unfused kernel plus torch's index_select, and the gathered
quantiser is checked against the CPU oracle on the gathered rows as well."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import synth
from test_gpu_grouped import CASES, make
from util import bf16_bits, f32_np, fp8_bytes

pytestmark = pytest.mark.gpu
BLK = mx.blockwise_fp8_config()
ROW = mx.rowwise_fp8_config()
NT = oracle.default_threads()


def u32(t):
    return t.to(torch.int64).to(torch.uint32)


@pytest.mark.parametrize("rows,K,R,div,group", [
    (64, 512, 128, 2, 128), (300, 7168, 2400, 8, 128), (1, 256, 8, 8, 128), (33, 384, 5, 1, 128),
    (50, 1024, 70, 1, -1), (50, 4096, 70, 3, -1), (17, 16384, 40, 2, -1),  # per-token: warp, block and long-row kernels
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_quantise_gathered_rows(dev, rows, K, R, div, group, dtype):
    g = torch.Generator().manual_seed(rows * 7 + R)
    x = synth.activations(rows, K, seed=rows + K).to(dtype)
    idx = torch.randint(0, rows * div, (R,), generator=g)
    cfg = BLK if group == 128 else ROW
    spec = (cfg.input_scale, cfg.weight_scale)
    kw = dict(scales_type=torch.float32, group_size_or_per_token=group)
    xd = x.to(dev)
    q, s = mx.quantize_dynamic_scaled_float8(xd, *spec, row_index=u32(idx).to(dev), index_div=div, **kw)
    q0, s0 = mx.quantize_dynamic_scaled_float8(xd.index_select(0, idx.to(dev) // div), *spec, **kw)
    torch.cuda.synchronize()
    assert q.shape == (R, K) and s.shape == s0.shape
    assert np.array_equal(fp8_bytes(q), fp8_bytes(q0))
    assert np.array_equal(f32_np(s)[:, :R], f32_np(s0)[:, :R])
    if dtype == torch.bfloat16:
        qo, so = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x.index_select(0, idx // div)), K if group == -1 else group,
                                                    threads=NT)
        assert np.array_equal(fp8_bytes(q), qo)
        assert np.array_equal(f32_np(s)[:, :R], so)


@pytest.mark.parametrize("rows,K,copies", [(64, 512, 2), (300, 7168, 8), (1, 256, 8), (33, 384, 1), (4096, 1024, 8), (50, 128, 3)])
def test_quantise_once_and_scatter_rows(dev, rows, K, copies):
    # input row r, quantised once, goes to the rows scatter_index[r * copies + j]: with a permutation as the index the
    # same bytes as the gather by its inverse, and as the oracle on the gathered rows
    g = torch.Generator().manual_seed(rows * 3 + copies)
    x = synth.activations(rows, K, seed=rows + K)
    dst = torch.randperm(rows * copies, generator=g)          # assignment a = r * copies + j lands in row dst[a]
    src = torch.empty_like(dst)
    src[dst] = torch.arange(rows * copies)                    # row d is assignment src[d]: the gather's index
    spec = (BLK.input_scale, BLK.weight_scale)
    kw = dict(scales_type=torch.float32, group_size_or_per_token=128)
    xd = x.to(dev)
    q, s = mx.quantize_dynamic_scaled_float8(xd, *spec, scatter_index=u32(dst).to(dev), **kw)
    q0, s0 = mx.quantize_dynamic_scaled_float8(xd, *spec, row_index=u32(src).to(dev), index_div=copies, **kw)
    torch.cuda.synchronize()
    R = rows * copies
    assert q.shape == (R, K) and s.shape == s0.shape
    assert np.array_equal(fp8_bytes(q), fp8_bytes(q0))
    assert np.array_equal(f32_np(s)[:, :R], f32_np(s0)[:, :R])
    qo, so = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x.index_select(0, src // copies)), 128, threads=NT)
    assert np.array_equal(fp8_bytes(q), qo)
    assert np.array_equal(f32_np(s)[:, :R], so)


def test_scatter_skips_destinations_outside_the_result(dev):
    rows, K = 16, 256
    x = synth.activations(rows, K, seed=3).to(dev)
    dst = torch.arange(rows * 2)
    dst[5] = 4000000000 % (1 << 32)          # far outside the 32 rows of the result
    q, s = mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32,
                                             group_size_or_per_token=128, scatter_index=u32(dst).to(dev))
    q0, s0 = mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32,
                                               group_size_or_per_token=128)
    torch.cuda.synchronize()
    keep = [a for a in range(rows * 2) if a != 5]
    assert np.array_equal(fp8_bytes(q)[keep], fp8_bytes(q0)[[a // 2 for a in keep]])


def test_scatter_argument_checks(dev):
    x = synth.activations(8, 256, seed=1).to(dev)
    idx = u32(torch.arange(16)).to(dev)
    kw = dict(scales_type=torch.float32, group_size_or_per_token=128)
    with pytest.raises(TypeError):
        mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scatter_index=torch.arange(16).to(dev), **kw)
    with pytest.raises(ValueError):   # not a whole number of destinations per row
        mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scatter_index=idx[:15], **kw)
    with pytest.raises(ValueError):
        mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scatter_index=idx, row_index=idx, **kw)
    with pytest.raises(TypeError):   # float32 input: the gather form's business
        mx.quantize_dynamic_scaled_float8(x.float(), BLK.input_scale, BLK.weight_scale, scatter_index=idx, **kw)


def test_gather_argument_checks(dev):
    x = synth.activations(8, 256, seed=1).to(dev)
    idx = torch.zeros(4, dtype=torch.int64)
    with pytest.raises(TypeError):
        mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32,
                                          group_size_or_per_token=128, row_index=idx.to(dev))
    with pytest.raises(ValueError):
        mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32,
                                          group_size_or_per_token=128, row_index=u32(idx).to(dev), index_div=0)
    # no rows asked for: nothing is launched
    q, s = mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32,
                                             group_size_or_per_token=128, row_index=u32(idx[:0]).to(dev))
    assert q.shape == (0, 256)


@pytest.mark.parametrize("counts,ids,E,N,K", CASES + [([300, 2000, 40], [2, -1, 0], 3, 512, 256)])
@pytest.mark.parametrize("out", [torch.float32, torch.bfloat16])
def test_grouped_matmul_scatters_rows(dev, counts, ids, E, N, K, out):
    a, b, sa, sb, off, eids = make(counts, ids, E, N, K, seed=sum(counts) + 5)
    T = a.shape[0]
    perm = torch.randperm(T, generator=torch.Generator().manual_seed(T))
    stats = torch.tensor([max(counts), len(counts)], dtype=torch.int64).to(torch.uint32)
    args = (a.to(dev), b.to(dev), sa.to(dev), sb.to(dev), off.to(dev), eids.to(dev), stats, BLK.input_scale, BLK.weight_scale)
    plain = mx.grouped_dynamic_scaled_fp8_matmul(*args, out_type=out, algo="tiled")
    scattered = mx.grouped_dynamic_scaled_fp8_matmul(*args, out_type=out, algo="tiled", out_row_index=u32(perm).to(dev))
    torch.cuda.synchronize()
    want = torch.empty_like(plain)
    want[perm.to(dev)] = plain
    assert torch.equal(scattered.view(torch.int32 if out == torch.float32 else torch.int16),
                       want.view(torch.int32 if out == torch.float32 else torch.int16))


def test_scatter_argument_checks(dev):
    a, b, sa, sb, off, eids = make([5, 11], [1, 0], 2, 384, 256, seed=3)
    stats = torch.tensor([11, 2], dtype=torch.int64).to(torch.uint32)
    args = (a.to(dev), b.to(dev), sa.to(dev), sb.to(dev), off.to(dev), eids.to(dev), stats, BLK.input_scale, BLK.weight_scale)
    with pytest.raises(TypeError):
        mx.grouped_dynamic_scaled_fp8_matmul(*args, out_row_index=torch.arange(16).to(dev))
    with pytest.raises(TypeError):
        mx.grouped_dynamic_scaled_fp8_matmul(*args, out_row_index=u32(torch.arange(15)).to(dev))
    with pytest.raises(ValueError):  # the one-thread-per-output kernel has no scatter
        mx.grouped_dynamic_scaled_fp8_matmul(*args, algo="naive", out_row_index=u32(torch.arange(16)).to(dev))
