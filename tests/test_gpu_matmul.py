"""GPU parity of the scaled FP8 matmuls.

  naive kernels  == CPU oracle bit for bit (f32 out): same summation order
  MFMA kernels   within max rel err 1e-2 of the oracle (bf16 and f32 out), and bit-exact
                 where the arithmetic is exact (small integers, power-of-two scales)
Shapes follow the reference's tests (test_naive_blockwise_fp8_matmul.mojo:194-200,
test_scaled_matmul.mojo:332-377, test_fp8_matmul_gpu.py:40-442) and BASELINE's configs;
at sizes the CPU cannot finish, the bit-exact-to-oracle naive kernel checks sampled rows."""
import os

import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import _lib, synth
from modular_amd.quant_config import InputScaleSpec, QuantConfig, ScaleGranularity, ScaleOrigin, WeightScaleSpec
from util import F32_BUDGET, assert_rel, bf16_bits, f32_np, fp8_bytes, fp8_from_bytes, rel_err

pytestmark = pytest.mark.gpu
BLK, ROW = mx.blockwise_fp8_config(), mx.rowwise_fp8_config()
NT = oracle.default_threads()
TOL = 1e-2  # BASELINE: max |rel err| <= 1e-2 against the fp32-accumulated reference result


def block_cfg(gm, gn, gk):
    return QuantConfig(InputScaleSpec(ScaleGranularity.BLOCK, ScaleOrigin.DYNAMIC, torch.float32, block_size=(gm, gk)),
                       WeightScaleSpec(ScaleGranularity.BLOCK, torch.float32, block_size=(gn, gk)))


def mm(a, b, sa, sb, cfg, dev, out=torch.float32, algo="auto"):
    c = mx.dynamic_scaled_matmul(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev), cfg.input_scale, cfg.weight_scale,
                                 out_type=out, algo=algo)
    torch.cuda.synchronize()
    return c


def make_block(M, N, K, seed, g=(1, 128, 128), pad_ld=True):
    gm, gn, gk = g
    a, b = synth.random_fp8((M, K), seed), synth.random_fp8((N, K), seed + 1)
    ld = -(-(-(-M // gm)) // 4) * 4 if pad_ld else -(-M // gm)
    sa = synth.random_scales((-(-K // gk), ld), seed + 2)
    sb = synth.random_scales((-(-N // gn), -(-K // gk)), seed + 3)
    return a, b, sa, sb


def oracle_block(a, b, sa, sb, g=(1, 128, 128), mode=0):
    return oracle.matmul_blockwise(fp8_bytes(a), fp8_bytes(b), sa.numpy(), sb.numpy(), gmnk=g, mode=mode, threads=NT)


# ---- naive kernel == oracle, bit for bit -------------------------------------------------

@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (120, 128, 128), (128, 129, 128), (128, 128, 129), (33, 70, 385)])
@pytest.mark.parametrize("g", [(1, 128, 128), (1, 64, 128), (1, 64, 16), (32, 128, 64)])
def test_naive_blockwise_is_the_oracle(dev, M, N, K, g):
    a, b, sa, sb = make_block(M, N, K, seed=M + N + K + g[1], g=g)
    c = mm(a, b, sa, sb, block_cfg(*g), dev, algo="naive")
    assert np.array_equal(f32_np(c), oracle_block(a, b, sa, sb, g))
    cb = mm(a, b, sa, sb, block_cfg(*g), dev, out=torch.bfloat16, algo="naive")
    want = oracle.matmul_blockwise(fp8_bytes(a), fp8_bytes(b), sa.numpy(), sb.numpy(), gmnk=g, c_dtype=oracle.BF16)
    assert np.array_equal(bf16_bits(cb), want)


def test_naive_rowwise_is_the_oracle(dev):
    for (M, N, K) in [(17, 512, 256), (124, 96, 512), (3, 40, 2050)]:
        a, b = synth.random_fp8((M, K), 1), synth.random_fp8((N, K), 2)
        sa, sb = synth.random_scales((1, M), 3, lo=0.01, hi=0.1), synth.random_scales((N, 1), 4, lo=0.001, hi=0.01)
        c = mm(a, b, sa, sb, ROW, dev, algo="naive")
        assert np.array_equal(f32_np(c), oracle.matmul_rowwise(fp8_bytes(a), fp8_bytes(b), sa.numpy(), sb.numpy(), threads=NT))


# ---- MFMA kernels: exact cases --------------------------------------------------------------

def exact_case(M, N, K, seed):
    rng = np.random.default_rng(seed)
    ai, bi = rng.integers(-4, 5, (M, K)), rng.integers(-4, 5, (N, K))
    a = fp8_from_bytes(oracle.e4m3fn_encode(ai.astype(np.float32)))
    b = fp8_from_bytes(oracle.e4m3fn_encode(bi.astype(np.float32)))
    kb, nb = -(-K // 128), -(-N // 128)
    ea, eb = rng.integers(-3, 4, (kb, -(-M // 4) * 4)), rng.integers(-3, 4, (nb, kb))
    want = np.zeros((M, N))
    for j in range(kb):
        part = ai[:, j * 128:(j + 1) * 128] @ bi[:, j * 128:(j + 1) * 128].T
        want += part * np.exp2(ea[j, :M])[:, None] * np.exp2(eb[np.arange(N) // 128, j])[None, :]
    return a, b, torch.from_numpy(np.exp2(ea).astype(np.float32)), torch.from_numpy(np.exp2(eb).astype(np.float32)), want


@pytest.mark.parametrize("algo,M,N,K", [
    ("tiled", 128, 128, 128), ("tiled", 130, 272, 512), ("tiled", 57, 100, 1040), ("tiled", 256, 384, 2048),
    ("skinny", 1, 64, 128), ("skinny", 8, 160, 512), ("skinny", 16, 100, 1040), ("skinny", 33, 48, 256),
    ("skinny", 64, 272, 640),
])
def test_mfma_blockwise_exact(dev, algo, M, N, K):
    a, b, sa, sb, want = exact_case(M, N, K, seed=M * 3 + N + K)
    c = mm(a, b, sa, sb, BLK, dev, algo=algo)
    got = f32_np(c).astype(np.float64)
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"{len(bad)} mismatches, first at {bad[:4].tolist()}: got {got[tuple(bad[0])]}, want {want[tuple(bad[0])]}"
    cb = mm(a, b, sa, sb, BLK, dev, out=torch.bfloat16, algo=algo)
    assert torch.equal(cb.cpu(), torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16))


@pytest.mark.parametrize("algo,M", [("tiled", 150), ("skinny", 5), ("skinny", 40)])
def test_mfma_rowwise_exact(dev, algo, M):
    rng = np.random.default_rng(M)
    N, K = 200, 768
    ai, bi = rng.integers(-4, 5, (M, K)), rng.integers(-4, 5, (N, K))
    a = fp8_from_bytes(oracle.e4m3fn_encode(ai.astype(np.float32)))
    b = fp8_from_bytes(oracle.e4m3fn_encode(bi.astype(np.float32)))
    sa = torch.from_numpy(np.exp2(rng.integers(-3, 3, (1, M))).astype(np.float32))
    sb = torch.from_numpy(np.exp2(rng.integers(-3, 3, (N, 1))).astype(np.float32))
    want = (ai @ bi.T) * sa.numpy().reshape(-1, 1) * sb.numpy().reshape(1, -1)
    c = mm(a, b, sa, sb, ROW, dev, algo=algo)
    assert np.array_equal(f32_np(c).astype(np.float64), want)


@pytest.mark.parametrize("sel", ["1408", "1416", "2408", "2416", "4432"])
@pytest.mark.parametrize("M,N,K", [(1, 64, 128), (8, 200, 1040), (16, 272, 640), (33, 100, 512), (64, 336, 1152)])
def test_every_decode_shape_is_exact(dev, tune, sel, M, N, K):
    """The decode kernel's shapes (weight rows per block, bytes in flight per wave) forced one by one, on ragged N and
    K: exact on integer data in both scale modes, so the choice between them cannot change a result."""
    tune(MAXFP8_SKINNY=sel)
    a, b, sa, sb, want = exact_case(M, N, K, seed=M + N + K)
    got = f32_np(mm(a, b, sa, sb, BLK, dev, algo="skinny")).astype(np.float64)
    assert np.array_equal(got, want), f"block mode, shape {sel}: {np.argwhere(got != want)[:4].tolist()}"
    rng = np.random.default_rng(K + M)
    ra = torch.from_numpy(np.exp2(rng.integers(-3, 3, (1, M))).astype(np.float32))
    rb = torch.from_numpy(np.exp2(rng.integers(-3, 3, (N, 1))).astype(np.float32))
    ai = oracle.e4m3fn_decode(fp8_bytes(a)).astype(np.float64)
    bi = oracle.e4m3fn_decode(fp8_bytes(b)).astype(np.float64)
    want_row = (ai @ bi.T) * ra.numpy().reshape(-1, 1) * rb.numpy().reshape(1, -1)
    got_row = f32_np(mm(a, b, ra, rb, ROW, dev, algo="skinny")).astype(np.float64)
    assert np.array_equal(got_row, want_row), f"row mode, shape {sel}"


@pytest.mark.parametrize("M,N,K", [(1, 272, 128), (1, 1000, 1040), (1, 2064, 8192), (2, 520, 8192), (2, 136, 4112),
                                   (3, 1032, 4096), (4, 264, 2048), (4, 4104, 4000)])
def test_decode_activations_through_lds(dev, tune, M, N, K):
    """With few tokens and a short enough share of K per wave the decode kernel copies the activations to LDS once
    instead of loading them slab by slab.  Same operands into the same MFMAs: bit-equal to the per-slab form on
    random data (both scale modes, K tails, ragged N), and exact on integer data."""
    for kind in ("block", "row"):
        if kind == "block":
            a, b = synth.random_fp8((M, K), M + K), synth.random_fp8((N, K), N + 1)
            kb = -(-K // 128)
            sa, sb = synth.random_scales((kb, -(-M // 4) * 4), 3), synth.random_scales((-(-N // 128), kb), 4)
            cfg = BLK
        else:
            a, b = synth.random_fp8((M, K), M + K), synth.random_fp8((N, K), N + 1)
            sa, sb = synth.random_scales((1, M), 3, lo=0.01, hi=0.1), synth.random_scales((N, 1), 4, lo=0.001, hi=0.01)
            cfg = ROW
        tune(MAXFP8_SKINNY_ALDS=None)
        got = mm(a, b, sa, sb, cfg, dev, algo="skinny")
        again = mm(a, b, sa, sb, cfg, dev, algo="skinny")
        tune(MAXFP8_SKINNY_ALDS="0")
        want = mm(a, b, sa, sb, cfg, dev, algo="skinny")
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), f"{kind} {M}x{N}x{K}"
        assert torch.equal(again.view(torch.int32), want.view(torch.int32)), f"{kind} {M}x{N}x{K}, second launch"
    tune(MAXFP8_SKINNY_ALDS=None)
    ea, eb, esa, esb, want = exact_case(M, N, K, seed=M + N)
    assert np.array_equal(f32_np(mm(ea, eb, esa, esb, BLK, dev, algo="skinny")).astype(np.float64), want)


@pytest.mark.parametrize("M,N,K", [(3, 16400, 4096), (12, 10256, 4096), (24, 10304, 4224), (40, 12288, 4096),
                                   (64, 8192, 2048), (20, 20480, 1536), (16, 16384, 16384), (8, 16384, 16384),
                                   (5, 4090, 2048), (32, 5120, 5120)])
def test_chosen_decode_shapes_match_the_scalar_kernel(dev, M, N, K):
    """Sizes that reach each shape through the kernel's own choice (16, 32 and 64 weight rows per block, both ring
    sizes), on integer data where both kernels are exact: equal to the scalar kernel bit for bit."""
    rng = np.random.default_rng(M + N)
    a = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (M, K)).astype(np.float32)))
    b = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (N, K)).astype(np.float32)))
    kb, nb = -(-K // 128), -(-N // 128)
    sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (kb, -(-M // 4) * 4))).astype(np.float32))
    sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (nb, kb))).astype(np.float32))
    assert torch.equal(mm(a, b, sa, sb, BLK, dev, algo="skinny"), mm(a, b, sa, sb, BLK, dev, algo="naive"))
    ra = torch.from_numpy(np.exp2(rng.integers(-3, 3, (1, M))).astype(np.float32))
    rb = torch.from_numpy(np.exp2(rng.integers(-3, 3, (N, 1))).astype(np.float32))
    assert torch.equal(mm(a, b, ra, rb, ROW, dev, algo="skinny"), mm(a, b, ra, rb, ROW, dev, algo="naive"))


def test_random_shapes_through_the_automatic_choice_are_exact(dev):
    """A seeded sweep of shapes over every regime of the automatic choice (decode kernel, K-split tiles, three-stage
    tiles, two regions, the persistent kernel), ragged and aligned, both scale modes, f32 and bf16 out: on integer
    data, where every kernel is exact, the result equals the scalar kernel's bit for bit."""
    rng = np.random.default_rng(2024)
    for it in range(60):
        kind = it % 6
        if kind == 0:
            M, N, K = int(rng.integers(1, 65)), int(rng.integers(1, 12000)), 16 * int(rng.integers(1, 300))
        elif kind == 1:
            M, N, K = int(rng.integers(33, 65)), 128 * int(rng.integers(40, 120)), 128 * int(rng.integers(16, 64))
        elif kind == 2:
            M, N, K = 256 * int(rng.integers(1, 6)), 256 * int(rng.integers(1, 40)), 128 * int(rng.integers(1, 24))
        elif kind == 3:
            M, N, K = int(rng.integers(65, 900)), int(rng.integers(1, 4000)), 16 * int(rng.integers(1, 200))
        elif kind == 4:
            M, N, K = int(rng.integers(100, 2100)), 8 * int(rng.integers(100, 1200)), 128 * int(rng.integers(1, 20))
        else:
            M, N, K = int(rng.integers(1, 33)), 16 * int(rng.integers(600, 1400)), 128 * int(rng.integers(30, 70))
        a = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (M, K)).astype(np.float32)))
        b = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (N, K)).astype(np.float32)))
        kb, nb = -(-K // 128), -(-N // 128)
        sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (kb, -(-M // 4) * 4))).astype(np.float32))
        sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (nb, kb))).astype(np.float32))
        ra = torch.from_numpy(np.exp2(rng.integers(-3, 3, (1, M))).astype(np.float32))
        rb = torch.from_numpy(np.exp2(rng.integers(-3, 3, (N, 1))).astype(np.float32))
        out = torch.bfloat16 if it % 2 else torch.float32
        for cfg, x, y in ((BLK, sa, sb), (ROW, ra, rb)):
            got, ref = mm(a, b, x, y, cfg, dev, out=out), mm(a, b, x, y, cfg, dev, out=out, algo="naive")
            assert torch.equal(got, ref), f"{M}x{N}x{K} {out} {'block' if cfg is BLK else 'row'}"


# ---- MFMA kernels: tolerance against the oracle ------------------------------------------

@pytest.mark.parametrize("algo,M,N,K", [
    ("tiled", 128, 128, 128), ("tiled", 120, 129, 128), ("tiled", 81, 1024, 2048), ("tiled", 300, 576, 1024),
    ("tiled", 257, 640, 3072), ("tiled", 64, 512, 4096),
    ("skinny", 1, 1024, 2048), ("skinny", 32, 1024, 2048), ("skinny", 2, 129, 512), ("skinny", 16, 640, 4096),
    ("skinny", 64, 256, 4096), ("auto", 81, 1024, 2048), ("auto", 7, 576, 7168),
])
@pytest.mark.parametrize("out", [torch.float32, torch.bfloat16])
def test_mfma_blockwise_vs_oracle(dev, algo, M, N, K, out):
    a, b, sa, sb = make_block(M, N, K, seed=M + N + K)
    ref = oracle_block(a, b, sa, sb)
    c = mm(a, b, sa, sb, BLK, dev, out=out, algo=algo)
    assert_rel(f32_np(c), ref, TOL, f"{algo} {M}x{N}x{K} {out}", F32_BUDGET if out == torch.float32 else None)


@pytest.mark.parametrize("algo,M,N,K", [
    ("tiled", 17, 512, 256), ("tiled", 124, 512, 512), ("tiled", 300, 1040, 1024),
    ("skinny", 1, 512, 256), ("skinny", 8, 1000, 8192), ("skinny", 17, 512, 256), ("auto", 3000, 512, 512),
])
def test_mfma_rowwise_vs_oracle(dev, algo, M, N, K):
    a, b = synth.random_fp8((M, K), M), synth.random_fp8((N, K), N)
    sa, sb = synth.random_scales((1, M), 3, lo=0.01, hi=0.1), synth.random_scales((N, 1), 4, lo=0.001, hi=0.01)
    ref = oracle.matmul_rowwise(fp8_bytes(a), fp8_bytes(b), sa.numpy(), sb.numpy(), threads=NT)
    for out in (torch.float32, torch.bfloat16):
        c = mm(a, b, sa, sb, ROW, dev, out=out, algo=algo)
        assert_rel(f32_np(c), ref, TOL, f"rowwise {algo} {M}x{N}x{K} {out}", F32_BUDGET if out == torch.float32 else None)


def test_mfma_keeps_13_bits_below_the_largest_product(dev):
    # Known answer that documents the hardware: 448*448 + 1*1 = 200705 is an exact f32, the
    # scalar kernel returns it, the matrix instruction drops the 1 (truncation inside the
    # instruction, not in this library's code).  The loss is bounded by 2^-12 of the largest product.
    a = torch.zeros((16, 128), dtype=torch.float32)
    b = torch.zeros((16, 128), dtype=torch.float32)
    a[:, 0], b[:, 0], a[:, 1], b[:, 1] = 448.0, 448.0, 1.0, 1.0
    a8, b8 = a.to(torch.float8_e4m3fn), b.to(torch.float8_e4m3fn)
    one = torch.ones((1, 16))
    assert float(mm(a8, b8, one, one[:, :1], BLK, dev, algo="naive")[0, 0]) == 200705.0
    for algo in ("tiled", "skinny"):
        got = float(mm(a8, b8, one, one[:, :1], BLK, dev, algo=algo)[0, 0])
        assert 200704.0 <= got <= 200705.0 and abs(got - 200705.0) <= 200704.0 * 2.0 ** -12, got


def test_tensor_scales(dev):
    cfg = QuantConfig(InputScaleSpec(ScaleGranularity.TENSOR, ScaleOrigin.DYNAMIC, torch.float32),
                      WeightScaleSpec(ScaleGranularity.TENSOR, torch.float32))
    a, b = synth.random_fp8((20, 256), 1), synth.random_fp8((144, 256), 2)
    sa, sb = torch.tensor([[0.031]]), torch.tensor([[0.0047]])
    ref = oracle.matmul_rowwise(fp8_bytes(a), fp8_bytes(b), sa.numpy(), sb.numpy(), tensor_scales=True)
    for algo in ("naive", "skinny", "tiled"):
        assert_rel(f32_np(mm(a, b, sa, sb, cfg, dev, algo=algo)), ref, TOL, algo, F32_BUDGET)


def test_pathological_weight_scale_column(dev):
    # test_scaled_matmul_pathological_bscale.mojo:14-38: a denormal weight scale gives finite ~0
    a, b = synth.random_fp8((17, 512), 1), synth.random_fp8((64, 512), 2)
    sa, sb = synth.random_scales((1, 17), 3), synth.random_scales((64, 1), 4)
    sb[5, 0] = 1e-40
    for algo in ("skinny", "tiled"):
        c = f32_np(mm(a, b, sa, sb, ROW, dev, out=torch.bfloat16, algo=algo))
        assert np.all(np.isfinite(c)) and np.all(np.abs(c[:, 5]) < 1e-30)


def test_row_strided_operands(dev):
    a_wide, b_wide = synth.random_fp8((40, 1024), 1).to(dev), synth.random_fp8((200, 1024), 2).to(dev)
    a, b = a_wide[:, 256:768], b_wide[:, 512:]
    sa, sb = synth.random_scales((4, 40), 3), synth.random_scales((2, 4), 4)
    ref = oracle_block(a.cpu().contiguous(), b.cpu().contiguous(), sa, sb)
    for algo in ("skinny", "tiled"):
        assert_rel(f32_np(mm(a, b, sa, sb, BLK, dev, algo=algo)), ref, TOL, algo, F32_BUDGET)


def test_empty(dev):
    a, b, sa, sb = make_block(0, 128, 256, 1)
    assert tuple(mm(a, b, sa, sb, BLK, dev).shape) == (0, 128)


# ---- configuration-sized problems, checked on sampled rows by the naive kernel ----------------
# Every (K, N) of the benchmark configurations at the M values named there; rows are sampled because the
# scalar-order kernel (bit-identical to the CPU oracle, tested above) needs a second per 24 rows at these sizes.

LLAMA8B = {"qkv": (4096, 6144), "gate_up": (4096, 28672), "down": (14336, 4096), "o_proj": (4096, 4096)}
DSV3 = {"q_a": (7168, 1536), "q_b": (1536, 24576), "kv_a": (7168, 576), "kv_b": (512, 32768), "o_proj": (16384, 7168),
        # the call the reference's FP8 MLA issues for q_a and kv_a: one matmul over the two weights stacked, N = 1536 + 576
        # (max/python/max/nn/attention/multi_latent_attention_fp8.py:595-603)
        "q_a_kv_a": (7168, 2112)}
CONFIG_CELLS = ([("single_linear", 64, 4096, 4096)]
                + [(f"llama8b_{n}", M, K, N) for n, (K, N) in LLAMA8B.items() for M in (1, 16, 128, 2048)]
                + [(f"dsv3_{n}", M, K, N) for n, (K, N) in DSV3.items() for M in (256, 1024, 4096)])

_operands = {}


def config_operands(K, N, dev):
    """weights of one (K, N) cell, quantised once and shared by the cell's M values"""
    if (K, N) not in _operands:
        _operands.clear()
        _operands[(K, N)] = synth.quantize_weight_block(synth.weights_f32(N, K, seed=1, device=dev))
    return _operands[(K, N)]


@pytest.mark.parametrize("name,M,K,N", CONFIG_CELLS, ids=[f"{c[0]}_m{c[1]}" for c in CONFIG_CELLS])
def test_config_shapes_blockwise(dev, name, M, K, N):
    x = synth.activations(M, K, seed=0, device=dev)
    w, sb = config_operands(K, N, dev)
    q, sa = mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32)
    c = mx.dynamic_scaled_matmul(q, w, sa, sb, BLK.input_scale, BLK.weight_scale)
    # 24 rows spread over the matrix, the last one included (the last tile row, where partial tiles live)
    rows = torch.unique(torch.cat([torch.arange(0, M, max(1, M // 23), device=dev)[:23], torch.tensor([M - 1], device=dev)]))
    ref = mx.dynamic_scaled_matmul(q[rows].contiguous(), w, sa[:, rows].contiguous(), sb, BLK.input_scale,
                                   BLK.weight_scale, out_type=torch.float32, algo="naive")
    torch.cuda.synchronize()
    fig = assert_rel(f32_np(c[rows]), f32_np(ref), TOL, f"config {name} {M}x{N}x{K}", natural_scale=True)
    line = (f"{name} M={M} K={K} N={N}: rel err {fig['rel_err']:.2e} (floor 2^-4 rms), {fig['rel_err_strict_floor']:.2e} "
            f"(floor 2^-8 rms), |err| <= {fig['err_over_rms']:.2e} rms, reference-style excess {fig['reference_style_excess']:.2f}"
            f" | {_lib.matmul_describe(M, N, K, True, True)}")
    print("[parity] " + line)
    # (the figures of a run are kept beside the run's other results)
    out_dir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out")
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "parity_figures.txt"), "a") as f:
        f.write(line + "\n")
    # one row against the CPU oracle itself
    r0 = int(rows[-1])
    cpu = oracle.matmul_blockwise(fp8_bytes(q[r0:r0 + 1]), fp8_bytes(w), f32_np(sa[:, r0:r0 + 1]), f32_np(sb), threads=NT)
    assert np.array_equal(f32_np(ref[-1:]), cpu)


DECODE70B = {"qkv": (8192, 10240), "gate_up": (8192, 57344), "down": (28672, 8192)}
DECODE_CELLS = [(n, M, K, N) for n, (K, N) in DECODE70B.items() for M in (1, 2, 4, 8)]


@pytest.mark.parametrize("name,M,K,N", DECODE_CELLS, ids=[f"{c[0]}_m{c[1]}" for c in DECODE_CELLS])
def test_config_shapes_decode_rowwise(dev, name, M, K, N):
    x = synth.activations(M, K, seed=0, outlier_frac=0.0, device=dev)
    if ("row", K, N) not in _operands:
        _operands.clear()
        _operands[("row", K, N)] = synth.quantize_weight_rowwise(synth.weights_f32(N, K, seed=1, device=dev))
    w, sb = _operands[("row", K, N)]
    q, sa = mx.quantize_dynamic_scaled_float8(x, ROW.input_scale, ROW.weight_scale, scales_type=torch.float32)
    assert tuple(sa.shape) == (1, M)
    c = mx.dynamic_scaled_matmul(q, w, sa, sb, ROW.input_scale, ROW.weight_scale)
    cols = torch.arange(0, N, 37, device=dev)
    ref = oracle.matmul_rowwise(fp8_bytes(q), fp8_bytes(w[cols]), f32_np(sa), f32_np(sb[cols]), threads=NT)
    torch.cuda.synchronize()
    assert_rel(f32_np(c[:, cols]), ref, TOL, f"decode {name} {M}x{N}x{K}", natural_scale=True)
    # linearity in the activation scale: doubling a_s doubles C exactly (power of two)
    c2 = mx.dynamic_scaled_matmul(q, w, sa * 2, sb, ROW.input_scale, ROW.weight_scale)
    assert torch.equal(c2.float(), c.float() * 2)
    _ = name


# ---- per-token / per-channel scales in bf16 and f16 ----------------------------------------------

@pytest.mark.parametrize("algo,M,N,K", [("tiled", 300, 1040, 1024), ("tiled", 2048, 512, 512), ("tiled", 1024, 1024, 256),
                                        ("skinny", 8, 1000, 2048), ("skinny", 40, 512, 256), ("auto", 96, 2304, 16384)])
@pytest.mark.parametrize("sdt", [torch.bfloat16, torch.float16])
def test_rowwise_scales_in_bf16_and_f16(dev, algo, M, N, K, sdt):
    """The reference's matmul takes its scales in bf16, f16 or f32 (fp8_quantization.mojo:996-1018; its Python
    wrapper even defaults to bf16) and widens them when the epilogue loads them (:1218-1240).  Every kernel does
    the same: the result equals the f32-scales result on the widened values bit for bit, whatever the kernel, and
    meets the oracle reading the 16-bit scales itself."""
    a, b = synth.random_fp8((M, K), M), synth.random_fp8((N, K), N)
    sa = synth.random_scales((1, M), 3, lo=0.01, hi=0.1).to(sdt)
    sb = synth.random_scales((N, 1), 4, lo=0.001, hi=0.01).to(sdt)
    odt = oracle.BF16 if sdt == torch.bfloat16 else oracle.F16
    bits = (lambda t: bf16_bits(t)) if sdt == torch.bfloat16 else (lambda t: t.numpy())
    ref = oracle.matmul_rowwise(fp8_bytes(a), fp8_bytes(b), bits(sa), bits(sb), threads=NT, scales_dtype=odt)
    assert np.array_equal(ref, oracle.matmul_rowwise(fp8_bytes(a), fp8_bytes(b), sa.float().numpy(), sb.float().numpy(), threads=NT))
    from modular_amd import _lib
    assert "naive" not in _lib.matmul_describe(M, N, K, False, True)
    for out in (torch.float32, torch.bfloat16):
        c = mm(a, b, sa, sb, ROW, dev, out=out, algo=algo)
        assert_rel(f32_np(c), ref, TOL, f"{sdt} scales {algo} {M}x{N}x{K} {out}", F32_BUDGET if out == torch.float32 else None)
        assert torch.equal(c, mm(a, b, sa.float(), sb.float(), ROW, dev, out=out, algo=algo))
    # the scalar kernel reads them too (it is the oracle's twin)
    assert np.array_equal(f32_np(mm(a, b, sa, sb, ROW, dev, algo="naive")), ref)


def test_tensor_scales_in_bf16(dev):
    cfg = QuantConfig(InputScaleSpec(ScaleGranularity.TENSOR, ScaleOrigin.DYNAMIC, torch.bfloat16),
                      WeightScaleSpec(ScaleGranularity.TENSOR, torch.bfloat16))
    a, b = synth.random_fp8((200, 512), 1), synth.random_fp8((272, 512), 2)
    sa, sb = torch.tensor([[0.031]]).to(torch.bfloat16), torch.tensor([[0.0047]]).to(torch.bfloat16)
    ref = oracle.matmul_rowwise(fp8_bytes(a), fp8_bytes(b), sa.float().numpy(), sb.float().numpy(), tensor_scales=True)
    for algo in ("naive", "tiled"):
        assert_rel(f32_np(mm(a, b, sa, sb, cfg, dev, algo=algo)), ref, TOL, algo, F32_BUDGET)
