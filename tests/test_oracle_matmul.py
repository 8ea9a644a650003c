"""Pins the oracle's scaled matmuls: float64 brute force on the reference test's
shapes and granularities (max/kernels/test/gpu/linalg/test_naive_blockwise_fp8_matmul.mojo:
115-138, 194-200, tolerance 1e-4), exactly representable cases (bit-exact), the
multiplication order, and the grouped semantics of
max/kernels/src/linalg/fp8_quantization.mojo:1745-1865 with the token lists of
max/kernels/test/gpu/linalg/test_grouped_matmul_sm100_blockwise_fp8.mojo:298-420."""
import numpy as np
import pytest

import oracle


def rand_fp8(rng, shape, std=1.0):
    x = (rng.standard_normal(shape) * std).astype(np.float32)
    return oracle.e4m3fn_encode(np.clip(x, -448, 448))


def brute_block(a, b, a_s, b_s, gm, gn, gk):
    A = oracle.e4m3fn_decode(a).astype(np.float64)
    B = oracle.e4m3fn_decode(b).astype(np.float64)
    M, K = A.shape
    N = B.shape[0]
    As = np.repeat(np.repeat(a_s.astype(np.float64), gk, axis=0)[:K], gm, axis=1)[:, :M]  # [K, M]
    Bs = np.repeat(np.repeat(b_s.astype(np.float64), gn, axis=0)[:N], gk, axis=1)[:, :K]  # [N, K]
    return (A * As.T) @ (B * Bs).T


@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (120, 128, 128), (128, 129, 128), (128, 128, 129), (33, 70, 385)])
@pytest.mark.parametrize("g", [(1, 128, 128), (1, 64, 128), (1, 64, 16), (32, 128, 64)])
@pytest.mark.parametrize("mode", [0, 1])
def test_blockwise_vs_float64(M, N, K, g, mode):
    rng = np.random.default_rng(M * 7 + N * 3 + K + g[1])
    gm, gn, gk = g
    a, b = rand_fp8(rng, (M, K)), rand_fp8(rng, (N, K))
    a_s = rng.uniform(0.5, 2.0, (-(-K // gk), -(-M // gm))).astype(np.float32)
    b_s = rng.uniform(0.5, 2.0, (-(-N // gn), -(-K // gk))).astype(np.float32)
    c = oracle.matmul_blockwise(a, b, a_s, b_s, gmnk=g, mode=mode)
    ref = brute_block(a, b, a_s, b_s, gm, gn, gk)
    np.testing.assert_allclose(c, ref, rtol=1e-4, atol=1e-4)


def test_blockwise_exact_small_integers():
    # integers |v| <= 4 and power-of-two scales: every product and partial sum is an
    # exact f32, so the result must equal integer arithmetic bit for bit
    rng = np.random.default_rng(5)
    M, N, K = 37, 150, 512
    ai = rng.integers(-4, 5, (M, K))
    bi = rng.integers(-4, 5, (N, K))
    a = oracle.e4m3fn_encode(ai.astype(np.float32))
    b = oracle.e4m3fn_encode(bi.astype(np.float32))
    ea = rng.integers(-3, 4, (K // 128, M))
    eb = rng.integers(-3, 4, (2, K // 128))
    a_s, b_s = np.exp2(ea).astype(np.float32), np.exp2(eb).astype(np.float32)
    want = np.zeros((M, N), dtype=np.float64)
    for j in range(K // 128):
        part = ai[:, j * 128:(j + 1) * 128] @ bi[:, j * 128:(j + 1) * 128].T
        want += part * np.exp2(ea[j])[:, None] * np.exp2(eb[np.arange(N) // 128, j])[None, :]
    for mode in (0, 1):
        c = oracle.matmul_blockwise(a, b, a_s, b_s, mode=mode)
        assert np.array_equal(c.astype(np.float64), want)
    cb = oracle.matmul_blockwise(a, b, a_s, b_s, c_dtype=oracle.BF16)
    import torch
    want_bf16 = torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(cb, want_bf16)


def test_blockwise_identity_weight_picks_scales():
    # B = identity (N = K = 256): C[m, n] = A[m, n] * a_s[n/128, m] * b_s[n/128, n/128]
    rng = np.random.default_rng(9)
    M, K = 5, 256
    a = rand_fp8(rng, (M, K))
    b = oracle.e4m3fn_encode(np.eye(K, dtype=np.float32))
    a_s = rng.uniform(0.5, 2.0, (2, M)).astype(np.float32)
    b_s = rng.uniform(0.5, 2.0, (2, 2)).astype(np.float32)
    c = oracle.matmul_blockwise(a, b, a_s, b_s)
    A = oracle.e4m3fn_decode(a)
    for m in range(M):
        for n in range(K):
            want = np.float32(np.float32(A[m, n] * np.float32(1.0)) * a_s[n // 128, m]) * b_s[n // 128, n // 128]
            assert c[m, n] == want


def test_blockwise_multiplication_order_is_left_to_right():
    # one K term: ((a*b)*a_s)*b_s.  Pick scales for which the other grouping rounds differently.
    rng = np.random.default_rng(1)
    a = oracle.e4m3fn_encode(np.array([[1.75]], dtype=np.float32))
    b = oracle.e4m3fn_encode(np.array([[1.25]], dtype=np.float32))
    found = 0
    for _ in range(2000):
        as_, bs_ = rng.uniform(0.5, 2.0, 2).astype(np.float32)
        left = np.float32(np.float32(np.float32(1.75 * 1.25) * as_) * bs_)
        right = np.float32(np.float32(1.75 * 1.25) * np.float32(as_ * bs_))
        if left != right:
            c = oracle.matmul_blockwise(a, b, np.array([[as_]], np.float32), np.array([[bs_]], np.float32),
                                        gmnk=(1, 1, 1))
            assert c[0, 0] == left
            found += 1
    assert found > 10


def brute_row(a, b, a_s, b_s):
    A = oracle.e4m3fn_decode(a).astype(np.float64)
    B = oracle.e4m3fn_decode(b).astype(np.float64)
    return (A @ B.T) * a_s.astype(np.float64).reshape(-1, 1) * b_s.astype(np.float64).reshape(1, -1)


@pytest.mark.parametrize("M,N,K", [(17, 512, 256), (124, 96, 512), (1, 40, 2048)])
def test_rowwise_vs_float64_and_order(M, N, K):
    rng = np.random.default_rng(M + N + K)
    a, b = rand_fp8(rng, (M, K)), rand_fp8(rng, (N, K))
    a_s = rng.uniform(0.01, 0.1, (1, M)).astype(np.float32)
    b_s = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float32)
    c = oracle.matmul_rowwise(a, b, a_s, b_s)
    np.testing.assert_allclose(c, brute_row(a, b, a_s, b_s), rtol=1e-4, atol=1e-6)
    # (acc * a_s) * b_s, reproduced from the unscaled sum
    raw = oracle.matmul_rowwise(a, b, np.ones((1, M), np.float32), np.ones((N, 1), np.float32))
    want = (raw * a_s.reshape(-1, 1)).astype(np.float32) * b_s.reshape(1, -1)
    assert np.array_equal(c, want.astype(np.float32))
    other = raw * (a_s.reshape(-1, 1) * b_s.reshape(1, -1)).astype(np.float32)
    assert not np.array_equal(c, other.astype(np.float32))


def test_rowwise_exact_and_tensor_scales():
    rng = np.random.default_rng(3)
    ai, bi = rng.integers(-4, 5, (9, 384)), rng.integers(-4, 5, (21, 384))
    a, b = oracle.e4m3fn_encode(ai.astype(np.float32)), oracle.e4m3fn_encode(bi.astype(np.float32))
    a_s = np.exp2(rng.integers(-3, 3, (1, 9))).astype(np.float32)
    b_s = np.exp2(rng.integers(-3, 3, (21, 1))).astype(np.float32)
    c = oracle.matmul_rowwise(a, b, a_s, b_s)
    assert np.array_equal(c, ((ai @ bi.T) * a_s.reshape(-1, 1) * b_s.reshape(1, -1)).astype(np.float32))
    ct = oracle.matmul_rowwise(a, b, np.array([[0.5]], np.float32), np.array([[4.0]], np.float32), tensor_scales=True)
    assert np.array_equal(ct, ((ai @ bi.T) * 2.0).astype(np.float32))


def make_grouped(rng, counts, ids, E, N, K, pad_rows=0):
    T = int(sum(counts)) + pad_rows
    a = rand_fp8(rng, (T, K))
    b = rand_fp8(rng, (E, N, K))
    ld = -(-T // 4) * 4
    a_s = rng.uniform(0.5, 2.0, (K // 128, ld)).astype(np.float32)
    b_s = rng.uniform(0.5, 2.0, (E, -(-N // 128), K // 128)).astype(np.float32)
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    return a, b, a_s, b_s, off, np.asarray(ids, dtype=np.int32)


@pytest.mark.parametrize("counts,ids", [
    ([20, 150, 30, 28], [0, 3, 2, 4]),   # sparse expert ids (reference: [20,1500,300,28], scaled down)
    ([5, 11], [1, 0]),                   # unaligned offsets
    ([3, 4], [0, 1]),
    ([7, 0, 9], [2, 1, 0]),              # an expert without tokens keeps its slot
])
def test_grouped_equals_per_expert_dense(counts, ids):
    rng = np.random.default_rng(sum(counts))
    E, N, K = 5, 256, 256
    a, b, a_s, b_s, off, ids = make_grouped(rng, counts, ids, E, N, K)
    c = oracle.grouped_matmul(a, b, a_s, b_s, off, ids, max(counts), len(counts))
    for z, e in enumerate(ids):
        r0, r1 = int(off[z]), int(off[z + 1])
        if r1 == r0:
            continue
        want = oracle.matmul_blockwise(a[r0:r1], b[e], a_s[:, r0:r1], b_s[e])
        assert np.array_equal(c[r0:r1], want)


def test_grouped_skip_zero_edges_and_untouched_rows():
    rng = np.random.default_rng(11)
    E, N, K = 3, 128, 128
    a, b, a_s, b_s, off, ids = make_grouped(rng, [4, 6, 2], [1, -1, 0], E, N, K, pad_rows=3)
    c = oracle.grouped_matmul(a, b, a_s, b_s, off, ids, 6, 3)
    assert np.all(c[4:10] == 0.0)                     # expert id -1: zeros are written
    assert np.all(np.isfinite(c[:4])) and np.all(np.isfinite(c[10:12]))
    assert np.all(np.isnan(c[12:]))                   # rows past the last offset are never written
    # only the first two slots active: the third slot's rows stay untouched
    c2 = oracle.grouped_matmul(a, b, a_s, b_s, off, ids, 6, 2)
    assert np.array_equal(c2[:10], c[:10]) and np.all(np.isnan(c2[10:]))
    # either scalar zero => nothing is written (test_grouped_matmul_dynamic_scaled_fp8.mojo:245-263)
    for mt, na in ((0, 3), (6, 0)):
        assert np.all(np.isnan(oracle.grouped_matmul(a, b, a_s, b_s, off, ids, mt, na)))
