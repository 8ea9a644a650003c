"""GPU parity of the grouped (MoE) blockwise FP8 matmul against the CPU oracle; cases
of max/kernels/test/gpu/linalg/test_grouped_matmul_sm100_blockwise_fp8.mojo:298-420
(token lists, sparse expert ids, unaligned offsets) and
test_grouped_matmul_dynamic_scaled_fp8.mojo:38-265 (zero edge cases)."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import synth
from util import F32_BUDGET, assert_rel, f32_np, fp8_bytes, fp8_from_bytes, u32_np

pytestmark = pytest.mark.gpu
BLK = mx.blockwise_fp8_config()
NT = oracle.default_threads()
TOL = 1e-2


def make(counts, ids, E, N, K, seed, extra_rows=0):
    T = int(sum(counts)) + extra_rows
    a, b = synth.random_fp8((T, K), seed), synth.random_fp8((E, N, K), seed + 1)
    ld = -(-T // 4) * 4
    sa = synth.random_scales((K // 128, ld), seed + 2)
    sb = synth.random_scales((E, -(-N // 128), K // 128), seed + 3)
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32)
    # expert_ids holds one entry per expert (the wrapper checks that); slots past the active ones are unused
    ids = torch.tensor(list(ids) + [-1] * (E - len(ids)), dtype=torch.int32)
    return a, b, sa, sb, off, ids


def run(a, b, sa, sb, off, ids, max_tokens, num_active, dev, out=torch.float32, algo="auto", fill=None):
    stats = torch.tensor([max_tokens, num_active], dtype=torch.int64).to(torch.uint32)
    c = mx.grouped_dynamic_scaled_fp8_matmul(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev), off.to(dev), ids.to(dev),
                                             stats, BLK.input_scale, BLK.weight_scale, out_type=out, algo=algo)
    torch.cuda.synchronize()
    return c


def ref(a, b, sa, sb, off, ids, max_tokens, num_active, mode=0):
    return oracle.grouped_matmul(fp8_bytes(a), fp8_bytes(b), sa.numpy(), sb.numpy(), u32_np(off), ids.numpy(),
                                 max_tokens, num_active, mode=mode, threads=NT)


CASES = [
    ([20, 1500, 300, 28], [0, 3, 2, 4], 5, 256, 512),
    ([5, 11], [1, 0], 2, 384, 256),
    ([3, 4], [0, 1], 2, 128, 128),
    ([707, 709], [0, 1], 2, 256, 256),
    ([7, 0, 129, 0, 128], [2, 1, 0, 3, 4], 5, 200, 384),
]


@pytest.mark.parametrize("counts,ids,E,N,K", CASES)
def test_naive_grouped_is_the_oracle(dev, counts, ids, E, N, K):
    args = make(counts, ids, E, N, K, seed=sum(counts))
    c = run(*args, max(counts), len(counts), dev, algo="naive")
    want = ref(*args, max(counts), len(counts))
    assert np.array_equal(f32_np(c), want)


@pytest.mark.parametrize("counts,ids,E,N,K", CASES)
@pytest.mark.parametrize("out", [torch.float32, torch.bfloat16])
def test_mfma_grouped_vs_oracle(dev, counts, ids, E, N, K, out):
    args = make(counts, ids, E, N, K, seed=sum(counts))
    c = run(*args, max(counts), len(counts), dev, out=out, algo="tiled")
    assert_rel(f32_np(c), ref(*args, max(counts), len(counts)), TOL, f"grouped {counts}",
               F32_BUDGET if out == torch.float32 else None)


def test_grouped_exact_and_skipped_expert(dev):
    rng = np.random.default_rng(4)
    counts, ids, E, N, K = [40, 130, 9], [1, -1, 0], 2, 256, 256
    T = sum(counts)
    ai, bi = rng.integers(-4, 5, (T, K)), rng.integers(-4, 5, (E, N, K))
    a = fp8_from_bytes(oracle.e4m3fn_encode(ai.astype(np.float32)))
    b = fp8_from_bytes(oracle.e4m3fn_encode(bi.astype(np.float32)))
    sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (2, -(-T // 4) * 4))).astype(np.float32))
    sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (E, 2, 2))).astype(np.float32))
    off = torch.tensor([0, 40, 170, 179], dtype=torch.int64).to(torch.uint32)
    idt = torch.tensor(ids, dtype=torch.int32)
    b = torch.cat([b, b[:1]])  # three slots need three entries in expert_ids, hence three experts
    sb = torch.cat([sb, sb[:1]])
    want = ref(a, b, sa, sb, off, idt, 130, 3)
    for algo in ("naive", "tiled"):
        c = f32_np(run(a, b, sa, sb, off, idt, 130, 3, dev, algo=algo))
        assert np.array_equal(c, want), algo
        assert np.all(c[40:170] == 0.0)


def test_grouped_zero_edges_and_untouched_rows(dev):
    from modular_amd import _lib
    counts, ids, E, N, K = [4, 6, 2], [1, 0, 1], 3, 128, 128
    a, b, sa, sb, off, idt = make(counts, ids, E, N, K, seed=3, extra_rows=5)
    T = a.shape[0]
    ad, bd, sad, sbd, offd, idd = (t.to(dev) for t in (a, b, sa, sb, off, idt))

    def raw(max_tokens, num_active, algo):
        c = torch.full((T, N), float("nan"), device=dev)
        st = _lib.lib().maxfp8_grouped_matmul_dynamic_scaled_fp8(
            c.data_ptr(), ad.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), offd.data_ptr(),
            idd.data_ptr(), T, N, K, E, max_tokens, num_active, sa.shape[1], _lib.F32,
            _lib.F32, algo, None)
        assert st == 0, _lib.last_error()
        torch.cuda.synchronize()
        return f32_np(c)

    for algo in (_lib.ALGO_NAIVE, _lib.ALGO_TILED):
        assert np.all(np.isnan(raw(0, 3, algo))) and np.all(np.isnan(raw(6, 0, algo)))
        full = raw(6, 3, algo)
        assert np.all(np.isfinite(full[:12])) and np.all(np.isnan(full[12:]))
        two = raw(6, 2, algo)
        assert np.array_equal(two[:10], full[:10]) and np.all(np.isnan(two[10:]))


def test_moe_config_sampled(dev):
    # 256 experts, top-8 of 4096 tokens with Zipf(1.1) popularity; down projection K=2048, N=7168.
    E, Kd, Nd = 256, 2048, 7168
    off, ids, counts, stats = synth.moe_routing(4096, E, 8, seed=0, device=dev)
    T = int(counts.sum())
    assert T == 32768
    x = synth.activations(T, Kd, seed=0, outlier_frac=0.0, device=dev)
    q, sa = mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32)
    w = torch.empty((E, Nd, Kd), dtype=torch.float8_e4m3fn, device=dev)
    sb = torch.empty((E, Nd // 128, Kd // 128), dtype=torch.float32, device=dev)
    for e0 in range(0, E, 32):
        wq, ws = synth.quantize_weight_block(synth.weights_f32(32 * Nd, Kd, seed=100 + e0, device=dev).reshape(32, Nd, Kd))
        w[e0:e0 + 32], sb[e0:e0 + 32] = wq, ws
    c = mx.grouped_dynamic_scaled_fp8_matmul(q, w, sa, sb, off, ids, stats, BLK.input_scale, BLK.weight_scale)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(c.float()).all())
    offs = u32_np(off).astype(np.int64)
    order = np.argsort(-counts.numpy())
    for e in list(order[:2]) + list(order[-3:]) + [17, 128]:   # biggest, smallest and two arbitrary experts
        r0, r1 = offs[e], offs[e + 1]
        if r1 == r0:
            continue
        rows = torch.arange(r0, r1, max(1, (r1 - r0) // 8), device=dev)[:8]
        refc = mx.dynamic_scaled_matmul(q[rows].contiguous(), w[e], sa[:, rows].contiguous(), sb[e], BLK.input_scale,
                                        BLK.weight_scale, out_type=torch.float32, algo="naive")
        torch.cuda.synchronize()
        assert_rel(f32_np(c[rows]), f32_np(refc), TOL, f"expert {e} rows {r0}:{r1}")


def test_random_groupings_are_exact(dev):
    """A seeded sweep of groupings (empty, tiny, mid-size and >= 1024-row slots side by side, skipped experts, rows
    past the last slot, ragged and aligned N): on integer data the automatic choice -- large-tile launch, 128-row
    tiles, 32-row tiles -- equals the scalar kernel bit for bit on every row that belongs to a slot."""
    rng = np.random.default_rng(77)
    for it in range(36):
        E = int(rng.integers(1, 24))
        active = int(rng.integers(1, E + 1))
        if it % 3 == 0:
            counts = rng.integers(0, 70, active)
        elif it % 3 == 1:
            counts = rng.choice([0, 1, 5, 31, 32, 33, 127, 128, 129, 300, 1023, 1024, 1025, 1300, 2600], active)
        else:
            counts = (rng.zipf(1.3, active) * 7 % 3000).astype(np.int64)
        ids = rng.permutation(E)[:active].astype(np.int32)
        ids[rng.random(active) < 0.1] = -1
        extra = int(rng.integers(0, 9)) if it % 4 == 0 else 0
        N = 8 * int(rng.integers(8, 160)) if it % 2 else 128 * int(rng.integers(1, 12))
        K = 128 * int(rng.integers(1, 12))
        if counts.sum() == 0:
            counts[0] = 3
        live = int(counts.sum())
        T = live + extra
        a = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (T, K)).astype(np.float32)))
        b = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (E, N, K)).astype(np.float32)))
        sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (K // 128, -(-T // 4) * 4))).astype(np.float32))
        sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (E, -(-N // 128), K // 128))).astype(np.float32))
        off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32)
        idt = torch.tensor(list(ids) + [-1] * (E - active), dtype=torch.int32)
        out = torch.bfloat16 if it % 2 else torch.float32
        got = run(a, b, sa, sb, off, idt, int(counts.max()), active, dev, out=out)
        want = run(a, b, sa, sb, off, idt, int(counts.max()), active, dev, out=out, algo="naive")
        assert torch.equal(got[:live], want[:live]), f"case {it}: counts {counts.tolist()}, N {N}, K {K}, {out}"
