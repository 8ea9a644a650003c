"""GPU parity of the grouped (MoE) FP8 matmul with per-token x per-channel scales against the
oracle (one rowwise matmul per slot, max/kernels/src/linalg/grouped_matmul.mojo:1440-1541):
the slot layouts of the blockwise grouped tests, Llama-4-Scout-like sizes, expert id -1, empty
slots, rows past the last active slot left alone."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import synth
from test_gpu_grouped import CASES
from util import F32_BUDGET, assert_rel, f32_np, fp8_bytes, u32_np

pytestmark = pytest.mark.gpu
NT = oracle.default_threads()
TOL = 1e-2


def make(counts, ids, E, N, K, seed, extra_rows=0):
    T = int(sum(counts)) + extra_rows
    a, b = synth.random_fp8((T, K), seed), synth.random_fp8((E, N, K), seed + 1)
    sa = synth.random_scales((T, 1), seed + 2)
    sb = synth.random_scales((E, N, 1), seed + 3)
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32)
    ids = torch.tensor(list(ids) + [-1] * (E - len(ids)), dtype=torch.int32)
    return a, b, sa, sb, off, ids


def run(a, b, sa, sb, off, ids, max_tokens, num_active, dev, out=torch.float32, prefill=None):
    stats = torch.tensor([max_tokens, num_active], dtype=torch.int64).to(torch.uint32)
    c = mx.grouped_matmul_rowwise_dynamic_scaled_fp8(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev), off.to(dev), ids.to(dev),
                                                     stats, out_type=out)
    torch.cuda.synchronize()
    return c


def ref(a, b, sa, sb, off, ids, num_active):
    return oracle.grouped_matmul_rowwise(fp8_bytes(a), fp8_bytes(b), sa.numpy(), sb.numpy(), u32_np(off), ids.numpy(),
                                         num_active, threads=NT)


@pytest.mark.parametrize("counts,ids,E,N,K", CASES + [([300, 1100, 2, 40, 0, 600], [5, 0, 2, 1, 3, 4], 6, 640, 1024)])
@pytest.mark.parametrize("out", [torch.float32, torch.bfloat16])
def test_cases(dev, counts, ids, E, N, K, out):
    args = make(counts, ids, E, N, K, seed=sum(counts))
    c = run(*args, max(counts), len(counts), dev, out=out)
    want = ref(*args, len(counts))
    assert_rel(f32_np(c), want, TOL, "grouped rowwise", abs_budget=F32_BUDGET if out == torch.float32 else None)


def test_minus_one_expert_empty_slots_and_spare_rows(dev):
    counts4, ids4 = [40, 0, 130, 1], [2, 1, -1, 0]
    a, b, sa, sb, off, ids_t = make(counts4, ids4, 4, 384, 512, seed=3, extra_rows=9)
    c = run(a, b, sa, sb, off, ids_t, max(counts4), 4, dev)
    want = ref(a, b, sa, sb, off, ids_t, 4)
    live = slice(0, sum(counts4))
    assert_rel(f32_np(c)[live], want[live], TOL, "grouped rowwise", abs_budget=F32_BUDGET)
    lo = sum(counts4[:2])
    assert not f32_np(c)[lo:lo + counts4[2]].any(), "expert -1 must give zeros"


@pytest.mark.parametrize("launches", ["one persistent launch", "two launches"])
def test_exact_integers_are_bit_identical(dev, tune, launches):
    tune(MAXFP8_GROUPED_PERSIST=None if launches == "one persistent launch" else "0")
    counts, ids, E, N, K = [33, 1200, 7], [1, 0, 2], 3, 256, 256
    g = torch.Generator().manual_seed(0)
    T = sum(counts)
    a = torch.randint(-2, 3, (T, K), generator=g).float().to(torch.float8_e4m3fn)
    b = torch.randint(-2, 3, (E, N, K), generator=g).float().to(torch.float8_e4m3fn)
    sa = (2.0 ** torch.randint(-3, 4, (T, 1), generator=g)).float()
    sb = (2.0 ** torch.randint(-3, 4, (E, N, 1), generator=g)).float()
    off = torch.tensor([0, 33, 1233, 1240], dtype=torch.int64).to(torch.uint32)
    ids_t = torch.tensor(ids, dtype=torch.int32)
    c = run(a, b, sa, sb, off, ids_t, 1200, 3, dev)
    want = ref(a, b, sa, sb, off, ids_t, 3)
    assert np.array_equal(f32_np(c), want)
    # against plain integer arithmetic too
    z = (a[:33].double() @ b[1].double().T) * sa[:33].double() * sb[1].double().reshape(1, -1)
    assert np.array_equal(f32_np(c)[:33], z.float().numpy())


def test_llama4_scout_like(dev):
    # 16 experts, hidden 5120, expert intermediate 8192 (gate_up: N = 16384): 2048 tokens, top-1
    E, N, K = 16, 2048, 5120          # N cut to keep the CPU oracle quick
    counts = np.random.default_rng(0).multinomial(2048, np.ones(E) / E).tolist()
    args = make(counts, list(range(E)), E, N, K, seed=1)
    c = run(*args, max(counts), E, dev, out=torch.bfloat16)
    assert_rel(f32_np(c), ref(*args, E), TOL, "scout-like")


def test_errors(dev):
    a, b, sa, sb, off, ids = make([4, 4], [0, 1], 2, 128, 128, seed=0)
    stats = torch.tensor([4, 2], dtype=torch.int64).to(torch.uint32)
    f = mx.grouped_matmul_rowwise_dynamic_scaled_fp8
    with pytest.raises(ValueError, match="per-token a_scales"):
        f(a.to(dev), b.to(dev), sa.to(dev).T.contiguous(), sb.to(dev), off.to(dev), ids.to(dev), stats)
    with pytest.raises(ValueError, match="per-channel b_scales"):
        f(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev)[:, :64], off.to(dev), ids.to(dev), stats)
    with pytest.raises(TypeError, match="float32"):
        f(a.to(dev), b.to(dev), sa.to(dev).bfloat16(), sb.to(dev).bfloat16(), off.to(dev), ids.to(dev), stats)
    with pytest.raises(TypeError, match="int32"):
        f(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev), off.to(dev), ids.to(dev).long(), stats)
    none = torch.tensor([0, 0], dtype=torch.int64).to(torch.uint32)
    assert f(a.to(dev), b.to(dev), sa.to(dev), sb.to(dev), off.to(dev), ids.to(dev), none).shape == (8, 128)


def test_block_and_row_scaled_launches_in_flight_together(dev):
    """Two streams, one sending block-scaled and one row-scaled grouped matmuls, both busy at the same time: the
    launches take their tile counters from one pool in device memory, so no two launches in flight may be handed the
    same set.  Every result equals the one the same call gives alone."""
    import test_gpu_grouped as blk
    counts, ids, E, N, K = [300, 1100, 2, 40, 0, 600, 31, 129], [5, 0, 2, 1, 3, 4, 6, 7], 8, 640, 1024
    stats = torch.tensor([max(counts), len(counts)], dtype=torch.int64).to(torch.uint32)
    ops_b = [t.to(dev) for t in blk.make(counts, ids, E, N, K, seed=21)]
    ops_r = [t.to(dev) for t in make(counts, ids, E, N, K, seed=22)]
    call_b = lambda: mx.grouped_dynamic_scaled_fp8_matmul(*ops_b, stats, blk.BLK.input_scale, blk.BLK.weight_scale,
                                                          out_type=torch.bfloat16)
    call_r = lambda: mx.grouped_matmul_rowwise_dynamic_scaled_fp8(*ops_r, stats, out_type=torch.bfloat16)
    want_b, want_r = call_b(), call_r()
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    got_b, got_r = [], []
    for _ in range(12):
        with torch.cuda.stream(s1):
            got_b.append(call_b())
        with torch.cuda.stream(s2):
            got_r.append(call_r())
    torch.cuda.synchronize()
    live = sum(counts)
    for i, (gb, gr) in enumerate(zip(got_b, got_r)):
        assert torch.equal(gb[:live], want_b[:live]), f"block-scaled launch {i}"
        assert torch.equal(gr[:live], want_r[:live]), f"row-scaled launch {i}"


def test_four_wave_launch_beside_the_persistent_one(dev, tune):
    """Row scaling on the two launches side by side (the slots' full 192-row tiles and the rests behind them on the grouped
    form of the four-wave kernel, the other rows on the persistent launch): the bits of the one persistent launch
    (MAXFP8_GROUPED_W4=0) on a sweep of groupings around the bounds of the rule that shares the rows out, with a skipped
    expert, rows past the last slot and a ragged N; one of them against the oracle."""
    rng = np.random.default_rng(21)
    for it in range(10):
        E = int(rng.integers(2, 14))
        active = int(rng.integers(1, E + 1))
        counts = rng.choice([0, 5, 33, 128, 129, 191, 192, 193, 225, 385, 700, 1300], active)
        ids = rng.permutation(E)[:active].astype(np.int32)
        if active > 1 and it % 3 == 0:
            ids[int(rng.integers(0, active))] = -1
        if counts.sum() == 0:
            counts[0] = 200
        N = 8 * int(rng.integers(8, 120)) if it % 2 else 128 * int(rng.integers(1, 9))
        K = 256 * int(rng.integers(2, 6))
        args = make(list(counts), list(ids), E, N, K, seed=it, extra_rows=int(it % 4 == 0) * 5)
        tune(MAXFP8_GROUPED_W4=None, MAXFP8_GROUPED_W4_ROWS="0")
        got = run(*args, int(counts.max()), active, dev, out=torch.bfloat16)
        tune(MAXFP8_GROUPED_W4="0")
        want = run(*args, int(counts.max()), active, dev, out=torch.bfloat16)
        live = int(counts.sum())
        assert torch.equal(got[:live], want[:live]), f"case {it}: counts {counts.tolist()}, ids {ids.tolist()}, N {N}, K {K}"
        if it == 1:
            assert_rel(f32_np(got)[:live], ref(*args, active)[:live], TOL, "grouped rowwise, two launches")
