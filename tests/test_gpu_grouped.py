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
from util import F32_BUDGET, assert_rel, bf16_bits, f32_np, fp8_bytes, fp8_from_bytes, u32_np

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


@pytest.mark.parametrize("proj,Kd,Nd", [("gate_up", 7168, 4096), ("down", 2048, 7168)])
def test_moe_config_sampled(dev, proj, Kd, Nd):
    # 256 experts, top-8 of 4096 tokens with Zipf(1.1) popularity; both expert matmuls of the DeepSeek-V3 layer
    # (gate_up: hidden 7168 -> 2 * 2048; down: 2048 -> 7168) at full size, 32768 routed rows.
    E = 256
    off, ids, counts, stats = synth.moe_routing(4096, E, 8, seed=0, device=dev)
    T = int(counts.sum())
    assert T == 32768
    x = synth.activations(T, Kd, seed=0, outlier_frac=0.01 if proj == "gate_up" else 0.0, device=dev)
    q, sa = mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32)
    del x
    w = torch.empty((E, Nd, Kd), dtype=torch.float8_e4m3fn, device=dev)
    sb = torch.empty((E, Nd // 128, Kd // 128), dtype=torch.float32, device=dev)
    for e0 in range(0, E, 16):
        wq, ws = synth.quantize_weight_block(synth.weights_f32(16 * Nd, Kd, seed=100 + e0, device=dev).reshape(16, Nd, Kd))
        w[e0:e0 + 16], sb[e0:e0 + 16] = wq, ws
    c = mx.grouped_dynamic_scaled_fp8_matmul(q, w, sa, sb, off, ids, stats, BLK.input_scale, BLK.weight_scale)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(c.float()).all())
    offs = u32_np(off).astype(np.int64)
    order = np.argsort(-counts.numpy())
    # the two biggest experts, the three smallest, two of medium size (a few 128-row tiles) and two arbitrary ones
    mid = [int(e) for e in order if 129 <= counts[e] <= 1023][:2]
    for e in list(order[:2]) + list(order[-3:]) + mid + [17, 128]:
        r0, r1 = offs[e], offs[e + 1]
        if r1 == r0:
            continue
        # rows spread over the slot, its last row included (the slot's ragged last tile)
        rows = torch.unique(torch.cat([torch.arange(r0, r1, max(1, (r1 - r0) // 8), device=dev)[:8], torch.tensor([r1 - 1], device=dev)]))
        refc = mx.dynamic_scaled_matmul(q[rows].contiguous(), w[e], sa[:, rows].contiguous(), sb[e], BLK.input_scale,
                                        BLK.weight_scale, out_type=torch.float32, algo="naive")
        torch.cuda.synchronize()
        assert_rel(f32_np(c[rows]), f32_np(refc), TOL, f"{proj}: expert {e} rows {r0}:{r1}", natural_scale=True)
    # one row of the biggest expert against the CPU oracle itself
    e = int(order[0])
    r = int(offs[e])
    cpu = oracle.matmul_blockwise(fp8_bytes(q[r:r + 1]), fp8_bytes(w[e]), f32_np(sa[:, r:r + 1]), f32_np(sb[e]), threads=NT)
    assert_rel(f32_np(c[r:r + 1]), cpu, TOL, f"{proj}: row {r} against the CPU oracle", natural_scale=True)


@pytest.mark.parametrize("launches", ["one persistent launch", "two launches"])
def test_random_groupings_are_exact(dev, tune, launches):
    """A seeded sweep of groupings (empty, tiny, mid-size and >= 1024-row slots side by side, skipped experts, rows
    past the last slot, ragged and aligned N): on integer data the automatic choice -- 256-row tiles, 128-row
    tiles, the weight-streaming form of at most 32 rows; as one persistent launch (the default) and as the two
    launches behind MAXFP8_GROUPED_PERSIST=0 -- equals the scalar kernel bit for bit on every row that belongs
    to a slot."""
    tune(MAXFP8_GROUPED_PERSIST=None if launches == "one persistent launch" else "0")
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


def test_four_wave_launch_beside_the_persistent_one_is_exact(dev, tune):
    """Block scaling with K an even number (at least four) of slabs: the slots' full 192-row tiles, and a rest of more
    than 32 rows behind them (more than 128 rows for a slot without a full tile), go to the grouped form of the
    four-wave kernel, the other rows to the persistent launch on a second stream.  A seeded sweep of groupings around
    those bounds (191 / 192 / 193, 224 / 225, 320 / 321, 128 / 129 rows, empty slots, skipped experts, rows past the
    last slot, ragged N) on integer data: every row that belongs to a slot equals the scalar kernel's bit for bit, with
    the rule's bounds at their defaults and moved (every rest to the four-wave launch; none)."""
    rng = np.random.default_rng(5)
    for it in range(30):
        hot, cold = [("32", "128"), ("0", "32"), ("128", "128")][it % 3]
        tune(MAXFP8_GROUPED_W4_ROWS="0", MAXFP8_GROUPED_W4_HOT_REST=hot, MAXFP8_GROUPED_W4_COLD_ROWS=cold)
        E = int(rng.integers(1, 24))
        active = int(rng.integers(1, E + 1))
        if it % 3 == 0:
            counts = rng.choice([0, 5, 128, 129, 191, 192, 193, 224, 225, 320, 321, 383, 384, 385, 1000], active)
        elif it % 3 == 1:
            counts = rng.choice([0, 1, 32, 33, 129, 192, 300, 1023, 1024, 1300, 2600], active)
        else:
            counts = (rng.zipf(1.3, active) * 97 % 3000).astype(np.int64)
        ids = rng.permutation(E)[:active].astype(np.int32)
        ids[rng.random(active) < 0.1] = -1
        extra = int(rng.integers(0, 9)) if it % 4 == 0 else 0
        N = 8 * int(rng.integers(8, 160)) if it % 2 else 128 * int(rng.integers(1, 12))
        K = 256 * int(rng.integers(2, 7))
        if counts.sum() == 0:
            counts[0] = 200
        live = int(counts.sum())
        T = live + extra
        a = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (T, K)).astype(np.float32)))
        b = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (E, N, K)).astype(np.float32)))
        sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (K // 128, -(-T // 4) * 4))).astype(np.float32))
        sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (E, -(-N // 128), K // 128))).astype(np.float32))
        off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32)
        idt = torch.tensor(list(ids) + [-1] * (E - active), dtype=torch.int32)
        got = run(a, b, sa, sb, off, idt, int(counts.max()), active, dev, out=torch.bfloat16, fill=None)
        want = run(a, b, sa, sb, off, idt, int(counts.max()), active, dev, out=torch.bfloat16, algo="naive")
        assert torch.equal(got[:live], want[:live]), f"case {it}: counts {counts.tolist()}, ids {ids.tolist()}, N {N}, K {K}"
    # a slot of more than 24 row tiles (its tiles are walked in groups of 12 row tiles) between small ones
    tune(MAXFP8_GROUPED_W4_ROWS="0", MAXFP8_GROUPED_W4_HOT_REST=None, MAXFP8_GROUPED_W4_COLD_ROWS=None)
    counts, N, K = np.array([40, 5003, 200, 7]), 776, 512
    T = int(counts.sum())
    a = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (T, K)).astype(np.float32)))
    b = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (4, N, K)).astype(np.float32)))
    sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (K // 128, -(-T // 4) * 4))).astype(np.float32))
    sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (4, -(-N // 128), K // 128))).astype(np.float32))
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32)
    idt = torch.tensor([2, 0, 3, 1], dtype=torch.int32)
    got = run(a, b, sa, sb, off, idt, 5003, 4, dev, out=torch.bfloat16)
    want = run(a, b, sa, sb, off, idt, 5003, 4, dev, out=torch.bfloat16, algo="naive")
    assert torch.equal(got, want), "a slot of 27 row tiles"


def test_four_wave_launch_with_a_row_index(dev, tune):
    """The row index on C (row m of the result is stored at row index[m]: the MoE layer's restore of the token order) on
    the two launches side by side: the four-wave kernel copies the index entries of a tile's rows into LDS and stores
    each row through them.  Integer data, groupings around the bounds of the rule that shares the rows out, ragged N,
    skipped experts: equal to the one-launch form's result, and to the result without an index permuted afterwards."""
    rng = np.random.default_rng(9)
    for it in range(12):
        E = int(rng.integers(1, 20))
        active = int(rng.integers(1, E + 1))
        counts = rng.choice([0, 5, 33, 129, 191, 192, 193, 225, 385, 1000, 1300], active)
        ids = rng.permutation(E)[:active].astype(np.int32)
        ids[rng.random(active) < 0.1] = -1
        if counts.sum() == 0:
            counts[0] = 200
        T = int(counts.sum())
        N = 8 * int(rng.integers(8, 160)) if it % 2 else 128 * int(rng.integers(1, 12))
        K = 256 * int(rng.integers(2, 6))
        a = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (T, K)).astype(np.float32))).to(dev)
        b = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (E, N, K)).astype(np.float32))).to(dev)
        sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (K // 128, -(-T // 4) * 4))).astype(np.float32)).to(dev)
        sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (E, -(-N // 128), K // 128))).astype(np.float32)).to(dev)
        off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32).to(dev)
        idt = torch.tensor(list(ids) + [-1] * (E - active), dtype=torch.int32).to(dev)
        perm = torch.from_numpy(rng.permutation(T).astype(np.int64)).to(dev)
        stats = torch.tensor([int(counts.max()), active], dtype=torch.int64).to(torch.uint32)

        def go(index):
            return mx.grouped_dynamic_scaled_fp8_matmul(a, b, sa, sb, off, idt, stats, BLK.input_scale, BLK.weight_scale,
                                                        out_type=torch.bfloat16, out_row_index=index)

        tune(MAXFP8_GROUPED_W4=None, MAXFP8_GROUPED_W4_ROWS="0")
        got, plain = go(perm.to(torch.uint32)), go(None)
        tune(MAXFP8_GROUPED_W4="0")
        want = go(perm.to(torch.uint32))
        torch.cuda.synchronize()
        what = f"case {it}: counts {counts.tolist()}, ids {ids.tolist()}, N {N}, K {K}"
        assert torch.equal(got, want), what + ": differs from the one-launch form"
        back = torch.empty_like(plain)
        back[perm] = plain
        assert torch.equal(got, back), what + ": differs from the plain result permuted"


def test_four_wave_launch_has_the_bits_of_the_one_launch_form(dev, tune):
    """Random (inexact) data on a skewed routing of 64 experts: both forms add a row's products up in the same order,
    so the two launches side by side give the bits of the one persistent launch -- also with a share of the chip forced
    on the four-wave launch that is too small and too large, and on twelve launches in a row (each block works its
    share out again, and the second stream is joined every time)."""
    off, ids, counts, stats = synth.moe_routing(1024, 64, 8, seed=3, zipf_a=1.1)
    T, N, K = int(counts.sum()), 1024, 1024
    a, b = synth.random_fp8((T, K), 11).to(dev), synth.random_fp8((64, N, K), 12).to(dev)
    sa = synth.random_scales((K // 128, T), 13).to(dev)
    sb = synth.random_scales((64, N // 128, K // 128), 14).to(dev)
    off, ids = off.to(dev), ids.to(dev)
    assert int(counts.max()) >= 192 and int((counts % 192 <= 32).sum()) > 0

    def launch():
        return mx.grouped_dynamic_scaled_fp8_matmul(a, b, sa, sb, off, ids, stats, BLK.input_scale, BLK.weight_scale,
                                                    out_type=torch.bfloat16)

    tune(MAXFP8_GROUPED_W4="0")
    want = launch()
    torch.cuda.synchronize()
    for share in (None, "-8", "-256"):
        tune(MAXFP8_GROUPED_W4=None, MAXFP8_GROUPED_W4_SHARE=share)
        outs = [launch() for _ in range(12)]
        torch.cuda.synchronize()
        for i, got in enumerate(outs):
            assert torch.equal(got, want), f"share {share}, launch {i}"
    r = int(torch.argmax(counts))
    row = int(counts[:r].sum())
    cpu = oracle.matmul_blockwise(fp8_bytes(a[row:row + 1]), fp8_bytes(b[r]), f32_np(sa[:, row:row + 1]), f32_np(sb[r]), threads=NT)
    assert_rel(f32_np(want[row:row + 1]), cpu, TOL, "a row of the largest slot against the CPU oracle", natural_scale=True)


@pytest.mark.parametrize("counts,N", [([1024] * 8, 2048), ([8] * 100, 1024), ([200] * 40, 512), ([100] * 30 + [1300] * 3, 768)])
def test_launches_of_one_kind_of_tile_many_times(dev, counts, N):
    """A grouping whose tiles are all of one kind (256-row tiles only; streaming tiles only; one mid-size kind) leaves
    most (kind, XCD) counters of the persistent launch without work from the start and the others empty at the same
    moment: the blocks' search for the next pair that still has tiles, and the counters' return to zero, decide the
    result.  More launches than there are counter sets (64), every one equal to the scalar kernel's result."""
    rng = np.random.default_rng(len(counts) + N)
    E, K = len(counts), 256
    T = sum(counts)
    a = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (T, K)).astype(np.float32)))
    b = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (E, N, K)).astype(np.float32)))
    sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (K // 128, -(-T // 4) * 4))).astype(np.float32))
    sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (E, -(-N // 128), K // 128))).astype(np.float32))
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32)
    idt = torch.arange(E, dtype=torch.int32)
    want = run(a, b, sa, sb, off, idt, max(counts), E, dev, out=torch.bfloat16, algo="naive")
    for launch in range(70):
        got = run(a, b, sa, sb, off, idt, max(counts), E, dev, out=torch.bfloat16)
        assert torch.equal(got, want), f"launch {launch}"


def test_recorded_launch_replays_beside_eager_launches(dev):
    """A grouped matmul recorded into a HIP graph keeps the counter set of the recording in every replay.  Replays run on
    one stream while more eager launches than there are counter sets (64) run on another: were the recorded launch's set
    one of those the eager launches draw from, a replay and an eager launch would sooner or later claim tiles from the
    same counters at the same time.  Every result of both streams equals the scalar kernel's."""
    rng = np.random.default_rng(77)
    counts, N, K = [300] * 24 + [20] * 40, 1024, 512
    E, T = len(counts), sum(counts)
    a = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (T, K)).astype(np.float32))).to(dev)
    b = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (E, N, K)).astype(np.float32))).to(dev)
    sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (K // 128, -(-T // 4) * 4))).astype(np.float32)).to(dev)
    sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (E, N // 128, K // 128))).astype(np.float32)).to(dev)
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32).to(dev)
    idt = torch.arange(E, dtype=torch.int32).to(dev)
    stats = torch.tensor([max(counts), E], dtype=torch.int64).to(torch.uint32)

    def launch(algo="auto"):
        return mx.grouped_dynamic_scaled_fp8_matmul(a, b, sa, sb, off, idt, stats, BLK.input_scale, BLK.weight_scale,
                                                    out_type=torch.bfloat16, algo=algo)

    want = launch("naive")
    launch()  # (outside the capture: the kernel's LDS attribute is set at the first launch)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = launch()
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    eager = []
    for i in range(72):
        if i % 6 == 0:
            recorded.zero_()
            graph.replay()  # on the current stream, beside the launches of the other
        with torch.cuda.stream(side):
            eager.append(launch())
        if i % 6 == 5:
            torch.cuda.synchronize()
            assert torch.equal(recorded, want), f"replay before eager launch {i}"
    torch.cuda.synchronize()
    for i, got in enumerate(eager):
        assert torch.equal(got, want), f"eager launch {i}"


def test_more_slots_than_the_persistent_launch_holds(dev):
    """600 active slots: more than the persistent launch's tables hold (512), so the two-launch form runs; exact on
    integer data like every other path."""
    rng = np.random.default_rng(5)
    E, N, K = 600, 128, 256
    counts = rng.integers(0, 5, E)
    counts[7] = 140
    T = int(counts.sum())
    a = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (T, K)).astype(np.float32)))
    b = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (E, N, K)).astype(np.float32)))
    sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (K // 128, -(-T // 4) * 4))).astype(np.float32))
    sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (E, 1, K // 128))).astype(np.float32))
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32)
    ids = torch.from_numpy(rng.permutation(E).astype(np.int32))
    got = run(a, b, sa, sb, off, ids, int(counts.max()), E, dev)
    want = run(a, b, sa, sb, off, ids, int(counts.max()), E, dev, algo="naive")
    assert torch.equal(got, want)


# ---- the layer above the op: quantized_grouped_matmul and Fp8Strategy -----------------------------------

def test_quantized_grouped_matmul_from_the_storage_layout(dev):
    """quant_ops.py:880-1007: bf16 rows sorted by expert, weights and block scales in STORAGE layout [E, K, N] /
    [E, K/128, N/128].  The entry point transposes both to the kernel's orientation, quantises x in 1 x 128 groups and
    runs the grouped matmul: against the oracle's quantiser + grouped matmul on the K-innermost operands."""
    from modular_amd import quant_ops
    counts, ids, E, N, K = [20, 1500, 300, 28], [0, 3, 2, 4], 5, 256, 512
    T = sum(counts)
    x = synth.activations(T, K, seed=3)
    w_nk, s_nk = synth.quantize_weight_block(synth.weights_f32(E * N, K, seed=4).reshape(E, N, K))   # kernel orientation
    w_store = w_nk.view(torch.uint8).transpose(1, 2).contiguous().view(torch.float8_e4m3fn)            # [E, K, N]
    s_store = s_nk.transpose(1, 2).contiguous()                                                         # [E, K/128, N/128]
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32)
    ids_t = torch.tensor(ids + [-1] * (E - len(ids)), dtype=torch.int32)
    stats = torch.tensor([max(counts), len(counts)], dtype=torch.int64).to(torch.uint32)
    wd, sd = w_store.to(dev), s_store.to(dev)
    y = quant_ops.quantized_grouped_matmul(x.to(dev), wd, sd, off.to(dev), ids_t.to(dev), stats.to(dev), BLK)
    torch.cuda.synchronize()
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (T, N)
    q, sa = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x), 128, threads=NT)
    want = oracle.grouped_matmul(q, fp8_bytes(w_nk), sa, s_nk.numpy(), u32_np(off), ids_t.numpy(), max(counts), len(counts), threads=NT)
    assert_rel(f32_np(y), want, TOL, "quantized_grouped_matmul", natural_scale=True)
    # the K-innermost copy is made once per storage tensor, and again after an in-place write
    n_cached = len(quant_ops._K_INNERMOST)
    y2 = quant_ops.quantized_grouped_matmul(x.to(dev), wd, sd, off.to(dev), ids_t.to(dev), stats, BLK)
    assert len(quant_ops._K_INNERMOST) == n_cached and torch.equal(y, y2)
    wd.view(torch.uint8)[3].zero_()   # expert 3 serves slot 1
    y3 = quant_ops.quantized_grouped_matmul(x.to(dev), wd, sd, off.to(dev), ids_t.to(dev), stats, BLK)
    assert len(quant_ops._K_INNERMOST) == n_cached, "the tensor's entry is replaced, not added to"
    # weights already in the kernel's orientation (transposed once at load time)
    y4 = quant_ops.quantized_grouped_matmul(x.to(dev), wd.view(torch.uint8).transpose(1, 2).contiguous().view(wd.dtype),
                                            sd.transpose(1, 2).contiguous(), off.to(dev), ids_t.to(dev), stats, BLK, k_innermost=True)
    assert torch.equal(y4, y3) and len(quant_ops._K_INNERMOST) == n_cached
    lo = counts[0] + counts[1]
    assert torch.equal(y3[:counts[0]], y[:counts[0]]) and torch.equal(y3[lo:], y[lo:]) and not y3[counts[0]:lo].float().any()


def test_quantized_grouped_matmul_per_channel_layout(dev):
    """The compressed-tensors FP8-dynamic layout (quant_ops.py:945-981): per-channel weight scales [E, N, 1] used as
    they are, per-token activation scales [1, T] handed to the kernel as [T, 1]."""
    from modular_amd import quant_ops
    ROWCFG = mx.rowwise_fp8_config()
    counts, ids, E, N, K = [40, 0, 130, 1], [2, 1, 3, 0], 4, 384, 512
    T = sum(counts)
    x = synth.activations(T, K, seed=5, outlier_frac=0.0)
    w_nk, s_nk = synth.quantize_weight_rowwise(synth.weights_f32(E * N, K, seed=6))
    w_nk, s_nk = w_nk.reshape(E, N, K), s_nk.reshape(E, N, 1)
    w_store = w_nk.view(torch.uint8).transpose(1, 2).contiguous().view(torch.float8_e4m3fn)
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32)
    ids_t = torch.tensor(ids, dtype=torch.int32)
    stats = torch.tensor([max(counts), len(counts)], dtype=torch.int64).to(torch.uint32)
    y = quant_ops.quantized_grouped_matmul(x.to(dev), w_store.to(dev), s_nk.to(dev), off.to(dev), ids_t.to(dev), stats, ROWCFG)
    torch.cuda.synchronize()
    q, sa = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x), K, threads=NT)          # [1, T]
    want = oracle.grouped_matmul_rowwise(q, fp8_bytes(w_nk), sa.reshape(T, 1), s_nk.numpy(), u32_np(off), ids_t.numpy(), len(counts), threads=NT)
    assert_rel(f32_np(y), want, TOL, "quantized_grouped_matmul, per-channel", natural_scale=True)


def test_fp8_strategy_methods(dev):
    """moe/quant_strategy.py:114-215: quantize / grouped_quantize / grouped_matmul / prepare_weight_scales /
    fused_silu_quantize do what the ops they forward to do."""
    counts, ids, E, N, K = [7, 0, 129, 0, 128], [2, 1, 0, 3, 4], 5, 256, 384
    T = sum(counts)
    st = mx.Fp8Strategy(BLK, torch.float8_e4m3fn)
    x = synth.activations(T, K, seed=7).to(dev)
    xq, xs = st.quantize(x, 128)
    q0, s0 = mx.quantize_dynamic_scaled_float8(x, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32, group_size_or_per_token=128)
    assert torch.equal(xq.view(torch.uint8), q0.view(torch.uint8)) and torch.equal(xs[:, :T], s0[:, :T]) and xs.dtype == torch.float32
    g2 = st.grouped_quantize(x, 128, None, None, None, None)
    assert torch.equal(g2[0].view(torch.uint8), xq.view(torch.uint8))
    w, sw = synth.quantize_weight_block(synth.weights_f32(E * N, K, seed=8).reshape(E, N, K))
    a, b = st.prepare_weight_scales(sw, sw, dev)
    assert a is sw and b is sw
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32).to(dev)
    ids_t = torch.tensor(ids, dtype=torch.int32, device=dev)
    stats = torch.tensor([max(counts), len(counts)], dtype=torch.int64).to(torch.uint32).to(dev)   # on the device: copied to the host inside
    inputs = (xq, xs, off, ids_t, stats)
    y = st.grouped_matmul(w.to(dev), sw.to(dev), expert_inputs=inputs)
    want = mx.grouped_dynamic_scaled_fp8_matmul(xq, w.to(dev), xs, sw.to(dev), off, ids_t, stats.cpu(), BLK.input_scale, BLK.weight_scale)
    assert torch.equal(y, want)
    hq, hs = st.fused_silu_quantize(y, expert_inputs=inputs)
    wq_, ws_ = mx.fused_silu_quantized(y, off, BLK)
    assert torch.equal(hq.view(torch.uint8), wq_.view(torch.uint8)) and torch.equal(hs, ws_)
    with pytest.raises(AssertionError):
        st.fused_silu_quantize(y, expert_inputs=inputs, clamp_activation=True)


@pytest.mark.parametrize("algo", ["auto", "naive"])
def test_offsets_beyond_the_rows_are_held_to_the_buffers(dev, algo):
    """expert_start_indices is read on the device.  Entries beyond T (a stale or damaged routing tensor) are held
    to T: the slot ends with the buffers, no row outside them is read or written."""
    counts, ids, E, N, K = [10, 30], [1, 0], 2, 256, 256
    a, b, sa, sb, off, ids_t = make(counts, ids, E, N, K, seed=9)
    good = run(a, b, sa, sb, off, ids_t, 40, 2, dev, algo=algo)
    wild = torch.tensor([0, 10, 1 << 30], dtype=torch.int64).to(torch.uint32)
    got = run(a, b, sa, sb, wild, ids_t, 40, 2, dev, algo=algo)
    assert torch.equal(good, got)
