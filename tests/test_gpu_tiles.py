"""Every tile shape, the split-K path and the workspace contract of the tiled MFMA matmul,
and the two tile kinds of the grouped kernel, on cases whose arithmetic is exact (small
integers, power-of-two scales: any summation order gives the same f32) plus tolerance checks
against the CPU oracle.  The shapes cut tiles in M, N and K and leave N off the 8-column store
width, which is where the edge handling of the kernels lives."""
import ctypes

import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import _lib, synth
from test_gpu_matmul import BLK, ROW, TOL, exact_case, make_block, mm, oracle_block
from test_gpu_grouped import make as make_grouped, ref as ref_grouped, run as run_grouped
from util import F32_BUDGET, assert_rel, f32_np, fp8_bytes, fp8_from_bytes

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tile", ["1", "2", "3", "4"])
@pytest.mark.parametrize("M,N,K", [(300, 392, 1040), (257, 100, 512), (64, 129, 384), (513, 520, 256)])
def test_each_tile_shape_exact(dev, tune, tile, M, N, K):
    tune(MAXFP8_TILE=tile)
    a, b, sa, sb, want = exact_case(M, N, K, seed=M + N + K)
    got = f32_np(mm(a, b, sa, sb, BLK, dev, algo="tiled")).astype(np.float64)
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"tile {tile}: {len(bad)} mismatches, first at {bad[:4].tolist()}"
    cb = mm(a, b, sa, sb, BLK, dev, out=torch.bfloat16, algo="tiled")
    assert torch.equal(cb.cpu(), torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16))


@pytest.mark.parametrize("tile", ["1", "2", "3"])
def test_each_tile_shape_rowwise(dev, tune, tile):
    tune(MAXFP8_TILE=tile)
    M, N, K = 300, 1044, 1024
    a, b = synth.random_fp8((M, K), M), synth.random_fp8((N, K), N)
    sa, sb = synth.random_scales((1, M), 3, lo=0.01, hi=0.1), synth.random_scales((N, 1), 4, lo=0.001, hi=0.01)
    ref = oracle.matmul_rowwise(fp8_bytes(a), fp8_bytes(b), sa.numpy(), sb.numpy())
    for out in (torch.float32, torch.bfloat16):
        assert_rel(f32_np(mm(a, b, sa, sb, ROW, dev, out=out, algo="tiled")), ref, TOL, f"tile {tile} {out}",
                   F32_BUDGET if out == torch.float32 else None)


@pytest.mark.parametrize("splits", ["2", "3", "4"])
@pytest.mark.parametrize("kind", ["block", "row"])
def test_split_k_exact(dev, tune, splits, kind):
    # forced split counts (at most one per 4 slabs); the shares are uneven (17 slabs)
    tune(MAXFP8_SPLITK=splits)
    M, N, K = 130, 264, 17 * 128
    if kind == "block":
        a, b, sa, sb, want = exact_case(M, N, K, seed=int(splits))
        cfg = BLK
    else:
        rng = np.random.default_rng(7)
        ai, bi = rng.integers(-4, 5, (M, K)), rng.integers(-4, 5, (N, K))
        a = fp8_from_bytes(oracle.e4m3fn_encode(ai.astype(np.float32)))
        b = fp8_from_bytes(oracle.e4m3fn_encode(bi.astype(np.float32)))
        sa = torch.from_numpy(np.exp2(rng.integers(-3, 3, (1, M))).astype(np.float32))
        sb = torch.from_numpy(np.exp2(rng.integers(-3, 3, (N, 1))).astype(np.float32))
        want = (ai @ bi.T) * sa.numpy().reshape(-1, 1) * sb.numpy().reshape(1, -1)
        cfg = ROW
    assert _lib.lib().maxfp8_matmul_workspace_bytes(M, N, K) >= int(splits) * M * N * 4
    got = f32_np(mm(a, b, sa, sb, cfg, dev, algo="tiled")).astype(np.float64)
    assert np.array_equal(got, want)
    cb = mm(a, b, sa, sb, cfg, dev, out=torch.bfloat16, algo="tiled")
    assert torch.equal(cb.cpu(), torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16))


def test_split_k_chosen_for_a_small_grid(dev):
    # 2 x 2 tiles of 128 on a 256-CU chip with K = 8192: the cost model splits K when it is
    # given workspace; with and without it the result meets the tolerance
    M, N, K = 256, 256, 8192
    assert _lib.lib().maxfp8_matmul_workspace_bytes(M, N, K) > 0
    a, b, sa, sb = make_block(M, N, K, seed=5)
    ref = oracle_block(a, b, sa, sb)
    c_split = f32_np(mm(a, b, sa, sb, BLK, dev, algo="tiled"))
    assert_rel(c_split, ref, TOL, "split-K", F32_BUDGET)
    c_plain = f32_np(_call_abi(a, b, sa, sb, dev, workspace=None))
    assert_rel(c_plain, ref, TOL, "no workspace", F32_BUDGET)


def _call_abi(a, b, sa, sb, dev, workspace, workspace_bytes=0, algo=2):
    """maxfp8_matmul_dynamic_scaled_fp8 through the C ABI, blockwise 1x128 / 128x128, f32 out."""
    L = _lib.lib()
    a, b, sa, sb = a.to(dev), b.to(dev), sa.to(dev), sb.to(dev)
    M, K = a.shape
    N = b.shape[0]
    c = torch.empty((M, N), dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    rc = L.maxfp8_matmul_dynamic_scaled_fp8(
        ctypes.c_void_p(c.data_ptr()), ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(b.data_ptr()),
        ctypes.c_void_p(sa.data_ptr()), ctypes.c_void_p(sb.data_ptr()), M, N, K, K, K, N,
        3, 3, 1, 128, 128, sa.shape[1], sb.shape[1], 2, 2, algo,
        ctypes.c_void_p(workspace), workspace_bytes, ctypes.c_void_p(stream))
    torch.cuda.synchronize()
    if rc != 0:
        raise RuntimeError((rc, L.maxfp8_last_error().decode()))
    return c


def test_workspace_contract(dev):
    M, N, K = 256, 256, 8192
    a, b, sa, sb = make_block(M, N, K, seed=9)
    need = _lib.lib().maxfp8_matmul_workspace_bytes(M, N, K)
    ws = torch.empty(need + 64, dtype=torch.uint8, device=dev)
    full = _call_abi(a, b, sa, sb, dev, ws.data_ptr(), need)
    # a workspace that is too small is not an error: the matmul runs unsplit
    small = _call_abi(a, b, sa, sb, dev, ws.data_ptr(), 1024)
    plain = _call_abi(a, b, sa, sb, dev, None)
    assert torch.equal(small, plain)
    assert_rel(f32_np(full), f32_np(plain), 1e-4, "split vs unsplit", F32_BUDGET)
    # a misaligned workspace is refused
    with pytest.raises(RuntimeError) as e:
        _call_abi(a, b, sa, sb, dev, ws.data_ptr() + 4, need)
    assert e.value.args[0][0] == -3  # MAXFP8_ERR_ALIGN


GROUPED = [
    # small tiles (<= 32 rows), big tiles, their boundaries, empty slots, a slot without expert
    ([0, 1, 31, 32, 33, 129, 300], [3, 0, 6, 1, -1, 2, 5], 7, 200, 384),
    ([32] * 6, [5, 4, 3, 2, 1, 0], 6, 100, 256),
    ([1, 257, 2, 128], [0, 1, 2, 3], 4, 392, 512),
    # slots of 1024 rows and more give their full 256-row tiles to the large-tile launch
    ([1030, 0, 2050, 31], [2, 1, -1, 0], 4, 392, 256),
    ([1024, 1279, 5], [1, 0, 2], 3, 264, 384),
]


@pytest.mark.parametrize("tile", ["0", "2", "3", "4"])
@pytest.mark.parametrize("counts,ids,E,N,K", GROUPED)
@pytest.mark.parametrize("out", [torch.float32, torch.bfloat16])
def test_grouped_tile_kinds(dev, tune, tile, counts, ids, E, N, K, out):
    tune(MAXFP8_TILE=tile)
    args = make_grouped(counts, ids, E, N, K, seed=sum(counts) + N)
    c = run_grouped(*args, max(counts), len(counts), dev, out=out, algo="tiled")
    assert_rel(f32_np(c), ref_grouped(*args, max(counts), len(counts)), TOL, f"grouped {counts} tile {tile}",
               F32_BUDGET if out == torch.float32 else None)


def test_grouped_small_tiles_exact(dev):
    # integer data and power-of-two scales through the small-tile path: bit-exact
    rng = np.random.default_rng(3)
    counts, E, N, K = [5, 32, 17, 0, 9], 5, 264, 640
    T = sum(counts)
    ai, bi = rng.integers(-4, 5, (T, K)), rng.integers(-4, 5, (E, N, K))
    a = fp8_from_bytes(oracle.e4m3fn_encode(ai.astype(np.float32)))
    b = fp8_from_bytes(oracle.e4m3fn_encode(bi.astype(np.float32).reshape(E * N, K))).reshape(E, N, K)
    kb, nb = K // 128, -(-N // 128)
    ea, eb = rng.integers(-3, 4, (kb, -(-T // 4) * 4)), rng.integers(-3, 4, (E, nb, kb))
    sa = torch.from_numpy(np.exp2(ea).astype(np.float32))
    sb = torch.from_numpy(np.exp2(eb).astype(np.float32))
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)).to(torch.uint32)
    ids = torch.tensor([4, 2, 0, 1, 3], dtype=torch.int32)
    want = np.zeros((T, N))
    for z, e in enumerate(ids.tolist()):
        r0, r1 = int(off[z]), int(off[z + 1])
        for j in range(kb):
            part = ai[r0:r1, j * 128:(j + 1) * 128] @ bi[e][:, j * 128:(j + 1) * 128].T
            want[r0:r1] += part * np.exp2(ea[j, r0:r1])[:, None] * np.exp2(eb[e][np.arange(N) // 128, j])[None, :]
    c = run_grouped(a, b, sa, sb, off, ids, max(counts), len(counts), dev, algo="tiled")
    assert np.array_equal(f32_np(c).astype(np.float64), want)


# Problems whose 256 x 256 tiles make a whole number of rounds plus a small rest run as two
# launches (a cut along N or along M, the rest in another tile shape): both sides of the cut
# are checked on sampled rows by the naive kernel, which is the oracle bit for bit.
@pytest.mark.parametrize("M,K,N,kind", [
    (2048, 4096, 28672, "block"),    # Llama-3.1-8B gate_up: 3.5 rounds -> cut along N
    (2040, 4096, 28600, "block"),    # the same with ragged edges on both axes
    (28672, 4096, 2048, "block"),    # the transposed problem -> cut along M
    (28600, 4096, 2040, "row"),
    (2048, 4096, 28672, "row"),
])
def test_two_region_launch(dev, tune, M, K, N, kind):
    # (with a workspace, shapes of whole 256 x 256 tiles now split their work between the blocks instead: that path
    # has its own tests below; here it is switched off so that the cut is what runs)
    tune(MAXFP8_STREAMK="0", MAXFP8_W4="0")
    assert " + " in _lib.matmul_describe(M, N, K, kind == "block"), "this shape is meant to run as two launches"
    cfg = BLK if kind == "block" else ROW
    x = synth.activations(M, K, seed=0, outlier_frac=0.0 if kind == "row" else 0.01, device=dev)
    wf = synth.weights_f32(N, K, seed=1, device=dev)
    w, sb = synth.quantize_weight_block(wf) if kind == "block" else synth.quantize_weight_rowwise(wf)
    q, sa = mx.quantize_dynamic_scaled_float8(x, cfg.input_scale, cfg.weight_scale, scales_type=torch.float32)
    c = mx.dynamic_scaled_matmul(q, w, sa, sb, cfg.input_scale, cfg.weight_scale)
    rows = torch.unique(torch.cat([torch.arange(0, M, max(1, M // 29), device=dev), torch.tensor([M - 1], device=dev)]))
    ref = mx.dynamic_scaled_matmul(q[rows].contiguous(), w, sa[:, rows].contiguous(), sb, cfg.input_scale,
                                   cfg.weight_scale, out_type=torch.float32, algo="naive")
    torch.cuda.synchronize()
    assert_rel(f32_np(c[rows]), f32_np(ref), TOL, f"two regions {M}x{N}x{K} {kind}")
    # and the f32 output path, against the same reference
    c32 = mx.dynamic_scaled_matmul(q, w, sa, sb, cfg.input_scale, cfg.weight_scale, out_type=torch.float32)
    assert_rel(f32_np(c32[rows]), f32_np(ref), TOL, f"two regions f32 {M}x{N}x{K} {kind}", abs_budget=F32_BUDGET)


# ---- persistent kernel (whole 256 x 256 tiles, bf16 out) -----------------------------------------
# Shapes: fewer tiles than CUs; two and four tiles per block; an uneven share (300 tiles);
# one slab per tile; a K tail.  The persistent kernel forms every sum in the order of the
# per-tile kernel, so the two agree bit for bit; exact cases pin both to the true result.
PERSIST_SHAPES = [(512, 512, 256), (4096, 8192, 256), (2560, 7680, 384), (8192, 8192, 128), (1024, 4096, 144), (256, 256, 1024)]


# The four-wave kernel (MAXFP8_W4=4 / 5 / 6: 128 x 256 / 160 x 256 / 192 x 256 tiles, one wave per SIMD; it takes the shapes whose K is an
# even number of slabs and leaves the others to the eight-wave kernel) makes the same sums in the same order and is held
# to the same bits.
FORMS = {"eight waves": "0", "four waves, 128 rows": "4", "four waves, 160 rows": "5", "four waves, 192 rows": "6"}


@pytest.mark.parametrize("M,N,K", PERSIST_SHAPES)
@pytest.mark.parametrize("kind", ["block", "row"])
@pytest.mark.parametrize("form", list(FORMS))
def test_persistent_kernel_equals_per_tile_kernel(dev, tune, M, N, K, kind, form):
    tune(MAXFP8_TILE="1", MAXFP8_W4=FORMS[form], MAXFP8_W4_SPLIT="0")   # (whole tiles only: pieces add up in another order)
    if kind == "block":
        a, b, sa, sb = make_block(M, N, K, seed=M + K)
        cfg = BLK
    else:
        a, b = synth.random_fp8((M, K), M), synth.random_fp8((N, K), N + 1)
        sa, sb = synth.random_scales((1, M), 3, lo=0.01, hi=0.1), synth.random_scales((N, 1), 4, lo=0.001, hi=0.01)
        cfg = ROW
    assert "persistent" in _lib.matmul_describe(M, N, K, kind == "block", False)
    ad, bd, sad, sbd = a.to(dev), b.to(dev), sa.to(dev), sb.to(dev)
    run = lambda: mx.dynamic_scaled_matmul(ad, bd, sad, sbd, cfg.input_scale, cfg.weight_scale, out_type=torch.bfloat16,
                                           algo="tiled")
    got = run()
    again = run()  # a second launch on the same stream: same bits
    tune(MAXFP8_PERSIST="0")
    want = run()
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert torch.equal(again.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(512, 768, 384), (2560, 7680, 144)])
@pytest.mark.parametrize("form", list(FORMS))
def test_persistent_kernel_exact(dev, tune, M, N, K, form):
    tune(MAXFP8_TILE="1", MAXFP8_W4=FORMS[form])
    a, b, sa, sb, want = exact_case(M, N, K, seed=M + N + K)
    cb = mm(a, b, sa, sb, BLK, dev, out=torch.bfloat16, algo="tiled")
    assert torch.equal(cb.cpu(), torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16))


@pytest.mark.parametrize("M,N,K", [(4096, 2112, 7168), (320, 264, 512), (1000, 8, 1024), (161, 1544, 768)])
@pytest.mark.parametrize("kind", ["block", "row"])
@pytest.mark.parametrize("rows", ["4", "5", "6"])
def test_four_wave_kernel_ragged_edges(dev, tune, M, N, K, kind, rows):
    # a last row tile past M and a last column tile past N (DeepSeek-V3's fused q_a + kv_a projection: N = 1536 + 576 = 2112 =
    # 8 tiles and a quarter): bit-equal to the per-tile kernel, and nothing written outside the result.  Through the C ABI,
    # so that the result can sit in the middle of a larger buffer.
    L = _lib.lib()
    if kind == "block":
        a, b, sa, sb = make_block(M, N, K, seed=M + N)
        gin, gw, g, a_ld, b_ld = _lib.GRAN_BLOCK, _lib.GRAN_BLOCK, (1, 128, 128), sa.shape[1], K // 128
    else:
        a, b = synth.random_fp8((M, K), M), synth.random_fp8((N, K), N + 1)
        sa, sb = synth.random_scales((1, M), 3, lo=0.01, hi=0.1), synth.random_scales((N, 1), 4, lo=0.001, hi=0.01)
        gin, gw, g, a_ld, b_ld = _lib.GRAN_COLWISE, _lib.GRAN_ROWWISE, (-1, -1, -1), M, 1
    a, b, sa, sb = a.to(dev), b.to(dev), sa.to(dev).contiguous(), sb.to(dev).contiguous()
    stream = torch.cuda.current_stream(dev).cuda_stream

    def run(c):
        st = L.maxfp8_matmul_dynamic_scaled_fp8(c.data_ptr(), a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), M, N, K,
                                                K, K, N, gin, gw, *g, a_ld, b_ld, _lib.BF16, _lib.F32, _lib.ALGO_TILED, None, 0, stream)
        assert st == 0, _lib.last_error()

    tune(MAXFP8_TILE="1", MAXFP8_W4=rows, MAXFP8_W4_SPLIT="0")
    assert "four waves" in _lib.matmul_describe(M, N, K, kind == "block", False)
    guard = torch.full((M + 2, N), -7.0, dtype=torch.bfloat16, device=dev)
    run(guard[1:M + 1])
    tune(MAXFP8_PERSIST="0")
    want = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    run(want)
    torch.cuda.synchronize()
    assert torch.equal(guard[1:M + 1].view(torch.int16), want.view(torch.int16))
    assert bool((guard[0] == -7.0).all()) and bool((guard[M + 1] == -7.0).all())


def test_persistent_kernel_leaves_other_outputs_alone(dev, tune):
    # f32 output, rows of C that are not 16-byte aligned and partial tiles stay with the per-tile kernel
    tune(MAXFP8_TILE="1")
    a, b, sa, sb, want = exact_case(512, 520, 256, seed=9)
    assert np.array_equal(f32_np(mm(a, b, sa, sb, BLK, dev, algo="tiled")).astype(np.float64), want)
    a, b, sa, sb, want = exact_case(512, 512, 256, seed=10)
    assert np.array_equal(f32_np(mm(a, b, sa, sb, BLK, dev, algo="tiled")).astype(np.float64), want)


@pytest.mark.parametrize("form", list(FORMS))
def test_persistent_kernel_many_tiles_per_block_repeated(dev, tune, form):
    # short K, sixteen tiles per block: the stores of one tile are still in flight when the next tile's first slab
    # is waited for.  Twelve launches with fresh activations, each compared with the per-tile kernel.
    tune(MAXFP8_TILE="1", MAXFP8_W4=FORMS[form], MAXFP8_W4_SPLIT="0")
    M, N, K = 8192, 32768, 256
    b = synth.random_fp8((N, K), 77).to(dev)
    sb = synth.random_scales((N // 128, K // 128), 78).to(dev)
    sa = synth.random_scales((K // 128, M), 79).to(dev)
    for seed in range(12):
        a = synth.random_fp8((M, K), 100 + seed).to(dev)
        tune(MAXFP8_PERSIST="1")
        got = mx.dynamic_scaled_matmul(a, b, sa, sb, BLK.input_scale, BLK.weight_scale, out_type=torch.bfloat16, algo="tiled")
        tune(MAXFP8_PERSIST="0")
        want = mx.dynamic_scaled_matmul(a, b, sa, sb, BLK.input_scale, BLK.weight_scale, out_type=torch.bfloat16, algo="tiled")
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"launch {seed}"


# ---- the four-wave kernel with its last round cut into pieces ------------------------------------------------------
# Tiles beyond the last whole round of the CUs are each cut along K into two to four pieces, a block per piece: the
# pieces' f32 sums travel through the workspace and the block with a tile's last slabs adds them up.  That changes the
# order of the f32 sums: bit-equal to the uncut kernel where every sum is exact, one bf16 step apart at most elsewhere.
TAIL_CUT_SHAPES = [(2040, 6144, 4096), (3000, 7000, 3584), (4096, 7168, 2048), (2048, 7168, 18432)]


def _tail_cut_operands(M, N, K, kind, exact, dev, seed=0):
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K + seed)
    if exact:   # small integers times powers of two: every partial sum is exact in f32, whatever its order
        a = torch.randint(-2, 3, (M, K), generator=g).float().to(torch.float8_e4m3fn)
        b = torch.randint(-2, 3, (N, K), generator=g).float().to(torch.float8_e4m3fn)
        if kind == "block":
            sa = torch.pow(2.0, torch.randint(-3, 2, (K // 128, -(-M // 4) * 4), generator=g).float())
            sb = torch.pow(2.0, torch.randint(-3, 2, (-(-N // 128), K // 128), generator=g).float())
        else:
            sa = torch.pow(2.0, torch.randint(-3, 2, (1, M), generator=g).float())
            sb = torch.pow(2.0, torch.randint(-3, 2, (N, 1), generator=g).float())
    elif kind == "block":
        a, b, sa, sb = make_block(M, N, K, seed=M + K + seed)
    else:
        a, b = synth.random_fp8((M, K), M + seed), synth.random_fp8((N, K), N + 1)
        sa, sb = synth.random_scales((1, M), 3, lo=0.01, hi=0.1), synth.random_scales((N, 1), 4, lo=0.001, hi=0.01)
    return [t.to(dev) for t in (a, b, sa, sb)]


def _one_bf16_step_apart(got, want):
    """|got - want| within a bf16 step of the element, or (sums that cancel to nearly nothing) within what reordering
    f32 sums of this size can move them: 2^-12 of the mean magnitude."""
    g, w = got.float(), want.float()
    assert bool(torch.isfinite(g).all())
    excess = ((g - w).abs() - (2.0 ** -7 * w.abs() + 2.0 ** -12 * w.abs().mean())).max().item()
    assert excess <= 0, f"further apart than a bf16 step: by {excess:.3g}"


@pytest.mark.parametrize("M,N,K", TAIL_CUT_SHAPES)
@pytest.mark.parametrize("kind", ["block", "row"])
@pytest.mark.parametrize("rows", ["4", "5", "6"])
def test_tail_cut_against_the_uncut_kernel(dev, tune, M, N, K, kind, rows):
    if kind == "row" and K > 4096:
        pytest.skip("one long-K case is enough")
    cfg = BLK if kind == "block" else ROW
    tune(MAXFP8_W4=rows, MAXFP8_W4_SPLIT="1")   # 1: wherever the shape has a cut, whatever the cost model says
    cut_text = _lib.matmul_describe(M, N, K, kind == "block", True)
    if "tail cut" not in cut_text:
        pytest.skip(f"no cut at this tile height: {cut_text}")
    assert "tail cut" not in _lib.matmul_describe(M, N, K, kind == "block", False)   # no workspace, no pieces
    for exact in (True, False):
        ops = _tail_cut_operands(M, N, K, kind, exact, dev)
        run = lambda: mx.dynamic_scaled_matmul(*ops, cfg.input_scale, cfg.weight_scale, out_type=torch.bfloat16, algo="tiled")
        tune(MAXFP8_W4=rows, MAXFP8_W4_SPLIT="1")
        got, again = run(), run()
        tune(MAXFP8_W4=rows, MAXFP8_W4_SPLIT="0")
        assert "tail cut" not in _lib.matmul_describe(M, N, K, kind == "block", True)
        want = run()
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), again.view(torch.int16)), "two launches, two results"
        if exact:
            assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        else:
            _one_bf16_step_apart(got, want)


@pytest.mark.parametrize("M,N,K", [(256, 1792, 4096), (384, 2304, 2048), (1024, 2112, 7168), (130, 520, 1024), (256, 7168, 8192), (128, 1024, 8192)])
@pytest.mark.parametrize("kind", ["block", "row"])
@pytest.mark.parametrize("rows", ["4", "5", "6"])
def test_every_tile_cut_against_the_uncut_kernel(dev, tune, M, N, K, kind, rows):
    """At most half a round of tiles: where the other plan is a K split (two launches, the shares' sums through memory)
    the four-wave kernel can cut EVERY tile into two to eight pieces, one block each, which exchange their sums inside the
    one launch.  Forced here wherever the shape allows it (the planner takes it where the pieces fill three quarters of
    the chip with at least 16 slabs each), against the same kernel uncut: equal on exact data, a bf16 step apart at most
    elsewhere, the same bits on two launches."""
    if kind == "row" and K > 4096:
        pytest.skip("one long-K case is enough")
    cfg = BLK if kind == "block" else ROW
    tune(MAXFP8_W4=rows, MAXFP8_W4_SPLIT="1")
    cut_text = _lib.matmul_describe(M, N, K, kind == "block", True)
    if "every tile cut" not in cut_text:
        pytest.skip(f"no such cut at this tile height: {cut_text}")
    assert "cut" not in _lib.matmul_describe(M, N, K, kind == "block", False)   # no workspace, no pieces
    for exact in (True, False):
        ops = _tail_cut_operands(M, N, K, kind, exact, dev)
        run = lambda: mx.dynamic_scaled_matmul(*ops, cfg.input_scale, cfg.weight_scale, out_type=torch.bfloat16, algo="tiled")
        tune(MAXFP8_W4=rows, MAXFP8_W4_SPLIT="1", MAXFP8_SPLITK=None)
        got, again = run(), run()
        tune(MAXFP8_W4=rows, MAXFP8_W4_SPLIT="0", MAXFP8_SPLITK="1")
        uncut = _lib.matmul_describe(M, N, K, kind == "block", True)
        assert "four waves" in uncut and "cut" not in uncut, uncut
        want = run()
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), again.view(torch.int16)), "two launches, two results"
        if exact:
            assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        else:
            _one_bf16_step_apart(got, want)
    assert _lib.lib().maxfp8_handovers_given_up() == 0


def test_planner_cuts_every_tile_where_it_measured_ahead(dev, tune):
    """The planner's own choice on a shape of the kind (DeepSeek-V3 fused q_a + kv_a at M = 1024): the cut form, and its
    result against the CPU oracle on sampled rows."""
    M, N, K = 1024, 2112, 7168
    assert "every tile cut" in _lib.matmul_describe(M, N, K, True, True)
    a, b, sa, sb = make_block(M, N, K, seed=5)
    c = mm(a, b, sa, sb, BLK, dev, out=torch.bfloat16)
    rows = [0, 127, 128, 500, 1023]
    ref = oracle_block(a.view(torch.uint8)[rows].view(a.dtype), b, sa[:, rows].contiguous(), sb)
    assert_rel(f32_np(c[rows]), ref, TOL, f"every tile cut {M}x{N}x{K}")


def test_tail_cut_against_the_oracle(dev, tune):
    tune(MAXFP8_W4="5", MAXFP8_W4_SPLIT="1")
    for (M, N, K) in [(2040, 6144, 1024), (2200, 7168, 512)]:
        if "tail cut" not in _lib.matmul_describe(M, N, K, True, True):
            continue
        a, b, sa, sb = make_block(M, N, K, seed=M)
        ref = oracle_block(a, b, sa, sb)
        c = mm(a, b, sa, sb, BLK, dev, out=torch.bfloat16, algo="tiled")
        assert_rel(f32_np(c), ref, TOL, f"tail cut {M}x{N}x{K}")
        return
    pytest.skip("no shape of this list has a cut on this chip")


def test_tail_cut_repeated_launches_with_fresh_data(dev, tune):
    """The pieces go through memory that other CUs (and other XCDs, whose L2 caches are not coherent with each other)
    wrote, behind flags that a launch raises and lowers again: thirty launches in a row, block-scaled and row-scaled
    taking turns (they share the flags), each with new activations, each against the uncut kernel.  A block that read a stale piece, or found a flag still up, would show here."""
    M, N, K = 2040, 6144, 2048
    tune(MAXFP8_W4="5", MAXFP8_W4_SPLIT="1")
    if "tail cut" not in _lib.matmul_describe(M, N, K, True, True):
        pytest.skip("no cut at this shape on this chip")
    L = _lib.lib()
    assert L.maxfp8_matmul_workspace_bytes(M, N, K) >= 160 * 256 * 4 * 8
    fixed = {kind: _tail_cut_operands(M, N, K, kind, False, dev) for kind in ("block", "row")}
    for seed in range(30):
        kind = "block" if seed % 2 == 0 else "row"
        cfg = BLK if kind == "block" else ROW
        _, b, sa, sb = fixed[kind]
        a = synth.random_fp8((M, K), 100 + seed).to(dev)
        run = lambda: mx.dynamic_scaled_matmul(a, b, sa, sb, cfg.input_scale, cfg.weight_scale, out_type=torch.bfloat16, algo="tiled")
        tune(MAXFP8_W4="5", MAXFP8_W4_SPLIT="1")
        got = run()
        tune(MAXFP8_W4="5", MAXFP8_W4_SPLIT="0")
        want = run()
        torch.cuda.synchronize()
        _one_bf16_step_apart(got, want)
    assert L.maxfp8_handovers_given_up() == 0


def test_random_large_shapes_through_the_four_wave_kernel_are_exact(dev, tune):
    """Random shapes of 700 ... 4300 rows through the four-wave kernel -- every tile height and the planner's own choice,
    the last round cut, uncut and as the planner decides, ragged M and N -- on small integers times powers of two:
    every sum is exact in any order, so the result equals the scalar kernel's bit for bit.  (The same generator ran 690
    cases, 1275 four-wave launches, 88 of them with a cut last round, without a mismatch.)"""
    rng = np.random.default_rng(11)
    launches = 0
    for it in range(24):
        M, N, K = int(rng.integers(700, 4300)), 8 * int(rng.integers(200, 1000)), 256 * int(rng.integers(2, 13))
        if it % 3 == 0:
            K = 512 * int(rng.integers(1, 7))
        tune(MAXFP8_W4=[None, "4", "5", "6"][it % 4], MAXFP8_W4_SPLIT=[None, "1", "0"][it % 3])
        a = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (M, K)).astype(np.float32))).to(dev)
        b = fp8_from_bytes(oracle.e4m3fn_encode(rng.integers(-4, 5, (N, K)).astype(np.float32))).to(dev)
        kb, nb = K // 128, -(-N // 128)
        sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (kb, -(-M // 4) * 4))).astype(np.float32)).to(dev)
        sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, (nb, kb))).astype(np.float32)).to(dev)
        ra = torch.from_numpy(np.exp2(rng.integers(-3, 3, (1, M))).astype(np.float32)).to(dev)
        rb = torch.from_numpy(np.exp2(rng.integers(-3, 3, (N, 1))).astype(np.float32)).to(dev)
        for kind, cfg, x, y in (("block", BLK, sa, sb), ("row", ROW, ra, rb)):
            text = _lib.matmul_describe(M, N, K, kind == "block", True)
            launches += "four waves" in text
            got = mx.dynamic_scaled_matmul(a, b, x, y, cfg.input_scale, cfg.weight_scale, out_type=torch.bfloat16)
            want = mx.dynamic_scaled_matmul(a, b, x, y, cfg.input_scale, cfg.weight_scale, out_type=torch.bfloat16, algo="naive")
            torch.cuda.synchronize()
            assert torch.equal(got, want), f"case {it}, {kind}: {M}x{N}x{K} [{text}]"
    assert launches >= 24 and _lib.lib().maxfp8_handovers_given_up() == 0


def test_tail_cut_on_two_streams_at_once(dev, tune):
    """Launches that overlap in time each bring a workspace of their own and draw a set of flags of their own: two
    streams issue the same matmul on different activations, back to back, sixteen times each without waiting for one
    another; every result equals what the same launch gives alone."""
    M, N, K = 2040, 6144, 2048
    tune(MAXFP8_W4="5", MAXFP8_W4_SPLIT="1")
    if "tail cut" not in _lib.matmul_describe(M, N, K, True, True):
        pytest.skip("no cut at this shape on this chip")
    L = _lib.lib()
    need = L.maxfp8_matmul_workspace_bytes(M, N, K)
    _, bd, sad, sbd = _tail_cut_operands(M, N, K, "block", False, dev)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    acts = [[synth.random_fp8((M, K), 300 + 16 * s_ + i).to(dev) for i in range(16)] for s_ in range(2)]
    outs = [[torch.empty((M, N), dtype=torch.bfloat16, device=dev) for _ in range(16)] for _ in range(2)]
    spaces = [torch.empty((need,), dtype=torch.uint8, device=dev) for _ in range(2)]

    def launch(a, out, ws, stream):
        st = L.maxfp8_matmul_dynamic_scaled_fp8(out.data_ptr(), a.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), M, N, K,
                                                K, K, N, _lib.GRAN_BLOCK, _lib.GRAN_BLOCK, 1, 128, 128, sad.shape[1], K // 128,
                                                _lib.BF16, _lib.F32, _lib.ALGO_TILED, ws.data_ptr(), need, stream.cuda_stream)
        assert st == 0, _lib.last_error()

    torch.cuda.synchronize()
    for i in range(16):
        for s_ in range(2):
            launch(acts[s_][i], outs[s_][i], spaces[s_], streams[s_])
    torch.cuda.synchronize()
    alone = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    for s_ in range(2):
        for i in range(16):
            launch(acts[s_][i], alone, spaces[0], torch.cuda.current_stream())
            torch.cuda.synchronize()
            assert torch.equal(outs[s_][i].view(torch.int16), alone.view(torch.int16)), f"stream {s_}, launch {i}"
    assert L.maxfp8_handovers_given_up() == 0


def test_tail_cut_recorded_into_a_graph(dev, tune):
    # A recorded launch replays with the arguments of the recording -- the set of flags among them.  The flags are
    # lowered by the launch that raised them, so a replay finds them as the recording did; recorded launches draw
    # their sets from a range that eager launches never get.  Four replays, each on new activations, eager launches
    # of the same shape in between, each replay against the eager result, bit for bit.
    M, N, K = 2040, 6144, 2048
    tune(MAXFP8_W4="5", MAXFP8_W4_SPLIT="1")
    if "tail cut" not in _lib.matmul_describe(M, N, K, True, True):
        pytest.skip("no cut at this shape on this chip")
    ad, bd, sad, sbd = _tail_cut_operands(M, N, K, "block", False, dev)
    L = _lib.lib()
    need = L.maxfp8_matmul_workspace_bytes(M, N, K)
    ws = torch.empty((need,), dtype=torch.uint8, device=dev)
    out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)

    def run(dst, stream):
        st = L.maxfp8_matmul_dynamic_scaled_fp8(dst.data_ptr(), ad.data_ptr(), bd.data_ptr(), sad.data_ptr(), sbd.data_ptr(), M, N, K,
                                                K, K, N, _lib.GRAN_BLOCK, _lib.GRAN_BLOCK, 1, 128, 128, sad.shape[1], K // 128,
                                                _lib.BF16, _lib.F32, _lib.ALGO_TILED, ws.data_ptr(), need, stream.cuda_stream)
        assert st == 0, _lib.last_error()

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(out, side)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            run(out, side)
    torch.cuda.current_stream().wait_stream(side)
    eager = torch.empty_like(out)
    for seed in range(4):
        ad.copy_(synth.random_fp8((M, K), 100 + seed).to(dev))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        run(eager, torch.cuda.current_stream())
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), eager.view(torch.int16)), f"replay {seed}"
    assert L.maxfp8_handovers_given_up() == 0


# ---- the persistent kernel with its work split along K ("stream-K") --------------------------------------------
# Matmuls of at least one 256 x 256 tile per block whose tiles are not whole rounds of the chip: every block takes the
# same number of slabs, and a tile that a block boundary cuts is begun by one block and finished by the next, its f32
# accumulators handed over through the workspace.  The sums keep the per-tile kernel's order: bit-equal results.
STREAMK_SHAPES = [(2560, 7680, 384), (4096, 7168, 2048), (5120, 5120, 640), (2048, 28672, 512), (4096, 7168, 16384)]


@pytest.mark.parametrize("M,N,K", STREAMK_SHAPES)
@pytest.mark.parametrize("kind", ["block", "row"])
def test_stream_k_equals_per_tile_kernel(dev, tune, M, N, K, kind):
    if kind == "row" and K > 4096:
        pytest.skip("one long-K case is enough")
    tune(MAXFP8_TILE="1", MAXFP8_STREAMK="2")     # 2: wherever the shape allows it, whatever the cost model says
    assert "stream-K" in _lib.matmul_describe(M, N, K, kind == "block", True)
    assert "stream-K" not in _lib.matmul_describe(M, N, K, kind == "block", False)   # no workspace, no hand-over
    if kind == "block":
        a, b, sa, sb = make_block(M, N, K, seed=M + K)
        cfg = BLK
    else:
        a, b = synth.random_fp8((M, K), M), synth.random_fp8((N, K), N + 1)
        sa, sb = synth.random_scales((1, M), 3, lo=0.01, hi=0.1), synth.random_scales((N, 1), 4, lo=0.001, hi=0.01)
        cfg = ROW
    ad, bd, sad, sbd = a.to(dev), b.to(dev), sa.to(dev), sb.to(dev)
    run = lambda: mx.dynamic_scaled_matmul(ad, bd, sad, sbd, cfg.input_scale, cfg.weight_scale, out_type=torch.bfloat16,
                                           algo="tiled")
    got = run()
    tune(MAXFP8_STREAMK="0", MAXFP8_W4="0")   # (the eight-wave persistent kernel: the four-wave one may cut its last round, in another order of sums)
    assert "stream-K" not in _lib.matmul_describe(M, N, K, kind == "block", True)
    persistent = run()
    tune(MAXFP8_PERSIST="0")
    per_tile = run()
    torch.cuda.synchronize()
    assert bool(torch.isfinite(got.float()).all())
    assert torch.equal(got.view(torch.int16), per_tile.view(torch.int16))
    assert torch.equal(persistent.view(torch.int16), per_tile.view(torch.int16))


def test_stream_k_scale_modes_take_turns(dev, tune):
    # Block-scaled and row-scaled launches share the hand-over flags in device memory, so they must share the numbering
    # of the launches too: with a counter each, the n-th row-scaled launch found its flags already set by the n-th
    # block-scaled one, and a block could take over accumulators that its predecessor had not written yet.
    M, N, K = 2560, 7680, 384   # 3 slabs per tile, 3.5 per block: the hand-over comes early in every block
    cases = []
    for kind in ("block", "row"):
        if kind == "block":
            a, b, sa, sb = make_block(M, N, K, seed=11)
            cfg = BLK
        else:
            a, b = synth.random_fp8((M, K), 5), synth.random_fp8((N, K), 6)
            sa, sb = synth.random_scales((1, M), 3, lo=0.01, hi=0.1), synth.random_scales((N, 1), 4, lo=0.001, hi=0.01)
            cfg = ROW
        ops = [t.to(dev) for t in (a, b, sa, sb)]
        cases.append((kind, cfg, ops))
    run = lambda cfg, ops: mx.dynamic_scaled_matmul(*ops, cfg.input_scale, cfg.weight_scale, out_type=torch.bfloat16, algo="tiled")
    tune(MAXFP8_TILE="1", MAXFP8_STREAMK="0", MAXFP8_PERSIST="0")
    want = {kind: run(cfg, ops) for kind, cfg, ops in cases}
    tune(MAXFP8_TILE="1", MAXFP8_STREAMK="2")
    for it in range(40):
        for kind, cfg, ops in cases:
            got = run(cfg, ops)
            assert torch.equal(got.view(torch.int16), want[kind].view(torch.int16)), f"{kind}, launch {it}"


def test_stream_k_shape_recorded_into_a_graph(dev, tune):
    # A recorded launch replays with the arguments of the recording, so the work-split kernel's flag value would repeat
    # and a replay would find its flags already set: under stream capture such a matmul runs as the persistent kernel
    # (the same sums in the same order).  Four replays, each on new activations, each against the eager result.
    M, N, K = 2560, 7680, 384
    a, b, sa, sb = make_block(M, N, K, seed=21)
    ad, bd, sad, sbd = a.to(dev), b.to(dev), sa.to(dev), sb.to(dev)
    run = lambda: mx.dynamic_scaled_matmul(ad, bd, sad, sbd, BLK.input_scale, BLK.weight_scale, out_type=torch.bfloat16, algo="tiled")
    tune(MAXFP8_TILE="1", MAXFP8_STREAMK="2")
    assert "stream-K" in _lib.matmul_describe(M, N, K, True, True)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            out = run()
    torch.cuda.current_stream().wait_stream(side)
    for seed in range(4):
        ad.copy_(synth.random_fp8((M, K), 100 + seed).to(dev))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = run()     # eager: the work-split kernel itself
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"replay {seed}"


def test_stream_k_exact(dev, tune):
    tune(MAXFP8_TILE="1", MAXFP8_STREAMK="2")
    M, N, K = 2560, 7680, 640
    a, b, sa, sb, want = exact_case(M, N, K, seed=M + N + K)
    assert "stream-K" in _lib.matmul_describe(M, N, K, True, True)
    cb = mm(a, b, sa, sb, BLK, dev, out=torch.bfloat16, algo="tiled")
    assert torch.equal(cb.cpu(), torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16))


def test_stream_k_repeated_launches_with_fresh_data(dev, tune):
    """The hand-over goes through memory that other CUs (and other XCDs, whose L2 caches are not coherent with each
    other) wrote: thirty launches in a row, each with new activations and a new workspace position, each compared with
    the per-tile kernel.  A block that read a stale partial sum or an old flag would show here."""
    tune(MAXFP8_TILE="1", MAXFP8_STREAMK="2")
    M, N, K = 2560, 7680, 1024
    b = synth.random_fp8((N, K), 77).to(dev)
    sb = synth.random_scales((N // 128, K // 128), 78).to(dev)
    sa = synth.random_scales((K // 128, M), 79).to(dev)
    L = _lib.lib()
    need = L.maxfp8_matmul_workspace_bytes(M, N, K)
    assert need == 64 << 20
    ws = torch.zeros((need + 4096,), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    for seed in range(30):
        a = synth.random_fp8((M, K), 100 + seed).to(dev)
        got = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        off = 256 * (seed % 3)      # the same slots again, and slots shifted against the last launch's
        tune(MAXFP8_TILE="1", MAXFP8_STREAMK="2", MAXFP8_PERSIST="1")
        st = L.maxfp8_matmul_dynamic_scaled_fp8(got.data_ptr(), a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), M, N, K,
                                                K, K, N, _lib.GRAN_BLOCK, _lib.GRAN_BLOCK, 1, 128, 128, M, K // 128, _lib.BF16,
                                                _lib.F32, _lib.ALGO_TILED, ws.data_ptr() + off, need, stream)
        assert st == 0, _lib.last_error()
        tune(MAXFP8_PERSIST="0")
        want = mx.dynamic_scaled_matmul(a, b, sa, sb, BLK.input_scale, BLK.weight_scale, out_type=torch.bfloat16, algo="tiled")
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"launch {seed}"
    assert L.maxfp8_handovers_given_up() == 0   # (no block ever stopped waiting for its predecessor)
