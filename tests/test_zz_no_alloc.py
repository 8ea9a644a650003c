"""The matmul entry point that allocates nothing (maxfp8_matmul_dynamic_scaled_fp8_noalloc): through the C ABI,
against the plain entry point with a caller-allocated workspace, bit for bit (both plan alike, so both add the same
partial sums in the same order), on two calls in a row, the second with a smaller input."""
import numpy as np
import pytest
import torch

import oracle
from modular_amd import _lib, synth
from util import assert_rel, f32_np, fp8_bytes

pytestmark = pytest.mark.gpu
NT = oracle.default_threads()


def both_entry_points(M, N, K, block, dev, seed, out=torch.bfloat16):
    L = _lib.lib()
    a, b = synth.random_fp8((M, K), seed).to(dev), synth.random_fp8((N, K), seed + 1).to(dev)
    if block:
        ld = -(-M // 4) * 4
        sa, sb = synth.random_scales((K // 128, ld), seed + 2).to(dev), synth.random_scales((-(-N // 128), K // 128), seed + 3).to(dev)
        gin, gw, g, a_ld, b_ld = _lib.GRAN_BLOCK, _lib.GRAN_BLOCK, (1, 128, 128), ld, K // 128
    else:
        sa, sb = synth.random_scales((1, M), seed + 2, lo=0.01, hi=0.1).to(dev), synth.random_scales((N, 1), seed + 3, lo=0.001, hi=0.01).to(dev)
        gin, gw, g, a_ld, b_ld = _lib.GRAN_COLWISE, _lib.GRAN_ROWWISE, (-1, -1, -1), M, 1
    odt = _lib.BF16 if out == torch.bfloat16 else _lib.F32
    need = L.maxfp8_matmul_workspace_bytes(M, N, K)
    ws = torch.empty((max(need, 16),), dtype=torch.uint8, device=dev)
    c_plain = torch.full((M, N), float("nan"), dtype=out, device=dev)
    c_noalloc = torch.full((M, N), float("nan"), dtype=out, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    st = L.maxfp8_matmul_dynamic_scaled_fp8(c_plain.data_ptr(), a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), M, N, K,
                                            K, K, N, gin, gw, *g, a_ld, b_ld, odt, _lib.F32, _lib.ALGO_AUTO,
                                            ws.data_ptr() if need else None, need, stream)
    assert st == 0, _lib.last_error()
    st = L.maxfp8_matmul_dynamic_scaled_fp8_noalloc(c_noalloc.data_ptr(), a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(),
                                                    M, N, K, K, K, N, gin, gw, *g, a_ld, b_ld, odt, _lib.F32, _lib.ALGO_AUTO, stream)
    assert st == 0, _lib.last_error()
    torch.cuda.synchronize()
    return c_plain, c_noalloc, (a, b, sa, sb), need


def test_noalloc_matmul_equals_the_plain_entry_point_twice_in_a_row(dev):
    L = _lib.lib()
    assert L.maxfp8_matmul_noalloc_max_scratch_bytes() == 48 << 20
    # first call: a K-split plan with ~8 MiB of partial sums; second call: a smaller one that reuses the same array
    # (whatever the first call left in it); then a row-scaled shape and one that needs no scratch at all
    for (M, N, K, block) in [(256, 576, 7168, True), (128, 512, 4096, True), (4096, 576, 7168, True), (100, 576, 7168, False), (2048, 1024, 512, True),
                              # 33 to 64 rows with a plan that does not split: both entry points run the tiles, not the
                              # weight-streaming kernel
                              (64, 28672, 4096, True), (48, 8192, 4096, False),
                              # a last round of tiles computed in pieces, their sums in the scratch: 48 MiB, all of the array
                              # (too long for the CPU oracle here: held to the plain entry point's bits, and that one to
                              # the uncut kernel by the tests of the tiles)
                              (4096, 7168, 16384, True)]:
        print(f"[no-alloc] {M}x{N}x{K} {'block' if block else 'row'}: {_lib.matmul_describe(M, N, K, block, True)}", flush=True)
        c_plain, c_noalloc, (a, b, sa, sb), need = both_entry_points(M, N, K, block, dev, seed=M + N)
        assert bool(torch.isfinite(c_noalloc.float()).all())
        assert torch.equal(c_plain, c_noalloc), f"{M}x{N}x{K}: the two entry points differ"
        if 2.0 * M * N * K > 2e11:
            assert "tail cut" in _lib.matmul_describe(M, N, K, block, True) and need == 48 << 20
            continue
        if block:
            ref = oracle.matmul_blockwise(fp8_bytes(a), fp8_bytes(b), sa.cpu().numpy(), sb.cpu().numpy(), threads=NT)
        else:
            ref = oracle.matmul_rowwise(fp8_bytes(a), fp8_bytes(b), sa.cpu().numpy(), sb.cpu().numpy(), threads=NT)
        assert_rel(f32_np(c_noalloc), ref, 1e-2, f"no-alloc {M}x{N}x{K}")


def test_noalloc_matmul_refuses_what_its_scratch_cannot_hold(dev):
    L = _lib.lib()
    limit = L.maxfp8_matmul_noalloc_max_scratch_bytes()
    M, N, K = 2048, 2304, 16384          # K split 3: 3 * 2048 * 2304 * 4 bytes = 54 MiB of partial sums
    assert "K split 3" in _lib.matmul_describe(M, N, K, True, True) and 3 * M * N * 4 > limit
    # (refused before anything is launched: the pointers are never used)
    st = L.maxfp8_matmul_dynamic_scaled_fp8_noalloc(16, 16, 16, 16, 16, M, N, K, K, K, N, _lib.GRAN_BLOCK, _lib.GRAN_BLOCK, 1, 128,
                                                    128, M, K // 128, _lib.BF16, _lib.F32, _lib.ALGO_AUTO, None)
    assert st == _lib.ERR_WORKSPACE and "static buffer holds" in _lib.last_error()
    with pytest.raises(ValueError):
        _lib.check(st)
