"""Oracle of the fused QKV matmul with paged-cache stores: the index arithmetic against an
independent gather, the value path against exact integer arithmetic and against a float64 matmul,
and the bf16 helpers against torch's CPU casts."""
import numpy as np
import pytest
import torch

import oracle
from qkv_cases import logical_rows, make_cache_case, make_operands
from util import fp8_bytes


def test_bf16_round_is_torch_cpu_cast():
    rng = np.random.default_rng(0)
    x = rng.integers(0, 2 ** 32, size=1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
    x = x[np.isfinite(x)]
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(oracle.bf16_round(x).view(np.uint32), want.view(np.uint32))
    assert np.array_equal(oracle.bf16_bits_of(want), torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))


@pytest.mark.parametrize("mnk", [(-1, -1, -1), (1, 1, -1), (1, 128, 128)])
def test_small_integers_land_exactly_where_they_belong(mnk):
    # fp8 operands in {-1, 0, 1}, scales 1 / 2 / 4, bias small integers: every value is an integer below 256, every rounding exact,
    # so Q and the cache must hold the integer matmul, found through an independent gather
    H, D, Hq, page, layers, nblocks = 2, 16, 3, 4, 3, 16
    prompt, cached = [5, 1, 0, 7], [3, 0, 2, 9]
    T, K = sum(prompt), 256
    q_dim, k_dim = Hq * D, H * D
    N = q_dim + 2 * k_dim
    rng = np.random.default_rng(1)
    ai = rng.integers(-1, 2, size=(T, K))
    wi = rng.integers(-1, 2, size=(N, K))
    a = fp8_bytes(torch.from_numpy(ai.astype(np.float32)).to(torch.float8_e4m3fn))
    w = fp8_bytes(torch.from_numpy(wi.astype(np.float32)).to(torch.float8_e4m3fn))
    if mnk == (-1, -1, -1):
        sa, sb = np.full((1, 1), 0.5, np.float32), np.full((1, 1), 4.0, np.float32)
        scale = np.full((T, N), 2.0)
    elif mnk == (1, 1, -1):
        sa = (2.0 ** rng.integers(0, 2, size=(1, T))).astype(np.float32)
        sb = (2.0 ** rng.integers(0, 2, size=(N, 1))).astype(np.float32)
        scale = sa.reshape(T, 1).astype(np.float64) * sb.reshape(1, N)
    else:
        sa = (2.0 ** rng.integers(0, 2, size=(K // 128, T))).astype(np.float32)
        sb = np.ones((-(-N // 128), K // 128), dtype=np.float32)
        sb[0, 1] = 2.0
        scale = None
    bias_f = rng.integers(-3, 4, size=N).astype(np.float32)
    bias = oracle.bf16_bits_of(bias_f)
    if scale is not None:
        want = (ai @ wi.T) * scale + bias_f
    else:
        want = np.zeros((T, N))
        for kb in range(K // 128):
            part = ai[:, kb * 128:(kb + 1) * 128] @ wi[:, kb * 128:(kb + 1) * 128].T
            want += part * sa[kb][:T, None].astype(np.float64) * np.repeat(sb[:, kb], 128)[:N][None, :]
        want += bias_f
    assert np.abs(want).max() < 256
    want32 = want.astype(np.float32)
    assert np.array_equal(oracle.bf16_round(want32), want32), "test data must be bf16-exact"
    ro, cl, lut = make_cache_case(prompt, cached, page, nblocks, seed=2)
    blocks = np.full((nblocks, 2, layers, page, H, D), 0x7FC0, dtype=np.uint16)
    layer = 1
    q = oracle.fused_qkv_matmul(a, w, sa, sb, mnk, ro, cl, lut, blocks, layer, q_dim, bias=bias)
    assert np.array_equal(q, oracle.bf16_bits_of(want32[:, :q_dim]))
    touched = np.zeros(blocks.shape[:4], dtype=bool)
    for b in range(len(prompt)):
        if prompt[b] == 0:
            continue
        rows = slice(int(ro[b]), int(ro[b + 1]))
        got_k = logical_rows(blocks, 0, layer, lut, b, cached[b], prompt[b], page)
        got_v = logical_rows(blocks, 1, layer, lut, b, cached[b], prompt[b], page)
        assert np.array_equal(got_k, oracle.bf16_bits_of(want32[rows, q_dim:q_dim + k_dim]))
        assert np.array_equal(got_v, oracle.bf16_bits_of(want32[rows, q_dim + k_dim:]))
        toks = np.arange(cached[b], cached[b] + prompt[b])
        touched[lut[b, toks // page].astype(np.int64), :, layer, toks % page] = True
    # nothing else was written: other layers, the cached prefix, unused pages
    assert np.all(blocks[~touched] == 0x7FC0)


def test_values_against_float64_and_k_only_mla_layout():
    H, D, page, layers, nblocks = 1, 64, 8, 2, 12
    prompt, cached = [9, 4], [7, 0]
    T, K = sum(prompt), 384
    a, w, sa, sb = make_operands(T, H * D, K, (1, 128, 128), seed=5)
    ro, cl, lut = make_cache_case(prompt, cached, page, nblocks, seed=6)
    blocks = np.zeros((nblocks, 1, layers, page, H, D), dtype=np.uint16)       # one plane: the MLA layout
    q = oracle.fused_qkv_matmul(fp8_bytes(a), fp8_bytes(w), sa.numpy(), sb.numpy(), (1, 128, 128), ro, cl, lut, blocks, 0, 0)
    assert q.shape == (T, 0)
    af, wf = a.double().numpy(), w.double().numpy()
    ref = np.zeros((T, H * D))
    for kb in range(K // 128):
        ref += (af[:, kb * 128:(kb + 1) * 128] @ wf[:, kb * 128:(kb + 1) * 128].T) * sa.numpy()[kb, :T, None] * \
            np.repeat(sb.numpy()[:, kb], 128)[:H * D][None, :]
    for b in range(2):
        got = logical_rows(blocks, 0, 0, lut, b, cached[b], prompt[b], page)
        gotf = (got.astype(np.uint32) << 16).view(np.float32)
        want = ref[int(ro[b]):int(ro[b + 1])]
        assert np.all(np.abs(gotf - want) <= np.abs(want) * 2.0 ** -8 + 1e-3)
    assert not blocks[:, :, 1].any()
