"""Pins the oracle's dynamic quantisation against (a) the reference test's own host
procedure (max/kernels/test/gpu/quantization/test_scaled_fp8_quantization.mojo:257-299)
re-stated with torch library routines on that test's shapes, and (b) closed forms
that a dropped clamp, a swapped division, a wrong scale index or a missing guard
would each break."""
import numpy as np
import pytest
import torch

import oracle
from util import bf16_bits, fp8_bytes

FP8 = torch.float8_e4m3fn


def torch_quant(x: torch.Tensor, G: int, ub: float = 1200.0):
    """The reference test's host loop with torch's IEEE f32 ops and its fp8 cast."""
    M, K = x.shape
    xf = x.float().reshape(M, K // G, G)
    amax = xf.abs().amax(-1)
    scale = torch.minimum(amax, torch.tensor(ub)) / torch.tensor(448.0)
    recip = 1.0 / scale
    recip = torch.where((scale == 0) | ~torch.isfinite(recip), torch.zeros(()), recip)
    q = (xf * recip[..., None]).clamp(-448.0, 448.0).to(FP8).reshape(M, K)
    return q, scale.t().contiguous()


# shapes of the reference test (test_scaled_fp8_quantization.mojo:707-750)
REF_SHAPES = [(1, 256), (2, 1024), (4, 16384), (2, 260), (4, 264), (1, 576), (4, 576)]


@pytest.mark.parametrize("M,K", REF_SHAPES)
@pytest.mark.parametrize("group", [-1, 128])
def test_reference_test_shapes(M, K, group):
    if group == 128 and K % 128:
        pytest.skip("group 128 needs K % 128 == 0 (the reference runs these shapes per-token only)")
    g = torch.Generator().manual_seed(M * 100003 + K)
    x = (torch.rand((M, K), generator=g) * 2 - 1).to(torch.bfloat16)  # random(in_host, -1.0, 1.0)
    G = K if group == -1 else group
    q, sc = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x), G)
    q_ref, sc_ref = torch_quant(x, G)
    assert sc.shape == (K // G, M)
    assert np.array_equal(sc.view(np.uint32), sc_ref.numpy().view(np.uint32))
    assert np.array_equal(q, fp8_bytes(q_ref))


def test_outlier_activations_match_torch():
    from modular_amd import synth
    x = synth.activations(8, 1024, seed=0)
    q, sc = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x), 128)
    q_ref, sc_ref = torch_quant(x, 128)
    assert np.array_equal(sc.view(np.uint32), sc_ref.numpy().view(np.uint32))
    assert np.array_equal(q, fp8_bytes(q_ref))


def test_power_of_two_amax_is_exact():
    # amax = 448 * 2^k  =>  scale = 2^k, recip = 2^-k, q = e4m3fn(x * 2^-k) exactly
    for k in (-20, -3, 0, 1):
        vals = np.array([448.0, -224.0, 3.5, 0.4375, -0.001953125, 0.0], dtype=np.float32)
        row = np.zeros(128, dtype=np.float32)
        row[: vals.size] = vals * np.float32(2.0 ** k)
        x = torch.from_numpy(row[None, :]).to(torch.bfloat16)
        assert torch.equal(x.float(), torch.from_numpy(row[None, :]))  # representable
        q, sc = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x), 128)
        assert sc[0, 0] == np.float32(2.0 ** k)
        assert np.array_equal(q[0, : vals.size], oracle.e4m3fn_encode(vals))
        assert np.array_equal(oracle.e4m3fn_decode(q[0, : vals.size]), vals)


def test_scale_is_amax_over_448_not_its_inverse():
    s, r = oracle.dynamic_scale(1.0)
    assert s == np.float32(1.0) / np.float32(448.0)
    assert r == np.float32(1.0) / s
    assert r != np.float32(448.0)  # 1/(1/448) rounds away from 448 in f32: two divisions, not one
    # the element equal to amax lands on +-448 after the clamp
    x = torch.ones((1, 128), dtype=torch.bfloat16)
    x[0, 5] = -1.0
    q, _ = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x), 128)
    assert q[0, 0] == 0x7E and q[0, 5] == 0xFE


def test_scale_ub_clamps_and_saturates():
    row = torch.zeros((1, 128), dtype=torch.float32)
    row[0, :4] = torch.tensor([3008.0, 1200.0, 600.0, -2000.0])
    q, sc = oracle.quantize_dynamic_scaled_fp8(bf16_bits(row.to(torch.bfloat16)), 128)
    assert sc[0, 0] == np.float32(1200.0) / np.float32(448.0)
    assert q[0, 0] == 0x7E and q[0, 3] == 0xFE          # beyond the bound: saturate
    assert q[0, 1] == 0x7E                              # the bound itself maps to 448
    assert oracle.e4m3fn_decode(q[0, 2:3])[0] == 224.0  # half the bound
    # custom bound
    q2, sc2 = oracle.quantize_dynamic_scaled_fp8(bf16_bits(row.to(torch.bfloat16)), 128, scale_ub=600.0)
    assert sc2[0, 0] == np.float32(600.0) / np.float32(448.0) and q2[0, 2] == 0x7E


def test_near_zero_groups_give_clean_zeros():
    # test_scaled_fp8_quantization.mojo:421-512: every input 1e-38, one exact zero per group
    M, K, G = 4, 512, 128
    x = torch.full((M, K), 1e-38, dtype=torch.float32).to(torch.bfloat16)
    x[:, ::G] = 0.0
    q, sc = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x), G)
    assert np.all(q == 0)
    assert np.all(sc > 0) and np.all(sc < 1e-38)  # the scale itself stays a denormal (unclamped)
    # all-zero group: scale 0, recip 0; -0 inputs keep their sign (-0 * 0 = -0)
    z = torch.zeros((1, 128), dtype=torch.bfloat16)
    z[0, 3] = -0.0
    q, sc = oracle.quantize_dynamic_scaled_fp8(bf16_bits(z), 128)
    assert sc[0, 0] == 0.0 and q[0, 3] == 0x80 and q[0, 0] == 0x00


def test_scales_are_transposed_and_padding_untouched():
    M, K, G, ld = 3, 384, 128, 4
    x = torch.zeros((M, K), dtype=torch.float32)
    for r in range(M):
        for g in range(K // G):
            x[r, g * G + 7] = 448.0 * 2.0 ** (r - 2 * g - 3)
    q, sc = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x.to(torch.bfloat16)), G, scales_ld=ld)
    assert sc.shape == (3, 4)
    for r in range(M):
        for g in range(K // G):
            assert sc[g, r] == np.float32(2.0 ** (r - 2 * g - 3))
    assert np.all(np.isnan(sc[:, M:]))


def test_f32_and_f16_inputs_and_bf16_scales():
    g = torch.Generator().manual_seed(7)
    x = torch.randn((2, 256), generator=g)
    q32, s32 = oracle.quantize_dynamic_scaled_fp8(x.numpy(), 128, in_dtype=oracle.F32)
    q_ref, s_ref = torch_quant(x, 128)
    assert np.array_equal(q32, fp8_bytes(q_ref)) and np.array_equal(s32, s_ref.numpy())
    xh = x.to(torch.float16)
    q16, s16 = oracle.quantize_dynamic_scaled_fp8(xh.view(torch.int16).numpy().view(np.uint16), 128, in_dtype=oracle.F16)
    q_ref, s_ref = torch_quant(xh, 128)
    assert np.array_equal(q16, fp8_bytes(q_ref)) and np.array_equal(s16, s_ref.numpy())
    # bf16 scales (parity unpinned beyond this closed form): amax = 448 * 2^k stays exact
    row = torch.zeros((1, 128))
    row[0, 0] = 448.0 * 2
    qb, sb = oracle.quantize_dynamic_scaled_fp8(bf16_bits(row.to(torch.bfloat16)), 128, scales_dtype=oracle.BF16)
    assert oracle.bf16_bits_to_f32(sb)[0, 0] == 2.0 and qb[0, 0] == 0x7E


def _rne_bf16(v):
    """Fraction -> the nearest bf16 value (ties to even) as a Fraction; normal range only."""
    from fractions import Fraction
    e = v.numerator.bit_length() - v.denominator.bit_length()
    if Fraction(2) ** e > v:
        e -= 1
    assert Fraction(2) ** e <= v < Fraction(2) ** (e + 1) and e >= -126
    step = Fraction(2) ** (e - 7)
    q = v / step
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return n * step


def test_bf16_scales_are_the_correctly_rounded_quotient():
    # Scales of dtype bf16 are bf16(min(amax, ub)) / bf16(448), one division rounded to bf16 (fp8_utils.mojo:24-60 with the
    # scales dtype as its type).  A compiler may divide in f32 and round the f32 quotient to bf16 instead: for operands of
    # 8 significant bits the two are the same number (an intermediate of at least 2 * 8 + 2 bits makes the second rounding
    # harmless), so exact rational arithmetic pins the value whichever way the reference's compiler lowers it.  Every
    # positive bf16 amax whose quotient is a normal number.
    from fractions import Fraction
    vals = (np.arange(1, 0x7F80, dtype=np.uint32) << 16).view(np.float32)
    vals = vals[vals >= np.float32(448.0 * 2.0 ** -126)]
    x = np.zeros((vals.size, 128), dtype=np.float32)
    x[:, 5] = -vals
    x[:, 90] = vals * 0.5
    q, sc = oracle.quantize_dynamic_scaled_fp8(oracle.bf16_bits_of(x), 128, scales_dtype=oracle.BF16)
    got = oracle.bf16_bits_to_f32(sc)[0, :vals.size]
    for i in range(0, vals.size, 1):
        a = Fraction(float(vals[i]))
        want = _rne_bf16(min(a, Fraction(1200)) / 448)
        assert Fraction(float(got[i])) == want, (i, float(vals[i]), float(got[i]), float(want))
    # and the bytes follow from the f32 value of that scale: x * (1 / scale), both in f32
    s32 = got.astype(np.float32)
    recip = np.float32(1.0) / s32
    want_q = oracle.e4m3fn_encode((x * recip[:, None]).astype(np.float32))
    assert np.array_equal(q, want_q)


def test_f16_scales_are_refused():
    # the quantisers restate f32 and bf16 scales only: f16 is refused before any buffer is written
    x = np.zeros((2, 128), dtype=np.uint16)
    with pytest.raises(ValueError):
        oracle.quantize_dynamic_scaled_fp8(x, 128, scales_dtype=oracle.F16)
    with pytest.raises(ValueError):
        oracle.rms_norm_fused_quantize(x, np.zeros(128, dtype=np.uint16), 1e-5, scales_dtype=oracle.F16)
