"""Pins the oracle's e4m3fn codec (oracle/maxfp8_oracle.c) against the committed
fixtures (made by torch's CPU cast, tests/golden/make_e4m3fn_vectors.py), against
torch's cast live, and against the closed form of the format."""
import os

import numpy as np
import torch

import oracle

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_decode_matches_fixture_and_closed_form():
    table = oracle.e4m3fn_decode_table()
    gold = np.fromfile(os.path.join(GOLD, "e4m3fn_decode_256.f32"), dtype="<f4")
    finite = ~np.isnan(gold)
    assert finite.sum() == 254 and np.isnan(table[0x7F]) and np.isnan(table[0xFF])
    assert np.array_equal(table[finite].view(np.uint32), gold[finite].view(np.uint32))
    # closed form: (-1)^s * 2^(e-7) * (1 + m/8), subnormals m/8 * 2^-6
    for b in range(256):
        s, e, m = b >> 7, (b >> 3) & 15, b & 7
        if e == 15 and m == 7:
            continue
        v = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        assert table[b] == np.float32(-v if s else v)
    assert table[0x7E] == 448.0 and table[0x01] == 2.0 ** -9
    assert np.signbit(table[0x80]) and table[0x80] == 0.0


def test_encode_all_bf16_matches_fixture():
    gold = np.fromfile(os.path.join(GOLD, "e4m3fn_encode_bf16_65536.u8"), dtype=np.uint8)
    x = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    mine = oracle.e4m3fn_encode(np.clip(x, -448.0, 448.0))
    ok = ~np.isnan(x)
    assert np.array_equal(mine[ok], gold[ok])
    assert np.all(mine[~ok] == 0x7F)  # every NaN encodes as 0x7f (sign dropped)


def test_encode_random_f32_matches_torch():
    rng = np.random.default_rng(123)
    bits = rng.integers(0, 2 ** 32, size=1 << 21, dtype=np.uint64).astype(np.uint32)
    mags = rng.standard_normal(1 << 21).astype(np.float32) * np.exp2(rng.integers(-14, 9, size=1 << 21)).astype(np.float32)
    for x in (bits.view(np.float32), mags):
        x = x[~np.isnan(x)]
        mine = oracle.e4m3fn_encode(np.clip(x, -448.0, 448.0))
        ref = torch.from_numpy(x.copy()).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(mine, ref)


def test_encode_named_cases():
    enc = lambda *v: oracle.e4m3fn_encode(np.array(v, dtype=np.float32)).tolist()
    # ties to even between representable neighbours (16,18,20 ; 240,256)
    assert enc(17.0, 19.0, 248.0) == [0x58, 0x5A, 0x78]  # 16, 20, 256
    # half of the smallest subnormal ties to zero, just above rounds up
    assert enc(2.0 ** -10, np.nextafter(np.float32(2.0 ** -10), np.float32(1))) == [0x00, 0x01]
    # sign survives rounding to zero
    assert enc(-1e-30, -0.0, 0.0) == [0x80, 0x80, 0x00]
    # saturation (satfinite) and NaN
    assert enc(448.0, 449.0, 464.0, 1e30, np.inf, -np.inf, -1000.0) == [0x7E] * 5 + [0xFE, 0xFE]
    assert enc(np.nan) == [0x7F]
    # round trip of every finite code
    table = oracle.e4m3fn_decode_table()
    codes = np.array([b for b in range(256) if b not in (0x7F, 0xFF)], dtype=np.uint8)
    assert np.array_equal(oracle.e4m3fn_encode(table[codes]), codes)
