"""Oracle of the MoE plumbing: moe_create_indices against the invariants of the reference's
test (same sizes) and against numpy's stable sort; fused_silu against closed forms and a
float64 evaluation."""
import numpy as np
import pytest
import torch

import oracle
from moe_checks import check_indices


@pytest.mark.parametrize("n,num_experts", [(197, 256), (2500, 256), (11, 256), (1, 256), (20660, 256), (100000, 256), (0, 8), (64, 3)])
def test_create_indices(n, num_experts):
    rng = np.random.default_rng(n + num_experts)
    ids = rng.integers(0, num_experts, n).astype(np.int32)
    out = oracle.moe_create_indices(ids, num_experts)
    check_indices(ids, num_experts, *out)
    order, start, restore, eids, stats = out
    assert np.array_equal(order, np.argsort(ids, kind="stable").astype(np.uint32))
    assert np.array_equal(eids, np.arange(num_experts))
    assert np.array_equal(start[1:], np.cumsum(np.bincount(ids, minlength=num_experts)))


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_fused_silu_closed_forms():
    I = 256
    x = torch.zeros((3, 2 * I), dtype=torch.bfloat16)
    x[0, :I], x[0, I:] = 0.0, 5.0          # silu(0) = 0
    x[1, :I], x[1, I:] = 40.0, 0.5         # exp(-40) vanishes in f32: silu(40) = 40 -> 20
    x[2, :I], x[2, I:] = -100.0, 3.0       # exp(100) overflows to inf: -100 / inf = -0 -> -0 * 3
    out = oracle.fused_silu(_bits(x), 3)
    got = torch.from_numpy(out.view(np.int16)).view(torch.bfloat16).float()
    assert torch.all(got[0] == 0) and torch.all(got[1] == 20.0) and torch.all(got[2] == 0)
    q, s = oracle.fused_silu(_bits(x), 3, quantize=True)
    assert np.all(s[:, 1] == np.float32(20.0) / np.float32(448.0)) and np.all(q[1] == 0x7E)
    # all-zero group: the scale floor 1e-4 / 448, bytes 0
    assert np.all(s[:, 0] == np.float32(1e-4) / np.float32(448.0)) and not q[0].any()
    # rows at and past `rows` are not touched
    q, s = oracle.fused_silu(_bits(x), 1, quantize=True)
    assert not q[1:].any() and np.all(np.isnan(s[:, 1:]))


def test_fused_silu_against_float64():
    gen = torch.Generator().manual_seed(0)
    x = (torch.randn((16, 1024), generator=gen) * 3).to(torch.bfloat16)
    out = oracle.fused_silu(_bits(x), 16)
    got = torch.from_numpy(out.view(np.int16)).view(torch.bfloat16).double()
    g, u = x[:, :512].double(), x[:, 512:].double()
    want = g / (1 + torch.exp(-g)) * u
    assert float(((got - want).abs() / (want.abs() + 1e-3)).max()) <= 2.0 ** -8   # one bf16 rounding
    q, s = oracle.fused_silu(_bits(x), 16, quantize=True)
    amax = want.reshape(16, 4, 128).abs().amax(-1)
    assert np.allclose(s.T, (amax / 448.0).numpy(), rtol=1e-6)
    deq = oracle.e4m3fn_decode_table()[q].reshape(16, 4, 128) * s.T[:, :, None]
    assert float((torch.from_numpy(deq).double() - want.reshape(16, 4, 128)).abs().max() / amax.max()) <= 2.0 ** -4
