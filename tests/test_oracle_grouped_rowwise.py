"""The grouped rowwise oracle is the per-slot composition of the pinned rowwise oracle; this pins
the composition (slot boundaries, expert lookup, -1, spare rows) against a float64 matmul."""
import numpy as np
import torch

import oracle
from modular_amd import synth
from util import fp8_bytes


def test_grouped_rowwise_composition():
    counts, ids, E, N, K = [5, 0, 17, 3], [2, 1, -1, 0], 3, 48, 256
    T = sum(counts) + 4
    a, b = synth.random_fp8((T, K), 0), synth.random_fp8((E, N, K), 1)
    sa, sb = synth.random_scales((T, 1), 2), synth.random_scales((E, N, 1), 3)
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    c = oracle.grouped_matmul_rowwise(fp8_bytes(a), fp8_bytes(b), sa.numpy(), sb.numpy(), off, np.array(ids, np.int32), 4)
    assert np.isnan(c[sum(counts):]).all(), "rows past the last active slot are not written"
    lo = 0
    for cnt, e in zip(counts, ids):
        rows = slice(lo, lo + cnt)
        lo += cnt
        if e < 0:
            assert not c[rows].any()
            continue
        want = (a[rows].double() @ b[e].double().T) * sa[rows].double() * sb[e].double().reshape(1, -1)
        assert np.allclose(c[rows], want.numpy(), rtol=1e-5, atol=1e-5)
