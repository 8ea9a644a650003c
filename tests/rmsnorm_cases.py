"""Inputs of the reference's fused RMSNorm + FP8 quantisation test
(max/kernels/test/gpu/nn/test_rms_norm_fused_fp8.mojo:31-57 data pattern, :171-173 gamma,
:270-330 shapes) and a numpy restatement of its host procedure (:60-126), used to pin the oracle."""
import numpy as np
import torch

SHAPES = [(16, 128), (32, 256), (8, 512), (64, 4096), (16, 8192), (16, 16384), (16, 32768)]
EPS = 1e-5


def pattern_input(rows, cols):
    i = np.arange(rows * cols) % 20
    val = np.where(i < 5, 0.05 + i * 0.05,
          np.where(i < 10, 0.3 + (i - 5) * 0.1,
          np.where(i < 15, 0.8 + (i - 10) * 0.2, 1.8 + (i - 15) * 0.3)))
    x = torch.from_numpy(val.astype(np.float32).reshape(rows, cols)).to(torch.bfloat16)
    g = torch.from_numpy((0.5 + (np.arange(cols) % 11) * 0.1).astype(np.float64)).to(torch.bfloat16)
    return x, g


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def host_procedure(x, g, eps, weight_offset, scale_ub, encode):
    """test_rms_norm_fused_fp8.mojo:60-126 in numpy f32: returns (bytes, scales)."""
    xf = x.float().numpy()
    gf = g.float().numpy() + np.float32(weight_offset)
    rows, cols = xf.shape
    out = np.zeros((rows, cols), dtype=np.uint8)
    scales = np.zeros(rows, dtype=np.float32)
    for r in range(rows):
        ms = np.float32(0.0)
        for v in xf[r]:
            ms = np.float32(ms + np.float32(v * v))
        ms = np.float32(ms / np.float32(cols))
        norm = np.float32(1.0) / np.sqrt(np.float32(ms + np.float32(eps)))
        scaled = (xf[r] * norm).astype(np.float32) * gf
        row_max = np.float32(np.abs(scaled).max()) if cols else np.float32(0)
        scale = np.float32(min(row_max, np.float32(scale_ub)) / np.float32(448.0))
        scales[r] = scale
        recip = np.float32(0.0) if scale == 0 else np.float32(1.0) / scale
        out[r] = encode(np.clip(scaled * recip, -448.0, 448.0).astype(np.float32))
    return out, scales
