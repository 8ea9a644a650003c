"""Oracle of the static per-tensor quantiser against torch's CPU cast and closed forms."""
import numpy as np
import torch

import oracle


def test_quantize_static_matches_torch_cpu_cast():
    gen = torch.Generator().manual_seed(0)
    x = (torch.randn((64, 512), generator=gen) * 5).to(torch.bfloat16)
    for scale in (0.02, 1.0, 0.3):
        s = np.float32(scale)
        q = oracle.quantize_static(x.view(torch.int16).numpy().view(np.uint16), float(s))
        want = (x.float() * float(np.float32(1.0) / s)).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(q, want)


def test_quantize_static_closed_forms():
    x = torch.tensor([[448.0, -448.0, 1000.0, 0.0, -0.0, 2.0 ** -9, 17.0, 19.0]], dtype=torch.float32)
    q = oracle.quantize_static(x.numpy(), 1.0, in_dtype=oracle.F32)
    assert q.tolist() == [[0x7E, 0xFE, 0x7E, 0x00, 0x80, 0x01, 0x58, 0x5A]]   # 17 -> 16, 19 -> 20 (ties to even)
    q = oracle.quantize_static(x.numpy(), 2.0, in_dtype=oracle.F32)
    assert q[0, 0] == 0x76 and q[0, 2] == 0x7E                                 # 224; 500 saturates
