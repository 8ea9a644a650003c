"""Oracle of the dynamic per-tensor quantiser against the formula of the reference's own test
(test_scaled_fp8_quantization.mojo:148-186) evaluated with torch's CPU casts."""
import numpy as np
import pytest
import torch

import oracle


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("M,K,dtype", [(1, 1024, torch.bfloat16), (4, 16384, torch.bfloat16), (4, 576, torch.float32),
                                       (2, 260, torch.bfloat16), (2, 264, torch.bfloat16)])
def test_tensor_quant_is_the_reference_tests_formula(M, K, dtype):
    g = torch.Generator().manual_seed(M * 131 + K)
    x = (torch.rand((M, K), generator=g) * 2 - 1).to(dtype)
    sdt = dtype  # the reference test pairs bf16 input with bf16 scales and f32 with f32
    src, idt = (_bits(x), oracle.BF16) if dtype == torch.bfloat16 else (x.numpy(), oracle.F32)
    q, sc = oracle.quantize_tensor_dynamic(src, in_dtype=idt, scales_dtype=oracle.BF16 if sdt == torch.bfloat16 else oracle.F32)
    # max |x| in the scales dtype, min with 1200, divided by 448 in the scales dtype
    amax = x.to(sdt).abs().max()
    scale = (torch.minimum(amax, torch.tensor(1200.0, dtype=sdt)) / torch.tensor(448.0, dtype=sdt)).to(sdt)
    recip = torch.tensor(1.0, dtype=torch.float32) / scale.float()
    want = (x.float() * recip).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(q, want)
    got_scale = torch.from_numpy(sc.view(np.int16)).view(torch.bfloat16).float() if sdt == torch.bfloat16 else torch.from_numpy(sc)
    assert got_scale.shape == (1, M) and torch.all(got_scale == scale.float())


def test_tensor_quant_zero_and_near_zero():
    # test_scaled_fp8_quantization.mojo:515-600: a denormal tensor maximum must give finite (zero) output
    x = np.zeros((3, 128), dtype=np.float32)
    q, sc = oracle.quantize_tensor_dynamic(x, in_dtype=oracle.F32)
    assert not q.any() and not sc.any()
    x[1, 5] = 1e-38
    x[2, 7] = -1e-39
    q, sc = oracle.quantize_tensor_dynamic(x, in_dtype=oracle.F32)
    assert np.all((q & 0x7F) == 0) and np.all(np.isfinite(sc)) and sc[0, 0] > 0
