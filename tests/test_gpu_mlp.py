"""The FP8 gated MLP block (`MLP`, mirroring max/python/max/nn/linear.py:865-1095) on the GPU.

Block-scaled with SiLU it is this package's kernels only: quantise, one matmul over the stacked gate / up
weights, silu(gate) * up (by default rounded to bf16 and quantised by `down_proj` like any input; with
`fuse_activation_quant=True` fused with that quantisation), and the down matmul.  Each stage
is checked against the CPU oracle ON THE GPU'S OWN INPUT of that stage (end to end, two correct runs differ
by more than a matmul's tolerance: a bf16 flip in gate_up moves the second quantiser's scales), the block
against float64 arithmetic on the dequantised weights, and the other routes (per-token scales, bias, clamp,
another activation) against the same block put together from its three `Linear`s."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import synth
from util import assert_rel, bf16_bits, f32_np, fp8_bytes

pytestmark = pytest.mark.gpu
NT = oracle.default_threads()
BLK = mx.blockwise_fp8_config()


def make_block_mlp(hidden, ffl, dev, **kw):
    mlp = mx.MLP(hidden, ffl, BLK, device=dev, **kw)
    parts = {}
    for name, (n, k, seed) in {"gate_proj": (ffl, hidden, 1), "up_proj": (ffl, hidden, 2), "down_proj": (hidden, ffl, 3)}.items():
        w = synth.weights_f32(n, k, seed=seed)
        wq, ws = synth.quantize_weight_block(w)
        getattr(mlp, name).weight.copy_(wq.to(dev))
        getattr(mlp, name).weight_scale.copy_(ws.to(dev))
        parts[name] = (wq, ws)
    return mlp, parts


@pytest.mark.parametrize("M,hidden,ffl", [(64, 512, 1024), (300, 1024, 3584), (2048, 512, 2048), (1, 256, 512)])
def test_block_scaled_mlp_stage_by_stage(dev, M, hidden, ffl):
    mlp, parts = make_block_mlp(hidden, ffl, dev, fuse_activation_quant=True)
    assert mlp._fused()
    # the projections' weights are the halves of one buffer: nothing is concatenated per call
    assert mlp.gate_proj.weight.data_ptr() == mlp.gate_up_weight.data_ptr()
    assert torch.equal(mlp.gate_up_weight[ffl:].view(torch.uint8), parts["up_proj"][0].to(dev).view(torch.uint8))
    x = synth.activations(M, hidden, seed=5)
    y = mlp(x.to(dev).reshape(1, M, hidden))
    torch.cuda.synchronize()
    assert tuple(y.shape) == (1, M, hidden) and y.dtype == torch.bfloat16

    # stage 1: quantise + stacked matmul
    xq, xs = mx.quantize_dynamic_scaled_float8(x.to(dev), BLK.input_scale, BLK.weight_scale, scales_type=torch.float32)
    gu = mx.dynamic_scaled_matmul(xq, mlp.gate_up_weight, xs, mlp.gate_up_weight_scale, BLK.input_scale, BLK.weight_scale)
    qo, so = oracle.quantize_dynamic_scaled_fp8(bf16_bits(x), 128, threads=NT)
    assert np.array_equal(fp8_bytes(xq), qo)
    w_gu = np.concatenate([fp8_bytes(parts["gate_proj"][0]), fp8_bytes(parts["up_proj"][0])])
    s_gu = np.concatenate([parts["gate_proj"][1].numpy(), parts["up_proj"][1].numpy()])
    assert_rel(f32_np(gu), oracle.matmul_blockwise(qo, w_gu, so, s_gu, threads=NT), 1e-2, "gate_up")
    # stage 2: silu(gate) * up, quantised (scales to the last bits of exp, bytes equal or neighbours)
    rows = torch.tensor([0, M], dtype=torch.int64).to(torch.uint32).to(dev)
    hq, hs = mx.fused_silu_quantized(gu, rows, BLK)
    want_q, want_s = oracle.fused_silu(bf16_bits(gu), M, quantize=True, threads=NT)
    # (the GPU's exp and the host's differ in the last bits, so now and then a product rounds to the neighbouring
    # bf16 value; where that product is its group's largest, the group's scale moves by that one bf16 step)
    got_s = f32_np(hs)
    close = np.isclose(got_s, want_s, rtol=2 * 2.0 ** -23, atol=0)
    assert close.mean() >= 0.99 and np.allclose(got_s, want_s, rtol=2.0 ** -7, atol=0)
    assert (fp8_bytes(hq) != want_q).mean() <= 5e-3
    # stage 3: the down matmul on the GPU's own quantised activations
    down = mx.dynamic_scaled_matmul(hq, mlp.down_proj.weight, hs, mlp.down_proj.weight_scale, BLK.input_scale, BLK.weight_scale)
    ref = oracle.matmul_blockwise(fp8_bytes(hq), fp8_bytes(parts["down_proj"][0]), f32_np(hs), parts["down_proj"][1].numpy(), threads=NT)
    assert_rel(f32_np(down), ref, 1e-2, "down")
    assert torch.equal(y.reshape(M, hidden), down), "the block is exactly its stages"

    # against float64 on the dequantised weights: quantisation noise only
    def deq(name):
        wq, ws = parts[name]
        return wq.double() * ws.double().repeat_interleave(128, 0).repeat_interleave(128, 1)[:wq.shape[0], :wq.shape[1]]
    xd = x.double()
    full = (torch.nn.functional.silu(xd @ deq("gate_proj").t()) * (xd @ deq("up_proj").t())) @ deq("down_proj").t()
    err = (y.reshape(M, hidden).double().cpu() - full).norm() / full.norm()
    assert err < 0.06, f"relative error {err:.3f} against float64 on dequantised weights"


@pytest.mark.parametrize("M,hidden,ffl", [(48, 512, 1024), (257, 1024, 3584)])
def test_block_scaled_mlp_default_route_quantises_like_a_linear(dev, M, hidden, ffl):
    """Without the opt-in the activations that reach the second matmul are what the reference's block hands it:
    silu(gate) rounded to bf16, times up, rounded to bf16 (two bf16 operations, linear.py:1072), quantised by
    down_proj's own rule (upper bound 1200, multiplication by the guarded reciprocal).  The fp8 bytes and scales are
    those of the oracle's quantiser on that bf16 tensor."""
    mlp, parts = make_block_mlp(hidden, ffl, dev)
    assert not mlp._fused() and mlp._silu_kernel()
    x = synth.activations(M, hidden, seed=8).to(dev)
    y = mlp(x)
    both = mx.quantized_matmul(x, mlp.gate_up_weight, mlp.gate_up_weight_scale, None, BLK)
    rows = torch.tensor([0, M], dtype=torch.int64).to(torch.uint32).to(dev)
    hidden_act = mx.fused_silu(both, rows, round_activation=True)
    assert torch.equal(y, mlp.down_proj(hidden_act)), "the block is its stages"
    # the stage in front of the second quantiser against float64 arithmetic with the two roundings: equal but for
    # activations within the last bit of exp of a bf16 rounding boundary, and those one bf16 step apart
    g64, u64 = both[:, :ffl].double().cpu(), both[:, ffl:].double().cpu()
    act = (g64 / (1.0 + torch.exp(-g64))).to(torch.float32).to(torch.bfloat16)
    want_h = (act.double() * u64).to(torch.float32).to(torch.bfloat16)
    got_bits, want_bits = bf16_bits(hidden_act).astype(np.int32), bf16_bits(want_h).astype(np.int32)
    assert (got_bits != want_bits).mean() <= 5e-3 and np.abs(got_bits - want_bits).max() <= 1
    # (the MoE kernel's single rounding is another tensor: the flag is not a no-op)
    once = mx.fused_silu(both, rows)
    assert np.array_equal(bf16_bits(once), oracle.fused_silu(bf16_bits(both), M, quantize=False, threads=NT)) or \
        (bf16_bits(once) != oracle.fused_silu(bf16_bits(both), M, quantize=False, threads=NT)).mean() <= 5e-3
    assert not torch.equal(once, hidden_act)
    # what down_proj quantises: bit-exact with the oracle's quantize_dynamic_scaled_fp8 on the same bf16 input
    hq, hs = mx.quantize_dynamic_scaled_float8(hidden_act, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32)
    want_q, want_s = oracle.quantize_dynamic_scaled_fp8(bf16_bits(hidden_act), 128, threads=NT)
    assert np.array_equal(fp8_bytes(hq), want_q) and np.array_equal(f32_np(hs)[:, :M], want_s)
    # ... and the three-Linear route with torch's bf16 silu and product between them: the same roundings, so the same
    # block element by element (where torch's exp and the kernel's differ in their last bit, a rare activation lands
    # on the other side of a bf16 boundary and moves an fp8 code in front of the second matmul)
    want = mlp.down_proj(torch.nn.functional.silu(mlp.gate_proj(x)) * mlp.up_proj(x))
    torch.cuda.synchronize()
    assert_rel(f32_np(y), f32_np(want), 2e-2, "default route against the three linears")
    # calling twice reuses the [0, rows] operand: no host tensor is built per call
    assert len(mlp._row_offsets) == 1 and mlp(x) is not None and len(mlp._row_offsets) == 1


@pytest.mark.parametrize("kw", [dict(has_bias=True), dict(activation_function="gelu"), dict(swiglu_limit=0.5)])
def test_block_scaled_mlp_other_routes(dev, kw):
    M, hidden, ffl = 48, 512, 1024
    mlp, _ = make_block_mlp(hidden, ffl, dev, **kw)
    assert not mlp._fused()
    if kw.get("has_bias"):
        for lin, seed in ((mlp.gate_proj, 1), (mlp.up_proj, 2), (mlp.down_proj, 3)):
            lin.bias.copy_(torch.randn(lin.bias.shape, generator=torch.Generator().manual_seed(seed)).to(torch.bfloat16))
    x = synth.activations(M, hidden, seed=6).to(dev)
    y = mlp(x)
    act = mx.MLP._ACTIVATIONS[mlp.activation_function]
    g, u = act(mlp.gate_proj(x)), mlp.up_proj(x)
    if mlp.swiglu_limit > 0:
        g, u = g.clamp(max=mlp.swiglu_limit), u.clamp(min=-mlp.swiglu_limit, max=mlp.swiglu_limit)
    want = mlp.down_proj(g * u)
    torch.cuda.synchronize()
    if kw.get("has_bias"):
        assert torch.equal(y, want)          # with bias the block IS its three linears
    else:                                    # one stacked matmul instead of two: other tile shapes, other summation order
        assert_rel(f32_np(y), f32_np(want), 2e-2, str(kw))


def test_per_token_mlp_runs_gate_and_up_as_one_matmul(dev):
    M, hidden, ffl = 40, 512, 768
    cfg = mx.rowwise_fp8_config()
    mlp = mx.MLP(hidden, ffl, cfg, device=dev)
    assert mlp._one_matmul and not mlp._fused()
    for lin, (n, k, seed) in ((mlp.gate_proj, (ffl, hidden, 1)), (mlp.up_proj, (ffl, hidden, 2)), (mlp.down_proj, (hidden, ffl, 3))):
        wq, ws = synth.quantize_weight_rowwise(synth.weights_f32(n, k, seed=seed))
        lin.weight.copy_(wq.to(dev))
        lin.weight_scale.copy_(ws.to(dev))
    x = synth.activations(M, hidden, seed=7, outlier_frac=0.0).to(dev)
    y = mlp(x)
    want = mlp.down_proj(torch.nn.functional.silu(mlp.gate_proj(x)) * mlp.up_proj(x))
    torch.cuda.synchronize()
    # (the same two roundings as torch's silu and product: element by element)
    assert_rel(f32_np(y), f32_np(want), 2e-2, "per-token MLP against its three linears")


def test_mlp_argument_checks(dev):
    with pytest.raises(ValueError):
        mx.MLP(256, 512, BLK, activation_function="swish")
