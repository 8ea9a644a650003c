"""GPU parity of the fused QKV matmul with paged-cache stores (and of the K-only cache matmul):
Q and every written cache element within tolerance of the oracle, bit-exact where the arithmetic
is exact, and every other cache element untouched.

Tolerance.  Block scaling rounds the f32 result to bf16 once: max rel err 1e-2 as for the plain
matmul.  The per-tensor / per-channel flavours follow the reference's epilogue, which rounds to
bf16 BEFORE multiplying by the (bf16) scale and rounds again: an accumulator that sits next to a
bf16 rounding boundary (the MFMA sum and the oracle's sequential sum differ in the last f32 bits)
flips the first rounding by one ulp and the second can add another, so two results of the same
arithmetic can be 2 bf16 ulps = 2^-6 apart; that is the bar there.  A bias is added after those
roundings, so errors are measured against the larger of the value before and after the bias.  Shapes follow
max/kernels/test/gpu/kv_cache/test_kv_cache_ragged_matmul_scale.mojo (8 kv heads x 128, 32 q heads,
page 512, ragged prompts over non-empty caches) plus decode and BASELINE-sized prefill."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import kernels
from modular_amd.kv_cache import KVCacheParams, PagedCacheValues
from qkv_cases import logical_rows, make_cache_case, make_operands
from util import bf16_bits, fp8_bytes

pytestmark = pytest.mark.gpu
NT = oracle.default_threads()
TOL = 1e-2
TOL_BF16_SCALING = 2.0 ** -6
FLOOR = 2.0 ** -4
POISON = 0x7FC0  # bf16 NaN


def as_i32(u):
    return torch.from_numpy(np.ascontiguousarray(u).view(np.int32))


def f32_of_bits(u):
    return (np.asarray(u).astype(np.uint32) << 16).view(np.float32)


def check_vals(got_bits, want_bits, bias_f, tol, what):
    got, want = f32_of_bits(got_bits).astype(np.float64), f32_of_bits(want_bits).astype(np.float64)
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    before = want - bias_f
    rms = np.sqrt(np.mean(before * before, axis=-1, keepdims=True))
    denom = np.maximum(np.maximum(np.abs(want), np.abs(before)), np.maximum(rms * FLOOR, 1e-30))
    e = float(np.max(np.abs(got - want) / denom)) if got.size else 0.0
    assert e <= tol, f"{what}: max rel err {e:.3e} > {tol}"


def run_case(dev, prompt, cached, Hq, H, D, K, mnk, page, layers, layer, nblocks, seed, algo="auto", bias=False,
             kv_dim=2, k_only=False, exact=False):
    T = sum(prompt)
    q_dim = 0 if k_only else Hq * D
    k_dim = H * D
    N = q_dim + (k_dim if (k_only or kv_dim == 1) else 2 * k_dim)
    a, w, sa, sb = make_operands(T, N, K, mnk, seed)
    if exact:  # small integers and power-of-two scales: every rounding is exact, the result must be bit-identical
        g = torch.Generator().manual_seed(seed)
        a = torch.randint(-1, 2, (T, K), generator=g).float().to(torch.float8_e4m3fn)
        w = torch.randint(-1, 2, (N, K), generator=g).float().to(torch.float8_e4m3fn)
        sa = torch.ones_like(sa) * 2.0
        sb = torch.ones_like(sb)
    ro, cl, lut = make_cache_case(prompt, cached, page, nblocks, seed + 7)
    params = KVCacheParams(torch.bfloat16, H, D, layers, page, is_mla=(kv_dim == 1))
    blocks_ref = np.full(params.blocks_shape(nblocks), POISON, dtype=np.uint16)
    blocks_gpu = torch.from_numpy(blocks_ref.view(np.int16).copy()).view(torch.bfloat16).to(dev)
    bias_t = None
    bias_bits = None
    if bias:
        bias_t = (torch.randn(N, generator=torch.Generator().manual_seed(seed + 9)) * (1.0 if exact else 8.0)).round().to(torch.bfloat16)
        bias_bits = bf16_bits(bias_t)
    coll = PagedCacheValues(blocks_gpu, as_i32(cl).to(dev), as_i32(lut).to(dev))
    if k_only:
        mx.matmul_k_cache_ragged_scaled_float8(params, a.to(dev), as_i32(ro).to(dev), w.to(dev), sa.to(dev), sb.to(dev),
                                               coll, mnk, layer, algo=algo)
        q = torch.empty((T, 0), dtype=torch.bfloat16)
    else:
        cfg = mx.blockwise_fp8_config() if mnk == (1, 128, 128) else None
        q = mx.fused_qkv_ragged_matmul_scaled_float8(params, a.to(dev), as_i32(ro).to(dev), w.to(dev), coll, layer, Hq,
                                                     sa.to(dev), sb.to(dev), bias=None if bias_t is None else bias_t.to(dev),
                                                     quant_config=cfg, algo=algo)
    torch.cuda.synchronize()
    q_ref = oracle.fused_qkv_matmul(fp8_bytes(a), fp8_bytes(w), sa.numpy(), sb.numpy(), mnk, ro, cl, lut, blocks_ref, layer,
                                    q_dim, bias=bias_bits, threads=NT)
    got_blocks = bf16_bits(blocks_gpu)
    written = blocks_ref != POISON
    # what the oracle left alone must be untouched on the GPU too (other layers, cached prefixes, free pages)
    assert np.array_equal(got_blocks[~written], blocks_ref[~written]), "the kernel wrote outside the new tokens"
    if exact:
        assert np.array_equal(bf16_bits(q), q_ref) and np.array_equal(got_blocks, blocks_ref)
        return
    tol = TOL if mnk == (1, 128, 128) else TOL_BF16_SCALING
    bias_f = f32_of_bits(bias_bits).astype(np.float64) if bias else np.zeros(N)
    if q_dim:
        check_vals(bf16_bits(q), q_ref, bias_f[:q_dim], tol, "Q")
    for b in range(len(prompt)):
        if prompt[b] == 0:
            continue
        for plane in range(1 if N - q_dim == k_dim else 2):
            got = logical_rows(got_blocks, plane, layer, lut, b, cached[b], prompt[b], page)
            want = logical_rows(blocks_ref, plane, layer, lut, b, cached[b], prompt[b], page)
            lo = q_dim + plane * k_dim
            check_vals(got, want, bias_f[lo:lo + k_dim], tol, f"sequence {b} plane {plane}")


LLAMA = dict(Hq=32, H=8, D=128, K=4096, page=512, layers=2, layer=1, nblocks=32)


@pytest.mark.parametrize("mnk", [(1, 128, 128), (1, 1, -1), (-1, -1, -1)])
@pytest.mark.parametrize("prompt,cached", [([100, 200, 300], [10, 20, 30]), ([1, 1, 1, 1], [511, 512, 0, 1023]),
                                           ([17, 0, 3], [500, 40, 0])])
def test_reference_shapes(dev, mnk, prompt, cached):
    run_case(dev, prompt, cached, mnk=mnk, seed=len(prompt) + sum(cached), **LLAMA)


@pytest.mark.parametrize("mnk", [(1, 128, 128), (1, 1, -1)])
@pytest.mark.parametrize("algo", ["tiled", "skinny"])
def test_exact_arithmetic_is_bit_identical(dev, mnk, algo):
    prompt = [5, 1, 0, 7] if algo == "skinny" else [130, 1, 0, 260]
    run_case(dev, prompt, [3, 0, 2, 9], Hq=3, H=2, D=16, K=256, mnk=mnk, page=4 if algo == "skinny" else 64, layers=3, layer=1,
             nblocks=16, seed=3, algo=algo, bias=True, exact=True)


@pytest.mark.parametrize("mnk", [(1, 128, 128), (1, 1, -1), (-1, -1, -1)])
def test_bias_and_both_kernels(dev, mnk):
    for algo, prompt in (("skinny", [3, 9, 1]), ("tiled", [70, 150, 33])):
        run_case(dev, prompt, [5, 0, 127], Hq=4, H=2, D=64, K=512, mnk=mnk, page=128, layers=1, layer=0, nblocks=8,
                 seed=11, algo=algo, bias=True)


def test_k_only_and_mla_layout(dev):
    # mo.k_matmul.ragged.paged.scale: everything goes to the key pages (test_kv_cache_ragged_matmul_scale.mojo:400-460)
    run_case(dev, [100, 200, 300], [10, 20, 30], mnk=(1, 128, 128), seed=1, k_only=True, **LLAMA)
    run_case(dev, [2, 4], [0, 10], mnk=(1, 128, 128), seed=2, k_only=True, **LLAMA)
    # MLA: one latent "head" of 576, a single plane per block
    run_case(dev, [33, 90], [3, 64], Hq=0, H=1, D=576, K=7168, mnk=(1, 128, 128), page=128, layers=2, layer=0, nblocks=4,
             seed=3, kv_dim=1, k_only=True)


def test_prefill_sized(dev):
    # Llama-3.1-8B QKV (N = 6144, K = 4096) over 2048 new tokens in 5 sequences
    run_case(dev, [700, 1, 512, 35, 800], [0, 4000, 12, 300, 90], mnk=(1, 128, 128), seed=5,
             Hq=32, H=8, D=128, K=4096, page=128, layers=2, layer=0, nblocks=64)


def test_errors(dev):
    params = KVCacheParams(torch.bfloat16, 2, 16, 1, 4)
    blocks = torch.zeros(params.blocks_shape(4), dtype=torch.bfloat16, device=dev)
    coll = PagedCacheValues(blocks, torch.zeros(1, dtype=torch.int32, device=dev), torch.zeros((1, 2), dtype=torch.int32, device=dev))
    a, w, sa, sb = make_operands(4, 3 * 16 + 64, 128, (1, 1, -1), 0)
    ro = torch.tensor([0, 4], dtype=torch.int32, device=dev)
    args = (params, a.to(dev), ro, w.to(dev), coll, 0, 3, sa.to(dev), sb.to(dev))
    mx.fused_qkv_ragged_matmul_scaled_float8(*args)
    with pytest.raises(ValueError, match="Can not infer"):
        mx.fused_qkv_ragged_matmul_scaled_float8(params, a.to(dev), ro, w.to(dev), coll, 0, 3, sa.to(dev).T.contiguous(), sb.to(dev))
    with pytest.raises(TypeError, match="uint32"):
        mx.fused_qkv_ragged_matmul_scaled_float8(params, a.to(dev), ro.long(), w.to(dev), coll, 0, 3, sa.to(dev), sb.to(dev))
    with pytest.raises(ValueError, match="N ="):
        mx.fused_qkv_ragged_matmul_scaled_float8(params, a.to(dev), ro, w.to(dev)[:100], coll, 0, 3, sa.to(dev), sb.to(dev)[:100])
    with pytest.raises(ValueError, match="cache geometry"):
        mx.fused_qkv_ragged_matmul_scaled_float8(params, a.to(dev), ro, w.to(dev), coll, 5, 3, sa.to(dev), sb.to(dev))
    # no sequences: nothing happens
    out = mx.fused_qkv_ragged_matmul_scaled_float8(params, a[:0].to(dev), ro[:1], w.to(dev), coll, 0, 3, sa.to(dev)[:, :0], sb.to(dev))
    assert out.shape == (0, 48)


@pytest.mark.parametrize("flavour", ["block", "rowwise", "tensor_dynamic", "static"])
def test_quantized_fused_qkv_matmul_equals_its_parts(dev, flavour):
    # the dispatcher = the quantiser of the config + the fused matmul; compared with the unfused linear
    # (quantized_matmul) whose K / V columns are read back from the cache
    from modular_amd.quant_config import InputScaleSpec, QuantConfig, QuantFormat, ScaleGranularity, ScaleOrigin, WeightScaleSpec
    Hq, H, D, K, page = 4, 2, 64, 512, 16
    prompt, cached = [40, 3, 90], [5, 0, 17]
    T, q_dim, k_dim = sum(prompt), Hq * D, H * D
    N = q_dim + 2 * k_dim
    g = torch.Generator().manual_seed(4)
    x = (torch.randn((T, K), generator=g) * 2).to(torch.bfloat16).to(dev)
    w = (torch.randn((N, K), generator=g) * 0.05)
    input_scale = None
    if flavour == "block":
        cfg = mx.blockwise_fp8_config()
        ws = torch.rand((-(-N // 128), K // 128), generator=g) * 0.01 + 0.001
        wq = (w / ws.repeat_interleave(128, 0)[:N].repeat_interleave(128, 1)).clamp(-448, 448).to(torch.float8_e4m3fn)
    elif flavour == "rowwise":
        cfg = mx.rowwise_fp8_config()
        ws = w.abs().amax(dim=1, keepdim=True) / 448
        wq = (w / ws).to(torch.float8_e4m3fn)
    else:
        origin = ScaleOrigin.STATIC if flavour == "static" else ScaleOrigin.DYNAMIC
        cfg = QuantConfig(InputScaleSpec(ScaleGranularity.TENSOR, origin, torch.float32),
                          WeightScaleSpec(ScaleGranularity.TENSOR, torch.float32), format=QuantFormat.COMPRESSED_TENSORS_FP8)
        if flavour == "static":
            ws = (w.abs().amax() / 448).reshape(1)
            wq = (w / ws).to(torch.float8_e4m3fn)
            input_scale = torch.tensor([0.03])
        else:
            ws = w.abs().amax(dim=1, keepdim=True) / 448      # fused QKV weights carry rowwise [N, 1] scales
            wq = (w / ws).to(torch.float8_e4m3fn)
    ro, cl, lut = make_cache_case(prompt, cached, page, 16, 1)
    params = KVCacheParams(torch.bfloat16, H, D, 1, page)
    blocks = torch.zeros(params.blocks_shape(16), dtype=torch.bfloat16, device=dev)
    coll = PagedCacheValues(blocks, as_i32(cl).to(dev), as_i32(lut).to(dev))
    q = mx.quantized_fused_qkv_matmul(params, x, wq.to(dev), coll, 0, as_i32(ro).to(dev), Hq, cfg, ws.to(dev), input_scale=input_scale)
    if flavour == "tensor_dynamic":
        # the unfused linear quantises per token there; build the per-tensor reference from the pieces
        xq, xs = mx.quantize_tensor_dynamic_scaled_float8(x, cfg.input_scale, cfg.weight_scale, scales_type=torch.float32)
        row = mx.rowwise_fp8_config()
        full = mx.dynamic_scaled_matmul(xq, wq.to(dev), xs, ws.to(dev), row.input_scale, row.weight_scale)
    else:
        full = mx.quantized_matmul(x, wq.to(dev), ws.to(dev) if flavour != "static" else ws, input_scale=input_scale, quant_config=cfg)
    torch.cuda.synchronize()
    full_np = full.float().cpu().numpy()
    # the unfused linear applies f32 scales once; the fused epilogue rounds both scales, their product and the
    # value to bf16 (the reference's epilogue): five roundings of 2^-9 .. 2^-8 each
    tol = TOL if flavour == "block" else 2.0 ** -5
    zero = np.zeros(N)
    check_vals(bf16_bits(q), bf16_bits(full[:, :q_dim].contiguous()), zero[:q_dim], tol, "Q")
    got_blocks = bf16_bits(blocks)
    for b in range(len(prompt)):
        rows = slice(int(ro[b]), int(ro[b + 1]))
        for plane in range(2):
            got = logical_rows(got_blocks, plane, 0, lut, b, cached[b], prompt[b], page)
            lo = q_dim + plane * k_dim
            want = bf16_bits(full[rows, lo:lo + k_dim].contiguous())
            check_vals(got, want, zero[:k_dim], tol, f"sequence {b} plane {plane}")
