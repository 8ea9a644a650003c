"""The expert matmuls of a block-scaled FP8 MoE layer (moe_fp8.py:487-616) end to end on the GPU,
against the same chain of oracle functions on the CPU: grouping, gather, quantise, grouped gate_up,
silu * up, quantise, grouped down, restore."""
import numpy as np
import pytest
import torch

import modular_amd as mx
import oracle
from modular_amd import synth
from util import assert_rel, bf16_bits, bf16_from_bits, f32_np, fp8_bytes

pytestmark = pytest.mark.gpu
NT = oracle.default_threads()
BLK = mx.blockwise_fp8_config()


def check_stages(x, router_idx, wgu, sgu, wd, sd, dev):
    """Each stage on the GPU against the oracle ON THE GPU'S OWN INPUT of that stage.  (End to end, two
    correct runs differ by percents of a row's rms: one bf16 rounding flip in gate_up can move a
    group's scale in the second quantiser and with it many fp8 codes.)"""
    seq, k = router_idx.shape
    E = wgu.shape[0]
    order, start, restore, eids, stats = mx.moe_create_indices(router_idx.reshape(-1).to(dev), E)
    o2, s2, r2, e2, st2 = oracle.moe_create_indices(router_idx.reshape(-1).numpy().astype(np.int32), E)
    for a, b in ((order, o2), (start, s2), (restore, r2), (stats, st2)):
        assert np.array_equal(a.cpu().numpy().view(np.uint32), b)
    assert np.array_equal(eids.cpu().numpy(), e2)
    stats_host = stats.cpu()

    def stage(t_gpu, w, ws, what):
        q, s = mx.quantize_dynamic_scaled_float8(t_gpu, BLK.input_scale, BLK.weight_scale, scales_type=torch.float32,
                                                 group_size_or_per_token=128)
        qo, so = oracle.quantize_dynamic_scaled_fp8(bf16_bits(t_gpu), 128, threads=NT)
        assert np.array_equal(fp8_bytes(q), qo) and np.array_equal(f32_np(s)[:, :so.shape[1]], so), what + ": quantiser"
        c = mx.grouped_dynamic_scaled_fp8_matmul(q, w.to(dev), s, ws.to(dev), start, eids, stats_host, BLK.input_scale,
                                                 BLK.weight_scale)
        co = oracle.grouped_matmul(qo, fp8_bytes(w), so, ws.numpy(), s2, e2, int(st2[0]), int(st2[1]), threads=NT)
        assert_rel(f32_np(c), co, 1e-2, what + ": grouped matmul")
        return c

    permuted = x.to(dev).index_select(0, order.to(torch.int64) // k)
    gate_up = stage(permuted, wgu, sgu, "gate_up")
    act = mx.fused_silu(gate_up, start)
    acto = f32_np(bf16_from_bits(oracle.fused_silu(bf16_bits(gate_up), gate_up.shape[0], threads=NT)))
    # silu's exp is not pinned to the last bit: one bf16 ulp
    assert np.all(np.abs(f32_np(act) - acto) <= np.abs(acto) * 2.0 ** -7 + 1e-30), "fused_silu"
    down = stage(act, wd, sd, "down")
    return down.index_select(0, restore.to(torch.int64)).reshape(seq, k, -1)


@pytest.mark.parametrize("seq,k,E,hidden,inter,zipf", [(64, 2, 8, 256, 128, 0.0), (300, 4, 16, 512, 256, 1.1), (1, 8, 32, 256, 128, 1.1)])
def test_expert_matmuls_fp8(dev, seq, k, E, hidden, inter, zipf):
    g = torch.Generator().manual_seed(seq + E)
    x = synth.activations(seq, hidden, seed=1)
    logits = torch.randn((seq, E), generator=g) - zipf * torch.log(torch.arange(1, E + 1).float())
    router_idx = logits.topk(k, dim=1).indices.to(torch.int32)
    wgu, sgu = zip(*[synth.quantize_weight_block(synth.weights_f32(2 * inter, hidden, seed=10 + e)) for e in range(E)])
    wd, sd = zip(*[synth.quantize_weight_block(synth.weights_f32(hidden, inter, seed=100 + e)) for e in range(E)])
    wgu, sgu, wd, sd = torch.stack(wgu), torch.stack(sgu), torch.stack(wd), torch.stack(sd)
    got = mx.expert_matmuls_fp8(x.to(dev), router_idx.to(dev), wgu.to(dev), sgu.to(dev), wd.to(dev), sd.to(dev), BLK)
    torch.cuda.synchronize()
    staged = check_stages(x, router_idx, wgu, sgu, wd, sd, dev)
    assert got.shape == (seq, k, hidden)
    assert torch.equal(got, staged), "the layer function is exactly its stages"
    free = mx.expert_matmuls_fp8(x.to(dev), router_idx.to(dev), wgu.to(dev), sgu.to(dev), wd.to(dev), sd.to(dev), BLK,
                                 host_sync=False)
    assert torch.equal(free, got), "upper bounds in place of the two host scalars change nothing"
    fused = mx.expert_matmuls_fp8(x.to(dev), router_idx.to(dev), wgu.to(dev), sgu.to(dev), wd.to(dev), sd.to(dev), BLK,
                                  fuse_activation_quant=True)
    rel = (fused.double() - got.double()).norm() / got.double().norm()
    assert rel < 0.02, f"one-kernel activation + quantisation: {rel:.4f} from the two-kernel form"
    # and against plain float64 arithmetic on the dequantised weights (quantisation error only)
    wgu_f = wgu.double() * sgu.double().repeat_interleave(128, 1).repeat_interleave(128, 2)[:, :2 * inter, :hidden]
    wd_f = wd.double() * sd.double().repeat_interleave(128, 1).repeat_interleave(128, 2)[:, :hidden, :inter]
    ref = torch.zeros((seq, k, hidden), dtype=torch.float64)
    for t in range(seq):
        for j in range(k):
            e = int(router_idx[t, j])
            gu = wgu_f[e] @ x[t].double()
            h = torch.nn.functional.silu(gu[:inter]) * gu[inter:]
            ref[t, j] = wd_f[e] @ h
    err = (got.double().cpu() - ref).norm() / ref.norm()
    assert err < 0.05, f"relative error {err:.3f} against float64 on dequantised weights"


def test_expert_matmuls_replay_from_a_graph(dev):
    """Without the host scalars nothing in the expert path waits for the GPU, so it records into a HIP graph.
    Every replay (with eager work and synchronisations between them, and new routing in the same buffers)
    must give the eager result."""
    seq, k, E, hidden, inter = 96, 4, 16, 512, 256
    wgu, sgu = zip(*[synth.quantize_weight_block(synth.weights_f32(2 * inter, hidden, seed=10 + e)) for e in range(E)])
    wd, sd = zip(*[synth.quantize_weight_block(synth.weights_f32(hidden, inter, seed=100 + e)) for e in range(E)])
    wgu, sgu, wd, sd = (torch.stack(t).to(dev) for t in (wgu, sgu, wd, sd))
    x = synth.activations(seq, hidden, seed=1).to(dev)
    g = torch.Generator().manual_seed(5)
    routing = lambda: torch.randn((seq, E), generator=g).topk(k, dim=1).indices.to(torch.int32)
    router_idx = routing().to(dev)
    run = lambda: mx.expert_matmuls_fp8(x, router_idx, wgu, sgu, wd, sd, BLK, host_sync=False)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        run()  # first calls outside the capture: they set the kernels' LDS attributes
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = run()
    for i in range(3):
        router_idx.copy_(routing())
        x.mul_(1.25)
        want = run()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i}"
