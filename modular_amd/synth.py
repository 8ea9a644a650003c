"""Seeded synthetic workloads for tests and the benchmark: activations, offline
weight quantisation and MoE routing.  This is data preparation with torch ops on
whatever device is asked for; none of it is on the measured path.

Recipes follow the reference's own tests: block weight scales
`scale = max(|w|_block, 1e-6) / 448, q = clamp(w / scale)`
(max/tests/integration/architectures/glm/test_mla_fp8_glm.py:76-96) and rowwise
`scale = absmax / 448` (max/tests/integration/nn/test_mlp_float8_gpu.py:103-125).
"""
from __future__ import annotations

import math

import torch

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0


def activations(M: int, K: int, seed: int = 0, outlier_frac: float = 0.01, outlier_scale: float = 20.0,
                device="cpu") -> torch.Tensor:
    """bf16 [M, K] ~ N(0,1) with ceil(outlier_frac*K) channels multiplied by outlier_scale."""
    g = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn((M, K), generator=g, device=device, dtype=torch.float32)
    n_out = math.ceil(outlier_frac * K) if outlier_frac > 0 else 0
    if n_out:
        cols = torch.randperm(K, generator=g, device=device)[:n_out]
        x[:, cols] *= outlier_scale
    return x.to(torch.bfloat16)


def weights_f32(N: int, K: int, seed: int = 1, std: float = 0.02, device="cpu") -> torch.Tensor:
    g = torch.Generator(device=device).manual_seed(seed)
    return torch.randn((N, K), generator=g, device=device, dtype=torch.float32) * std


def quantize_weight_block(w: torch.Tensor, block: int = 128) -> tuple[torch.Tensor, torch.Tensor]:
    """w [..., N, K] f32 -> (q e4m3fn [..., N, K], scales f32 [..., ceil(N/b), ceil(K/b)])."""
    *lead, N, K = w.shape
    nb, kb = -(-N // block), -(-K // block)
    wp = torch.zeros((*lead, nb * block, kb * block), dtype=torch.float32, device=w.device)
    wp[..., :N, :K] = w
    blocks = wp.reshape(*lead, nb, block, kb, block)
    amax = blocks.abs().amax(dim=(-3, -1))                       # [..., nb, kb]
    scale = amax.clamp(min=1e-6) / FP8_MAX
    q = (blocks / scale[..., :, None, :, None]).clamp(-FP8_MAX, FP8_MAX)
    q = q.reshape(*lead, nb * block, kb * block)[..., :N, :K].contiguous().to(FP8)
    return q, scale.contiguous()


def quantize_weight_rowwise(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """w [N, K] f32 -> (q e4m3fn [N, K], scales f32 [N, 1])."""
    amax = w.abs().amax(dim=1, keepdim=True).clamp(min=1e-6)
    scale = amax / FP8_MAX
    q = (w / scale).clamp(-FP8_MAX, FP8_MAX).to(FP8)
    return q, scale.contiguous()


def random_fp8(shape, seed: int, device="cpu", std: float = 1.0) -> torch.Tensor:
    """e4m3fn tensor of N(0, std) values (already 'quantised' data for GEMM tests)."""
    g = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn(shape, generator=g, device=device, dtype=torch.float32) * std
    return x.clamp(-FP8_MAX, FP8_MAX).to(FP8)


def random_scales(shape, seed: int, device="cpu", lo: float = 0.5, hi: float = 2.0) -> torch.Tensor:
    g = torch.Generator(device=device).manual_seed(seed)
    return (torch.rand(shape, generator=g, device=device, dtype=torch.float32) * (hi - lo) + lo)


def moe_routing(tokens: int, num_experts: int, top_k: int, seed: int = 0, zipf_a: float = 1.1,
                device="cpu"):
    """Top-k routing with Zipf(zipf_a) expert popularity.

    Returns (expert_start_indices uint32 [E+1], expert_ids int32 [E], counts int64 [E],
    usage_stats_host uint32 [2] on the CPU = [max tokens per expert, active experts]).
    Every expert keeps a slot, including those with no tokens
    (max/kernels/src/nn/moe.mojo:548-558, 584-588).
    """
    g = torch.Generator(device="cpu").manual_seed(seed)
    perm = torch.randperm(num_experts, generator=g)
    rank = torch.empty(num_experts, dtype=torch.float32)
    rank[perm] = torch.arange(1, num_experts + 1, dtype=torch.float32)
    logp = -zipf_a * torch.log(rank)
    logits = torch.randn((tokens, num_experts), generator=g) + logp
    top = torch.topk(torch.softmax(logits, dim=-1), top_k, dim=-1).indices  # [tokens, k]
    counts = torch.bincount(top.reshape(-1), minlength=num_experts)
    offsets = torch.zeros(num_experts + 1, dtype=torch.int64)
    offsets[1:] = torch.cumsum(counts, 0)
    stats = torch.tensor([int(counts.max()), num_experts], dtype=torch.int64).to(torch.uint32)
    return (offsets.to(torch.uint32).to(device), torch.arange(num_experts, dtype=torch.int32, device=device),
            counts, stats)
