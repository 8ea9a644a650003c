"""Shared builders of the fused-QKV / paged-cache tests: ragged batches, a lookup table that
scatters pages over the block pool, and an independent read-back of the cache."""
import numpy as np
import torch

from modular_amd import synth


def make_cache_case(prompt_lens, cache_sizes, page_size, num_blocks, seed):
    """row_offsets [B+1], cache_lengths [B], lookup_table [B, max_pages] (unused entries = 0xFFFFFFFF
    would fault a careless kernel; they are set to num_blocks, which the kernels must never read
    for a live token).  Pages are handed out from a random permutation of the pool."""
    B = len(prompt_lens)
    ro = np.zeros(B + 1, dtype=np.uint32)
    ro[1:] = np.cumsum(prompt_lens)
    cl = np.asarray(cache_sizes, dtype=np.uint32)
    pages = [-(-(int(p) + int(c)) // page_size) for p, c in zip(prompt_lens, cache_sizes)]
    max_pages = max(max(pages), 1)
    assert sum(pages) <= num_blocks
    perm = np.random.default_rng(seed).permutation(num_blocks)
    lut = np.full((B, max_pages), num_blocks, dtype=np.uint32)
    nxt = 0
    for b in range(B):
        lut[b, :pages[b]] = perm[nxt:nxt + pages[b]]
        nxt += pages[b]
    return ro, cl, lut


def logical_rows(kv_blocks, kv_idx, layer, lut, b, first, count, page_size):
    """Tokens [first, first + count) of sequence b from plane kv_idx of `layer`, [count, heads * head_dim],
    read with one fancy-index gather (not the per-token formula of the code under test)."""
    toks = np.arange(first, first + count)
    plane = kv_blocks[:, kv_idx, layer]                      # [blocks, page, heads, head_dim]
    rows = plane[lut[b, toks // page_size].astype(np.int64), toks % page_size]
    return rows.reshape(count, -1)


def make_operands(T, N, K, mnk, seed, std=1.0):
    a = synth.random_fp8((T, K), seed, std=std)
    w = synth.random_fp8((N, K), seed + 1, std=std)
    if mnk == (-1, -1, -1):
        sa = synth.random_scales((1, 1), seed + 2)
        sb = synth.random_scales((1, 1), seed + 3)
    elif mnk == (1, 1, -1):
        sa = synth.random_scales((1, T), seed + 2)
        sb = synth.random_scales((N, 1), seed + 3)
    else:
        sa = synth.random_scales((-(-K // 128), -(-T // 4) * 4), seed + 2)
        sb = synth.random_scales((-(-N // 128), -(-K // 128)), seed + 3)
    return a, w, sa, sb
