"""The two small records of the paged KV cache that the fused QKV matmul needs
(max/python/max/nn/kv_cache/cache_params.py:703-780, PagedCacheValues of
max/python/max/nn/kv_cache): geometry and the device tensors of one replica.
Cache management itself (allocation, eviction, prefix reuse) is not part of this package."""
from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass
class KVCacheParams:
    dtype: torch.dtype
    n_kv_heads: int
    head_dim: int
    num_layers: int
    page_size: int = 128
    is_mla: bool = False

    @property
    def kv_dim(self) -> int:
        """Planes per block: K and V, or the single latent plane of MLA."""
        return 1 if self.is_mla else 2

    def blocks_shape(self, num_blocks: int) -> tuple[int, ...]:
        return (num_blocks, self.kv_dim, self.num_layers, self.page_size, self.n_kv_heads, self.head_dim)


@dataclass
class PagedCacheValues:
    kv_blocks: torch.Tensor      # [num_blocks, kv_dim, num_layers, page_size, n_kv_heads, head_dim]
    cache_lengths: torch.Tensor  # uint32 / int32 [batch]: tokens already in the cache per sequence
    lookup_table: torch.Tensor   # uint32 / int32 [batch, max_pages]: block index of each page
    max_lengths: torch.Tensor | None = None  # [steps, 2] on the host; not read by the matmul
