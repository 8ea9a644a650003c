// Argument block shared by the tiled, skinny and grouped matmul kernels.
#pragma once
#include <stdint.h>

namespace maxfp8 {

// Where a fused QKV matmul puts its columns (max/kernels/src/nn/kv_cache_ragged.mojo:1122-1307):
// columns [0, q_dim) go to C, [q_dim, q_dim + k_dim) to the K pages and the rest to the V pages
// of a paged cache [num_blocks, 2, num_layers, page_size, kv_heads, head_dim] (bf16).  Row m is
// token (m - row_offsets[b]) + cache_lengths[b] of sequence b, which lives in page
// lookup_table[b, token / page_size] at slot token % page_size (max/kernels/src/kv_cache/types.mojo:2274-2296).
struct KvStore {
  uint16_t* k_base;               // element (block 0, K, layer, 0, 0, 0)
  uint16_t* v_base;               // element (block 0, V, layer, 0, 0, 0)
  const uint32_t* lookup_table;   // [batch, lut_ld]
  const uint32_t* cache_lengths;  // [batch]
  const uint32_t* row_offsets;    // [batch + 1]
  const uint16_t* bias;           // [N] bf16 or null
  int64_t block_stride;           // elements between consecutive blocks
  int64_t lut_ld;
  int64_t num_blocks;
  int q_dim, k_dim;
  int row_elems;                  // kv_heads * head_dim
  int page_size, batch;
  int bf16_scaling;               // per-tensor / per-channel flavour: scales are applied in bf16
};

struct GemmArgs {
  const uint8_t* a;        // [M, K] e4m3fn, row stride lda bytes
  const uint8_t* b;        // [N, K] e4m3fn (per expert when grouped), row stride ldb bytes
  void* c;                 // [M, N] bf16 or f32, row stride ldc elements
  const float* a_scales;   // block: [ceil(K/128), a_scales_ld]; row/tensor: element m * a_scale_stride
  const float* b_scales;   // block: [ceil(N/128), b_scales_ld]; row/tensor: element n * b_scale_stride
  int M, N, K;
  int64_t lda, ldb, ldc;
  int64_t a_scales_ld, b_scales_ld;
  int64_t a_scale_stride, b_scale_stride;
  int c_dtype;
  int scales_dtype;        // row / tensor scaling: MAXFP8_F32, MAXFP8_BF16 or MAXFP8_F16 (block scaling is always f32)
  int c_vec_ok;            // C base and ldc allow 4-element vector stores
  int c_vec8_ok;           // ... and 8-element ones (16-byte aligned rows)
  // grouped only
  const uint32_t* offsets;
  const int32_t* expert_ids;
  int num_active;
  int small_rows;            // a tile with at most this many rows left for it uses the small tile shape (0: none does)
  int big_rows, big_bm;      // slots with at least big_rows rows give their full big_bm-row tiles to the large-tile launch (0: none)
  int heads_elsewhere;       // the persistent launch: the rows of w4_grouped_head_rows are the four-wave launch's, it has no L tiles
  int w4_hot_rest, w4_cold_rows;  // ... see w4_grouped_head_rows
  // The large-tile launch as a fixed set of blocks that share the chip with the other launch (0: one block per tile):
  int big_tile_rows;         // upper bound of the number of big_bm-row tiles over all slots
  float share_bias;          // scales the other launch's estimated work when the blocks decide how many of them stay
  int64_t b_expert_stride;   // bytes between experts in b
  int64_t bs_expert_stride;  // elements between experts in b_scales
  const uint32_t* c_row_index;  // grouped only, optional: row m of the result is stored at row c_row_index[m] of c
  // batched only: blockIdx.z (tiled) / blockIdx.y (skinny) steps the five base pointers, in elements
  int64_t a_batch, b_batch, c_batch, a_scales_batch, b_scales_batch;
  // split-K / skinny only
  float* workspace;
  int splits;
  // work split along K of the persistent kernel: which set of hand-over flags this launch uses, and the value a flag takes
  int streamk_slot;
  unsigned int streamk_seq;
  // four-wave kernel only: slabs per block of the tail (the tiles beyond the last whole round of the chip, cut evenly along
  // K among the blocks; 0: every tile is computed whole by one block)
  int tail_units;           // the four-wave kernel: slabs of a run of its cut tail (0: whole tiles only)
  // fused QKV only
  int kv_on;
  KvStore kv;
};

#if defined(__HIPCC__)
// Rows of a slot that go to the grouped form of the four-wave kernel (192 x 256 tiles) when it runs beside the persistent
// launch: the slot's full 192-row tiles; what is left behind them when that is more than hot_rest rows (one more tile,
// stored up to the slot's end); a slot without a full tile whole when it has more than cold_rows rows.  The persistent
// launch keeps the other rows.
__device__ __forceinline__ int w4_grouped_head_rows(int rows, int hot_rest, int cold_rows) {
  const int full = rows / 192 * 192;
  if (full == 0) return rows > cold_rows ? rows : 0;
  return rows - full > hot_rest ? rows : full;
}

// Element idx of a row / tensor scale vector of the given dtype, widened to f32 (exact): how the reference's
// epilogue reads its scales (max/kernels/src/linalg/fp8_quantization.mojo:1218-1240: load, cast, multiply in f32).
__device__ __forceinline__ float scale_at(const float* base, int64_t idx, int dtype) {
  if (dtype == 2 /* MAXFP8_F32 */) return base[idx];
  const uint16_t h = reinterpret_cast<const uint16_t*>(base)[idx];
  if (dtype == 0 /* MAXFP8_BF16 */) return __uint_as_float((uint32_t)h << 16);
  return (float)__builtin_bit_cast(_Float16, h);
}

// offsets (elements from k_base / v_base) of the cache rows that receive rows m[0..R); -1 for a
// row that is not live or that the lookup table has no page for (nothing is stored then).  The R
// binary searches run in lockstep with a trip count that only depends on the batch size, so
// their dependent loads overlap instead of queueing up behind each other.
template <int R>
__device__ __forceinline__ void kv_row_offsets(const KvStore& kv, const int64_t (&m)[R], const bool (&live)[R], int64_t (&off)[R]) {
  int low[R], high[R];
#pragma unroll
  for (int r = 0; r < R; ++r) { low[r] = 0; high[r] = kv.batch; }
  const int steps = kv.batch > 1 ? 32 - __builtin_clz((unsigned)(kv.batch - 1)) : 0;
  for (int s = 0; s < steps; ++s) {
    uint32_t first[R];
    int mid[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      mid[r] = (low[r] + high[r]) >> 1;  // == low[r] once the search has narrowed to one sequence
      first[r] = live[r] ? kv.row_offsets[mid[r]] : 0u;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (m[r] >= (int64_t)first[r]) low[r] = mid[r];  // the last sequence whose first row is <= m
      else high[r] = mid[r];
    }
  }
  uint32_t token[R], page[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    token[r] = live[r] ? (uint32_t)(m[r] - kv.row_offsets[low[r]]) + kv.cache_lengths[low[r]] : 0u;
    page[r] = token[r] / (uint32_t)kv.page_size;
  }
  uint32_t block[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const bool ok = live[r] && (int64_t)page[r] < kv.lut_ld;
    block[r] = ok ? kv.lookup_table[(int64_t)low[r] * kv.lut_ld + page[r]] : 0xffffffffu;
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t slot = token[r] - page[r] * (uint32_t)kv.page_size;
    off[r] = (int64_t)block[r] < kv.num_blocks ? (int64_t)block[r] * kv.block_stride + (int64_t)slot * kv.row_elems : -1;
  }
}

__device__ __forceinline__ int64_t kv_row_offset(const KvStore& kv, int64_t m) {
  const int64_t mm[1] = {m};
  const bool live[1] = {true};
  int64_t off[1];
  kv_row_offsets<1>(kv, mm, live, off);
  return off[0];
}

// destination of column n (and the columns after it up to the next multiple of 8) of row m
__device__ __forceinline__ uint16_t* kv_dst(const KvStore& kv, void* c, int64_t ldc, int64_t m, int64_t row_off, int n) {
  if (n < kv.q_dim) return reinterpret_cast<uint16_t*>(c) + m * ldc + n;
  if (n < kv.q_dim + kv.k_dim) return kv.k_base + row_off + (n - kv.q_dim);
  return kv.v_base + row_off + (n - kv.q_dim - kv.k_dim);
}

// the arguments of batch `b` of a batched matmul
__device__ __forceinline__ GemmArgs batch_view(const GemmArgs& p, int64_t b) {
  GemmArgs q = p;
  q.a += b * p.a_batch;
  q.b += b * p.b_batch;
  q.c = reinterpret_cast<uint8_t*>(p.c) + b * p.c_batch * (p.c_dtype == 0 /* bf16 */ ? 2 : 4);
  q.a_scales += b * p.a_scales_batch;
  q.b_scales += b * p.b_scales_batch;
  return q;
}
#endif

// the four-wave kernel's tail cut: blocks, slabs of a run (0: none at this shape), bytes of workspace
struct W4Split { int blocks; int unit; size_t bytes; };

}  // namespace maxfp8
