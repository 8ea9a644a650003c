// Argument block shared by the tiled, skinny and grouped matmul kernels.
#pragma once
#include <stdint.h>

namespace maxfp8 {

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
  int c_vec_ok;            // C base and ldc allow 4-element vector stores
  int c_vec8_ok;           // ... and 8-element ones (16-byte aligned rows)
  // grouped only
  const uint32_t* offsets;
  const int32_t* expert_ids;
  int num_active;
  int small_rows;            // slots with at most this many rows use the small tile (0: none do)
  int big_rows, big_bm;      // slots with at least big_rows rows give their full big_bm-row tiles to the large-tile launch (0: none)
  int64_t b_expert_stride;   // bytes between experts in b
  int64_t bs_expert_stride;  // elements between experts in b_scales
  // batched only: blockIdx.z (tiled) / blockIdx.y (skinny) steps the five base pointers, in elements
  int64_t a_batch, b_batch, c_batch, a_scales_batch, b_scales_batch;
  // split-K / skinny only
  float* workspace;
  int splits;
};

#if defined(__HIPCC__)
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

}  // namespace maxfp8
