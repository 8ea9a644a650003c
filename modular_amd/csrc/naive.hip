// One-thread-per-output scaled FP8 matmuls in the reference's own summation order.
// They are the on-device stand-in for the CPU restatement at sizes the CPU cannot
// finish: this file is compiled with -ffp-contract=off so that every product and
// sum is rounded exactly as in a scalar host loop, and the e4m3fn decode is done in
// software so nothing is shared with the MFMA kernels these results are held against.
//
//   blockwise: acc += ((a*b)*a_s[k/gk, m/gm])*b_s[n/gn, k/gk], k ascending
//              (max/kernels/src/linalg/fp8_quantization.mojo:1576-1624)
//   rowwise:   ((sum_k a*b) * a_s[m]) * b_s[n]   (fp8_quantization.mojo:1218-1240)
//   grouped:   blockwise per expert slot; expert id -1 writes zeros
//              (fp8_quantization.mojo:1745-1865)
#include "common.h"

namespace maxfp8 {

__device__ __forceinline__ void store_out(void* c, int c_dtype, int64_t idx, float v) {
  if (c_dtype == MAXFP8_BF16) reinterpret_cast<uint16_t*>(c)[idx] = (uint16_t)f32_to_bf16_bits(v);
  else reinterpret_cast<float*>(c)[idx] = v;
}

__device__ __forceinline__ float load_scale(const void* s, int dtype, int64_t idx) {
  if (dtype == MAXFP8_BF16) return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(s)[idx]);
  if (dtype == MAXFP8_F16) return (float)reinterpret_cast<const _Float16*>(s)[idx];
  return reinterpret_cast<const float*>(s)[idx];
}

__device__ __forceinline__ float blockwise_dot(const uint8_t* ar, const uint8_t* br, const float* a_scales,
                                               const float* b_scales_row, int64_t K, int64_t gk,
                                               int64_t a_scales_ld, int64_t a_col) {
  float acc = 0.0f;
  for (int64_t k = 0; k < K; ++k) {
    const float as = a_scales[(k / gk) * a_scales_ld + a_col];
    const float bs = b_scales_row[k / gk];
    float p = e4m3fn_to_f32_sw(ar[k]) * e4m3fn_to_f32_sw(br[k]);
    p = p * as;
    p = p * bs;
    acc = acc + p;
  }
  return acc;
}

__global__ __launch_bounds__(256) void naive_blockwise_kernel(
    void* c, const uint8_t* a, const uint8_t* b, const float* a_scales, const float* b_scales, int64_t M,
    int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t gm, int64_t gn, int64_t gk,
    int64_t a_scales_ld, int64_t b_scales_ld, int c_dtype, int64_t a_batch, int64_t b_batch, int64_t c_batch,
    int64_t as_batch, int64_t bs_batch) {
  a += blockIdx.z * a_batch;
  b += blockIdx.z * b_batch;
  c = reinterpret_cast<uint8_t*>(c) + blockIdx.z * c_batch * (c_dtype == MAXFP8_BF16 ? 2 : 4);
  a_scales += blockIdx.z * as_batch;
  b_scales += blockIdx.z * bs_batch;
  const int64_t n = (int64_t)blockIdx.x * 16 + (threadIdx.x & 15);
  const int64_t m = (int64_t)blockIdx.y * 16 + (threadIdx.x >> 4);
  if (m >= M || n >= N) return;
  const float acc = blockwise_dot(a + m * lda, b + n * ldb, a_scales, b_scales + (n / gn) * b_scales_ld, K, gk,
                                  a_scales_ld, m / gm);
  store_out(c, c_dtype, m * ldc + n, acc);
}

__global__ __launch_bounds__(256) void naive_rowwise_kernel(
    void* c, const uint8_t* a, const uint8_t* b, const void* a_scales, const void* b_scales, int64_t M,
    int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t a_stride, int64_t b_stride,
    int c_dtype, int scales_dtype) {
  const int64_t n = (int64_t)blockIdx.x * 16 + (threadIdx.x & 15);
  const int64_t m = (int64_t)blockIdx.y * 16 + (threadIdx.x >> 4);
  if (m >= M || n >= N) return;
  const uint8_t* ar = a + m * lda;
  const uint8_t* br = b + n * ldb;
  float acc = 0.0f;
  for (int64_t k = 0; k < K; ++k) acc += e4m3fn_to_f32_sw(ar[k]) * e4m3fn_to_f32_sw(br[k]);
  float v = acc * load_scale(a_scales, scales_dtype, m * a_stride);
  v = v * load_scale(b_scales, scales_dtype, n * b_stride);
  store_out(c, c_dtype, m * ldc + n, v);
}

__global__ __launch_bounds__(256) void naive_grouped_kernel(
    void* c, const uint8_t* a, const uint8_t* b, const float* a_scales, const float* b_scales,
    const uint32_t* offsets, const int32_t* expert_ids, int64_t T, int64_t N, int64_t K, int64_t a_scales_ld,
    int c_dtype) {
  const int z = blockIdx.z;
  // (held inside the T rows the buffers have, whatever the routing tensor says)
  const int64_t o0 = offsets[z], o1 = offsets[z + 1];
  const int64_t r0 = o0 < T ? o0 : T, r1 = o1 < T ? o1 : T;
  const int64_t n = (int64_t)blockIdx.x * 16 + (threadIdx.x & 15);
  const int64_t ml = (int64_t)blockIdx.y * 16 + (threadIdx.x >> 4);
  if (n >= N || ml >= r1 - r0) return;
  const int64_t m = r0 + ml;
  const int32_t e = expert_ids[z];
  float acc = 0.0f;
  if (e >= 0) {
    const int64_t kb = (K + 127) / 128, nb = (N + 127) / 128;
    acc = blockwise_dot(a + m * K, b + ((int64_t)e * N + n) * K, a_scales,
                        b_scales + ((int64_t)e * nb + n / 128) * kb, K, 128, a_scales_ld, m);
  }
  store_out(c, c_dtype, m * N + n, acc);
}

int naive_blockwise_dispatch(void* c, const void* a, const void* b, const void* a_scales, const void* b_scales,
                             int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t gm,
                             int64_t gn, int64_t gk, int64_t a_scales_ld, int64_t b_scales_ld, int c_dtype,
                             int64_t batch, int64_t a_batch, int64_t b_batch, int64_t c_batch, int64_t as_batch,
                             int64_t bs_batch, hipStream_t stream) {
  const int64_t gy = ceil_div(M, 16);
  if (gy > 65535) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "naive matmul: M = %lld too large (limit 1048560)", (long long)M);
  hipLaunchKernelGGL(naive_blockwise_kernel, dim3((unsigned)ceil_div(N, 16), (unsigned)gy, (unsigned)batch), dim3(256), 0,
                     stream, c, (const uint8_t*)a, (const uint8_t*)b, (const float*)a_scales, (const float*)b_scales, M, N,
                     K, lda, ldb, ldc, gm, gn, gk, a_scales_ld, b_scales_ld, c_dtype, a_batch, b_batch, c_batch, as_batch,
                     bs_batch);
  return launch_status("naive_blockwise");
}

int naive_rowwise_dispatch(void* c, const void* a, const void* b, const void* a_scales, const void* b_scales,
                           int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                           int64_t a_stride, int64_t b_stride, int c_dtype, int scales_dtype, hipStream_t stream) {
  const int64_t gy = ceil_div(M, 16);
  if (gy > 65535) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "naive matmul: M = %lld too large (limit 1048560)", (long long)M);
  hipLaunchKernelGGL(naive_rowwise_kernel, dim3((unsigned)ceil_div(N, 16), (unsigned)gy), dim3(256), 0, stream, c,
                     (const uint8_t*)a, (const uint8_t*)b, a_scales, b_scales, M, N, K, lda, ldb, ldc, a_stride,
                     b_stride, c_dtype, scales_dtype);
  return launch_status("naive_rowwise");
}

int naive_grouped_dispatch(void* c, const void* a, const void* b, const void* a_scales, const void* b_scales,
                           const uint32_t* offsets, const int32_t* expert_ids, int64_t T, int64_t N, int64_t K,
                           int64_t max_tokens, int64_t num_active, int64_t a_scales_ld, int c_dtype,
                           hipStream_t stream) {
  const int64_t gy = ceil_div(max_tokens, 16);
  if (gy > 65535 || num_active > 65535)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "naive grouped matmul: launch bounds exceeded (max_tokens %lld, slots %lld)",
                (long long)max_tokens, (long long)num_active);
  hipLaunchKernelGGL(naive_grouped_kernel, dim3((unsigned)ceil_div(N, 16), (unsigned)gy, (unsigned)num_active),
                     dim3(256), 0, stream, c, (const uint8_t*)a, (const uint8_t*)b, (const float*)a_scales,
                     (const float*)b_scales, offsets, expert_ids, T, N, K, a_scales_ld, c_dtype);
  return launch_status("naive_grouped");
}

}  // namespace maxfp8
