// Dynamic activation quantisation for gfx950: bf16/f16/f32 [M, K] -> e4m3fn [M, K]
// plus one scale per (row, group), stored transposed as scales[group, row].
//
// Arithmetic (max/kernels/src/linalg/fp8_quantization.mojo:509-583,
// max/kernels/src/internal_utils/fp8_utils.mojo:24-143):
//   amax  = max |x| over the group (f32)
//   scale = min(amax, scale_ub) / 448          (correctly rounded division)
//   recip = scale == 0 ? 0 : 1 / scale         (0 when that is inf or nan)
//   q     = e4m3fn(clamp(x * recip, -448, 448)) (round to nearest even)
//
// Kernels:
//   quant_g128_bf16   group 128, bf16 in, f32 scales.  One pass: 16 lanes own one
//                     group (16-byte loads), amax by DPP inside the 16-lane row,
//                     8-byte packed fp8 stores.  A block covers 16 rows x (4*U)
//                     groups so the transposed scale stores of one group are 64
//                     contiguous bytes.
//   quant_row_bf16    per-token (group == K), bf16 in, f32 scales.  One block per
//                     row, the row is kept in registers between the amax and the
//                     convert pass.
//   quant_generic     every other dtype / group size / alignment: one block per
//                     (row, group), two passes over the group.
#include "common.h"

namespace maxfp8 {

// Batched launches (blockIdx.y = batch) step the three base pointers by these element counts.
struct BatchStep { int64_t in, out, scales; };
// Optional row gather: output row r is quantised from input row index[r] / div (index == nullptr: row r).
struct RowGather { const uint32_t* index; uint32_t div; };

// 16 bytes of the input.  STREAM: a non-temporal load, for inputs too large for the 256 MB memory-side cache -- a stream
// marked so reads faster (7.0 against 6.2 TB/s on a read-only kernel; these kernels 7-9 % on 470 MB of input) -- while a
// smaller input, usually still in that cache from the kernel that wrote it, is better off with plain loads (3 % here).
constexpr int64_t kStreamInputBytes = (int64_t)1 << 28;
template <bool STREAM>
__device__ __forceinline__ uint4 load_input(const uint4* p) {
  if constexpr (STREAM) {
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    const u4 v = __builtin_nontemporal_load(reinterpret_cast<const u4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
  } else {
    return *p;
  }
}

// ---------------------------------------------------------------------------
template <int U, bool STREAM>
__global__ __launch_bounds__(256) void quant_g128_bf16_kernel(
    uint8_t* __restrict__ out, float* __restrict__ scales, const uint16_t* __restrict__ in,
    int M, int ngroups, int nxb, int64_t in_stride, int64_t out_stride, int64_t scales_ld,
    float scale_ub, BatchStep bs, RowGather rg) {
  in += blockIdx.y * bs.in;
  out += blockIdx.y * bs.out;
  scales += blockIdx.y * bs.scales;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int seg = lane >> 4, sl = lane & 15;
  const int rb = blockIdx.x / nxb, xb = blockIdx.x - rb * nxb;
  const int row = rb * 16 + wave * 4 + seg;
  // Each wave owns 4 rows (one per 16-lane segment) and the block's U consecutive groups.
  const int gbase = xb * U;
  const bool row_ok = row < M;
  const int64_t src_row = (rg.index && row_ok) ? (int64_t)(rg.index[row] / rg.div) : row;

  uint4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int g = gbase + u;
    if (row_ok && g < ngroups)
      v[u] = load_input<STREAM>(reinterpret_cast<const uint4*>(in + src_row * in_stride + (int64_t)g * 128 + sl * 8));
    else
      v[u] = make_uint4(0, 0, 0, 0);
  }

  float my_scale = 0.0f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[i]));
    amax = row16_max(amax);
    float scale, recip;
    dynamic_scale_f32(amax, scale_ub, scale, recip);
    if (sl == u) my_scale = scale;
    int lo = 0, hi = 0;
    lo = cvt_pk_e4m3fn(clamp448(f[0] * recip), clamp448(f[1] * recip), lo, false);
    lo = cvt_pk_e4m3fn(clamp448(f[2] * recip), clamp448(f[3] * recip), lo, true);
    hi = cvt_pk_e4m3fn(clamp448(f[4] * recip), clamp448(f[5] * recip), hi, false);
    hi = cvt_pk_e4m3fn(clamp448(f[6] * recip), clamp448(f[7] * recip), hi, true);
    const int g = gbase + u;
    if (row_ok && g < ngroups)
      *reinterpret_cast<uint2*>(out + (int64_t)row * out_stride + (int64_t)g * 128 + sl * 8) =
          make_uint2((uint32_t)lo, (uint32_t)hi);
  }
  if (row_ok && sl < U && gbase + sl < ngroups) scales[(int64_t)(gbase + sl) * scales_ld + row] = my_scale;
}

// ---------------------------------------------------------------------------
// The same quantisation with `copies` destinations: input row r is quantised once and written to the output rows
// dst_index[r * copies + j], j < copies (rows of `out`, columns of `scales`).  What a row gather with repeated source
// rows costs top_k times over -- the loads and the arithmetic -- is paid once; the stores are the gather form's.
// A destination outside [0, out_rows) is skipped.
template <int U>
__global__ __launch_bounds__(256) void quant_g128_bf16_scatter_kernel(
    uint8_t* __restrict__ out, float* __restrict__ scales, const uint16_t* __restrict__ in,
    int M, int ngroups, int nxb, int64_t in_stride, int64_t out_stride, int64_t scales_ld,
    float scale_ub, const uint32_t* __restrict__ dst_index, int copies, int64_t out_rows) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int seg = lane >> 4, sl = lane & 15;
  const int rb = blockIdx.x / nxb, xb = blockIdx.x - rb * nxb;
  const int row = rb * 16 + wave * 4 + seg;
  const int gbase = xb * U;
  const bool row_ok = row < M;

  uint4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int g = gbase + u;
    if (row_ok && g < ngroups)
      v[u] = *reinterpret_cast<const uint4*>(in + (int64_t)row * in_stride + (int64_t)g * 128 + sl * 8);
    else
      v[u] = make_uint4(0, 0, 0, 0);
  }
  float my_scale = 0.0f;
  uint2 code[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[i]));
    amax = row16_max(amax);
    float scale, recip;
    dynamic_scale_f32(amax, scale_ub, scale, recip);
    if (sl == u) my_scale = scale;
    int lo = 0, hi = 0;
    lo = cvt_pk_e4m3fn(clamp448(f[0] * recip), clamp448(f[1] * recip), lo, false);
    lo = cvt_pk_e4m3fn(clamp448(f[2] * recip), clamp448(f[3] * recip), lo, true);
    hi = cvt_pk_e4m3fn(clamp448(f[4] * recip), clamp448(f[5] * recip), hi, false);
    hi = cvt_pk_e4m3fn(clamp448(f[6] * recip), clamp448(f[7] * recip), hi, true);
    code[u] = make_uint2((uint32_t)lo, (uint32_t)hi);
  }
  if (!row_ok) return;
  for (int j = 0; j < copies; ++j) {
    const int64_t dst = dst_index[(int64_t)row * copies + j];
    if (dst >= out_rows) continue;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (gbase + u < ngroups)
        *reinterpret_cast<uint2*>(out + dst * out_stride + (int64_t)(gbase + u) * 128 + sl * 8) = code[u];
    }
    if (sl < U && gbase + sl < ngroups) scales[(int64_t)(gbase + sl) * scales_ld + dst] = my_scale;
  }
}

// ---------------------------------------------------------------------------
// One block (256 threads) per row, group == K.  NV 16-byte vectors per thread are
// held in registers; K <= 256 * 8 * NV.
template <int NV, bool STREAM>
__global__ __launch_bounds__(256) void quant_row_bf16_kernel(
    uint8_t* __restrict__ out, float* __restrict__ scales, const uint16_t* __restrict__ in,
    int K, int64_t in_stride, int64_t out_stride, float scale_ub, BatchStep bs, RowGather rg) {
  in += blockIdx.y * bs.in;
  out += blockIdx.y * bs.out;
  scales += blockIdx.y * bs.scales;
  __shared__ float red[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const uint16_t* src = in + (rg.index ? (int64_t)(rg.index[row] / rg.div) : (int64_t)row) * in_stride;
  const int nvec = K >> 3;
  uint4 v[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = tid + i * 256;
    v[i] = idx < nvec ? load_input<STREAM>(reinterpret_cast<const uint4*>(src) + idx) : make_uint4(0, 0, 0, 0);
  }
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      amax = fmaxf(amax, fabsf(__uint_as_float(w[j] << 16)));
      amax = fmaxf(amax, fabsf(__uint_as_float(w[j] & 0xffff0000u)));
    }
  }
  amax = wave_max(amax);
  if ((tid & 63) == 0) red[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  float scale, recip;
  dynamic_scale_f32(amax, scale_ub, scale, recip);
  if (tid == 0) scales[row] = scale;
  uint8_t* dst = out + (int64_t)row * out_stride;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = tid + i * 256;
    if (idx < nvec) {
      const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
      float f[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        f[2 * j] = __uint_as_float(w[j] << 16);
        f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      }
      int lo = 0, hi = 0;
      lo = cvt_pk_e4m3fn(clamp448(f[0] * recip), clamp448(f[1] * recip), lo, false);
      lo = cvt_pk_e4m3fn(clamp448(f[2] * recip), clamp448(f[3] * recip), lo, true);
      hi = cvt_pk_e4m3fn(clamp448(f[4] * recip), clamp448(f[5] * recip), hi, false);
      hi = cvt_pk_e4m3fn(clamp448(f[6] * recip), clamp448(f[7] * recip), hi, true);
      reinterpret_cast<uint2*>(dst)[idx] = make_uint2((uint32_t)lo, (uint32_t)hi);
    }
  }
}

// ---------------------------------------------------------------------------
__device__ __forceinline__ float load_elem(const void* p, int dtype, int64_t i) {
  if (dtype == MAXFP8_BF16) return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
  if (dtype == MAXFP8_F16) return (float)reinterpret_cast<const _Float16*>(p)[i];
  return reinterpret_cast<const float*>(p)[i];
}

__device__ __forceinline__ uint8_t encode_one(float v) {
  return (uint8_t)(cvt_pk_e4m3fn(v, 0.0f, 0, false) & 0xff);
}

// 1 / scale as the dynamic quantisers use it: 0 for a zero scale or a reciprocal that overflows
__device__ __forceinline__ float guarded_recip(float scale) {
  float r = 0.0f;
  if (scale != 0.0f) {
    r = 1.0f / scale;
    if (isinf(r) || isnan(r)) r = 0.0f;
  }
  return r;
}

// One block per (row, group); any group size, dtype and alignment.
__global__ __launch_bounds__(256) void quant_generic_kernel(
    uint8_t* __restrict__ out, void* __restrict__ scales, const void* __restrict__ in,
    int ngroups, int G, int64_t in_stride, int64_t out_stride, int64_t scales_ld,
    int in_dtype, int scales_dtype, float scale_ub, BatchStep bs, RowGather rg) {
  in = reinterpret_cast<const uint8_t*>(in) + blockIdx.y * bs.in * (in_dtype == MAXFP8_F32 ? 4 : 2);
  out += blockIdx.y * bs.out;
  scales = reinterpret_cast<uint8_t*>(scales) + blockIdx.y * bs.scales * (scales_dtype == MAXFP8_F32 ? 4 : 2);
  __shared__ float red[4];
  const int row = blockIdx.x / ngroups, g = blockIdx.x - row * ngroups;
  const int tid = threadIdx.x;
  const int64_t base = (rg.index ? (int64_t)(rg.index[row] / rg.div) : (int64_t)row) * in_stride + (int64_t)g * G;
  float amax = 0.0f;
  for (int i = tid; i < G; i += 256) amax = fmaxf(amax, fabsf(load_elem(in, in_dtype, base + i)));
  amax = wave_max(amax);
  if ((tid & 63) == 0) red[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  float scale, recip;
  if (scales_dtype == MAXFP8_BF16) {
    // scale is formed in f32 from bf16-rounded operands and rounded to bf16 once more
    const float a = bf16_bits_to_f32(f32_to_bf16_bits(amax));
    const float ub = bf16_bits_to_f32(f32_to_bf16_bits(scale_ub));
    const uint32_t sb = f32_to_bf16_bits(fminf(a, ub) / 448.0f);
    scale = bf16_bits_to_f32(sb);
    float r = 0.0f;
    if (scale != 0.0f) {
      r = 1.0f / scale;
      if (isinf(r) || isnan(r)) r = 0.0f;
    }
    recip = r;
    if (tid == 0) reinterpret_cast<uint16_t*>(scales)[(int64_t)g * scales_ld + row] = (uint16_t)sb;
  } else {
    dynamic_scale_f32(amax, scale_ub, scale, recip);
    if (tid == 0) reinterpret_cast<float*>(scales)[(int64_t)g * scales_ld + row] = scale;
  }
  uint8_t* dst = out + (int64_t)row * out_stride + (int64_t)g * G;
  for (int i = tid; i < G; i += 256) dst[i] = encode_one(clamp448(load_elem(in, in_dtype, base + i) * recip));
}

// ---------------------------------------------------------------------------
// RMSNorm fused with per-row dynamic quantisation (max/kernels/src/nn/normalization.mojo:3996-4175):
//   inv_rms = rsqrt(sum x^2 / K + eps);  g' = gamma + weight_offset (f32)
//   row_max = max |x * g'| * inv_rms;  (scale, recip) from row_max
//   out = e4m3fn(clamp(((x * inv_rms) * g') * recip))
// One block (256 threads) per row; the row and gamma stay in registers between the two
// reductions and the convert pass: the activations are read once (2 bytes in, 1 byte out per
// element -- the unfused pair of kernels moves 2 + 2 + 2 + 1).
template <int NV, bool STREAM>
__global__ __launch_bounds__(256) void rmsnorm_quant_row_bf16_kernel(
    uint8_t* __restrict__ out, float* __restrict__ scales, const uint16_t* __restrict__ in,
    const uint16_t* __restrict__ gamma, int K, int64_t in_stride, int64_t out_stride, float epsilon,
    float weight_offset, float scale_ub) {
  __shared__ float red_s[4], red_m[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const uint16_t* src = in + (int64_t)row * in_stride;
  const int nvec = K >> 3;
  uint4 v[NV], g[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = tid + i * 256;
    v[i] = idx < nvec ? load_input<STREAM>(reinterpret_cast<const uint4*>(src) + idx) : make_uint4(0, 0, 0, 0);
    g[i] = idx < nvec ? reinterpret_cast<const uint4*>(gamma)[idx] : make_uint4(0, 0, 0, 0);
  }
  float ssq = 0.0f, amax = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
    const uint32_t gw[4] = {g[i].x, g[i].y, g[i].z, g[i].w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float x0 = __uint_as_float(w[j] << 16), x1 = __uint_as_float(w[j] & 0xffff0000u);
      const float g0 = __uint_as_float(gw[j] << 16) + weight_offset, g1 = __uint_as_float(gw[j] & 0xffff0000u) + weight_offset;
      ssq += x0 * x0;
      ssq += x1 * x1;
      amax = fmaxf(amax, fabsf(x0 * g0));
      amax = fmaxf(amax, fabsf(x1 * g1));
    }
  }
  ssq = wave_sum(ssq);
  amax = wave_max(amax);
  if ((tid & 63) == 0) { red_s[tid >> 6] = ssq; red_m[tid >> 6] = amax; }
  __syncthreads();
  ssq = (red_s[0] + red_s[1]) + (red_s[2] + red_s[3]);
  amax = fmaxf(fmaxf(red_m[0], red_m[1]), fmaxf(red_m[2], red_m[3]));
  const float inv_rms = 1.0f / __fsqrt_rn(ssq / (float)K + epsilon);
  float scale, recip;
  dynamic_scale_f32(amax * inv_rms, scale_ub, scale, recip);
  if (tid == 0) scales[row] = scale;
  uint8_t* dst = out + (int64_t)row * out_stride;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = tid + i * 256;
    if (idx < nvec) {
      const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
      const uint32_t gw[4] = {g[i].x, g[i].y, g[i].z, g[i].w};
      float f[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float g0 = __uint_as_float(gw[j] << 16) + weight_offset, g1 = __uint_as_float(gw[j] & 0xffff0000u) + weight_offset;
        f[2 * j] = ((__uint_as_float(w[j] << 16) * inv_rms) * g0) * recip;
        f[2 * j + 1] = ((__uint_as_float(w[j] & 0xffff0000u) * inv_rms) * g1) * recip;
      }
      int lo = 0, hi = 0;
      lo = cvt_pk_e4m3fn(clamp448(f[0]), clamp448(f[1]), lo, false);
      lo = cvt_pk_e4m3fn(clamp448(f[2]), clamp448(f[3]), lo, true);
      hi = cvt_pk_e4m3fn(clamp448(f[4]), clamp448(f[5]), hi, false);
      hi = cvt_pk_e4m3fn(clamp448(f[6]), clamp448(f[7]), hi, true);
      reinterpret_cast<uint2*>(dst)[idx] = make_uint2((uint32_t)lo, (uint32_t)hi);
    }
  }
}

// any dtype, alignment and row length: three passes over global memory
__global__ __launch_bounds__(256) void rmsnorm_quant_generic_kernel(
    uint8_t* __restrict__ out, void* __restrict__ scales, const void* __restrict__ in, const void* __restrict__ gamma,
    int K, int64_t in_stride, int64_t out_stride, int in_dtype, int scales_dtype, float epsilon, float weight_offset,
    float scale_ub) {
  __shared__ float red_s[4], red_m[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int64_t base = (int64_t)row * in_stride;
  float ssq = 0.0f, amax = 0.0f;
  for (int i = tid; i < K; i += 256) {
    const float x = load_elem(in, in_dtype, base + i);
    ssq += x * x;
    amax = fmaxf(amax, fabsf(x * (load_elem(gamma, in_dtype, i) + weight_offset)));
  }
  ssq = wave_sum(ssq);
  amax = wave_max(amax);
  if ((tid & 63) == 0) { red_s[tid >> 6] = ssq; red_m[tid >> 6] = amax; }
  __syncthreads();
  ssq = (red_s[0] + red_s[1]) + (red_s[2] + red_s[3]);
  amax = fmaxf(fmaxf(red_m[0], red_m[1]), fmaxf(red_m[2], red_m[3]));
  const float inv_rms = 1.0f / __fsqrt_rn(ssq / (float)K + epsilon);
  const float row_max = amax * inv_rms;
  float scale, recip;
  if (scales_dtype == MAXFP8_BF16) {
    const float a = bf16_bits_to_f32(f32_to_bf16_bits(row_max));
    const float ub = bf16_bits_to_f32(f32_to_bf16_bits(scale_ub));
    const uint32_t sb = f32_to_bf16_bits(fminf(a, ub) / 448.0f);
    scale = bf16_bits_to_f32(sb);
    float r = 0.0f;
    if (scale != 0.0f) {
      r = 1.0f / scale;
      if (isinf(r) || isnan(r)) r = 0.0f;
    }
    recip = r;
    if (tid == 0) reinterpret_cast<uint16_t*>(scales)[row] = (uint16_t)sb;
  } else {
    dynamic_scale_f32(row_max, scale_ub, scale, recip);
    if (tid == 0) reinterpret_cast<float*>(scales)[row] = scale;
  }
  uint8_t* dst = out + (int64_t)row * out_stride;
  for (int i = tid; i < K; i += 256) {
    const float gq = load_elem(gamma, in_dtype, i) + weight_offset;
    dst[i] = encode_one(clamp448(((load_elem(in, in_dtype, base + i) * inv_rms) * gq) * recip));
  }
}

// ---------------------------------------------------------------------------
// Static per-tensor quantisation: out = e4m3fn(clamp(f32(x) * (1 / scale)))
// (max/kernels/src/linalg/fp8_quantization.mojo:89-141; the op ignores scale_is_inverted and
// always multiplies by 1 / scale, builtin_kernels/quantization.mojo:1292-1310).
__global__ __launch_bounds__(256) void quant_static_bf16_kernel(uint8_t* __restrict__ out, const uint16_t* __restrict__ in,
                                                                int64_t rows, int kvec, int64_t in_stride,
                                                                int64_t out_stride, float recip, const void* scale_ptr,
                                                                int scales_dtype) {
  if (scale_ptr) recip = guarded_recip(load_elem(scale_ptr, scales_dtype, 0));
  const int64_t total = rows * kvec;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / kvec;
    const int c = (int)(i - r * kvec);
    const uint4 v = reinterpret_cast<const uint4*>(in + r * in_stride)[c];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float f[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = __uint_as_float(w[j] << 16) * recip;
      f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u) * recip;
    }
    int lo = 0, hi = 0;
    lo = cvt_pk_e4m3fn(clamp448(f[0]), clamp448(f[1]), lo, false);
    lo = cvt_pk_e4m3fn(clamp448(f[2]), clamp448(f[3]), lo, true);
    hi = cvt_pk_e4m3fn(clamp448(f[4]), clamp448(f[5]), hi, false);
    hi = cvt_pk_e4m3fn(clamp448(f[6]), clamp448(f[7]), hi, true);
    reinterpret_cast<uint2*>(out + r * out_stride)[c] = make_uint2((uint32_t)lo, (uint32_t)hi);
  }
}

__global__ __launch_bounds__(256) void quant_static_generic_kernel(uint8_t* __restrict__ out, const void* __restrict__ in,
                                                                   int64_t rows, int64_t K, int64_t in_stride,
                                                                   int64_t out_stride, int in_dtype, float recip,
                                                                   const void* scale_ptr, int scales_dtype) {
  if (scale_ptr) recip = guarded_recip(load_elem(scale_ptr, scales_dtype, 0));
  const int64_t total = rows * K;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / K, c = i - r * K;
    out[r * out_stride + c] = encode_one(clamp448(load_elem(in, in_dtype, r * in_stride + c) * recip));
  }
}

// ---------------------------------------------------------------------------
// Dynamic per-tensor quantisation (max/kernels/src/linalg/fp8_quantization.mojo:209-360, 596-775):
// one scale for the whole tensor, written to every scales[0, row].  Three launches, no scratch
// memory: row amax -> scales[row] (as the scales dtype, like the reference's first kernel), one
// block turns them into the tensor's scale in place, then the static-scale kernel quantises with
// the scale it reads from scales[0].  (The reference's second kernel reads and overwrites the
// per-row values in one launch, so what its later blocks see depends on block order; here every
// row gets the scale of the true tensor maximum.)
__global__ __launch_bounds__(256) void row_amax_kernel(void* __restrict__ scales, const void* __restrict__ in, int64_t K,
                                                       int64_t in_stride, int in_dtype, int scales_dtype, int vec_bf16) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x;
  float amax = 0.0f;
  if (vec_bf16) {
    const uint4* src = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(in) + row * in_stride);
    for (int64_t i = tid; i < (K >> 3); i += 256) {
      const uint4 v = src[i];
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        amax = fmaxf(amax, fabsf(__uint_as_float(w[j] << 16)));
        amax = fmaxf(amax, fabsf(__uint_as_float(w[j] & 0xffff0000u)));
      }
    }
  } else {
    for (int64_t i = tid; i < K; i += 256) amax = fmaxf(amax, fabsf(load_elem(in, in_dtype, row * in_stride + i)));
  }
  amax = wave_max(amax);
  if ((tid & 63) == 0) red[tid >> 6] = amax;
  __syncthreads();
  if (tid == 0) {
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    if (scales_dtype == MAXFP8_BF16) reinterpret_cast<uint16_t*>(scales)[row] = (uint16_t)f32_to_bf16_bits(amax);
    else reinterpret_cast<float*>(scales)[row] = amax;
  }
}

__global__ __launch_bounds__(1024) void tensor_scale_kernel(void* __restrict__ scales, int64_t rows, int scales_dtype,
                                                            float scale_ub) {
  __shared__ float red[16];
  const int tid = threadIdx.x;
  float amax = 0.0f;
  for (int64_t r = tid; r < rows; r += 1024) amax = fmaxf(amax, load_elem(scales, scales_dtype, r));
  amax = wave_max(amax);
  if ((tid & 63) == 0) red[tid >> 6] = amax;
  __syncthreads();
  amax = 0.0f;
#pragma unroll
  for (int w = 0; w < 16; ++w) amax = fmaxf(amax, red[w]);
  if (scales_dtype == MAXFP8_BF16) {
    const float ub = bf16_bits_to_f32(f32_to_bf16_bits(scale_ub));
    const uint16_t sb = (uint16_t)f32_to_bf16_bits(fminf(amax, ub) / 448.0f);
    for (int64_t r = tid; r < rows; r += 1024) reinterpret_cast<uint16_t*>(scales)[r] = sb;
  } else {
    const float scale = fminf(amax, scale_ub) / 448.0f;
    for (int64_t r = tid; r < rows; r += 1024) reinterpret_cast<float*>(scales)[r] = scale;
  }
}

// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void cast_f32_to_e4m3fn_kernel(uint8_t* out, const float* in, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < n; i += stride) out[i] = encode_one(clamp448(in[i]));
}

// pairs of f32 -> bf16 through pack_bf16x2, the convert the matmul epilogues use
__global__ __launch_bounds__(256) void cast_f32_to_bf16_kernel(uint16_t* out, const float* in, int64_t n) {
  int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 2;
  const int64_t stride = (int64_t)gridDim.x * 512;
  for (; i < n; i += stride) {
    const uint32_t w = pack_bf16x2(in[i], i + 1 < n ? in[i + 1] : 0.f);
    out[i] = (uint16_t)w;
    if (i + 1 < n) out[i + 1] = (uint16_t)(w >> 16);
  }
}

__global__ __launch_bounds__(256) void cast_e4m3fn_to_f32_kernel(float* out, const uint8_t* in, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < n; i += stride) {
    v2f f = __builtin_amdgcn_cvt_pk_f32_fp8((int)in[i], false);
    out[i] = f.x;
  }
}

__global__ __launch_bounds__(256) void copy_bytes_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, int64_t nvec) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < nvec; i += stride) dst[i] = src[i];
}

// ---------------------------------------------------------------------------
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int quantize_dispatch(void* out_fp8, void* out_scales, const void* in, int64_t M, int64_t K,
                      int64_t in_row_stride, int64_t out_row_stride, int64_t G, int64_t scales_ld,
                      int in_dtype, int scales_dtype, float scale_ub, int64_t batch, int64_t in_batch_stride,
                      int64_t out_batch_stride, int64_t scales_batch_stride, const uint32_t* row_index, uint32_t index_div,
                      hipStream_t stream) {
  const BatchStep bs = {in_batch_stride, out_batch_stride, scales_batch_stride};
  const RowGather rg = {row_index, index_div ? index_div : 1u};
  const unsigned nb = (unsigned)batch;
  const int64_t ngroups = K / G;
  const bool fast_types = in_dtype == MAXFP8_BF16 && scales_dtype == MAXFP8_F32;
  // (a row gather reads its source rows more than once -- the MoE layer each token's row top_k times, far apart in
  // time -- and wants them kept in the memory-side cache)
  const bool stream_in = M * K * 2 * batch >= kStreamInputBytes && row_index == nullptr;
  const bool vec_ok = aligned16(in) && (in_row_stride % 8 == 0) && (reinterpret_cast<uintptr_t>(out_fp8) % 8 == 0) &&
                      (out_row_stride % 8 == 0) && (in_batch_stride % 8 == 0) && (out_batch_stride % 8 == 0);
  if (fast_types && vec_ok && G == 128) {
    constexpr int U = 4;
    const int64_t nxb = ceil_div(ngroups, U);
    const int64_t blocks = ceil_div(M, 16) * nxb;
    if (blocks < (int64_t)1 << 31) {
      auto kern = stream_in ? quant_g128_bf16_kernel<U, true> : quant_g128_bf16_kernel<U, false>;
      hipLaunchKernelGGL(kern, dim3((unsigned)blocks, nb), dim3(256), 0, stream,
                         (uint8_t*)out_fp8, (float*)out_scales, (const uint16_t*)in, (int)M, (int)ngroups,
                         (int)nxb, in_row_stride, out_row_stride, scales_ld, scale_ub, bs, rg);
      return launch_status("quant_g128_bf16");
    }
  }
  if (fast_types && vec_ok && G == K && K % 8 == 0 && K <= 256 * 8 * 16 && M < ((int64_t)1 << 31)) {
    const int nvec = (int)(K / 8);
    const int nv = (nvec + 255) / 256;
    uint8_t* o = (uint8_t*)out_fp8;
    float* s = (float*)out_scales;
    const uint16_t* x = (const uint16_t*)in;
#define LAUNCH_ROW(NV)                                                                                          \
  hipLaunchKernelGGL((stream_in ? quant_row_bf16_kernel<NV, true> : quant_row_bf16_kernel<NV, false>), dim3((unsigned)M, nb), \
                     dim3(256), 0, stream, o, s, x, (int)K, in_row_stride, out_row_stride, scale_ub, bs, rg)
    if (nv <= 1) LAUNCH_ROW(1);
    else if (nv <= 2) LAUNCH_ROW(2);
    else if (nv <= 4) LAUNCH_ROW(4);
    else if (nv <= 8) LAUNCH_ROW(8);
    else LAUNCH_ROW(16);
#undef LAUNCH_ROW
    return launch_status("quant_row_bf16");
  }
  const int64_t blocks = M * ngroups;
  if (blocks >= (int64_t)1 << 31) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize: M * K/group_size = %lld exceeds the grid limit", (long long)blocks);
  hipLaunchKernelGGL(quant_generic_kernel, dim3((unsigned)blocks, nb), dim3(256), 0, stream, (uint8_t*)out_fp8,
                     out_scales, in, (int)ngroups, (int)G, in_row_stride, out_row_stride, scales_ld, in_dtype,
                     scales_dtype, scale_ub, bs, rg);
  return launch_status("quant_generic");
}

// bf16 in, f32 scales, groups of 128, 16-byte aligned rows: what the scatter form takes (-1: not this)
int quantize_scatter_dispatch(void* out_fp8, void* out_scales, const void* in, int64_t M, int64_t K, int64_t in_row_stride,
                              int64_t out_row_stride, int64_t scales_ld, float scale_ub, const uint32_t* dst_index,
                              int64_t copies, int64_t out_rows, hipStream_t stream) {
  const bool vec_ok = aligned16(in) && (in_row_stride % 8 == 0) && (reinterpret_cast<uintptr_t>(out_fp8) % 8 == 0) && (out_row_stride % 8 == 0);
  constexpr int U = 4;
  const int64_t ngroups = K / 128, nxb = ceil_div(ngroups, U), blocks = ceil_div(M, 16) * nxb;
  if (!vec_ok || K % 128 != 0 || blocks >= (int64_t)1 << 31 || copies > 0x7fffffff) return -1;
  hipLaunchKernelGGL(quant_g128_bf16_scatter_kernel<U>, dim3((unsigned)blocks), dim3(256), 0, stream, (uint8_t*)out_fp8,
                     (float*)out_scales, (const uint16_t*)in, (int)M, (int)ngroups, (int)nxb, in_row_stride, out_row_stride,
                     scales_ld, scale_ub, dst_index, (int)copies, out_rows);
  return launch_status("quant_g128_bf16_scatter");
}

int rmsnorm_quantize_dispatch(void* out_fp8, void* out_scales, const void* in, const void* gamma, int64_t rows, int64_t K,
                              int64_t in_row_stride, int64_t out_row_stride, int in_dtype, int scales_dtype, float epsilon,
                              float weight_offset, float scale_ub, hipStream_t stream) {
  const bool fast = in_dtype == MAXFP8_BF16 && scales_dtype == MAXFP8_F32 && aligned16(in) && aligned16(gamma) &&
                    (in_row_stride % 8 == 0) && (reinterpret_cast<uintptr_t>(out_fp8) % 8 == 0) && (out_row_stride % 8 == 0) &&
                    (K % 8 == 0) && K <= 256 * 8 * 16;
  if (fast) {
    const int64_t nv = ceil_div(K / 8, 256);
    uint8_t* o = (uint8_t*)out_fp8;
    float* s = (float*)out_scales;
    const bool stream_in = rows * K * 2 >= kStreamInputBytes;
#define LAUNCH_RMS(NV)                                                                                          \
  hipLaunchKernelGGL((stream_in ? rmsnorm_quant_row_bf16_kernel<NV, true> : rmsnorm_quant_row_bf16_kernel<NV, false>), \
                     dim3((unsigned)rows), dim3(256), 0, stream, o, s, (const uint16_t*)in, (const uint16_t*)gamma, (int)K, \
                     in_row_stride, out_row_stride, epsilon, weight_offset, scale_ub)
    if (nv <= 1) LAUNCH_RMS(1);
    else if (nv <= 2) LAUNCH_RMS(2);
    else if (nv <= 4) LAUNCH_RMS(4);
    else if (nv <= 8) LAUNCH_RMS(8);
    else LAUNCH_RMS(16);
#undef LAUNCH_RMS
    return launch_status("rmsnorm_quant_row_bf16");
  }
  hipLaunchKernelGGL(rmsnorm_quant_generic_kernel, dim3((unsigned)rows), dim3(256), 0, stream, (uint8_t*)out_fp8, out_scales,
                     in, gamma, (int)K, in_row_stride, out_row_stride, in_dtype, scales_dtype, epsilon, weight_offset, scale_ub);
  return launch_status("rmsnorm_quant_generic");
}

// scale_ptr == nullptr: quantise with the host value `scale`; otherwise with element 0 of scale_ptr
static int quantize_by_scale(void* out_fp8, const void* in, int64_t rows, int64_t K, int64_t in_row_stride,
                             int64_t out_row_stride, int in_dtype, float scale, const void* scale_ptr, int scales_dtype,
                             hipStream_t stream) {
  const float recip = 1.0f / scale;
  const bool fast = in_dtype == MAXFP8_BF16 && aligned16(in) && (in_row_stride % 8 == 0) && (K % 8 == 0) &&
                    (reinterpret_cast<uintptr_t>(out_fp8) % 8 == 0) && (out_row_stride % 8 == 0);
  const int64_t items = fast ? rows * (K / 8) : rows * K;
  const unsigned blocks = (unsigned)(ceil_div(items, 256) < 16384 ? ceil_div(items, 256) : 16384);
  if (fast)
    hipLaunchKernelGGL(quant_static_bf16_kernel, dim3(blocks), dim3(256), 0, stream, (uint8_t*)out_fp8, (const uint16_t*)in,
                       rows, (int)(K / 8), in_row_stride, out_row_stride, recip, scale_ptr, scales_dtype);
  else
    hipLaunchKernelGGL(quant_static_generic_kernel, dim3(blocks), dim3(256), 0, stream, (uint8_t*)out_fp8, in, rows, K,
                       in_row_stride, out_row_stride, in_dtype, recip, scale_ptr, scales_dtype);
  return launch_status("quantize_static");
}

int quantize_static_dispatch(void* out_fp8, const void* in, int64_t rows, int64_t K, int64_t in_row_stride,
                             int64_t out_row_stride, int in_dtype, float scale, hipStream_t stream) {
  return quantize_by_scale(out_fp8, in, rows, K, in_row_stride, out_row_stride, in_dtype, scale, nullptr, MAXFP8_F32, stream);
}

int quantize_tensor_dispatch(void* out_fp8, void* out_scales, const void* in, int64_t rows, int64_t K, int64_t in_row_stride,
                             int64_t out_row_stride, int in_dtype, int scales_dtype, float scale_ub, hipStream_t stream) {
  const int vec = in_dtype == MAXFP8_BF16 && aligned16(in) && (in_row_stride % 8 == 0) && (K % 8 == 0);
  hipLaunchKernelGGL(row_amax_kernel, dim3((unsigned)rows), dim3(256), 0, stream, out_scales, in, K, in_row_stride, in_dtype,
                     scales_dtype, vec);
  hipLaunchKernelGGL(tensor_scale_kernel, dim3(1), dim3(1024), 0, stream, out_scales, rows, scales_dtype, scale_ub);
  return quantize_by_scale(out_fp8, in, rows, K, in_row_stride, out_row_stride, in_dtype, 1.0f, out_scales, scales_dtype, stream);
}

int cast_f32_to_e4m3fn_dispatch(void* out, const float* in, int64_t n, hipStream_t stream) {
  const unsigned blocks = (unsigned)(ceil_div(n, 256) < 65536 ? ceil_div(n, 256) : 65536);
  hipLaunchKernelGGL(cast_f32_to_e4m3fn_kernel, dim3(blocks), dim3(256), 0, stream, (uint8_t*)out, in, n);
  return launch_status("cast_f32_to_e4m3fn");
}

int cast_f32_to_bf16_dispatch(void* out, const float* in, int64_t n, hipStream_t stream) {
  const int64_t pairs = ceil_div(n, 2);
  const unsigned blocks = (unsigned)(ceil_div(pairs, 256) < 65536 ? ceil_div(pairs, 256) : 65536);
  hipLaunchKernelGGL(cast_f32_to_bf16_kernel, dim3(blocks), dim3(256), 0, stream, (uint16_t*)out, in, n);
  return launch_status("cast_f32_to_bf16");
}

int cast_e4m3fn_to_f32_dispatch(float* out, const void* in, int64_t n, hipStream_t stream) {
  const unsigned blocks = (unsigned)(ceil_div(n, 256) < 65536 ? ceil_div(n, 256) : 65536);
  hipLaunchKernelGGL(cast_e4m3fn_to_f32_kernel, dim3(blocks), dim3(256), 0, stream, out, (const uint8_t*)in, n);
  return launch_status("cast_e4m3fn_to_f32");
}

int copy_bytes_dispatch(void* dst, const void* src, int64_t n, hipStream_t stream) {
  const int64_t nvec = n / 16;
  const unsigned blocks = (unsigned)(ceil_div(nvec, 256) < 16384 ? ceil_div(nvec, 256) : 16384);
  hipLaunchKernelGGL(copy_bytes_kernel, dim3(blocks), dim3(256), 0, stream, (uint4*)dst, (const uint4*)src, nvec);
  return launch_status("copy_bytes");
}

}  // namespace maxfp8
