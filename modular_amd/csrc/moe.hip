// The MoE steps on either side of the grouped FP8 matmul:
//
//   * moe_create_indices: groups the (token, expert) assignments by expert -- a stable bucket
//     sort of topk_ids (semantics: max/kernels/src/nn/moe.mojo:435-590).  The reference hands
//     out expert slots in the order in which its blocks reach an atomic lock, so its
//     expert_ids is some permutation of 0..E-1; here slot z is expert z and tokens keep their
//     order inside a slot, which is one of the reference's possible results and the same on
//     every run.  Three small launches (count, scan, scatter), no atomics, no scratch memory:
//     the counts travel in expert_start_indices.
//   * fused_silu / fused_silu_quantized: silu(gate) * up on the rows that row_offsets says
//     are in use, written as the input dtype or quantised to e4m3fn with one scale per
//     128 outputs, scales transposed (max/kernels/src/shmem/ep_comm.mojo:4409-4500, 4505-4624).
//     Note the quantiser of this op: scale = max(amax, 1e-4) / 448 and out / scale (a division),
//     not the min(amax, ub) / 448 and x * (1 / scale) of quantize_dynamic_scaled_fp8.
#include "common.h"

namespace maxfp8 {

// ---- moe_create_indices -----------------------------------------------------------------------
// block e counts the assignments to expert e; the count waits in expert_start_indices[e + 1].
// V ids per thread and iteration: a multiple of 4 (16-byte loads, topk_ids 16-byte aligned) or 1.  Every block reads all of topk_ids from
// L2, so what counts is loads in flight: one id per load and iteration took 49 us for 32768 ids, four per load with
// four loads in flight take a fifth of that.
template <int V>
__device__ __forceinline__ void moe_load_ids(const int32_t* __restrict__ topk_ids, int i, int n, int (&id)[V]) {
  if constexpr (V % 4 == 0) {
    if (i + V - 1 < n) {
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        const int4 v = *reinterpret_cast<const int4*>(topk_ids + i + 4 * q);
        id[4 * q] = v.x; id[4 * q + 1] = v.y; id[4 * q + 2] = v.z; id[4 * q + 3] = v.w;
      }
      return;
    }
  }
#pragma unroll
  for (int j = 0; j < V; ++j) id[j] = i + j < n ? topk_ids[i + j] : -1;  // (-1: no expert)
}
template <int V>
__global__ __launch_bounds__(256) void moe_count_kernel(uint32_t* __restrict__ expert_start_indices,
                                                        const int32_t* __restrict__ topk_ids, int n) {
  __shared__ int red[4];
  const int e = blockIdx.x, tid = threadIdx.x;
  int cnt = 0;
#pragma unroll 4
  for (int i = tid * V; i < n; i += 256 * V) {
    int id[V];
    moe_load_ids<V>(topk_ids, i, n, id);
#pragma unroll
    for (int j = 0; j < V; ++j) cnt += id[j] == e;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) cnt += __shfl_xor(cnt, o, 64);
  if ((tid & 63) == 0) red[tid >> 6] = cnt;
  __syncthreads();
  if (tid == 0) {
    expert_start_indices[e + 1] = (uint32_t)(red[0] + red[1] + red[2] + red[3]);
    if (e == 0) expert_start_indices[0] = 0;
  }
}
__global__ __launch_bounds__(1024) void moe_scan_kernel(uint32_t* __restrict__ expert_start_indices,
                                                        int32_t* __restrict__ expert_ids,
                                                        uint32_t* __restrict__ expert_usage_stats, int num_experts) {
  __shared__ uint32_t wave_sum[16], wave_max_s[16];
  __shared__ uint32_t carry;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) carry = 0;
  uint32_t mx = 0;
  __syncthreads();
  for (int base = 0; base < num_experts; base += 1024) {
    const int z = base + tid;
    const uint32_t c = z < num_experts ? expert_start_indices[z + 1] : 0u;
    mx = c > mx ? c : mx;
    uint32_t incl = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const uint32_t up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    uint32_t before = carry;
    for (int w = 0; w < wave; ++w) before += wave_sum[w];
    if (z < num_experts) {
      expert_start_indices[z + 1] = before + incl;
      expert_ids[z] = z;
    }
    __syncthreads();
    if (tid == 1023) carry = before + incl;
    __syncthreads();
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint32_t other = __shfl_xor(mx, o, 64);
    mx = other > mx ? other : mx;
  }
  if (lane == 0) wave_max_s[wave] = mx;
  __syncthreads();
  if (tid == 0) {
    uint32_t m = 0;
    for (int w = 0; w < 16; ++w) m = wave_max_s[w] > m ? wave_max_s[w] : m;
    expert_usage_stats[0] = m;                       // most tokens on one expert
    expert_usage_stats[1] = (uint32_t)num_experts;   // every expert keeps a slot (moe.mojo:584-588)
  }
}

// block e writes the positions of its assignments, in order, from expert_start_indices[e] on: 256 * V ids per
// iteration, thread t the V consecutive ids from 256 * V * iteration + V * t, a prefix sum of the threads' hit counts
// (shuffles inside a wave, LDS across the four waves; the two halves of wave_cnt take turns, so one barrier per iteration).
// An iteration costs 0.7 us whatever it holds -- the scan and the barrier, with one block of four waves per CU -- so V = 16 where
// the pointer allows: 32768 ids in 8 iterations (41 us with one id per thread and iteration, 23 with four, 12 with sixteen)
template <int V>
__global__ __launch_bounds__(256) void moe_scatter_kernel(uint32_t* __restrict__ token_expert_order,
                                                          uint32_t* __restrict__ restore_token_order,
                                                          const uint32_t* __restrict__ expert_start_indices,
                                                          const int32_t* __restrict__ topk_ids, int n) {
  __shared__ int wave_cnt[2][4];
  const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t base = expert_start_indices[e];
  if (expert_start_indices[e + 1] == base) return;
  int turn = 0;
  for (int i0 = 0; i0 < n; i0 += 256 * V, turn ^= 1) {
    const int i = i0 + tid * V;
    int id[V];
    moe_load_ids<V>(topk_ids, i, n, id);
    int c = 0;
#pragma unroll
    for (int j = 0; j < V; ++j) c += id[j] == e;
    int incl = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    if (lane == 63) wave_cnt[turn][wave] = incl;
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (w < wave) before += wave_cnt[turn][w];
      total += wave_cnt[turn][w];
    }
    uint32_t pos = base + (uint32_t)(before + incl - c);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      if (id[j] == e) {
        token_expert_order[pos] = (uint32_t)(i + j);
        restore_token_order[i + j] = pos;
        ++pos;
      }
    }
    base += (uint32_t)total;
  }
}

int moe_create_indices_dispatch(uint32_t* token_expert_order, uint32_t* expert_start_indices, uint32_t* restore_token_order,
                                int32_t* expert_ids, uint32_t* expert_usage_stats, const int32_t* topk_ids, int64_t n,
                                int64_t num_experts, hipStream_t stream) {
  const bool vec = (reinterpret_cast<uintptr_t>(topk_ids) & 15) == 0;
  if (vec) hipLaunchKernelGGL(moe_count_kernel<4>, dim3((unsigned)num_experts), dim3(256), 0, stream, expert_start_indices, topk_ids, (int)n);
  else hipLaunchKernelGGL(moe_count_kernel<1>, dim3((unsigned)num_experts), dim3(256), 0, stream, expert_start_indices, topk_ids, (int)n);
  hipLaunchKernelGGL(moe_scan_kernel, dim3(1), dim3(1024), 0, stream, expert_start_indices, expert_ids, expert_usage_stats,
                     (int)num_experts);
  if (n > 0) {
    if (vec)
      hipLaunchKernelGGL(moe_scatter_kernel<16>, dim3((unsigned)num_experts), dim3(256), 0, stream, token_expert_order,
                         restore_token_order, expert_start_indices, topk_ids, (int)n);
    else
      hipLaunchKernelGGL(moe_scatter_kernel<1>, dim3((unsigned)num_experts), dim3(256), 0, stream, token_expert_order,
                         restore_token_order, expert_start_indices, topk_ids, (int)n);
  }
  return launch_status("moe_create_indices");
}

// ---- fused SiLU(gate) * up --------------------------------------------------------------------
// a / b, correctly rounded (the IEEE quotient), at a third of the IEEE sequence's cost on the common path.  One Newton
// step turns the hardware's reciprocal (within an ulp) into the correctly rounded one -- unless b's mantissa is all ones --
// and with that, a quotient estimate, its exact residual and one correction give the correctly rounded quotient
// (Markstein's sequence) as long as no product underflows or overflows.  Everything outside those conditions takes the
// IEEE division, in a branch the wave skips unless one of its lanes needs it.  (Checked on the CPU against the IEEE
// quotient: the same operations and acceptance tests on 1.8e9 operand pairs -- random, bf16 numerators, divisors whose
// mantissa is (nearly) all ones, zeros and tiny numerators, quotients of the quantiser's size -- with the reciprocal
// off by -1, 0 and +1 ulp: no difference.)
__device__ __forceinline__ float refined_rcp(float b) {
  const float y0 = __builtin_amdgcn_rcpf(b);
  return fmaf(fmaf(-b, y0, 1.0f), y0, y0);
}
// a / b given y = refined_rcp(b); to be trusted where div_b_ok(b) and div_q_ok(a, result)
__device__ __forceinline__ float div_by(float a, float b, float y) {
  const float q0 = a * y;
  const float q = fmaf(fmaf(-b, q0, a), y, q0);
  return a == 0.0f ? q0 : q;  // (keeps the sign of a zero quotient)
}
__device__ __forceinline__ bool div_b_ok(float b) {
  return b >= 0x1p-63f && b < 0x1p64f && (__float_as_uint(b) & 0x007fffffu) != 0x007fffffu;
}
__device__ __forceinline__ bool div_q_ok(float a, float q) {
  return a == 0.0f || (fabsf(a) >= 0x1p-63f && fabsf(q) >= 0x1p-63f && fabsf(q) < 0x1p64f);
}
// Eight quotients a[j] / b[j] (SHARED: one divisor b[0] for all) with one test for the lane and one branch for the wave
template <bool SHARED>
__device__ __forceinline__ void exact_div8(const float (&a)[8], const float (&b)[8], float (&q)[8]) {
  bool ok = true;
  float y = 0.f;
  if constexpr (SHARED) {
    y = refined_rcp(b[0]);
    ok = div_b_ok(b[0]);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if constexpr (!SHARED) {
      y = refined_rcp(b[j]);
      ok = ok && div_b_ok(b[j]);
    }
    q[j] = div_by(a[j], b[SHARED ? 0 : j], y);
    ok = ok && div_q_ok(a[j], q[j]);
  }
  if (__builtin_amdgcn_ballot_w64(!ok) != 0ull) {
    if (!ok) {
#pragma unroll
      for (int j = 0; j < 8; ++j) q[j] = a[j] / b[SHARED ? 0 : j];
    }
  }
}

// gate / (1 + exp(-gate)) * up, every step rounded to f32 (ep_comm.mojo:4494-4497), for eight outputs.
// (1 + exp(-gate) = inf, gate < -88: outside the fast division's range, and gate / inf = -0 is what the IEEE division gives)
// ROUND_ACT: the activation is rounded to bf16 before the product, as where silu and the multiplication are two bf16
// operations (the dense gated MLP, max/python/max/nn/linear.py:1072: ops.silu(gate) * up).
template <bool ROUND_ACT>
__device__ __forceinline__ void silu_mul8(const float (&gate)[8], const float (&up)[8], float (&f)[8]) {
  float d[8], sig[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) d[j] = 1.0f + expf(-gate[j]);
  exact_div8<false>(gate, d, sig);
  if constexpr (ROUND_ACT) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w = pack_bf16x2(sig[2 * j], sig[2 * j + 1]);
      sig[2 * j] = __uint_as_float(w << 16);
      sig[2 * j + 1] = __uint_as_float(w & 0xffff0000u);
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) f[j] = sig[j] * up[j];
}

// 16 lanes own 128 consecutive outputs of one row (8 each): one 16-byte load of gate and of up
// per lane; QUANT: amax over the 16 lanes by DPP, 8-byte packed fp8 store, lane 0 writes the scale.
template <bool QUANT, bool ROUND_ACT = false>
__global__ __launch_bounds__(256) void fused_silu_bf16_kernel(void* __restrict__ out, float* __restrict__ scales,
                                                              const uint16_t* __restrict__ in,
                                                              const uint32_t* __restrict__ row_offsets, int num_offsets,
                                                              int64_t max_rows, int inter, int64_t in_stride,
                                                              int64_t out_stride, int64_t scales_ld) {
  // (the buffers hold max_rows rows: an offset beyond that -- a stale or damaged routing tensor -- must not
  // turn into accesses outside them)
  const uint32_t rows_dev = row_offsets[num_offsets - 1];
  const int64_t rows = (int64_t)rows_dev < max_rows ? (int64_t)rows_dev : max_rows;
  const int groups = inter >> 7;
  const int tid = threadIdx.x, sub = tid & 15;
  const int64_t total = rows * groups;
  for (int64_t item = (int64_t)blockIdx.x * 16 + (tid >> 4); item < total; item += (int64_t)gridDim.x * 16) {
    const int64_t m = item / groups;
    const int g = (int)(item - m * groups);
    const uint16_t* src = in + m * in_stride + g * 128 + sub * 8;
    const uint4 gv = *reinterpret_cast<const uint4*>(src);
    const uint4 uv = *reinterpret_cast<const uint4*>(src + inter);
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
    float gate[8], up[8], f[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      gate[2 * j] = __uint_as_float(gw[j] << 16);
      gate[2 * j + 1] = __uint_as_float(gw[j] & 0xffff0000u);
      up[2 * j] = __uint_as_float(uw[j] << 16);
      up[2 * j + 1] = __uint_as_float(uw[j] & 0xffff0000u);
    }
    silu_mul8<ROUND_ACT>(gate, up, f);
    if constexpr (!QUANT) {
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = pack_bf16x2(f[2 * j], f[2 * j + 1]);
      *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(out) + m * out_stride + g * 128 + sub * 8) =
          make_uint4(w[0], w[1], w[2], w[3]);
    } else {
      float amax = 0.0f;
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(f[j]));
      amax = row16_max(amax);
      const float scale = fmaxf(amax, 1e-4f) / 448.0f;
      const float divisor[8] = {scale, scale, scale, scale, scale, scale, scale, scale};
      float q[8];
      exact_div8<true>(f, divisor, q);   // (one reciprocal and one test of the divisor for the lane's eight quotients)
#pragma unroll
      for (int j = 0; j < 8; ++j) q[j] = clamp448(q[j]);
      int lo = 0, hi = 0;
      lo = cvt_pk_e4m3fn(q[0], q[1], lo, false);
      lo = cvt_pk_e4m3fn(q[2], q[3], lo, true);
      hi = cvt_pk_e4m3fn(q[4], q[5], hi, false);
      hi = cvt_pk_e4m3fn(q[6], q[7], hi, true);
      *reinterpret_cast<uint2*>(reinterpret_cast<uint8_t*>(out) + m * out_stride + g * 128 + sub * 8) =
          make_uint2((uint32_t)lo, (uint32_t)hi);
      if (sub == 0) scales[(int64_t)g * scales_ld + m] = scale;
    }
  }
}

int fused_silu_dispatch(void* out, float* scales, const void* in, const uint32_t* row_offsets, int64_t num_offsets,
                        int64_t max_rows, int64_t inter, int64_t in_stride, int64_t out_stride, int64_t scales_ld,
                        int mode, hipStream_t stream) {
  const bool quant = mode == 1;
  // the number of rows in use is only known on the device: the grid is sized for max_rows and
  // walks the items in strides
  const int64_t items = max_rows * (inter / 128);
  const unsigned blocks = (unsigned)(ceil_div(items, 16) < 8192 ? ceil_div(items, 16) : 8192);
  if (quant)
    hipLaunchKernelGGL(fused_silu_bf16_kernel<true>, dim3(blocks), dim3(256), 0, stream, out, scales, (const uint16_t*)in,
                       row_offsets, (int)num_offsets, max_rows, (int)inter, in_stride, out_stride, scales_ld);
  else if (mode == 2)
    hipLaunchKernelGGL((fused_silu_bf16_kernel<false, true>), dim3(blocks), dim3(256), 0, stream, out, scales, (const uint16_t*)in,
                       row_offsets, (int)num_offsets, max_rows, (int)inter, in_stride, out_stride, scales_ld);
  else
    hipLaunchKernelGGL(fused_silu_bf16_kernel<false>, dim3(blocks), dim3(256), 0, stream, out, scales, (const uint16_t*)in,
                       row_offsets, (int)num_offsets, max_rows, (int)inter, in_stride, out_stride, scales_ld);
  return launch_status(quant ? "fused_silu_quantized" : "fused_silu");
}

}  // namespace maxfp8
