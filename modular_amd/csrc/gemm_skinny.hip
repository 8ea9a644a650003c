// Weight-streaming scaled FP8 matmul for small M (decode): C[M,N] = A[M,K] . B[N,K]^T,
// M <= 16 * MT.
//
// The bytes that matter are the N*K weight bytes, read exactly once.  A block owns
// 16*NTW consecutive weight rows; its 4 waves take the 128-byte K slabs round-robin
// (so the block reads 512 contiguous bytes of every row per step).  A lane loads 32
// bytes of one weight row per slab straight into the MFMA row-operand registers
// (no LDS staging: nothing is reused), the activations are the MFMA column operand
// (tokens >= M read as zero through the buffer descriptor), and
// v_mfma_f32_16x16x128_f8f6f4 does the dot products: 16 weight rows x 16 token
// columns per instruction, so no M-padding to a 128-row tile.  Partial sums of the
// 4 waves meet in LDS; wave-ordered summation keeps the result deterministic.
//
// Scaling follows gemm_tiled.hip: block mode promotes every slab with
// a_s[slab, m] * b_s[n/128, slab]; row/tensor mode scales once at the end
// (max/kernels/src/linalg/fp8_quantization.mojo:1218-1240, 1576-1624).
#include "common.h"
#include "gemm_args.h"

namespace maxfp8 {

__device__ __forceinline__ __amdgpu_buffer_rsrc_t sk_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
__device__ __forceinline__ v4i sk_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff) {
  return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
}
__device__ __forceinline__ uint32_t sk_clamp_u32(int64_t v) {
  return v > 0xfffffff0ll ? 0xfffffff0u : (v < 0 ? 0u : (uint32_t)v);
}

template <int NTW, int MT, bool BLOCKSCALE>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(GemmArgs p) {
  constexpr int WAVES = 4;
  __shared__ float red[WAVES][MT * NTW * 4][64];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lm = lane & 15, lq = lane >> 4;
  const int n0 = blockIdx.x * (16 * NTW);
  const int cols_here = (p.N - n0) < 16 * NTW ? (p.N - n0) : 16 * NTW;

  const uint8_t* b_tile = p.b + (int64_t)n0 * p.ldb;
  const __amdgpu_buffer_rsrc_t b_rsrc = sk_rsrc(b_tile, sk_clamp_u32((int64_t)(cols_here - 1) * p.ldb + p.K));
  const __amdgpu_buffer_rsrc_t a_rsrc = sk_rsrc(p.a, sk_clamp_u32((int64_t)(p.M - 1) * p.lda + p.K));

  // lane's two 16-byte chunks of a slab: bytes [16*lq, +16) and [64 + 16*lq, +16)
  uint32_t b_off[NTW], a_off[MT];
#pragma unroll
  for (int t = 0; t < NTW; ++t) b_off[t] = (uint32_t)(t * 16 + lm) * (uint32_t)p.ldb + lq * 16;
#pragma unroll
  for (int t = 0; t < MT; ++t) a_off[t] = (uint32_t)(t * 16 + lm) * (uint32_t)p.lda + lq * 16;

  const int nslab = (p.K + 127) / 128;
  const bool k_tail = (p.K & 127) != 0;

  v4f acc[MT][NTW];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NTW; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  int as_m[MT];
  const float* bs_row = nullptr;
  if constexpr (BLOCKSCALE) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = t * 16 + lm;
      as_m[t] = m < p.M ? m : p.M - 1;
    }
    bs_row = p.b_scales + (int64_t)(n0 / 128) * p.b_scales_ld;
  }

  v8i wf[NTW], af[MT];
  float sc[MT];
  auto load_slab = [&](int slab) {
    const uint32_t koff = (uint32_t)slab * 128u;
    uint32_t kill0 = 0, kill1 = 0;
    if (k_tail) {
      if (koff + lq * 16 >= (uint32_t)p.K) kill0 = 0x80000000u;
      if (koff + 64 + lq * 16 >= (uint32_t)p.K) kill1 = 0x80000000u;
    }
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      const v4i lo = sk_load16(b_rsrc, (b_off[t] + koff) | kill0);
      const v4i hi = sk_load16(b_rsrc, (b_off[t] + koff + 64) | kill1);
      wf[t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const v4i lo = sk_load16(a_rsrc, (a_off[t] + koff) | kill0);
      const v4i hi = sk_load16(a_rsrc, (a_off[t] + koff + 64) | kill1);
      af[t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
    if constexpr (BLOCKSCALE) {
      const float bs = bs_row[slab];
#pragma unroll
      for (int t = 0; t < MT; ++t) sc[t] = p.a_scales[(int64_t)slab * p.a_scales_ld + as_m[t]] * bs;
    }
  };

  // The compiler software-pipelines this loop (the loads of the next slab do not
  // depend on the MFMAs of this one); UNROLL slabs are in flight per wave.
  constexpr int UNROLL = (NTW * 2 + MT * 2) <= 8 ? 4 : 2;
#pragma unroll UNROLL
  for (int slab = wave; slab < nslab; slab += WAVES) {
    load_slab(slab);
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if constexpr (BLOCKSCALE) {
          const v4f zero = {0.f, 0.f, 0.f, 0.f};
          const v4f part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[nt], af[mt], zero, 0, 0, 0, 0, 0, 0);
          acc[mt][nt] += part * sc[mt];
        } else {
          acc[mt][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[nt], af[mt], acc[mt][nt], 0, 0, 0, 0, 0, 0);
        }
      }
    }
  }

  // ---- reduce the 4 waves' partial sums (fixed order) and store ----------------------
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[wave][(mt * NTW + nt) * 4 + v][lane] = acc[mt][nt][v];
  __syncthreads();

  // (mt, nt) pairs are dealt to the waves round-robin
  for (int pair = wave; pair < MT * NTW; pair += WAVES) {
    const int mt = pair / NTW, nt = pair - mt * NTW;
    const int m = mt * 16 + lm;
    const int n = n0 + nt * 16 + lq * 4;
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = pair * 4 + i;
      v[i] = ((red[0][r][lane] + red[1][r][lane]) + red[2][r][lane]) + red[3][r][lane];
    }
    if (m >= p.M || n >= p.N) continue;
    if constexpr (!BLOCKSCALE) {
      const float a_s = p.a_scales[(int64_t)m * p.a_scale_stride];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int nn = (n + i < p.N) ? n + i : p.N - 1;
        const float t = v[i] * a_s;
        v[i] = t * p.b_scales[(int64_t)nn * p.b_scale_stride];
      }
    }
    if (p.c_dtype == MAXFP8_BF16) {
      uint16_t* dst = reinterpret_cast<uint16_t*>(p.c) + (int64_t)m * p.ldc + n;
      if (p.c_vec_ok && n + 3 < p.N) {
        const uint32_t lo = f32_to_bf16_bits(v[0]) | (f32_to_bf16_bits(v[1]) << 16);
        const uint32_t hi = f32_to_bf16_bits(v[2]) | (f32_to_bf16_bits(v[3]) << 16);
        *reinterpret_cast<uint2*>(dst) = make_uint2(lo, hi);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < p.N) dst[i] = (uint16_t)f32_to_bf16_bits(v[i]);
      }
    } else {
      float* dst = reinterpret_cast<float*>(p.c) + (int64_t)m * p.ldc + n;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < p.N) dst[i] = v[i];
    }
  }
}

template <int NTW, int MT, bool BLOCKSCALE>
static int launch_skinny(const GemmArgs& p, hipStream_t stream) {
  const int64_t blocks = ceil_div(p.N, 16 * NTW);
  hipLaunchKernelGGL((gemm_skinny_kernel<NTW, MT, BLOCKSCALE>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
  return launch_status("gemm_skinny");
}

template <int MT, bool BLOCKSCALE>
static int pick_ntw(const GemmArgs& p, hipStream_t stream) {
  // enough blocks to keep 256 CUs streaming: prefer >= 4 blocks per CU
  const int64_t n16 = ceil_div(p.N, 16);
  if (MT <= 2 && n16 >= 4 * 1024 * 4 / 4) return launch_skinny<4, MT, BLOCKSCALE>(p, stream);
  if (n16 >= 2 * 1024) return launch_skinny<2, MT, BLOCKSCALE>(p, stream);
  return launch_skinny<1, MT, BLOCKSCALE>(p, stream);
}

int gemm_skinny_max_m() { return 64; }

int gemm_skinny_dispatch(const GemmArgs& p, bool blockscale, hipStream_t stream) {
  if (p.M > 64) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "skinny matmul: M = %d exceeds 64", p.M);
  const int mt = (p.M + 15) / 16;
  if (blockscale) {
    if (mt <= 1) return pick_ntw<1, true>(p, stream);
    if (mt <= 2) return pick_ntw<2, true>(p, stream);
    return pick_ntw<4, true>(p, stream);
  }
  if (mt <= 1) return pick_ntw<1, false>(p, stream);
  if (mt <= 2) return pick_ntw<2, false>(p, stream);
  return pick_ntw<4, false>(p, stream);
}

}  // namespace maxfp8
