// LDS-staged MFMA GEMM for scaled FP8 on gfx950:  C[M,N] = A[M,K] . B[N,K]^T.
//
// One block owns a BM x BN tile of C and walks K in slabs of 128 bytes (one scale
// group).  Per slab the block copies BM + BN rows of 128 fp8 bytes into LDS
// (16-byte chunks, chunk index XOR-swizzled with (row >> 1) & 7 so that the
// 16-lane MFMA fragment reads hit 64 distinct banks), and every wave issues
// v_mfma_f32_16x16x128_f8f6f4 on its (BM/WAVES_M) x (BN/WAVES_N) sub-tile.
//
// The weight fragment is the MFMA's row operand and the activation fragment its
// column operand, so a lane ends up with 4 consecutive n for ONE m: the
// per-token scale is a single register per 16-row group and the bf16 results
// leave as 8-byte stores.
//
// Block scaling (1x128 activation groups, 128x128 weight blocks): each slab's
// product is formed in a fresh accumulator P (MFMA with C = 0) and promoted with
// acc += P * (a_s[slab, m] * b_s[n/128, slab]) -- the per-slab promotion of
// max/kernels/src/linalg/matmul/gpu/sm100/blockwise_fp8.mojo:376-392, which sums
// the same terms as the reference's naive kernel
// (max/kernels/src/linalg/fp8_quantization.mojo:1576-1624) in a different order.
// Row/tensor scaling: acc accumulates over all of K inside the MFMA and is scaled
// once, (acc * a_s[m]) * b_s[n]  (fp8_quantization.mojo:1218-1240).
//
// Grouped (MoE) mode maps blocks to (expert slot, m-tile, n-tile) from the
// device-resident offsets, so no host synchronisation is needed
// (semantics: fp8_quantization.mojo:1745-1865).
#include "common.h"
#include "gemm_args.h"

namespace maxfp8 {

// raw buffer descriptor: out-of-range offsets read as zero, which handles the
// M and N edges of partial tiles.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

__device__ __forceinline__ v4i buffer_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff) {
  return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
}

__device__ __forceinline__ uint32_t clamp_u32(int64_t v) {
  return v > 0xfffffff0ll ? 0xfffffff0u : (v < 0 ? 0u : (uint32_t)v);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool BLOCKSCALE, bool GROUPED>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, (BM * BN <= 128 * 128) ? 2 : 1) void gemm_tiled_kernel(GemmArgs p) {
  constexpr int NTHREADS = WAVES_M * WAVES_N * 64;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int CA = BM * 8 / NTHREADS, CB = BN * 8 / NTHREADS;
  constexpr int STAGE_BYTES = (BM + BN) * 128;
  static_assert(CA >= 1 && CB >= 1, "tile too small for the block");
  static_assert(!BLOCKSCALE || (WN <= 128 && 128 % WN == 0), "a wave's columns must sit inside one 128-wide scale block");

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // ---- block -> tile --------------------------------------------------------
  int64_t row_begin, row_end;  // rows of A/C this block may touch: [row_begin, row_end)
  int n0;
  const uint8_t* bptr = p.b;
  const float* bs_ptr = p.b_scales;
  bool zero_fill = false;
  if constexpr (GROUPED) {
    // blockIdx.y walks the m-tiles of all active slots in slot order: a block-wide
    // prefix sum over the slots' tile counts locates (slot, tile) without the host.
    __shared__ int s_slot, s_tile, s_wave_sum[NTHREADS / 64], s_carry;
    if (tid == 0) { s_slot = -1; s_tile = 0; s_carry = 0; }
    __syncthreads();
    for (int z0 = 0; z0 < p.num_active; z0 += NTHREADS) {
      const int z = z0 + tid;
      int t = 0;
      if (z < p.num_active) t = ((int)(p.offsets[z + 1] - p.offsets[z]) + BM - 1) / BM;
      int incl = t;  // inclusive scan inside the wave
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
      }
      if (lane == 63) s_wave_sum[wave] = incl;
      __syncthreads();
      int before = s_carry;
      for (int w = 0; w < wave; ++w) before += s_wave_sum[w];
      const int excl = before + incl - t;
      if (t > 0 && (int)blockIdx.y >= excl && (int)blockIdx.y < excl + t) { s_slot = z; s_tile = blockIdx.y - excl; }
      __syncthreads();
      if (tid == NTHREADS - 1) s_carry = before + incl;
      __syncthreads();
      if (s_slot >= 0 || (int)blockIdx.y < s_carry) break;
    }
    const int slot = s_slot;
    if (slot < 0) return;
    row_begin = (int64_t)p.offsets[slot] + (int64_t)s_tile * BM;
    row_end = p.offsets[slot + 1];
    n0 = blockIdx.x * BN;
    const int e = p.expert_ids[slot];
    if (e < 0) zero_fill = true;
    else {
      bptr += (int64_t)e * p.b_expert_stride;
      bs_ptr += (int64_t)e * p.bs_expert_stride;
    }
  } else {
    // 1-D grid.  Consecutive block ids land on different XCDs (8 of them, each
    // with its own L2), so give each XCD a contiguous run of tiles, and walk the
    // tiles in column-major groups of GROUP_M rows for L2 reuse of A and B.
    const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
    const int total = tiles_m * tiles_n;
    int pid = blockIdx.x;
    {
      const int xcd = pid & 7, local = pid >> 3;
      const int base = total >> 3, rem = total & 7;
      pid = xcd * base + (xcd < rem ? xcd : rem) + local;
    }
    constexpr int GROUP_M = 8;
    const int per_group = GROUP_M * tiles_n;
    const int group = pid / per_group;
    const int first_m = group * GROUP_M;
    const int gsize = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
    const int in_group = pid - group * per_group;
    const int tm = first_m + in_group % gsize;
    const int tn = in_group / gsize;
    row_begin = (int64_t)tm * BM;
    row_end = p.M;
    n0 = tn * BN;
  }
  const int rows_here = (int)((row_end - row_begin) < BM ? (row_end - row_begin) : BM);
  const int cols_here = (p.N - n0) < BN ? (p.N - n0) : BN;

  // ---- epilogue helpers --------------------------------------------------------
  const int lm = lane & 15, lq = lane >> 4;
  auto store4 = [&](int64_t m, int n, float v0, float v1, float v2, float v3) {
    // caller guarantees m is valid; n..n+3 may cross N
    if (p.c_dtype == MAXFP8_BF16) {
      uint16_t* dst = reinterpret_cast<uint16_t*>(p.c) + m * p.ldc + n;
      if (p.c_vec_ok && n + 3 < p.N) {
        const uint32_t lo = f32_to_bf16_bits(v0) | (f32_to_bf16_bits(v1) << 16);
        const uint32_t hi = f32_to_bf16_bits(v2) | (f32_to_bf16_bits(v3) << 16);
        *reinterpret_cast<uint2*>(dst) = make_uint2(lo, hi);
      } else {
        const float v[4] = {v0, v1, v2, v3};
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < p.N) dst[i] = (uint16_t)f32_to_bf16_bits(v[i]);
      }
    } else {
      float* dst = reinterpret_cast<float*>(p.c) + m * p.ldc + n;
      if (p.c_vec_ok && n + 3 < p.N) {
        *reinterpret_cast<float4*>(dst) = make_float4(v0, v1, v2, v3);
      } else {
        const float v[4] = {v0, v1, v2, v3};
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < p.N) dst[i] = v[i];
      }
    }
  };

  if (GROUPED && zero_fill) {
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      const int ml = wm * WM + mt * 16 + lm;
      if (ml >= rows_here) continue;
#pragma unroll
      for (int nt = 0; nt < TN; ++nt) {
        const int n = n0 + wn * WN + nt * 16 + lq * 4;
        if (n < p.N) store4(row_begin + ml, n, 0.f, 0.f, 0.f, 0.f);
      }
    }
    return;
  }

  // ---- global -> LDS copy plan ---------------------------------------------------
  // chunk q = tid + i*NTHREADS: row q>>3 of the tile, 16-byte chunk q&7 of the slab.
  const uint8_t* a_tile = p.a + row_begin * p.lda;
  const uint8_t* b_tile = bptr + (int64_t)n0 * p.ldb;
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a_tile, clamp_u32((int64_t)(rows_here - 1) * p.lda + p.K));
  const __amdgpu_buffer_rsrc_t b_rsrc = make_rsrc(b_tile, clamp_u32((int64_t)(cols_here - 1) * p.ldb + p.K));
  const int crow = tid >> 3, cchunk = tid & 7;
  constexpr int ROWS_PER_PASS = NTHREADS / 8;
  const uint32_t a_voff = (uint32_t)crow * (uint32_t)p.lda + cchunk * 16;
  const uint32_t b_voff = (uint32_t)crow * (uint32_t)p.ldb + cchunk * 16;
  const uint32_t a_step = (uint32_t)ROWS_PER_PASS * (uint32_t)p.lda;
  const uint32_t b_step = (uint32_t)ROWS_PER_PASS * (uint32_t)p.ldb;
  // ROWS_PER_PASS is a multiple of 16, so the swizzle term does not depend on i
  const uint32_t lds_wr = crow * 128 + ((cchunk ^ ((crow >> 1) & 7)) << 4);
  const bool k_tail = (p.K & 127) != 0;

  v4i ra[CA], rb[CB];
  auto gload = [&](int slab) {
    uint32_t koff = (uint32_t)slab * 128u;
    uint32_t kill = 0;
    if (k_tail && koff + cchunk * 16 >= (uint32_t)p.K) kill = 0x80000000u;  // past K: force out of range
#pragma unroll
    for (int i = 0; i < CA; ++i) ra[i] = buffer_load16(a_rsrc, (a_voff + i * a_step + koff) | kill);
#pragma unroll
    for (int i = 0; i < CB; ++i) rb[i] = buffer_load16(b_rsrc, (b_voff + i * b_step + koff) | kill);
  };
  auto sstore = [&](int buf) {
    uint8_t* sa = smem + buf * STAGE_BYTES;
    uint8_t* sb = sa + BM * 128;
#pragma unroll
    for (int i = 0; i < CA; ++i) *reinterpret_cast<v4i*>(sa + lds_wr + i * ROWS_PER_PASS * 128) = ra[i];
#pragma unroll
    for (int i = 0; i < CB; ++i) *reinterpret_cast<v4i*>(sb + lds_wr + i * ROWS_PER_PASS * 128) = rb[i];
  };

  // ---- fragment read plan ----------------------------------------------------------
  // lane (lm, lq) reads row lm of a 16-row group, logical chunks 2*lq and 2*lq+1.
  const int sw = (lm >> 1) & 7;
  const uint32_t frag0 = lm * 128 + (((2 * lq) ^ sw) << 4);
  const uint32_t frag1 = lm * 128 + (((2 * lq + 1) ^ sw) << 4);
  const uint32_t a_frag_base = (uint32_t)(wm * WM) * 128;
  const uint32_t b_frag_base = (uint32_t)(BM + wn * WN) * 128;

  v4f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  const int nslab = (p.K + 127) / 128;

  // per-slab scales: a_s for this lane's TM rows, b_s for the wave's 128-block
  float as_cur[TM], as_nxt[TM];
  float bs_cur = 1.f, bs_nxt = 1.f;
  int64_t as_col[TM];
  const float* bs_row = nullptr;
  if constexpr (BLOCKSCALE) {
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      int ml = wm * WM + mt * 16 + lm;
      if (ml >= rows_here) ml = rows_here - 1;  // stay inside the scale matrix
      as_col[mt] = row_begin + ml;
    }
    bs_row = bs_ptr + (int64_t)((n0 + wn * WN) / 128) * p.b_scales_ld;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) as_nxt[mt] = p.a_scales[as_col[mt]];
    bs_nxt = bs_row[0];
  }

  gload(0);
  sstore(0);
  __syncthreads();

  for (int slab = 0; slab < nslab; ++slab) {
    const int buf = slab & 1;
    const bool more = slab + 1 < nslab;
    if (more) gload(slab + 1);
    if constexpr (BLOCKSCALE) {
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) as_cur[mt] = as_nxt[mt] * bs_nxt;
      bs_cur = bs_nxt;
      (void)bs_cur;
      if (more) {
#pragma unroll
        for (int mt = 0; mt < TM; ++mt) as_nxt[mt] = p.a_scales[(int64_t)(slab + 1) * p.a_scales_ld + as_col[mt]];
        bs_nxt = bs_row[slab + 1];
      }
    }

    const uint8_t* sa = smem + buf * STAGE_BYTES;
    v8i af[TM], bf[TN];
#pragma unroll
    for (int t = 0; t < TM; ++t) {
      const v4i lo = *reinterpret_cast<const v4i*>(sa + a_frag_base + t * 2048 + frag0);
      const v4i hi = *reinterpret_cast<const v4i*>(sa + a_frag_base + t * 2048 + frag1);
      af[t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
#pragma unroll
    for (int t = 0; t < TN; ++t) {
      const v4i lo = *reinterpret_cast<const v4i*>(sa + b_frag_base + t * 2048 + frag0);
      const v4i hi = *reinterpret_cast<const v4i*>(sa + b_frag_base + t * 2048 + frag1);
      bf[t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
        if constexpr (BLOCKSCALE) {
          const v4f zero = {0.f, 0.f, 0.f, 0.f};
          const v4f part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[nt], af[mt], zero, 0, 0, 0, 0, 0, 0);
          acc[mt][nt] += part * as_cur[mt];
        } else {
          acc[mt][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[nt], af[mt], acc[mt][nt], 0, 0, 0, 0, 0, 0);
        }
      }
    }
    if (more) sstore(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue ------------------------------------------------------------------
#pragma unroll
  for (int mt = 0; mt < TM; ++mt) {
    const int ml = wm * WM + mt * 16 + lm;
    if (ml >= rows_here) continue;
    const int64_t m = row_begin + ml;
    float a_s = 1.f;
    if constexpr (!BLOCKSCALE) a_s = p.a_scales[m * p.a_scale_stride];
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
      const int n = n0 + wn * WN + nt * 16 + lq * 4;
      if (n >= p.N) continue;
      v4f v = acc[mt][nt];
      if constexpr (!BLOCKSCALE) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int nn = (n + i < p.N) ? n + i : p.N - 1;
          const float t = v[i] * a_s;
          v[i] = t * p.b_scales[(int64_t)nn * p.b_scale_stride];
        }
      }
      store4(m, n, v[0], v[1], v[2], v[3]);
    }
  }
}

// ---------------------------------------------------------------------------------
template <int BM, int BN, int WAVES_M, int WAVES_N, bool BLOCKSCALE, bool GROUPED>
static int launch_tiled(const GemmArgs& p, dim3 grid, hipStream_t stream, const char* name) {
  constexpr int smem = 2 * (BM + BN) * 128;
  auto kern = gemm_tiled_kernel<BM, BN, WAVES_M, WAVES_N, BLOCKSCALE, GROUPED>;
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", name, smem, hipGetErrorString(e));
    attr_done = true;
  }
  hipLaunchKernelGGL(kern, grid, dim3(WAVES_M * WAVES_N * 64), smem, stream, p);
  return launch_status(name);
}

int gemm_tiled_dispatch(const GemmArgs& p, bool blockscale, hipStream_t stream) {
  const int64_t tiles = ceil_div(p.M, 128) * ceil_div(p.N, 128);
  if (tiles >= ((int64_t)1 << 31)) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "tiled matmul: too many tiles");
  const dim3 grid((unsigned)tiles);
  if (blockscale) return launch_tiled<128, 128, 2, 2, true, false>(p, grid, stream, "gemm_tiled_block");
  return launch_tiled<128, 128, 2, 2, false, false>(p, grid, stream, "gemm_tiled_row");
}

int gemm_grouped_dispatch(const GemmArgs& p, int64_t T, hipStream_t stream) {
  // every active slot owns at most ceil(cnt/128) m-tiles: sum <= T/128 + num_active
  const int64_t m_tiles = T / 128 + p.num_active;
  if (m_tiles > 65535) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped matmul: %lld row tiles exceed the launch limit", (long long)m_tiles);
  const dim3 grid((unsigned)ceil_div(p.N, 128), (unsigned)m_tiles);
  return launch_tiled<128, 128, 2, 2, true, true>(p, grid, stream, "gemm_grouped_block");
}

}  // namespace maxfp8
