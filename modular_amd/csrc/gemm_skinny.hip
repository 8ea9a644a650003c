// Weight-streaming scaled FP8 matmul for small M (decode): C[M,N] = A[M,K] . B[N,K]^T,
// M <= 16 * MT.
//
// The bytes that matter are the N*K weight bytes, read exactly once, so the kernel is
// shaped by what HBM likes (measured on MI355X with read-only kernels: whole 128-byte lines
// per row and long runs per wave reach ~6.2 TB/s on these shapes; half lines taken by
// alternating waves stay at ~4.6 TB/s):
//
//   * a block owns 16*NTW consecutive weight rows; each of its 4 or 8 waves owns a contiguous
//     share of K and walks it in 128-byte slabs;
//   * weight slabs travel by LDS-DMA (`buffer_load_dwordx4 ... lds`), one instruction per
//     8 rows x 128 bytes (whole cache lines), into a ring of DEPTH slots that is private to
//     the wave -- no barrier in the loop, DEPTH slabs of weights in flight per wave;
//   * the MFMA row operand (16 weight rows x 128 K bytes) is read back from LDS with the
//     same conflict-free chunk swizzle as the tiled kernel; the activations are the column
//     operand, loaded straight from global memory / L2 (tokens >= M read as zero through the
//     buffer descriptor): v_mfma_f32_16x16x128_f8f6f4 computes 16 weight rows x 16 tokens
//     per instruction, so M is never padded to a 128-row tile;
//   * the waves' partial sums meet in LDS in a fixed order (deterministic result).
//
// Scaling follows gemm_tiled.hip: block mode promotes every slab with
// a_s[slab, m] * b_s[n/128, slab]; row/tensor mode scales once at the end
// (max/kernels/src/linalg/fp8_quantization.mojo:1218-1240, 1576-1624).
#include <stdlib.h>

#include <type_traits>
#include <utility>

#include "common.h"
#include "gemm_args.h"
#include "tuning.h"

namespace maxfp8 {

typedef __attribute__((address_space(3))) void* sk_lds_ptr_t;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t sk_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
// Cache policy of the weight copies: non-temporal.  A weight byte is read once per launch; marked so, the stream does not
// displace what the memory-side cache and the L2 hold, and the chip reads 7.0 instead of 6.2 TB/s (a read-only kernel,
// one block of eight 16 KB rings per CU, the same matrix with and without the bit).
constexpr int kWeightStream = 2;

__device__ __forceinline__ v4i sk_load16(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
__device__ __forceinline__ float sk_load_f32(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ uint32_t sk_clamp_u32(int64_t v) {
  return v > 0xfffffff0ll ? 0xfffffff0u : (v < 0 ? 0u : (uint32_t)v);
}

// ALDS: the activations of a wave's share of K are copied to LDS once, before the loop (at most kSkinnyALdsBytes per
// wave), instead of two loads per slab and 16-token group: on a launch that is a single round of blocks those loads
// are half of the loop's vector-memory instructions and cost 8 % of the kernel, whatever they fetch.
constexpr int kSkinnyALdsBytes = 8192;
template <int NTW, int MT, bool BLOCKSCALE, int RING_KB, int NWAVES, bool ALDS = false>
struct SkinnyCfg {
  static constexpr int WAVES = NWAVES;
  static constexpr int SLOT = NTW * 2048;                    // one slab of the block's rows
  // VMEM instructions a wave issues per slab, in this order: activations, scales, weight DMA
  static constexpr int PER = (ALDS ? 0 : 2 * MT) + (BLOCKSCALE ? MT + 1 : 0) + 2 * NTW;
  // slabs in flight per wave: RING_KB of weights, limited by the 6-bit vmcnt counter and by the
  // registers the activation fragments of the in-flight slabs take (96)
  static constexpr int D_BYTES = RING_KB * 1024 / SLOT, D_CNT = 63 / PER + 1, D_REGS = 96 / (MT * 8);
  static constexpr int D_MIN = D_BYTES < D_CNT ? (D_BYTES < D_REGS ? D_BYTES : D_REGS) : (D_CNT < D_REGS ? D_CNT : D_REGS);
  static constexpr int DEPTH = D_MIN < 2 ? 2 : D_MIN;
  static constexpr int RING = DEPTH * SLOT;                  // per wave
  static constexpr int RED = WAVES * MT * NTW * 4 * 64 * 4;  // reduction buffer (reuses the rings)
  static constexpr int RINGS = WAVES * RING > RED ? WAVES * RING : RED;
  static constexpr int SMEM = RINGS;  // (ALDS: plus WAVES * M * the share's bytes, added at the launch)
};

template <int NTW, int MT, bool BLOCKSCALE, int RING_KB, int NWAVES, bool ALDS = false>
__global__ __launch_bounds__(NWAVES * 64) void gemm_skinny_kernel(GemmArgs p_in) {
  const GemmArgs p = gridDim.y == 1 ? p_in : batch_view(p_in, blockIdx.y);
  using Cfg = SkinnyCfg<NTW, MT, BLOCKSCALE, RING_KB, NWAVES, ALDS>;
  static_assert(!ALDS || MT == 1, "activations in LDS: one 16-token group");
  constexpr int WAVES = Cfg::WAVES, DEPTH = Cfg::DEPTH, SLOT = Cfg::SLOT, PER = Cfg::PER;
  static_assert((DEPTH - 1) * PER < 64, "vmcnt is a 6-bit counter");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lm = lane & 15, lq = lane >> 4;
  const int n0 = blockIdx.x * (16 * NTW);
  const int cols_here = (p.N - n0) < 16 * NTW ? (p.N - n0) : 16 * NTW;

  const uint8_t* b_tile = p.b + (int64_t)n0 * p.ldb;
  const __amdgpu_buffer_rsrc_t b_rsrc = sk_rsrc(b_tile, sk_clamp_u32((int64_t)(cols_here - 1) * p.ldb + p.K));
  const __amdgpu_buffer_rsrc_t a_rsrc = sk_rsrc(p.a, sk_clamp_u32((int64_t)(p.M - 1) * p.lda + p.K));

  const int nslab = (p.K + 127) / 128;
  const bool k_tail = (p.K & 127) != 0;
  // this wave's slabs: [s_begin, s_end)
  const int per_wave = (nslab + WAVES - 1) / WAVES;
  const int s_begin = wave * per_wave;
  const int s_end = (s_begin + per_wave) < nslab ? (s_begin + per_wave) : nslab;

  // weight DMA: lane (cr = lane >> 3, cp = lane & 7) moves logical chunk cp ^ cr of row cr (then
  // row 8 + cr) of a 16-row group to LDS position lane * 16: row r, chunk c is stored at c ^ (r & 7)
  const int cr = lane >> 3, cp = lane & 7;
  const int cchunk = cp ^ cr;
  const uint32_t w_voff = (uint32_t)cr * (uint32_t)p.ldb + cchunk * 16;
  const uint32_t w_half = 8u * (uint32_t)p.ldb;
  const uint32_t w_tile = 16u * (uint32_t)p.ldb;
  // activation operand: lane (m = lm, lq) holds K bytes [16*lq, +16) and [64 + 16*lq, +16) of token m
  uint32_t a_off[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) a_off[t] = (uint32_t)(t * 16 + lm) * (uint32_t)p.lda + lq * 16;
  // fragment read: row lm of a 16-row group, logical chunks lq and lq + 4
  const uint32_t frag0 = lm * 128 + ((lq ^ (lm & 7)) << 4);
  const uint32_t frag1 = lm * 128 + (((lq + 4) ^ (lm & 7)) << 4);
  uint8_t* ring = smem + wave * Cfg::RING;
  // ALDS: token t's bytes of this wave's share of K sit at a_lds + t * a_tok; lane (lm, lq) reads token min(lm, M - 1)
  // (the columns of C past M are never stored, so what their lanes multiply does not matter)
  [[maybe_unused]] const uint32_t a_tok = ((uint32_t)per_wave * 128u + 1023u) & ~1023u;  // (whole copies: 1024 bytes each)
  [[maybe_unused]] uint8_t* a_lds = smem + Cfg::RINGS + wave * ((uint32_t)p.M * a_tok);
  [[maybe_unused]] const uint32_t a_rd = (uint32_t)(lm < p.M ? lm : p.M - 1) * a_tok + lq * 16;
  if constexpr (ALDS) {
    // one instruction moves 1024 consecutive bytes of a token; bytes past K or past the share are not fetched (zeros)
    const uint32_t share_begin = (uint32_t)s_begin * 128u, share_end = (uint32_t)(s_end > s_begin ? s_end : s_begin) * 128u;
    const uint32_t k_end = share_end < (uint32_t)p.K ? share_end : (uint32_t)p.K;
    for (int t = 0; t < p.M; ++t)
      for (uint32_t piece = 0; piece < a_tok; piece += 1024u) {
        const uint32_t k = share_begin + piece + lane * 16u;
        const uint32_t kill = k < k_end ? 0u : 0x80000000u;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (sk_lds_ptr_t)(a_lds + t * a_tok + piece), 16, ((uint32_t)t * (uint32_t)p.lda + k) | kill, 0, 0, 0);
      }
  }

  __amdgpu_buffer_rsrc_t as_rsrc = sk_rsrc(nullptr, 0), bs_rsrc = sk_rsrc(nullptr, 0);
  uint32_t as_voff[MT];
  if constexpr (BLOCKSCALE) {
    as_rsrc = sk_rsrc(p.a_scales, sk_clamp_u32(((int64_t)(nslab - 1) * p.a_scales_ld + p.M) * 4));
    bs_rsrc = sk_rsrc(p.b_scales + (int64_t)(n0 / 128) * p.b_scales_ld, (uint32_t)nslab * 4u);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = t * 16 + lm;
      as_voff[t] = (uint32_t)(m < p.M ? m : p.M - 1) * 4u;
    }
  }

  v4f acc[MT][NTW];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NTW; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  v8i af[DEPTH][MT];
  float as_v[DEPTH][MT], bs_v[DEPTH];

  // Issues the PER loads of one slab into pipeline slot d.  Slabs past the wave's range are
  // issued "out of range" (zeros, no traffic), so every slot always carries exactly PER
  // instructions and the wait counts below are exact.
  auto issue = [&](int slab, auto d_c) {
    constexpr int d = decltype(d_c)::value;
    const bool live = slab < s_end;
    const int sl = live ? slab : s_begin;
    // (wave-uniform by construction; said so explicitly, or the loads' scalar offsets end up in vector registers
    // and every load in a loop over the lanes' values)
    const uint32_t koff = __builtin_amdgcn_readfirstlane((uint32_t)sl * 128u);
    const uint32_t koff_hi = __builtin_amdgcn_readfirstlane(koff + 64u);
    uint32_t kill0 = live ? 0u : 0x80000000u, kill1 = kill0, killw = kill0;
    if (k_tail) {
      if (koff + lq * 16 >= (uint32_t)p.K) kill0 = 0x80000000u;
      if (koff + 64 + lq * 16 >= (uint32_t)p.K) kill1 = 0x80000000u;
      if (koff + cchunk * 16 >= (uint32_t)p.K) killw = 0x80000000u;
    }
    if constexpr (!ALDS) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const v4i lo = sk_load16(a_rsrc, a_off[t] | kill0, koff);
        const v4i hi = sk_load16(a_rsrc, a_off[t] | kill1, koff_hi);
        af[d][t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
    }
    if constexpr (BLOCKSCALE) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
        as_v[d][t] = sk_load_f32(as_rsrc, as_voff[t], (uint32_t)sl * (uint32_t)p.a_scales_ld * 4u);
      bs_v[d] = sk_load_f32(bs_rsrc, 0, (uint32_t)sl * 4u);
    }
    uint8_t* slot = ring + d * SLOT;
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (sk_lds_ptr_t)(slot + t * 2048), 16, w_voff | killw,
                                               koff + t * w_tile, 0, kWeightStream);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (sk_lds_ptr_t)(slot + t * 2048 + 1024), 16, w_voff | killw,
                                               koff + t * w_tile + w_half, 0, kWeightStream);
    }
  };
  auto compute = [&](auto d_c, [[maybe_unused]] int slab) {
    constexpr int d = decltype(d_c)::value;
    // the slot's loads are the oldest in flight: everything issued for the DEPTH-1 younger slots may stay
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 1) * PER) : "memory");
    const uint8_t* slot = ring + d * SLOT;
    if constexpr (ALDS) {
      // (a slab past the share's end multiplies zeros -- its weights were not fetched -- with whatever this reads)
      const uint32_t at = (uint32_t)(slab < s_end ? slab - s_begin : 0) * 128u;
      const v4i lo = *reinterpret_cast<const v4i*>(a_lds + a_rd + at);
      const v4i hi = *reinterpret_cast<const v4i*>(a_lds + a_rd + at + 64);
      af[d][0] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
      const v4i lo = *reinterpret_cast<const v4i*>(slot + nt * 2048 + frag0);
      const v4i hi = *reinterpret_cast<const v4i*>(slot + nt * 2048 + frag1);
      const v8i wf = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if constexpr (BLOCKSCALE) {
          const v4f zero = {0.f, 0.f, 0.f, 0.f};
          const v4f part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af[d][mt], zero, 0, 0, 0, 0, 0, 0);
          acc[mt][nt] += part * (as_v[d][mt] * bs_v[d]);
        } else {
          acc[mt][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af[d][mt], acc[mt][nt], 0, 0, 0, 0, 0, 0);
        }
      }
    }
    // the fragment reads must have left LDS before the slot is refilled
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  };
  auto for_each_slot = [&](auto&& f) {
    [&]<int... D>(std::integer_sequence<int, D...>) { (f(std::integral_constant<int, D>{}), ...); }
    (std::make_integer_sequence<int, DEPTH>{});
  };

  for_each_slot([&](auto d_c) { issue(s_begin + decltype(d_c)::value, d_c); });
  for (int base = s_begin; base < s_end; base += DEPTH) {
    for_each_slot([&](auto d_c) {
      constexpr int d = decltype(d_c)::value;
      compute(d_c, base + d);
      issue(base + DEPTH + d, d_c);
    });
  }
  // drain: the last DEPTH issues were out of range, but they still target LDS slots
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // ---- reduce the 4 waves' partial sums (fixed order) and store ----------------------
  float* red = reinterpret_cast<float*>(smem);  // [WAVES][MT*NTW*4][64]
  constexpr int RSTRIDE = MT * NTW * 4 * 64;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[wave * RSTRIDE + ((mt * NTW + nt) * 4 + v) * 64 + lane] = acc[mt][nt][v];
  __syncthreads();

  // (mt, nt) pairs are dealt to the waves round-robin
  for (int pair = wave; pair < MT * NTW; pair += WAVES) {
    const int mt = pair / NTW, nt = pair - mt * NTW;
    const int m = mt * 16 + lm;
    const int n = n0 + nt * 16 + lq * 4;
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = (pair * 4 + i) * 64 + lane;
      float sum = red[r];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) sum += red[w * RSTRIDE + r];
      v[i] = sum;
    }
    if (m >= p.M || n >= p.N) continue;
    if (p.kv_on) {
      // fused QKV: the reference's bf16 roundings, then C or the row's K / V page (see tile_body)
      const int64_t row_off = kv_row_offset(p.kv, m);
      float a_s = 1.f;
      if constexpr (!BLOCKSCALE) a_s = p.a_scales[(int64_t)m * p.a_scale_stride];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int nn = (n + i < p.N) ? n + i : p.N - 1;
        float r = bf16_round(v[i]);
        if constexpr (!BLOCKSCALE) {
          const float sc = bf16_round(bf16_round(a_s) * bf16_round(p.b_scales[(int64_t)nn * p.b_scale_stride]));
          r = bf16_round(r * sc);
        }
        if (p.kv.bias) r = bf16_round(r + bf16_bits_to_f32(p.kv.bias[nn]));
        v[i] = r;
      }
      if (row_off < 0 && n >= p.kv.q_dim) continue;
      uint16_t* dst = kv_dst(p.kv, p.c, p.ldc, m, row_off, n);
      if (p.c_vec_ok && n + 3 < p.N) {
        const uint32_t lo = pack_bf16x2(v[0], v[1]);
        const uint32_t hi = pack_bf16x2(v[2], v[3]);
        *reinterpret_cast<uint2*>(dst) = make_uint2(lo, hi);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < p.N) dst[i] = (uint16_t)f32_to_bf16_bits(v[i]);
      }
      continue;
    }
    if constexpr (!BLOCKSCALE) {
      const float a_s = scale_at(p.a_scales, (int64_t)m * p.a_scale_stride, p.scales_dtype);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int nn = (n + i < p.N) ? n + i : p.N - 1;
        const float t = v[i] * a_s;
        v[i] = t * scale_at(p.b_scales, (int64_t)nn * p.b_scale_stride, p.scales_dtype);
      }
    }
    if (p.c_dtype == MAXFP8_BF16) {
      uint16_t* dst = reinterpret_cast<uint16_t*>(p.c) + (int64_t)m * p.ldc + n;
      if (p.c_vec_ok && n + 3 < p.N) {
        const uint32_t lo = pack_bf16x2(v[0], v[1]);
        const uint32_t hi = pack_bf16x2(v[2], v[3]);
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

int compute_units();
template <int NTW, int MT, bool BLOCKSCALE, int RING_KB, int NWAVES, bool ALDS = false>
static int launch_skinny_r(const GemmArgs& p, int64_t batch, hipStream_t stream) {
  if constexpr (MT == 1 && !ALDS) {
    // few tokens, a share of K per wave that fits, and a weight matrix small enough that the launch is about one round of
    // blocks: the activations go to LDS once (84 MB, M = 1: 17.8 -> 17.0 us; on a 470 MB matrix, where blocks come and
    // go, the per-slab loads cost nothing and this form measured 1 % slower).  Not for the fused QKV epilogue's build, a
    // rare caller at these sizes, to keep the number of kernels down.
    // The extra LDS must not cost a resident block: all blocks of such a launch sit on the chip at once, and a CU's share
    // of them has to fit its 160 KB with the activations added (10240 x 8192 at M = 2: 18.3 -> 16.6 us; at M = 4, where
    // a CU's three blocks would need 192 KB: 18.5 -> 20.2, so that case keeps the per-slab loads).
    const int64_t per_wave = ceil_div(ceil_div(p.K, 128), NWAVES);
    const int64_t a_bytes = (int64_t)p.M * ((per_wave * 128 + 1023) / 1024 * 1024);  // per wave
    const int64_t blocks_per_cu = ceil_div(ceil_div((int64_t)p.N, 16 * NTW) * batch, (int64_t)compute_units());
    using Plain = SkinnyCfg<NTW, MT, BLOCKSCALE, RING_KB, NWAVES, false>;
    if (tuning().skinny_alds && !p.kv_on && (int64_t)p.N * p.K < ((int64_t)1 << 27) && a_bytes <= kSkinnyALdsBytes &&
        blocks_per_cu * (Plain::SMEM + NWAVES * a_bytes) <= 160 * 1024)
      return launch_skinny_r<NTW, MT, BLOCKSCALE, RING_KB, NWAVES, true>(p, batch, stream);
  }
  using Cfg = SkinnyCfg<NTW, MT, BLOCKSCALE, RING_KB, NWAVES, ALDS>;
  auto kern = gemm_skinny_kernel<NTW, MT, BLOCKSCALE, RING_KB, NWAVES, ALDS>;
  static PerDeviceFlag attr;
  bool& attr_done = attr.here();
  constexpr int smem_all = Cfg::SMEM + (ALDS ? NWAVES * kSkinnyALdsBytes : 0);
  constexpr int smem_max = smem_all < 160 * 1024 ? smem_all : 160 * 1024;  // (what a launch asks for was checked against the CU's LDS)
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem_max);
    if (e != hipSuccess) MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "gemm_skinny: cannot reserve %d bytes of LDS: %s", smem_max, hipGetErrorString(e));
    attr_done = true;
  }
  int smem = Cfg::SMEM;
  if constexpr (ALDS) {
    const int64_t per_wave = ceil_div(ceil_div(p.K, 128), NWAVES);
    smem += NWAVES * (int)(p.M * ((per_wave * 128 + 1023) / 1024 * 1024));
  }
  const int64_t blocks = ceil_div(p.N, 16 * NTW);
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks, (unsigned)batch), dim3(NWAVES * 64), smem, stream, p);
  return launch_status("gemm_skinny");
}

// Shape choice.  A block re-reads its M x K activations for every 16 * NTW weight rows, through L1 and L2, so the
// activation traffic is M / (16 * NTW) times the weight traffic, and all blocks are resident at once, so a CU's
// share is ceil(blocks / CUs) blocks.  The shape with the smallest
//     ceil(blocks / CUs) * (16 * NTW + M + 8)        (8: ring fill and the epilogue of a block, in the same unit)
// wins; 64-row blocks count 25 % more (one block per CU: 32 KB of weights in flight per wave, but fewer waves to
// hide latency with) and need K >= 4096 (with few slabs per wave the long epilogue shows).  Measured on Llama-70B /
// Llama-8B / DeepSeek-V3 decode shapes in both scale modes the rule lands on the fastest shape or within 4 % of it;
// e.g. M = 64, N = 8192, K = 28672: 32 rows per block, 75 us (16 rows: 122); M = 32, N = 10240, K = 8192: 64 rows,
// 23 us (16 rows: 33); M = 32, N = 5120, K = 5120: 32 rows, 12 us (16 rows: 18); N = 4096: 16 rows, one block per CU.
// 32-row blocks keep 16 KB per wave in flight when M <= 16 and the weights exceed 256 MB, else 8 KB.
// (8 waves per block were tried for the small-N shapes and were no faster.)  Every shape splits K over its four waves
// in the same way and adds the partial sums in the same order: the result does not depend on the choice.
// The tuning switch `skinny` = <ntw>4<ringKB>, e.g. 1408 or 2416, forces a shape for tuning runs.
int compute_units();
static int skinny_shape(int64_t M, int64_t N, int64_t K) {
  const int64_t cus = compute_units();
  int best = 1;
  float best_cost = 0.f;
  for (int ntw = 1; ntw <= 4; ntw *= 2) {
    if (ntw == 4 && K < 4096) break;
    const int64_t blocks = ceil_div(N, 16 * ntw);
    float cost = (float)ceil_div(blocks, cus) * (float)(16 * ntw + M + 8);
    if (ntw == 4) cost *= K >= 8192 ? 1.25f : 1.35f;  // (one block per CU: its start and end weigh more the shorter K is)
    if (ntw == 1 || cost < best_cost) { best = ntw; best_cost = cost; }
  }
  // (16 KB rings for 32-row blocks -- the selector 2416 -- were ahead on the largest matrices while the chip read 6.2
  // TB/s; with the weight copies marked non-temporal 8 KB rings are: 68.6 against 72.2 us on 57344 x 8192 at M = 1)
  if (best == 4) return 4432;
  if (best == 2) return 2408;
  return 1408;
}

template <int MT, bool BLOCKSCALE>
static int pick_ntw(const GemmArgs& p, int64_t batch, hipStream_t stream) {
  int sel = tuning().skinny;
  if (!sel) sel = skinny_shape(p.M, p.N, p.K);
  switch (sel) {
    case 1408: return launch_skinny_r<1, MT, BLOCKSCALE, 8, 4>(p, batch, stream);
    case 1416: return launch_skinny_r<1, MT, BLOCKSCALE, 16, 4>(p, batch, stream);
    case 2416: return launch_skinny_r<2, MT, BLOCKSCALE, 16, 4>(p, batch, stream);
    case 2408: return launch_skinny_r<2, MT, BLOCKSCALE, 8, 4>(p, batch, stream);
    case 4432: return launch_skinny_r<4, MT, BLOCKSCALE, 32, 4>(p, batch, stream);
    default: MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "skinny matmul: unknown shape selector %d", sel);
  }
}

// ---- read-only probe ---------------------------------------------------------------------------
// The weight traffic of gemm_skinny_kernel and nothing else: same grid, block size, rows per block, split of K over
// the waves, LDS ring, ring depth, DMA instructions and wait counts as the matmul of an M <= 16 row-scaled problem, but
// no activations, no MFMA, no reduction and no stores (one dword per slab is read back from LDS so that the ring is
// consumed in order).  Its time is what this access pattern can reach on the memory system: the matmul is measured
// against it.
template <int NTW, int RING_KB, int NWAVES>
__global__ __launch_bounds__(NWAVES * 64) void skinny_read_probe_kernel(const uint8_t* b, int N, int K, int64_t ldb, uint32_t* sink) {
  using Cfg = SkinnyCfg<NTW, 1, false, RING_KB, NWAVES>;
  constexpr int WAVES = Cfg::WAVES, DEPTH = Cfg::DEPTH, SLOT = Cfg::SLOT, PER = 2 * NTW;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * (16 * NTW);
  const int cols_here = (N - n0) < 16 * NTW ? (N - n0) : 16 * NTW;
  const __amdgpu_buffer_rsrc_t b_rsrc = sk_rsrc(b + (int64_t)n0 * ldb, sk_clamp_u32((int64_t)(cols_here - 1) * ldb + K));
  const int nslab = (K + 127) / 128;
  const int per_wave = (nslab + WAVES - 1) / WAVES;
  const int s_begin = wave * per_wave;
  const int s_end = (s_begin + per_wave) < nslab ? (s_begin + per_wave) : nslab;
  const int cr = lane >> 3, cp = lane & 7;
  const uint32_t w_voff = (uint32_t)cr * (uint32_t)ldb + (cp ^ cr) * 16;
  const uint32_t w_half = 8u * (uint32_t)ldb, w_tile = 16u * (uint32_t)ldb;
  uint8_t* ring = smem + wave * Cfg::RING;
  uint32_t seen = 0;
  auto issue = [&](int slab, auto d_c) {
    constexpr int d = decltype(d_c)::value;
    const bool live = slab < s_end;
    const uint32_t koff = (uint32_t)(live ? slab : s_begin) * 128u;
    const uint32_t killw = live ? 0u : 0x80000000u;
    uint8_t* slot = ring + d * SLOT;
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (sk_lds_ptr_t)(slot + t * 2048), 16, w_voff | killw, koff + t * w_tile, 0, kWeightStream);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (sk_lds_ptr_t)(slot + t * 2048 + 1024), 16, w_voff | killw, koff + t * w_tile + w_half, 0, kWeightStream);
    }
  };
  auto consume = [&](auto d_c) {
    constexpr int d = decltype(d_c)::value;
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 1) * PER) : "memory");
    seen ^= *reinterpret_cast<const uint32_t*>(ring + d * SLOT + lane * 4);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  };
  auto for_each_slot = [&](auto&& f) {
    [&]<int... D>(std::integer_sequence<int, D...>) { (f(std::integral_constant<int, D>{}), ...); }
    (std::make_integer_sequence<int, DEPTH>{});
  };
  for_each_slot([&](auto d_c) { issue(s_begin + decltype(d_c)::value, d_c); });
  for (int base = s_begin; base < s_end; base += DEPTH) {
    for_each_slot([&](auto d_c) {
      constexpr int d = decltype(d_c)::value;
      consume(d_c);
      issue(base + DEPTH + d, d_c);
    });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // (never true for the data the benchmark streams; keeps the reads alive)
  if (seen == 0x9e3779b9u && sink) sink[0] = seen;
}

template <int NTW, int RING_KB, int NWAVES>
static int launch_read_probe(const void* b, int64_t N, int64_t K, int64_t ldb, hipStream_t stream) {
  using Cfg = SkinnyCfg<NTW, 1, false, RING_KB, NWAVES>;
  auto kern = skinny_read_probe_kernel<NTW, RING_KB, NWAVES>;
  static PerDeviceFlag attr;
  bool& attr_done = attr.here();
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::SMEM);
    if (e != hipSuccess) MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "read probe: cannot reserve %d bytes of LDS: %s", Cfg::SMEM, hipGetErrorString(e));
    attr_done = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)ceil_div(N, 16 * NTW)), dim3(NWAVES * 64), Cfg::SMEM, stream, (const uint8_t*)b, (int)N, (int)K,
                     ldb, (uint32_t*)nullptr);
  return launch_status("skinny_read_probe");
}

int gemm_skinny_read_probe(const void* b, int64_t M, int64_t N, int64_t K, int64_t ldb, hipStream_t stream) {
  int sel = tuning().skinny;
  if (!sel) sel = skinny_shape(M, N, K);
  switch (sel) {
    case 1408: return launch_read_probe<1, 8, 4>(b, N, K, ldb, stream);
    case 1416: return launch_read_probe<1, 16, 4>(b, N, K, ldb, stream);
    case 2416: return launch_read_probe<2, 16, 4>(b, N, K, ldb, stream);
    case 2408: return launch_read_probe<2, 8, 4>(b, N, K, ldb, stream);
    case 4432: return launch_read_probe<4, 32, 4>(b, N, K, ldb, stream);
    default: MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "read probe: unknown shape selector %d", sel);
  }
}

int gemm_skinny_max_m() { return 64; }

// What MAXFP8_ALGO_AUTO gives the weight-streaming kernel: every matmul of at most 32 rows (but see below), and those
// of 33 to 64 rows whose weights take less than 32 MB.  With four 16-token groups per weight fragment every block re-reads 64 rows of
// activations through its L1 (about 8 TB/s over the chip) and its time grows with M, while the three-stage 128 x 128
// tiles share the activations through LDS, split K over the chip when their column tiles are few, and take the same
// time from 1 to 128 rows: at M = 64 they measured 54 us against 75 (N = 8192, K = 28672), 19 against 36 (2304 x
// 16384), 25 against 32 (10240 x 8192), 30 against 40 (28672 x 4096).  Their floor is two launches, 16 to 17 us:
// below 32 MB of weights the streaming kernel stays ahead (4096 x 4096: 12 us; 6144 x 4096: 14).
// From 25 rows on the tiles are already ahead where K is long and N narrow (M = 32: 48 us against 53 on 8192 x 28672,
// 17 against 21 on 4096 x 14336 and on 2304 x 16384); at 24 rows and below the streaming kernel wins or ties.
bool gemm_skinny_preferred(int64_t M, int64_t N, int64_t K) {
  const bool small_weights = N * K < ((int64_t)1 << 25);
  if (M <= 24) return true;
  if (M <= 32) return small_weights || K < 12288 || N >= 10240;
  return M <= 64 && small_weights;
}

int gemm_skinny_dispatch(const GemmArgs& p, bool blockscale, int64_t batch, hipStream_t stream) {
  if (p.M > 64) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "skinny matmul: M = %d exceeds 64", p.M);
  const int mt = (p.M + 15) / 16;
  if (blockscale) {
    if (mt <= 1) return pick_ntw<1, true>(p, batch, stream);
    if (mt <= 2) return pick_ntw<2, true>(p, batch, stream);
    return pick_ntw<4, true>(p, batch, stream);
  }
  if (mt <= 1) return pick_ntw<1, false>(p, batch, stream);
  if (mt <= 2) return pick_ntw<2, false>(p, batch, stream);
  return pick_ntw<4, false>(p, batch, stream);
}

}  // namespace maxfp8
