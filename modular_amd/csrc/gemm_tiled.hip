// LDS-staged MFMA GEMM for scaled FP8 on gfx950:  C[M,N] = A[M,K] . B[N,K]^T.
//
// One block owns a BM x BN tile of C and walks K in slabs of 128 bytes (one scale group).
//
//   * global -> LDS copies are `buffer_load_dwordx4 ... lds` (LDS DMA): no staging registers,
//     no ds_write.  A wave-instruction moves 8 tile rows x 128 bytes; lane (r = lane >> 3,
//     p = lane & 7) fetches the logical 16-byte chunk p ^ (row & 7) of its row, so the bytes
//     land in LDS already swizzled for conflict-free MFMA fragment reads.  Rows past the tile
//     edge read as zero through the buffer descriptor, so partial tiles need no branches.
//   * NS LDS stages (2 or 3; 4 measured no better), one barrier per slab, DMA issued NS-1 slabs ahead.
//   * every wave issues v_mfma_f32_16x16x128_f8f6f4 on its (BM/WAVES_M) x (BN/WAVES_N)
//     sub-tile.  The weight fragment is the MFMA's row operand and the activation fragment its
//     column operand, so a lane ends up with 4 consecutive n for ONE m: the per-token scale is
//     a single register per 16-row group and bf16 results leave as 8-byte stores.  Weight
//     fragments of the slab stay in registers; activation fragments stream 16 rows at a time,
//     one step ahead of the MFMAs that use them.
//
// Block scaling (1x128 activation groups, 128x128 weight blocks): each slab's product is formed
// in a fresh accumulator P (MFMA with C = 0) and promoted with
// acc += P * (a_s[slab, m] * b_s[n/128, slab]) -- the per-slab promotion of
// max/kernels/src/linalg/matmul/gpu/sm100/blockwise_fp8.mojo:376-392, which sums the same terms
// as the reference's naive kernel (max/kernels/src/linalg/fp8_quantization.mojo:1576-1624) in a
// different order.  The slab's activation scales travel through LDS with the tile (one more
// LDS-DMA instruction per wave).  Row/tensor scaling: acc accumulates over all of K inside the
// MFMA and is scaled once, (acc * a_s[m]) * b_s[n]  (fp8_quantization.mojo:1218-1240).
//
// Grouped (MoE) mode maps blocks to (expert slot, m-tile, n-tile) from the device-resident
// offsets with a block-wide prefix sum, so no host synchronisation is needed
// (semantics: fp8_quantization.mojo:1745-1865).  Its large-tile launch and the launch of the rest
// run side by side on two streams (gemm_grouped_dispatch).
//
// Matmuls made of whole 256 x 256 tiles with bf16 output run in gemm_persist_kernel: one block
// per CU, the slab stream carried across tile boundaries, tiles stored through a small LDS side
// buffer while the next tile is already being multiplied.
//
// Why the tiles are what they are (measured on MI355X): LDS serves ~128 B/clk/CU to
// ds_read_b128 and LDS-DMA together, the L1 -> LDS path ~50 B/clk/CU, and an MFMA retires in
// 32 clocks per SIMD, so a 64 x 64 wave tile is LDS-bound at two thirds of the MFMA rate and a
// 128 x 64 wave tile is balanced.  Accumulators must be ordinary VGPRs for the promotion, which
// caps the wave tile at 128 x 64 with two waves per SIMD.
#include <stdlib.h>

#include <atomic>
#include <mutex>
#include <utility>
#include "common.h"
#include "gemm_args.h"
#include "gemm_device.h"
#include "tuning.h"

namespace maxfp8 {

// The activation scales of a slab in LDS.  The copy puts its lanes' values at consecutive words, and a lane may fetch
// any row: word i of the scale area gets the row that puts the TM scales a lane needs in the main loop -- rows lm,
// lm + 16, ... of its wave's WM = 16 * TM rows -- four by four at neighbouring words (word wm * WM + (mt / 4) * 64 +
// lm * 4 + mt % 4: the 16 lane rows of a read cover 256 consecutive bytes, every bank once), so that they come back in
// one or two 16-byte LDS reads instead of TM narrow ones.
// (Wave tiles whose TM is not a multiple of 4 keep the rows in order: their scales would come back in reads that
// straddle 16-byte boundaries, which measured a quarter slower than narrow reads on the 192-row tiles.)
template <int WM>
__device__ __forceinline__ int scale_word_row(int i) {
  constexpr int TM = WM / 16;
  if constexpr (TM % 4 != 0) return i;
  const int in_wave = i % WM, mt = (in_wave / 64) * 4 + in_wave % 4, lm = (in_wave % 64) / 4;
  return (i / WM) * WM + mt * 16 + lm;
}

// byte offset, in a stage's scale area, of the first scale of lane row lm of a wave whose rows begin at wave_row0
template <int TM>
__device__ __forceinline__ uint32_t scale_read_offset(int wave_row0, int lm) {
  return (uint32_t)(wave_row0 + (TM % 4 == 0 ? lm * 4 : lm)) * 4u;
}
// a lane's TM scales: 16-byte reads of neighbouring words where TM allows, else one word per 16-row group
template <int TM>
struct ScaleRow { float v[TM]; __device__ __forceinline__ float operator[](int i) const { return v[i]; } };
template <int TM>
__device__ __forceinline__ ScaleRow<TM> read_scales(const uint8_t* at) {
  ScaleRow<TM> out;
  if constexpr (TM % 4 == 0) {
#pragma unroll
    for (int i = 0; i < TM / 4; ++i) {
      const v4f q = *reinterpret_cast<const v4f*>(at + i * 256);
      out.v[4 * i] = q[0]; out.v[4 * i + 1] = q[1]; out.v[4 * i + 2] = q[2]; out.v[4 * i + 3] = q[3];
    }
  } else {
#pragma unroll
    for (int i = 0; i < TM; ++i) out.v[i] = *reinterpret_cast<const float*>(at + i * 64);
  }
  return out;
}

// One BM x BN tile of C: rows [row_begin, row_end) (at most BM of them are used) by columns
// [n0, n0 + BN) of the weight matrix at bptr / scales at bs_ptr.  Called by every thread of a
// block of WAVES_M * WAVES_N waves with `smem` = the block's dynamic LDS.
template <int BM, int BN, int WAVES_M, int WAVES_N, int NS, bool BLOCKSCALE, bool GROUPED, bool KV = false, int B_POLICY = 0>
__device__ __forceinline__ void tile_body(const GemmArgs& p, uint8_t* smem, const int64_t row_begin, const int64_t row_end,
                                          const int n0, const uint8_t* bptr, const float* bs_ptr) {
  constexpr int NWAVES = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int IA = BM / 8 / NWAVES, IB = BN / 8 / NWAVES;  // LDS-DMA instructions per wave and slab
  // one stage: A rows, B rows, then (block scaling) the slab's activation scales, 64 per copy
  constexpr int SCALE_ROWS = BM < 64 ? 64 : BM;
  constexpr int SCALE_BYTES = BLOCKSCALE ? SCALE_ROWS * 4 : 0;
  constexpr int STAGE_BYTES = (BM + BN) * 128 + SCALE_BYTES;
  constexpr int PER = IA + IB + (BLOCKSCALE ? 1 : 0);  // LDS-DMA instructions per wave and slab
  static_assert(NWAVES % 2 == 0 && IA >= 1 && IB >= 1, "tile / wave layout");
  static_assert(NS >= 2 && NS <= 4 && (NS - 2) * PER < 64, "two to four LDS stages; the wait count must fit the vmcnt field");
  static_assert(!BLOCKSCALE || SCALE_ROWS % 64 == 0, "scale rows are copied 64 at a time");
  static_assert(!BLOCKSCALE || (WN <= 128 && 128 % WN == 0), "a wave's columns must sit inside one 128-wide scale block");

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int rows_here = (int)((row_end - row_begin) < BM ? (row_end - row_begin) : BM);
  const int cols_here = (p.N - n0) < BN ? (p.N - n0) : BN;

  const int lm = lane & 15, lq = lane >> 4;
  // A lane ends up with 8 consecutive columns of one row (see the weight fragment plan below):
  // one 16-byte store for bf16, two for f32.
  auto store8 = [&](int64_t m, int n, const v4f& lo, const v4f& hi) {
    const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (p.c_dtype == MAXFP8_BF16) {
      uint16_t* dst = reinterpret_cast<uint16_t*>(p.c) + m * p.ldc + n;
      if (p.c_vec8_ok && n + 7 < p.N) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
        *reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (n + i < p.N) dst[i] = (uint16_t)f32_to_bf16_bits(v[i]);
      }
    } else {
      float* dst = reinterpret_cast<float*>(p.c) + m * p.ldc + n;
      if (p.c_vec_ok && n + 7 < p.N) {
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (n + i < p.N) dst[i] = v[i];
      }
    }
  };

  // ---- global -> LDS copy plan (LDS DMA) ------------------------------------------------
  const uint8_t* a_tile = p.a + row_begin * p.lda;
  const uint8_t* b_tile = bptr + (int64_t)n0 * p.ldb;
  const __amdgpu_buffer_rsrc_t a_rsrc = t2_rsrc(a_tile, t2_clamp_u32((int64_t)(rows_here - 1) * p.lda + p.K));
  const __amdgpu_buffer_rsrc_t b_rsrc = t2_rsrc(b_tile, t2_clamp_u32((int64_t)(cols_here - 1) * p.ldb + p.K));
  const int cr = lane >> 3, cp = lane & 7;
  // tile row of instruction i is (i*NWAVES + wave)*8 + cr, so row & 7 == cr and (row >> 3) & 1 ==
  // wave & 1.  Activation rows keep logical chunk c at c ^ (row & 7); weight rows at
  // c ^ (4 * ((row >> 3) & 1) + (row & 3)), which is what keeps their fragment reads (rows
  // 0-3 and 8-11 of a 32-row group in one instruction) free of bank conflicts.
  const int cchunk = cp ^ cr;
  const int cchunk_b = cp ^ (((wave & 1) << 2) | (cr & 3));
  const uint32_t a_voff = (uint32_t)(wave * 8 + cr) * (uint32_t)p.lda + cchunk * 16;
  const uint32_t b_voff = (uint32_t)(wave * 8 + cr) * (uint32_t)p.ldb + cchunk_b * 16;
  const uint32_t a_istep = (uint32_t)(NWAVES * 8) * (uint32_t)p.lda;
  const uint32_t b_istep = (uint32_t)(NWAVES * 8) * (uint32_t)p.ldb;
  const int nslab = (p.K + 127) / 128;
  // split-K (dense only): blockIdx.y takes a contiguous share of the slabs and leaves raw f32
  // partial sums in the workspace for the reduction kernel
  int slab_begin = 0, slab_end = nslab;
  bool partial_out = false;
  if constexpr (!GROUPED) {
    if (p.splits > 1) {
      const int per = (nslab + p.splits - 1) / p.splits;
      slab_begin = blockIdx.y * per;
      slab_end = (slab_begin + per) < nslab ? (slab_begin + per) : nslab;
      partial_out = true;
    }
  }
  // activation scales of the tile: element (slab, row_begin + r); rows past the tile read as 0
  const int s_chunk = wave % (SCALE_ROWS / 64);
  __amdgpu_buffer_rsrc_t s_rsrc = t2_rsrc(nullptr, 0);
  uint32_t s_voff = 0, s_slab_step = 0;
  if constexpr (BLOCKSCALE) {
    s_rsrc = t2_rsrc(p.a_scales + row_begin, t2_clamp_u32(((int64_t)(nslab - 1) * p.a_scales_ld + rows_here) * 4));
    const int r = scale_word_row<WM>(s_chunk * 64 + lane);
    s_voff = r < rows_here ? (uint32_t)r * 4u : 0x80000000u;
    s_slab_step = (uint32_t)p.a_scales_ld * 4u;
  }

  // LDS-DMA instruction idx (0 .. PER-1) of a wave's share of a slab
  // (dead = 0x80000000 puts every lane out of range: nothing is fetched and the copy only writes
  // zeros into a stage that is not read again; that keeps the loop free of branches)
  auto dma_one = [&](int slab, int buf, int idx, uint32_t dead) {
    const uint32_t koff = (uint32_t)slab * 128u;
    uint32_t kill = dead, kill_b = dead;
    if (koff + cchunk * 16 >= (uint32_t)p.K) kill = 0x80000000u;
    if (koff + cchunk_b * 16 >= (uint32_t)p.K) kill_b = 0x80000000u;
    uint8_t* sa = smem + buf * STAGE_BYTES + wave * 1024;
    uint8_t* sb = sa + BM * 128;
    if (idx < IA) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(sa + idx * NWAVES * 1024), 16, a_voff | kill,
                                               koff + idx * a_istep, 0, 0);
    } else if (idx < IA + IB) {
      const int i = idx - IA;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (lds_ptr_t)(sb + i * NWAVES * 1024), 16, b_voff | kill_b,
                                               koff + i * b_istep, 0, B_POLICY);
    } else if constexpr (BLOCKSCALE) {
      // 64 scales of the slab's row of the transposed scale matrix per wave; with more waves
      // than 64-row chunks the extra waves repeat a chunk (same bytes to the same place), so
      // every wave issues the same number of DMA instructions per slab.
      uint8_t* ss = smem + buf * STAGE_BYTES + (BM + BN) * 128 + s_chunk * 256;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(s_rsrc, (lds_ptr_t)ss, 4, s_voff | dead,
                                               (uint32_t)slab * s_slab_step, 0, 0);
    }
  };
  auto dma = [&](int slab, int buf, uint32_t dead) {
#pragma unroll
    for (int idx = 0; idx < PER; ++idx) dma_one(slab, buf, idx, dead);
  };

  // ---- fragment read plan -------------------------------------------------------------------
  // lane (lm, lq) holds K bytes [16*lq, +16) and [64 + 16*lq, +16) of row lm: logical chunks
  // lq and lq + 4, stored at chunk ^ (row & 7).  (Both MFMA operands use the same K order,
  // which is all the dot product needs; measured conflict-free, unlike chunks 2*lq, 2*lq+1.)
  const int sw = lm & 7;
  const uint32_t frag0 = lm * 128 + ((lq ^ sw) << 4);
  const uint32_t frag1 = lm * 128 + (((lq + 4) ^ sw) << 4);
  const uint32_t a_frag_base = (uint32_t)(wm * WM) * 128;
  const uint32_t b_frag_base = (uint32_t)(BM + wn * WN) * 128;
  auto read_frag = [&](const uint8_t* base) -> v8i {
    const v4i lo = *reinterpret_cast<const v4i*>(base + frag0);
    const v4i hi = *reinterpret_cast<const v4i*>(base + frag1);
    return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  // Weight fragments come in pairs (t = 2q, 2q+1) over 32 weight rows: MFMA row i of the even
  // fragment is weight row 8*(i/4) + i%4 of the group, of the odd fragment 4 more.  The MFMA
  // leaves rows 4*(lane/16) .. +3 in a lane, so the pair gives a lane 8 consecutive columns of C.
  static_assert(TN % 2 == 0, "weight fragments are read in pairs");
  const int wrow = 8 * (lm >> 2) + (lm & 3);                      // row in the 32-row group (even fragment)
  const int wsw = (((wrow >> 3) & 1) << 2) | (wrow & 3);          // same for the odd fragment (rows + 4)
  const uint32_t wfrag0 = wrow * 128 + ((lq ^ wsw) << 4);
  const uint32_t wfrag1 = wrow * 128 + (((lq + 4) ^ wsw) << 4);
  auto read_wfrag = [&](const uint8_t* base, int t) -> v8i {
    const uint8_t* g = base + (t >> 1) * 4096 + (t & 1) * 512;
    const v4i lo = *reinterpret_cast<const v4i*>(g + wfrag0);
    const v4i hi = *reinterpret_cast<const v4i*>(g + wfrag1);
    return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };

  v4f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  // number of this wave's 16-row groups that hold rows of the tile (wave-uniform)
  constexpr bool SKIP_ROWS = GROUPED && BM <= 64;  // (in big tiles the branches cost more than the MFMAs saved)
  int mt_live = TM;
  if constexpr (SKIP_ROWS) {
    const int left = __builtin_amdgcn_readfirstlane(rows_here) - wm * WM;
    mt_live = left <= 0 ? 0 : ((left + 15) >> 4 < TM ? (left + 15) >> 4 : TM);
  }
  const float* bs_row = nullptr;
  if constexpr (BLOCKSCALE) bs_row = bs_ptr + (int64_t)((n0 + wn * WN) / 128) * p.b_scales_ld;
  const uint32_t s_rd = (uint32_t)((BM + BN) * 128) + scale_read_offset<TM>(wm * WM, lm);

  // NS LDS stages, one barrier per slab, DMA issued NS-1 slabs ahead.  At the top of slab j a
  // wave waits until its own DMA of slab j has landed (the younger ones may stay in flight:
  // LDS-DMA is the only VMEM traffic of the loop, so the count is exact), then the barrier makes
  // every wave's part of slab j visible and proves that slab j-1's buffer is no longer read, and
  // the DMA of slab j+NS-1 is sent into that buffer.
#pragma unroll
  for (int st = 0; st < NS - 1; ++st)
    dma(slab_begin + st, st, slab_begin + st < slab_end ? 0u : 0x80000000u);

  // the weight-block scale of the NEXT slab is fetched before this slab's DMA is issued, so
  // that waiting for it never waits for the youngest DMA
  float bs_nxt = 1.f;
  if constexpr (BLOCKSCALE) bs_nxt = bs_row[slab_begin];

  int buf = 0;
  for (int slab = slab_begin; slab < slab_end; ++slab) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 2) * PER) : "memory");  // the NS - 2 younger slabs may stay in flight
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const float bs = bs_nxt;
    if constexpr (BLOCKSCALE) {
      if (slab + 1 < slab_end) bs_nxt = bs_row[slab + 1];
    }
    asm volatile("" ::: "memory");
    // The DMA of slab + NS - 1 is issued in pieces between the MFMA groups below: a wave that
    // sends its whole share at once sits in the VMEM issue queue for most of the copy's
    // duration, and since the barrier lines all waves up, the matrix pipe idles meanwhile.
    const uint32_t dead = slab + NS - 1 < slab_end ? 0u : 0x80000000u;
    const int dma_slab = slab + NS - 1, dma_buf = buf == 0 ? NS - 1 : buf - 1;
    constexpr int SPREAD = (NS == 2 && TM >= 4) ? TM / 2 : TM;

    const uint8_t* sa = smem + buf * STAGE_BYTES;
    float s_cur[TM];
    if constexpr (BLOCKSCALE) {
const ScaleRow<TM> a_sc = read_scales<TM>(sa + s_rd);
      #pragma unroll
      for (int mt = 0; mt < TM; ++mt) s_cur[mt] = a_sc[mt] * bs;
    }
    v8i bf[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) bf[t] = read_wfrag(sa + b_frag_base, t);
    v8i af = read_frag(sa + a_frag_base);
    [[maybe_unused]] v4f part[2][TN];  // block scaling: products of the current and of the previous 16-row group
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      // 16-row groups past the end of a short tile (an expert with few tokens) are skipped:
      // their fragments are not read and their MFMAs not issued
      if (!SKIP_ROWS || mt < mt_live) {
        v8i af_next = af;
        if (mt + 1 < TM) af_next = read_frag(sa + a_frag_base + (mt + 1) * 2048);
        if constexpr (BLOCKSCALE) {
          // the group's MFMAs first, then the promotions of the PREVIOUS group: the matrix pipe works on
          // this group while the VALU folds the last one in
          const v4f zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int nt = 0; nt < TN; ++nt)
            part[mt & 1][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[nt], af, zero, 0, 0, 0, 0, 0, 0);
          if constexpr (!SKIP_ROWS) {
            if (mt > 0) {
#pragma unroll
              for (int nt = 0; nt < TN; ++nt) acc[mt - 1][nt] += part[(mt - 1) & 1][nt] * s_cur[mt - 1];
            }
            if (mt == TM - 1) {
#pragma unroll
              for (int nt = 0; nt < TN; ++nt) acc[mt][nt] += part[mt & 1][nt] * s_cur[mt];
            }
          } else {
#pragma unroll
            for (int nt = 0; nt < TN; ++nt) acc[mt][nt] += part[mt & 1][nt] * s_cur[mt];
          }
        } else {
#pragma unroll
          for (int nt = 0; nt < TN; ++nt)
            acc[mt][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[nt], af, acc[mt][nt], 0, 0, 0, 0, 0, 0);
        }
        af = af_next;
      }
#pragma unroll
      for (int idx = 0; idx < PER; ++idx)
        if (idx * SPREAD / PER == mt) dma_one(dma_slab, dma_buf, idx, dead);
    }
    buf = buf + 1 == NS ? 0 : buf + 1;
  }
  // the copies issued for slabs past the end only write zeros, but they write them into LDS: they
  // must have landed before the stage memory is reused below or handed to the next block
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- epilogue -----------------------------------------------------------------------------
  if (partial_out) {
    float* ws = p.workspace + (int64_t)blockIdx.y * p.M * p.N;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      const int ml = wm * WM + mt * 16 + lm;
      if (ml >= rows_here) continue;
      float* row = ws + (row_begin + ml) * p.N;
#pragma unroll
      for (int q = 0; q < TN / 2; ++q) {
        const int n = n0 + wn * WN + q * 32 + lq * 8;
        if (n >= p.N) continue;
        const v4f lo = acc[mt][2 * q], hi = acc[mt][2 * q + 1];
        if ((p.N & 3) == 0 && n + 7 < p.N) {
          *reinterpret_cast<float4*>(row + n) = make_float4(lo[0], lo[1], lo[2], lo[3]);
          *reinterpret_cast<float4*>(row + n + 4) = make_float4(hi[0], hi[1], hi[2], hi[3]);
        } else {
          const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (n + i < p.N) row[n + i] = v[i];
        }
      }
    }
    return;
  }
  if constexpr (KV) {
    // Fused QKV: bf16 only.  The value takes the reference's roundings -- the accumulator is
    // rounded to bf16 first, per-tensor / per-channel scales are multiplied in bf16, the bias is
    // added in bf16 (kv_cache_ragged.mojo:1210-1245) -- and goes to C or to the row's K / V page.
    // Columns outside, rows inside: 8 weight scales and 8 bias values live at a time.
    //
    // Tiles with all their columns: the finished bf16 values are staged in the wave's 16 KB of stage
    // memory (as the plain epilogue does) and each row's cache offset is looked up ONCE per wave and
    // parked in LDS after the staging area (KV kernels are launched with that much more LDS), so
    // that a store instruction writes 8 rows x one whole 128-byte line to C or to the rows' pages.
    if constexpr (WN == 64 && WM % 64 == 0) {
      if (p.c_vec8_ok && n0 + BN <= p.N) {
        __syncthreads();  // every wave has finished reading the stages
        uint8_t* wbuf = smem + wave * (WM * WN * 2);
        int64_t* otab = reinterpret_cast<int64_t*>(smem + NWAVES * (WM * WN * 2) + wave * (WM * 8));
        {
          constexpr int R = WM / 64;
          int64_t rows[R], off[R];
          bool live[R];
#pragma unroll
          for (int j = 0; j < R; ++j) {
            int r = j * 64 + lane;
            asm volatile("" : "+v"(r));  // keeps the page lookups here, out of the registers of the main loop
            rows[j] = row_begin + wm * WM + r;
            live[j] = wm * WM + r < rows_here;
          }
          kv_row_offsets<R>(p.kv, rows, live, off);
#pragma unroll
          for (int j = 0; j < R; ++j) otab[j * 64 + lane] = off[j];
        }
        static_for<TN / 2>([&](auto qc) {
          constexpr int q = decltype(qc)::value;
          const int n = n0 + wn * WN + q * 32 + lq * 8;
          float b_s[8], bias[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            b_s[i] = 1.f;
            if constexpr (!BLOCKSCALE) b_s[i] = bf16_round(p.b_scales[(int64_t)(n + i) * p.b_scale_stride]);
            bias[i] = p.kv.bias ? bf16_bits_to_f32(p.kv.bias[n + i]) : 0.f;
          }
#pragma unroll
          for (int mt = 0; mt < TM; ++mt) {
            const int r = mt * 16 + lm;
            float a_s = 1.f;
            if constexpr (!BLOCKSCALE) {
              const int64_t mm = row_begin + wm * WM + r;
              a_s = bf16_round(p.a_scales[(mm < p.M ? mm : p.M - 1) * p.a_scale_stride]);
            }
            const v4f lo = acc[mt][2 * q], hi = acc[mt][2 * q + 1];
            const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              w[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
              if constexpr (!BLOCKSCALE) {
                const uint32_t sc = pack_bf16x2(a_s * b_s[2 * i], a_s * b_s[2 * i + 1]);
                w[i] = pack_bf16x2(__uint_as_float(w[i] << 16) * __uint_as_float(sc << 16),
                                   __uint_as_float(w[i] & 0xffff0000u) * __uint_as_float(sc & 0xffff0000u));
              }
              if (p.kv.bias)
                w[i] = pack_bf16x2(__uint_as_float(w[i] << 16) + bias[2 * i], __uint_as_float(w[i] & 0xffff0000u) + bias[2 * i + 1]);
            }
            *reinterpret_cast<uint4*>(wbuf + r * (WN * 2) + (((q * 4 + lq) ^ (r & 7)) * 16)) = make_uint4(w[0], w[1], w[2], w[3]);
          }
        });
        // (a wave reads back only what it wrote itself; LDS operations of a wave execute in order)
        const int rr = lane >> 3, cc = lane & 7;
        const int n = n0 + wn * WN + cc * 8;
#pragma unroll
        for (int i = 0; i < WM / 8; ++i) {
          const int r = i * 8 + rr;
          const uint4 v = *reinterpret_cast<const uint4*>(wbuf + r * (WN * 2) + ((cc ^ (r & 7)) * 16));
          const int64_t off = otab[r];
          if (wm * WM + r < rows_here && !(off < 0 && n >= p.kv.q_dim))
            *reinterpret_cast<uint4*>(kv_dst(p.kv, p.c, p.ldc, row_begin + wm * WM + r, off, n)) = v;
        }
        return;
      }
    }
    float a_s[TM];
    int64_t row_off[TM], rows[TM];
    bool live[TM];
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      int ml = wm * WM + mt * 16 + lm;
      asm volatile("" : "+v"(ml));  // keeps the page lookups here, out of the registers of the main loop
      live[mt] = ml < rows_here;
      rows[mt] = row_begin + ml;
      a_s[mt] = 1.f;
      if constexpr (!BLOCKSCALE)
        if (live[mt]) a_s[mt] = bf16_round(p.a_scales[rows[mt] * p.a_scale_stride]);
    }
    kv_row_offsets<TM>(p.kv, rows, live, row_off);
    static_for<TN / 2>([&](auto qc) {  // (a plain unrolled loop leaves acc indexed at run time here)
      constexpr int q = decltype(qc)::value;
      const int n = n0 + wn * WN + q * 32 + lq * 8;
      if (n >= p.N) return;
      float b_s[8], bias[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int nn = (n + i < p.N) ? n + i : p.N - 1;
        b_s[i] = 1.f;
        if constexpr (!BLOCKSCALE) b_s[i] = bf16_round(p.b_scales[(int64_t)nn * p.b_scale_stride]);
        bias[i] = p.kv.bias ? bf16_bits_to_f32(p.kv.bias[nn]) : 0.f;
      }
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
        const int ml = wm * WM + mt * 16 + lm;
        if (ml >= rows_here) continue;
        if (row_off[mt] < 0 && n >= p.kv.q_dim) continue;
        const v4f lo = acc[mt][2 * q], hi = acc[mt][2 * q + 1];
        const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          w[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
          if constexpr (!BLOCKSCALE) {
            const float s0 = a_s[mt] * b_s[2 * i], s1 = a_s[mt] * b_s[2 * i + 1];
            const uint32_t sc = pack_bf16x2(s0, s1);
            w[i] = pack_bf16x2(__uint_as_float(w[i] << 16) * __uint_as_float(sc << 16),
                               __uint_as_float(w[i] & 0xffff0000u) * __uint_as_float(sc & 0xffff0000u));
          }
          if (p.kv.bias)
            w[i] = pack_bf16x2(__uint_as_float(w[i] << 16) + bias[2 * i], __uint_as_float(w[i] & 0xffff0000u) + bias[2 * i + 1]);
        }
        uint16_t* dst = kv_dst(p.kv, p.c, p.ldc, row_begin + ml, row_off[mt], n);
        if (p.c_vec8_ok && n + 7 < p.N) {
          *reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (n + i < p.N) dst[i] = (uint16_t)(w[i >> 1] >> ((i & 1) * 16));
        }
      }
    });
    return;
  }
  // bf16 tiles with all their columns go through LDS, so that a store instruction writes whole
  // 128-byte lines (8 lanes per row of the wave's WM x WN part) instead of 64-byte halves: each
  // wave owns WM * WN * 2 bytes of the stage memory, written with the 16-byte chunk index XORed
  // with the row (conflict-free in both directions).
  constexpr int CH = WN * 2 / 16;  // 16-byte chunks per row of a wave's part
  constexpr bool LDS_STORE = !GROUPED && CH == 8 && NWAVES * WM * WN * 2 <= NS * STAGE_BYTES;
  if constexpr (LDS_STORE) {
    if (p.c_dtype == MAXFP8_BF16 && p.c_vec8_ok && n0 + BN <= p.N) {
      __syncthreads();  // every wave has finished reading the stages
      uint8_t* wbuf = smem + wave * (WM * WN * 2);
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
        const int r = mt * 16 + lm;
        float a_s = 1.f;
        if constexpr (!BLOCKSCALE) {
          const int64_t mm = row_begin + wm * WM + r;
          a_s = scale_at(p.a_scales, (mm < p.M ? mm : p.M - 1) * p.a_scale_stride, p.scales_dtype);
        }
#pragma unroll
        for (int q = 0; q < TN / 2; ++q) {
          v4f lo = acc[mt][2 * q], hi = acc[mt][2 * q + 1];
          if constexpr (!BLOCKSCALE) {
            const int n = n0 + wn * WN + q * 32 + lq * 8;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float t_lo = lo[i] * a_s, t_hi = hi[i] * a_s;
              lo[i] = t_lo * scale_at(p.b_scales, (int64_t)(n + i) * p.b_scale_stride, p.scales_dtype);
              hi[i] = t_hi * scale_at(p.b_scales, (int64_t)(n + 4 + i) * p.b_scale_stride, p.scales_dtype);
            }
          }
          const int chunk = (q * 4 + lq) ^ (r & 7);
          *reinterpret_cast<uint4*>(wbuf + r * (WN * 2) + chunk * 16) =
              make_uint4(pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]), pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3]));
        }
      }
      // (a wave reads back only what it wrote itself: no barrier, the compiler orders the LDS accesses)
      const int rr = lane >> 3, cc = lane & 7;
      uint16_t* cbase = reinterpret_cast<uint16_t*>(p.c) + (row_begin + wm * WM) * p.ldc + n0 + wn * WN + cc * 8;
#pragma unroll
      for (int i = 0; i < WM / 8; ++i) {
        const int r = i * 8 + rr;
        const uint4 v = *reinterpret_cast<const uint4*>(wbuf + r * (WN * 2) + ((cc ^ (r & 7)) * 16));
        if (wm * WM + r < rows_here) *reinterpret_cast<uint4*>(cbase + (int64_t)r * p.ldc) = v;
      }
      return;
    }
  }
#pragma unroll
  for (int mt = 0; mt < TM; ++mt) {
    const int ml = wm * WM + mt * 16 + lm;
    if (ml >= rows_here) continue;
    const int64_t m = row_begin + ml;
    int64_t cm = m;  // the row of C that receives row m
    if constexpr (GROUPED)
      if (p.c_row_index) cm = p.c_row_index[m];
    float a_s = 1.f;
    if constexpr (!BLOCKSCALE) a_s = scale_at(p.a_scales, m * p.a_scale_stride, p.scales_dtype);
#pragma unroll
    for (int q = 0; q < TN / 2; ++q) {
      const int n = n0 + wn * WN + q * 32 + lq * 8;
      if (n >= p.N) continue;
      v4f lo = acc[mt][2 * q], hi = acc[mt][2 * q + 1];
      if constexpr (!BLOCKSCALE) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n_lo = (n + i < p.N) ? n + i : p.N - 1;
          const int n_hi = (n + 4 + i < p.N) ? n + 4 + i : p.N - 1;
          const float t_lo = lo[i] * a_s, t_hi = hi[i] * a_s;
          lo[i] = t_lo * scale_at(bs_ptr, (int64_t)n_lo * p.b_scale_stride, p.scales_dtype);  // (bs_ptr: this expert's scales when grouped)
          hi[i] = t_hi * scale_at(bs_ptr, (int64_t)n_hi * p.b_scale_stride, p.scales_dtype);
        }
      }
      store8(cm, n, lo, hi);
    }
  }
}

// B_STREAM: the matmul is one row of tiles, so every weight byte is read once: the weight copies are marked non-temporal
template <int BM, int BN, int WAVES_M, int WAVES_N, int NS, bool BLOCKSCALE, bool KV = false, bool B_STREAM = false>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, (WAVES_M * WAVES_N <= 4) ? 2 : 1) void gemm_tiled_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  // ---- block -> tile: XCD de-interleave, then groups of GROUP_M row tiles share weight columns
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;
  int pid = blockIdx.x;
  {
    const int xcd = pid & 7, local = pid >> 3;
    const int base = total >> 3, rem = total & 7;
    pid = xcd * base + (xcd < rem ? xcd : rem) + local;
  }
  int tm, tn;
  tile_coords(pid, tiles_m, tiles_n, tm, tn);
  const GemmArgs q = gridDim.z == 1 ? p : batch_view(p, blockIdx.z);
  tile_body<BM, BN, WAVES_M, WAVES_N, NS, BLOCKSCALE, false, KV, B_STREAM ? kStreamOnce : 0>(q, smem, (int64_t)tm * BM, q.M, tn * BN, q.b,
                                                                                              q.b_scales);
}

// ---- persistent variant ------------------------------------------------------------------------
// For matmuls made of whole BM x BN tiles with bf16 output.  One block per CU walks its share of
// the tiles and the slab stream never stops at a tile boundary: while the last slab of a tile is
// multiplied, slab 0 of the block's next tile is already being copied into the other stage.  The
// finished tile leaves through a 2 KB LDS side buffer of the wave's own (16 rows at a time, so
// that a store instruction still writes whole 128-byte lines), which keeps the stage memory free
// for those copies; the stores of one tile drain while the next one is multiplied.
//
// The wait at the top of a tile's first slab must not wait for those stores.  Vector memory
// operations of a wave complete in order, and after the copy of that slab the wave issued exactly
// NSTORE unconditional stores, so the copy has landed once at most NSTORE operations are
// outstanding.  (This is why only whole tiles run here: a predicated store that the compiler
// may skip would make the count a guess.)
//
// Same arithmetic, in the same order, as tile_body: results are bit-equal to gemm_tiled_kernel's.
//
// SPLIT (work split along K, "stream-K"): the work is counted in units of one slab of one tile, in
// tile order, and block l takes the units [l * U / G, (l + 1) * U / G): the same number for every
// block, whatever the number of tiles -- 448 tiles on 256 CUs are 1.75 tiles each instead of two
// rounds of which the second is three quarters empty.  A tile that a block boundary cuts is begun
// by block l - 1 (slabs 0 .. s - 1) and finished by block l (slabs s .. end).  The f32
// accumulators travel through the workspace, so the tile's sum is formed in the same order as by
// one block and the result stays bit-equal to the other kernels'.  A block works in the order
//     1. the tile it begins (the LAST of its range): accumulators -> workspace slot l + 1, then flag l + 1
//     2. its whole tiles
//     3. the tile it finishes (the FIRST of its range): waits for flag l, accumulators <- slot l
// so that what a block waits for is the first thing its predecessor does, and that depends on nothing:
// no block ever waits for a block that waits (with the host's rule of at least one tile per block a tile
// has at most two parts).  The hand-over crosses CUs and possibly XCDs, whose L2 caches are not coherent
// with each other: partial sums and flags are written and read with the device-scope cache policy (write
// through / miss always), the flag only after the writer's stores have completed.  Flags hold the launch's
// sequence number, so nothing has to be cleared between launches.  The wait is bounded; a block that gives
// up (its predecessor never ran: a hung GPU) poisons its tile with NaN instead of hanging too.
constexpr int kStreamkSlots = 64, kStreamkMaxBlocks = 512;
static __device__ unsigned int g_streamk_flags[kStreamkSlots * kStreamkMaxBlocks];
static __device__ unsigned int g_streamk_gave_up;   // hand-overs a block stopped waiting for (their tiles hold NaN)

// PROBE (measurement aid, results meaningless): 1 the same loop with every copy reading tile (0, 0) and slabs 0..7 over
// and over, so that the operands stay in L2, one job of K / 128 slabs per block; 2 the same without copies, waits and
// barriers -- the MFMA loop on what the prologue left in LDS.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool BLOCKSCALE, bool SPLIT, int PROBE = 0>
__device__ __forceinline__ void persist_body(const GemmArgs& p, uint8_t* smem) {
  static_assert(!(SPLIT && PROBE != 0), "the probe has no hand-over");
  constexpr int NS = 2;
  constexpr int NWAVES = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int IA = BM / 8 / NWAVES, IB = BN / 8 / NWAVES;
  constexpr int SCALE_BYTES = BLOCKSCALE ? BM * 4 : 0;
  constexpr int STAGE_BYTES = (BM + BN) * 128 + SCALE_BYTES;
  constexpr int PER = IA + IB + (BLOCKSCALE ? 1 : 0);
  constexpr int SIDE_BYTES = 16 * WN * 2;  // a wave's side buffer: 16 rows of its part of the tile
  constexpr int NSTORE = TM * 2;           // 16-byte stores per lane and tile
  constexpr int PARTIAL_BYTES = BM * BN * 4;  // the accumulators of a tile: one workspace slot
  static_assert(WN == 64 && BM % 64 == 0 && NWAVES % 2 == 0 && IA >= 1 && IB >= 1 && TN % 2 == 0, "tile / wave layout");
  static_assert(NSTORE < 64, "the count must fit the vmcnt field");

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lm = lane & 15, lq = lane >> 4;
  const int nslab = (p.K + 127) / 128;

  // ---- this block's jobs.  A job is (tile, first slab, end slab, kind): WHOLE tiles start from zero and store C;
  // a HEAD starts from zero and hands its accumulators on; a TAIL takes them over and stores C.
  enum { WHOLE = 0, HEAD = 1, TAIL = 2 };
  struct Job { int tile, s0, s1, kind; };
  const int tiles_m = p.M / BM, tiles_n = p.N / BN, total = tiles_m * tiles_n;
  const int xcd = blockIdx.x & 7;
  int njobs;
  // persistent: every 'nb'-th tile of the XCD's contiguous run (blocks are dealt to the XCDs round-robin)
  const int run_begin = xcd * (total >> 3) + (xcd < (total & 7) ? xcd : (total & 7));
  const int run_len = (total >> 3) + (xcd < (total & 7) ? 1 : 0);
  const int nb = ((int)gridDim.x - xcd + 7) >> 3;
  const int my = blockIdx.x >> 3;
  // split: logical block number l = position in XCD order, so that neighbours in l share an L2 but for 7 pairs
  const int per_xcd = (int)gridDim.x >> 3;           // (the host launches a multiple of 8 blocks)
  const int l = xcd * per_xcd + my;
  int t_first = 0, t_last = 0, s_first = 0, s_last_end = 0, nwhole = 0;
  bool has_head = false, has_tail = false;
  if constexpr (SPLIT) {
    const int64_t U = (int64_t)total * nslab, G = gridDim.x;
    const int64_t ub = (int64_t)l * U / G, ue = (int64_t)(l + 1) * U / G;
    t_first = (int)(ub / nslab);
    s_first = (int)(ub - (int64_t)t_first * nslab);
    t_last = (int)((ue - 1) / nslab);
    s_last_end = (int)(ue - (int64_t)t_last * nslab);
    has_tail = s_first != 0;
    has_head = s_last_end != nslab;
    nwhole = t_last - t_first + 1 - (has_tail ? 1 : 0) - (has_head ? 1 : 0);
    njobs = nwhole + (has_tail ? 1 : 0) + (has_head ? 1 : 0);
  } else if constexpr (PROBE != 0) {
    njobs = 1;
  } else {
    njobs = my < run_len ? (run_len - my + nb - 1) / nb : 0;
  }
  if (njobs <= 0) return;
  auto get_job = [&](int k) -> Job {
    if constexpr (SPLIT) {
      if (has_head && k == 0) return Job{t_last, 0, s_last_end, HEAD};
      const int w = k - (has_head ? 1 : 0);
      if (w < nwhole) return Job{t_first + (has_tail ? 1 : 0) + w, 0, nslab, WHOLE};
      return Job{t_first, s_first, nslab, TAIL};
    } else {
      return Job{run_begin + my + k * nb, 0, nslab, WHOLE};
    }
  };

  // ---- global -> LDS copy plan: as in tile_body, with the tile's position in the scalar offset
  const __amdgpu_buffer_rsrc_t a_rsrc = t2_rsrc(p.a, t2_clamp_u32((int64_t)(p.M - 1) * p.lda + p.K));
  const __amdgpu_buffer_rsrc_t b_rsrc = t2_rsrc(p.b, t2_clamp_u32((int64_t)(p.N - 1) * p.ldb + p.K));
  const int cr = lane >> 3, cp = lane & 7;
  const int cchunk = cp ^ cr;
  const int cchunk_b = cp ^ (((wave & 1) << 2) | (cr & 3));
  const uint32_t a_voff = (uint32_t)(wave * 8 + cr) * (uint32_t)p.lda + cchunk * 16;
  const uint32_t b_voff = (uint32_t)(wave * 8 + cr) * (uint32_t)p.ldb + cchunk_b * 16;
  const uint32_t a_istep = (uint32_t)(NWAVES * 8) * (uint32_t)p.lda;
  const uint32_t b_istep = (uint32_t)(NWAVES * 8) * (uint32_t)p.ldb;
  const int s_chunk = wave % (BM / 64);
  __amdgpu_buffer_rsrc_t s_rsrc = t2_rsrc(nullptr, 0);
  uint32_t s_voff = 0, s_slab_step = 0;
  if constexpr (BLOCKSCALE) {
    s_rsrc = t2_rsrc(p.a_scales, t2_clamp_u32(((int64_t)(nslab - 1) * p.a_scales_ld + p.M) * 4));
    s_voff = (uint32_t)scale_word_row<WM>(s_chunk * 64 + lane) * 4u;
    s_slab_step = (uint32_t)p.a_scales_ld * 4u;
  }
  struct TileAt { uint32_t a, b, s; };  // byte offsets of a tile's activation rows, weight rows and activation scales
  auto tile_at = [&](int tm, int tn) {
    if constexpr (PROBE != 0) return TileAt{0u, 0u, 0u};
    return TileAt{(uint32_t)(tm * BM) * (uint32_t)p.lda, (uint32_t)(tn * BN) * (uint32_t)p.ldb, (uint32_t)(tm * BM) * 4u};
  };
  auto dma_one = [&](const TileAt& at, int slab, int buf, int idx, uint32_t dead) {
    if constexpr (PROBE != 0) slab &= 7;
    const uint32_t koff = (uint32_t)slab * 128u;
    uint32_t kill = dead, kill_b = dead;
    if (koff + cchunk * 16 >= (uint32_t)p.K) kill = 0x80000000u;
    if (koff + cchunk_b * 16 >= (uint32_t)p.K) kill_b = 0x80000000u;
    uint8_t* sa = smem + buf * STAGE_BYTES + wave * 1024;
    uint8_t* sb = sa + BM * 128;
    if (idx < IA) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(sa + idx * NWAVES * 1024), 16, a_voff | kill,
                                               at.a + koff + idx * a_istep, 0, 0);
    } else if (idx < IA + IB) {
      const int i = idx - IA;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (lds_ptr_t)(sb + i * NWAVES * 1024), 16, b_voff | kill_b,
                                               at.b + koff + i * b_istep, 0, 0);
    } else if constexpr (BLOCKSCALE) {
      uint8_t* ss = smem + buf * STAGE_BYTES + (BM + BN) * 128 + s_chunk * 256;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(s_rsrc, (lds_ptr_t)ss, 4, s_voff | dead, at.s + (uint32_t)slab * s_slab_step, 0, 0);
    }
  };

  // ---- fragment read plan: as in tile_body
  const int sw = lm & 7;
  const uint32_t frag0 = lm * 128 + ((lq ^ sw) << 4);
  const uint32_t frag1 = lm * 128 + (((lq + 4) ^ sw) << 4);
  const uint32_t a_frag_base = (uint32_t)(wm * WM) * 128;
  const uint32_t b_frag_base = (uint32_t)(BM + wn * WN) * 128;
  auto read_frag = [&](const uint8_t* base) -> v8i {
    const v4i lo = *reinterpret_cast<const v4i*>(base + frag0);
    const v4i hi = *reinterpret_cast<const v4i*>(base + frag1);
    return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  const int wrow = 8 * (lm >> 2) + (lm & 3);
  const int wsw = (((wrow >> 3) & 1) << 2) | (wrow & 3);
  const uint32_t wfrag0 = wrow * 128 + ((lq ^ wsw) << 4);
  const uint32_t wfrag1 = wrow * 128 + (((lq + 4) ^ wsw) << 4);
  auto read_wfrag = [&](const uint8_t* base, int t) -> v8i {
    const uint8_t* g = base + (t >> 1) * 4096 + (t & 1) * 512;
    const v4i lo = *reinterpret_cast<const v4i*>(g + wfrag0);
    const v4i hi = *reinterpret_cast<const v4i*>(g + wfrag1);
    return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  const uint32_t s_rd = (uint32_t)((BM + BN) * 128) + scale_read_offset<TM>(wm * WM, lm);
  uint8_t* wbuf = smem + NS * STAGE_BYTES + wave * SIDE_BYTES;
  const int rr = lane >> 3, cc = lane & 7;
  const __amdgpu_buffer_rsrc_t c_rsrc = t2_rsrc(p.c, t2_clamp_u32(((int64_t)(p.M - 1) * p.ldc + p.N) * 2));
  const uint32_t c_row_bytes = (uint32_t)p.ldc * 2u;
  const uint32_t c_lane = (uint32_t)rr * c_row_bytes + (uint32_t)cc * 16u;

  // ---- hand-over of accumulators between blocks (SPLIT): slot i = PARTIAL_BYTES at workspace + i * PARTIAL_BYTES,
  // a wave's part at wave * (PARTIAL_BYTES / NWAVES), fragment (mt, nt) as 64 lanes x 16 bytes.  Cache policy 17 =
  // sc0 | sc1: device scope (stores go through to memory, loads do not hit a line of this XCD's L2).
  typedef unsigned int v4u __attribute__((ext_vector_type(4)));
  [[maybe_unused]] const __amdgpu_buffer_rsrc_t w_rsrc =
      SPLIT ? t2_rsrc(p.workspace, t2_clamp_u32((int64_t)gridDim.x * PARTIAL_BYTES)) : t2_rsrc(nullptr, 0);
  [[maybe_unused]] unsigned int* const flags = g_streamk_flags + (size_t)p.streamk_slot * kStreamkMaxBlocks;
  constexpr int kDeviceScope = 17;

  Job cur = get_job(0);
  int tm, tn;
  tile_coords(cur.tile, tiles_m, tiles_n, tm, tn);
  if constexpr (PROBE != 0) tm = tn = 0;
  TileAt cur_at = tile_at(tm, tn);
#pragma unroll
  for (int idx = 0; idx < PER; ++idx) dma_one(cur_at, cur.s0, 0, idx, 0u);
  if constexpr (PROBE == 2) {
#pragma unroll
    for (int idx = 0; idx < PER; ++idx) dma_one(cur_at, 1, 1, idx, 0u);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  }
  float bs_nxt = 1.f;
  if constexpr (BLOCKSCALE) bs_nxt = p.b_scales[(int64_t)((tn * BN + wn * WN) / 128) * p.b_scales_ld + cur.s0];

  // (probe: the core clock's cycle counter and the constant 100 MHz counter, around the slab loop)
  [[maybe_unused]] uint64_t probe_c0 = 0, probe_r0 = 0;
  if constexpr (PROBE != 0) {
    probe_c0 = clock64();
    probe_r0 = wall_clock64();
  }
  int buf = 0;
  bool stored = false;  // the wave's last vector memory operations are a tile's NSTORE stores
  for (int k = 0; k < njobs; ++k) {
    const bool has_next = k + 1 < njobs;
    Job nxt = cur;
    int tm2 = tm, tn2 = tn;
    if (has_next) {
      nxt = get_job(k + 1);
      tile_coords(nxt.tile, tiles_m, tiles_n, tm2, tn2);
    }
    const TileAt next_at = tile_at(tm2, tn2);
    const float* bs_row = nullptr;
    if constexpr (BLOCKSCALE) bs_row = p.b_scales + (int64_t)((tn * BN + wn * WN) / 128) * p.b_scales_ld;

    v4f acc[TM][TN];
    bool took_over = false;
    if constexpr (SPLIT) {
      if (cur.kind == TAIL) {
        // the predecessor's first job: in practice long done.  Every lane reads the same word.
        took_over = true;
        bool there = false;
        for (int spin = 0; spin < (1 << 22); ++spin) {
          if (__hip_atomic_load(flags + l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.streamk_seq) { there = true; break; }
          __builtin_amdgcn_s_sleep(16);
        }
        asm volatile("" ::: "memory");
        if (!there && tid == 0) atomicAdd(&g_streamk_gave_up, 1u);
        // (the slot's address is formed here, out of sight of the optimiser: hoisted out of the job loop, the 32
        // fragment offsets would sit in scalar registers for the whole kernel)
        uint32_t base = (uint32_t)l * PARTIAL_BYTES + (uint32_t)wave * (PARTIAL_BYTES / NWAVES);
        asm volatile("" : "+s"(base));
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const v4u v = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (uint32_t)lane * 16u, base + (uint32_t)(i * TN + j) * 1024u, kDeviceScope);
            acc[i][j] = there ? v4f{__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)}
                              : v4f{__builtin_nanf(""), __builtin_nanf(""), __builtin_nanf(""), __builtin_nanf("")};
          }
      }
    }
    if (!took_over) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
    }

    for (int slab = cur.s0; slab < cur.s1; ++slab) {
      if constexpr (PROBE != 2) {
        if (slab == cur.s0 && stored && !took_over) {
          asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NSTORE) : "memory");
        } else {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
      }
      const float bs = bs_nxt;
      if constexpr (BLOCKSCALE) {
        if (slab + 1 < cur.s1) bs_nxt = bs_row[PROBE != 0 ? ((slab + 1) & 7) : slab + 1];
      }
      asm volatile("" ::: "memory");
      // the copy issued during this slab: the job's next slab, or the first slab of the next job
      const bool last = slab + 1 == cur.s1;
      const uint32_t dead = (last && !has_next) ? 0x80000000u : 0u;
      const TileAt dat = last ? next_at : cur_at;
      const int dma_slab = last ? nxt.s0 : slab + 1, dma_buf = buf ^ 1;
      constexpr int SPREAD = TM >= 4 ? TM / 2 : TM;

      const uint8_t* sa = smem + buf * STAGE_BYTES;
      float s_cur[TM];
      if constexpr (BLOCKSCALE) {
const ScaleRow<TM> a_sc = read_scales<TM>(sa + s_rd);
        #pragma unroll
        for (int mt = 0; mt < TM; ++mt) s_cur[mt] = a_sc[mt] * bs;
      }
      v8i bf[TN];
#pragma unroll
      for (int t = 0; t < TN; ++t) bf[t] = read_wfrag(sa + b_frag_base, t);
      v8i af = read_frag(sa + a_frag_base);
      [[maybe_unused]] v4f part[2][TN];
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
        v8i af_next = af;
        if (mt + 1 < TM) af_next = read_frag(sa + a_frag_base + (mt + 1) * 2048);
        if constexpr (BLOCKSCALE) {
          const v4f zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int nt = 0; nt < TN; ++nt)
            part[mt & 1][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[nt], af, zero, 0, 0, 0, 0, 0, 0);
          // Issue order, pinned: one MFMA of this group, then four promotions of the previous one, four times.
          // (Left to itself the scheduler put each group's promotions straight behind its own MFMAs and
          // filled the wait with idle cycles.)
          if (mt > 0) {
#pragma unroll
            for (int nt = 0; nt < TN; ++nt) {
              __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
              __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // VALU
            }
          } else {
            __builtin_amdgcn_sched_group_barrier(0x008, TN, 0);
          }
          if (mt > 0) {
#pragma unroll
            for (int nt = 0; nt < TN; ++nt) acc[mt - 1][nt] += part[(mt - 1) & 1][nt] * s_cur[mt - 1];
          }
          if (mt == TM - 1) {
#pragma unroll
            for (int nt = 0; nt < TN; ++nt) acc[mt][nt] += part[mt & 1][nt] * s_cur[mt];
          }
        } else {
#pragma unroll
          for (int nt = 0; nt < TN; ++nt)
            acc[mt][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[nt], af, acc[mt][nt], 0, 0, 0, 0, 0, 0);
        }
        af = af_next;
        if constexpr (PROBE != 2) {
#pragma unroll
          for (int idx = 0; idx < PER; ++idx)
            if (idx * SPREAD / PER == mt) dma_one(dat, dma_slab, dma_buf, idx, dead);
        }
      }
      buf ^= 1;
    }
    if constexpr (PROBE != 0) {
      if (p.workspace != nullptr && tid == 0) {
        uint64_t* out = reinterpret_cast<uint64_t*>(p.workspace) + 2 * blockIdx.x;
        out[0] = clock64() - probe_c0;
        out[1] = wall_clock64() - probe_r0;
      }
    }
    // the first weight-block scale of the next job travels while this one is stored
    if constexpr (BLOCKSCALE) bs_nxt = p.b_scales[(int64_t)((tn2 * BN + wn * WN) / 128) * p.b_scales_ld + nxt.s0];

    bool handed_on = false;
    if constexpr (SPLIT) {
      if (cur.kind == HEAD) {
        // ---- the accumulators go to the successor's slot; the flag follows once every wave's stores have completed
        handed_on = true;
        uint32_t base = (uint32_t)(l + 1) * PARTIAL_BYTES + (uint32_t)wave * (PARTIAL_BYTES / NWAVES);
        asm volatile("" : "+s"(base));
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const v4f a4 = acc[i][j];
            const v4u v = {__float_as_uint(a4[0]), __float_as_uint(a4[1]), __float_as_uint(a4[2]), __float_as_uint(a4[3])};
            buffer_store_b128_guarded<kDeviceScope>(v, w_rsrc, (uint32_t)lane * 16u, base + (uint32_t)(i * TN + j) * 1024u);
          }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        if (tid == 0) __hip_atomic_store(flags + l + 1, p.streamk_seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        stored = false;
      }
    }
    if (!handed_on) {
      // ---- the tile leaves, 16 rows of the wave's part at a time
      // (row scaling: every scale of the tile is loaded before the first store, so that no later wait for a
      // load also waits for the stores in front of it)
      float b_s[TN / 2][8], a_s_all[TM];
      if constexpr (!BLOCKSCALE) {
#pragma unroll
        for (int q = 0; q < TN / 2; ++q)
#pragma unroll
          for (int i = 0; i < 8; ++i)
            b_s[q][i] = scale_at(p.b_scales, (int64_t)(tn * BN + wn * WN + q * 32 + lq * 8 + i) * p.b_scale_stride, p.scales_dtype);
#pragma unroll
        for (int mt = 0; mt < TM; ++mt)
          a_s_all[mt] = scale_at(p.a_scales, ((int64_t)tm * BM + wm * WM + mt * 16 + lm) * p.a_scale_stride, p.scales_dtype);
        asm volatile("" ::: "memory");
      }
      // (C goes out through a buffer descriptor: one 32-bit lane offset for all of a lane's stores, the rest scalar)
      const uint32_t c_tile = ((uint32_t)(tm * BM + wm * WM) * (uint32_t)p.ldc + (uint32_t)(tn * BN + wn * WN)) * 2u;
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
        float a_s = 1.f;
        if constexpr (!BLOCKSCALE) a_s = a_s_all[mt];
#pragma unroll
        for (int q = 0; q < TN / 2; ++q) {
          v4f lo = acc[mt][2 * q], hi = acc[mt][2 * q + 1];
          if constexpr (!BLOCKSCALE) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float t_lo = lo[i] * a_s, t_hi = hi[i] * a_s;
              lo[i] = t_lo * b_s[q][i];
              hi[i] = t_hi * b_s[q][4 + i];
            }
          }
          // (written and read back through the same vector type: to the compiler a store through one type and a load
          // through another need not alias, and it may then move the load in front of the store)
          *reinterpret_cast<v4u*>(wbuf + lm * (WN * 2) + (((q * 4 + lq) ^ (lm & 7)) * 16)) =
              v4u{pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]), pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3])};
        }
        // (a wave reads back only what it wrote itself, and its LDS operations execute in order)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int r = i * 8 + rr;
          const v4u v = *reinterpret_cast<const v4u*>(wbuf + r * (WN * 2) + ((cc ^ (r & 7)) * 16));
          // (non-temporal: C is not read again here, and its lines should not push the operands out of L2)
          buffer_store_b128_guarded<2>(v, c_rsrc, c_lane, c_tile + (uint32_t)(mt * 16 + i * 8) * c_row_bytes);
        }
      }
      stored = true;
    }
    cur = nxt;
    tm = tm2;
    tn = tn2;
    cur_at = next_at;
  }
  // the last copies (of nothing: every lane out of range) still write zeros into the stages: they
  // must have landed before the block's LDS goes to another block
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool BLOCKSCALE>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, 1) void gemm_persist_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  persist_body<BM, BN, WAVES_M, WAVES_N, BLOCKSCALE, false>(p, smem);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool BLOCKSCALE, int PROBE>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, 1) void gemm_persist_probe_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  persist_body<BM, BN, WAVES_M, WAVES_N, BLOCKSCALE, false, PROBE>(p, smem);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool BLOCKSCALE>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, 1) void gemm_streamk_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  persist_body<BM, BN, WAVES_M, WAVES_N, BLOCKSCALE, true>(p, smem);
}

// ---- grouped (MoE) matmul ---------------------------------------------------------------------
// Slot z owns rows [offsets[z], offsets[z+1]).  blockIdx.y counts row tiles over all slots,
// blockIdx.x is the column tile; a block finds its (slot, tile) with a block-wide prefix sum of
// tiles_of(slot) over the device-resident offsets: no host synchronisation, no list of tiles.
// Rows [begin, end) of slot z, held inside [0, M): the activations, their scales and C have M rows, so offsets
// beyond that (a stale or damaged routing tensor) must not turn into accesses outside them.
__device__ __forceinline__ void grouped_slot_rows(const GemmArgs& p, int z, int64_t& begin, int64_t& end) {
  const int64_t M = p.M, b = p.offsets[z], e = p.offsets[z + 1];
  begin = b < M ? b : M;
  end = e < M ? e : M;
  if (end < begin) end = begin;
}
__device__ __forceinline__ int grouped_slot_count(const GemmArgs& p, int z) {
  int64_t b, e;
  grouped_slot_rows(p, z, b, e);
  return (int)(e - b);
}

template <int NWAVES, typename TilesOf>
__device__ __forceinline__ bool grouped_find_tile(const GemmArgs& p, const int by, TilesOf tiles_of, int& slot, int& tile) {
  constexpr int NTHREADS = NWAVES * 64;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  __shared__ int s_slot, s_tile, s_wave_sum[NWAVES], s_carry;
  if (tid == 0) { s_slot = -1; s_tile = 0; s_carry = 0; }
  __syncthreads();
  for (int z0 = 0; z0 < p.num_active; z0 += NTHREADS) {
    const int z = z0 + tid;
    int t = 0;
    if (z < p.num_active) t = tiles_of(grouped_slot_count(p, z));
    int incl = t;
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
    if (t > 0 && by >= excl && by < excl + t) { s_slot = z; s_tile = by - excl; }
    __syncthreads();
    if (tid == NTHREADS - 1) s_carry = before + incl;
    __syncthreads();
    if (s_slot >= 0 || by < s_carry) break;
  }
  slot = s_slot;
  tile = s_tile;
  return slot >= 0;
}

// a slot without an expert (id -1) writes zeros
template <int NTHREADS>
__device__ __forceinline__ void grouped_zero_tile(const GemmArgs& p, int64_t row_begin, int rows_here, int n0, int bn) {
  const int cols_here = (p.N - n0) < bn ? (p.N - n0) : bn;
  for (int i = threadIdx.x; i < rows_here * cols_here; i += NTHREADS) {
    int64_t m = row_begin + i / cols_here;
    if (p.c_row_index) m = p.c_row_index[m];
    const int n = n0 + i % cols_here;
    if (p.c_dtype == MAXFP8_BF16) reinterpret_cast<uint16_t*>(p.c)[m * p.ldc + n] = 0;
    else reinterpret_cast<float*>(p.c)[m * p.ldc + n] = 0.f;
  }
}

// rows of a slot that the large-tile launch takes: the full big_bm-row tiles of slots with at
// least big_rows rows
__device__ __forceinline__ int grouped_head_rows(const GemmArgs& p, int rows) {
  return (p.big_rows > 0 && rows >= p.big_rows) ? (rows / p.big_bm) * p.big_bm : 0;
}

// The rows the large-tile launch leaves: BM-row tiles, and one SBM-row tile with one more LDS stage
// for what is at most small_rows (<= SBM) rows (such tiles only stream weights, so what they need is bytes in
// flight).
template <int BM, int BN, int WAVES_M, int WAVES_N, int NS, int SBM, int SWAVES_M, int SWAVES_N, int SNS, bool BLOCKSCALE = true>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, (WAVES_M * WAVES_N <= 4) ? 2 : 1) void gemm_grouped_kernel(GemmArgs p) {
  static_assert(WAVES_M * WAVES_N == SWAVES_M * SWAVES_N, "both tile kinds run on the same block");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  constexpr int NWAVES = WAVES_M * WAVES_N;
  int slot, tile;
  const int by = blockIdx.y, bx = blockIdx.x;
  const bool found = grouped_find_tile<NWAVES>(p, by, [&](int rows_total) {
    const int rows = rows_total - grouped_head_rows(p, rows_total);
    return rows <= p.small_rows ? (rows > 0 ? 1 : 0) : (rows + BM - 1) / BM;
  }, slot, tile);
  if (!found) return;
  int64_t slot_begin, row_end;
  grouped_slot_rows(p, slot, slot_begin, row_end);
  const int64_t rest_begin = slot_begin + grouped_head_rows(p, (int)(row_end - slot_begin));
  const int64_t row_begin = rest_begin + (int64_t)tile * BM;
  const bool small = row_end - row_begin <= p.small_rows;  // also the last tile of a longer slot, when few rows are left for it
  const int n0 = bx * BN;
  const int e = p.expert_ids[slot];
  if (e < 0) {
    grouped_zero_tile<NWAVES * 64>(p, row_begin, (int)((row_end - row_begin) < BM ? (row_end - row_begin) : BM), n0, BN);
    return;
  }
  const uint8_t* bptr = p.b + (int64_t)e * p.b_expert_stride;
  const float* bs_ptr = p.b_scales + (int64_t)e * p.bs_expert_stride;
  if (small) tile_body<SBM, BN, SWAVES_M, SWAVES_N, SNS, BLOCKSCALE, true>(p, smem, row_begin, row_end, n0, bptr, bs_ptr);
  else tile_body<BM, BN, WAVES_M, WAVES_N, NS, BLOCKSCALE, true>(p, smem, row_begin, row_end, n0, bptr, bs_ptr);
}

// The full BM-row tiles (BM == big_bm) of the slots with at least big_rows rows.
//
// Two launch forms.  One block per tile: grid (column tiles, upper bound of row tiles).  Or, with
// p.big_tile_rows > 0, a one-dimensional grid of at most one block per CU whose blocks walk the same
// (row tile, column tile) pairs with the grid's stride, so that this launch and gemm_grouped_kernel,
// sent down another stream, share the chip: these tiles are bound by the matrix pipe, most of the
// other launch's by HBM, and a block of this kernel fills a CU's LDS, so the two never share a CU.
// How many blocks stay is decided on the device, where the group sizes are: every block adds up the
// work of both launches (tiles x the per-tile costs of the host's cost model) and the blocks past this
// launch's share of the chip exit at once, leaving their CUs to the other launch.
template <int BM, int BN, int WAVES_M, int WAVES_N, int NS, bool BLOCKSCALE = true>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, 1) void gemm_grouped_large_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  constexpr int NWAVES = WAVES_M * WAVES_N;
  const int ncol = (p.N + BN - 1) / BN;
  int first = blockIdx.y * ncol + blockIdx.x, stride = 0, last = first + 1;
  if (p.big_tile_rows > 0) {
    __shared__ int s_big, s_mid, s_tiny;
    if (threadIdx.x == 0) { s_big = 0; s_mid = 0; s_tiny = 0; }
    __syncthreads();
    int big = 0, mid = 0, tiny = 0;
    for (int z = threadIdx.x; z < p.num_active; z += NWAVES * 64) {
      const int rows = grouped_slot_count(p, z);
      const int head = grouped_head_rows(p, rows), rest = rows - head;
      big += head / BM;
      if (rest > p.small_rows) mid += (rest + 127) / 128;
      else if (rest > 0) tiny += 1;
    }
    if (big) atomicAdd(&s_big, big);
    if (mid) atomicAdd(&s_mid, mid);
    if (tiny) atomicAdd(&s_tiny, tiny);
    __syncthreads();
    const float nslab = (float)((p.K + 127) / 128), ncol_small = (float)((p.N + 127) / 128);
    const float w_big = (float)s_big * (float)ncol * (nslab * 1.63f + 11.4f);
    // (two of the other launch's blocks share a CU; tiles of at most small_rows rows only stream their weights)
    const float w_rest = p.share_bias * 0.5f * ncol_small * ((float)s_mid * (nslab * 0.96f + 11.4f) + (float)s_tiny * (nslab * 0.5f + 6.0f));
    int keep = (int)((float)gridDim.x * w_big / (w_big + w_rest + 1e-9f) + 0.5f);
    keep = keep < 8 ? 8 : keep;
    keep = (keep + 7) & ~7;  // whole rounds of the 8 XCDs
    if (keep > (int)gridDim.x) keep = (int)gridDim.x;
    if ((int)blockIdx.x >= keep) return;
    first = blockIdx.x;
    stride = keep;
    last = p.big_tile_rows * ncol;
  }
  for (int t = first; t < last; t += stride) {
    if (stride) __syncthreads();  // every wave is done with the last tile's LDS (and with the tile search's variables)
    const int by = t / ncol, bx = t - by * ncol;
    int slot, tile;
    if (!grouped_find_tile<NWAVES>(p, by, [&](int rows_total) { return grouped_head_rows(p, rows_total) / BM; }, slot, tile)) return;
    int64_t slot_begin, slot_end;
    grouped_slot_rows(p, slot, slot_begin, slot_end);
    const int64_t row_begin = slot_begin + (int64_t)tile * BM;  // (a full tile of the slot: row_begin + BM <= slot_end <= M)
    const int n0 = bx * BN;
    const int e = p.expert_ids[slot];
    if (e < 0) {
      grouped_zero_tile<NWAVES * 64>(p, row_begin, BM, n0, BN);
    } else {
      tile_body<BM, BN, WAVES_M, WAVES_N, NS, BLOCKSCALE, true>(p, smem, row_begin, row_begin + BM, n0, p.b + (int64_t)e * p.b_expert_stride,
                                                                 p.b_scales + (int64_t)e * p.bs_expert_stride);
    }
    if (!stride) return;
  }
}

// ---- grouped matmul as one persistent launch ---------------------------------------------------
// One block of 8 waves per CU takes tiles of four kinds from four counters in device memory until all are gone:
//   L   every full 256-row tile of a slot with at least big_rows rows           256 x 256, 2 stages (matrix-pipe bound)
//   M2  a rest of 129 ... 255 rows                                               256 x 128, 3 stages
//   M1  a rest of small_rows + 1 ... 128 rows                                    128 x 256, 3 stages
//   S   a rest of at most small_rows (<= 32) rows                                512 weight rows streamed through eight
//       rings of 16 KB, one per wave, 64 rows each (HBM bound: 128 KB in flight per CU, no barrier)
// A CU holds one kind at a time -- the L and M tiles fill its registers and LDS, the S rings its LDS -- so the chip is
// shared out by CUs: the first blocks start with the S tiles and go on to M1, M2 and L when none are left, the others
// take L, M2, M1, S.  How many start with S follows from the device-resident group sizes and the per-tile times below;
// whichever kind runs out first, its blocks move on, so the estimate only has to be roughly right.  While both are busy
// the S blocks stream weights at the rate their rings allow and the other CUs keep the matrix pipes busy, instead of
// the two kinds taking turns on the whole chip.
//
// Every block builds the same four prefix tables over the slots in LDS (row tiles of each kind before slot z); a
// claimed index is a (row tile, column tile) pair, column tiles fastest, found by bisection.  No list of tiles in
// memory, no host synchronisation.  The result of a tile does not depend on which block computes it.
constexpr int kGroupedCtrSlots = 64;      // sets handed to launches that run when they are issued ...
constexpr int kGroupedCtrSlotsAll = 128;  // ... and as many again for launches recorded into a HIP graph
constexpr int kGroupedMaxSlots = 512;   // slots (active experts) the LDS tables hold
// Per launch in flight: a counter per (kind, XCD) and one that counts the blocks that are done.  All zero when the
// module is loaded; the last block of a launch to finish puts its set back to zero, so a set is clean whenever a
// launch takes it (sets are handed out round-robin: 64 grouped matmuls are never in flight together).
constexpr int kGroupedCtrStride = 33;
static __device__ unsigned int g_grouped_ctr[kGroupedCtrSlotsAll * kGroupedCtrStride];

// One wave: C[rows of the slot, 16 * NTW weight rows from n0 + 16 * NTW * wave] over the whole of K.  The weight slabs
// (16 * NTW rows x 128 bytes) travel by LDS-DMA through the wave's own ring of DEPTH slots, the activations (at most
// 16 * MT rows, read by every wave of the chip that works on this slot: L1 / L2 hits) and the scales straight to
// registers; wait counts are exact because every slot always carries PER instructions (slabs past the end are issued
// out of range).
template <int MT, int NTW, int DEPTH, bool BLOCKSCALE>
__device__ __forceinline__ void grouped_stream_body(const GemmArgs& p, uint8_t* smem, const int64_t row_begin, const int rows_here,
                                                    const int n0, const uint8_t* bptr, const float* bs_ptr) {
  constexpr int SLOT = NTW * 2048, PER = 2 * MT + (BLOCKSCALE ? MT + 1 : 0) + 2 * NTW;
  static_assert((DEPTH - 1) * PER < 64, "vmcnt is a 6-bit counter");
  static_assert(!BLOCKSCALE || 128 % (16 * NTW) == 0, "a wave's weight rows must sit inside one 128-row scale block");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lm = lane & 15, lq = lane >> 4;
  const int nw = n0 + wave * (16 * NTW);
  if (nw >= p.N) return;  // (wave-uniform; the body has no barrier)
  const int wrows = (p.N - nw) < 16 * NTW ? (p.N - nw) : 16 * NTW;
  const __amdgpu_buffer_rsrc_t b_rsrc = t2_rsrc(bptr + (int64_t)nw * p.ldb, t2_clamp_u32((int64_t)(wrows - 1) * p.ldb + p.K));
  const __amdgpu_buffer_rsrc_t a_rsrc = t2_rsrc(p.a + row_begin * p.lda, t2_clamp_u32((int64_t)(rows_here - 1) * p.lda + p.K));
  const int nslab = (p.K + 127) / 128;
  const bool k_tail = (p.K & 127) != 0;
  const int cr = lane >> 3, cp = lane & 7;
  const int cchunk = cp ^ cr;
  const uint32_t w_voff = (uint32_t)cr * (uint32_t)p.ldb + cchunk * 16;
  const uint32_t w_half = 8u * (uint32_t)p.ldb, w_tile = 16u * (uint32_t)p.ldb;
  uint32_t a_off[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) a_off[t] = (uint32_t)(t * 16 + lm) * (uint32_t)p.lda + lq * 16;
  const uint32_t frag0 = lm * 128 + ((lq ^ (lm & 7)) << 4);
  const uint32_t frag1 = lm * 128 + (((lq + 4) ^ (lm & 7)) << 4);
  uint8_t* ring = smem + wave * (DEPTH * SLOT);

  __amdgpu_buffer_rsrc_t as_rsrc = t2_rsrc(nullptr, 0), bs_rsrc = t2_rsrc(nullptr, 0);
  uint32_t as_voff[MT];
  if constexpr (BLOCKSCALE) {
    as_rsrc = t2_rsrc(p.a_scales + row_begin, t2_clamp_u32(((int64_t)(nslab - 1) * p.a_scales_ld + rows_here) * 4));
    bs_rsrc = t2_rsrc(bs_ptr + (int64_t)(nw / 128) * p.b_scales_ld, (uint32_t)nslab * 4u);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = t * 16 + lm;
      as_voff[t] = (uint32_t)(m < rows_here ? m : rows_here - 1) * 4u;
    }
  }
  v4f acc[MT][NTW];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NTW; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
  v8i af[DEPTH][MT];
  float as_v[DEPTH][MT], bs_v[DEPTH];

  auto load16 = [&](__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
  };
  auto issue = [&](int slab, auto d_c) {
    constexpr int d = decltype(d_c)::value;
    const bool live = slab < nslab;
    const int sl = live ? slab : 0;
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
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const v4i lo = load16(a_rsrc, a_off[t] | kill0, koff);
      const v4i hi = load16(a_rsrc, a_off[t] | kill1, koff_hi);
      af[d][t] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
    if constexpr (BLOCKSCALE) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
        as_v[d][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(as_rsrc, as_voff[t], (uint32_t)sl * (uint32_t)p.a_scales_ld * 4u, 0));
      bs_v[d] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(bs_rsrc, 0, (uint32_t)sl * 4u, 0));
    }
    uint8_t* slot = ring + d * SLOT;
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (lds_ptr_t)(slot + t * 2048), 16, w_voff | killw, koff + t * w_tile, 0, kStreamOnce);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (lds_ptr_t)(slot + t * 2048 + 1024), 16, w_voff | killw, koff + t * w_tile + w_half, 0, kStreamOnce);
    }
  };
  auto compute = [&](auto d_c) {
    constexpr int d = decltype(d_c)::value;
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 1) * PER) : "memory");
    const uint8_t* slot = ring + d * SLOT;
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
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the fragments have left LDS before the slot is refilled
  };
  static_for<DEPTH>([&](auto d_c) { issue(decltype(d_c)::value, d_c); });
  for (int base = 0; base < nslab; base += DEPTH) {
    static_for<DEPTH>([&](auto d_c) {
      compute(d_c);
      issue(base + DEPTH + decltype(d_c)::value, d_c);
    });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the last issues were out of range, but they still target the ring

  // lane (lm, lq) holds rows 4 * lq .. + 3 of a 16-row weight group for token lm: four consecutive columns of C
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int ml = mt * 16 + lm;
    if (ml >= rows_here) continue;
    const int64_t m = row_begin + ml;
    const int64_t cm = p.c_row_index ? (int64_t)p.c_row_index[m] : m;
    float a_s = 1.f;
    if constexpr (!BLOCKSCALE) a_s = scale_at(p.a_scales, m * p.a_scale_stride, p.scales_dtype);
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
      const int n = nw + nt * 16 + lq * 4;
      if (n >= p.N) continue;
      float v[4] = {acc[mt][nt][0], acc[mt][nt][1], acc[mt][nt][2], acc[mt][nt][3]};
      if constexpr (!BLOCKSCALE) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int nn = (n + i < p.N) ? n + i : p.N - 1;
          const float t = v[i] * a_s;
          v[i] = t * scale_at(bs_ptr, (int64_t)nn * p.b_scale_stride, p.scales_dtype);
        }
      }
      if (p.c_dtype == MAXFP8_BF16) {
        uint16_t* dst = reinterpret_cast<uint16_t*>(p.c) + cm * p.ldc + n;
        if (p.c_vec_ok && n + 3 < p.N) {
          *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < p.N) dst[i] = (uint16_t)f32_to_bf16_bits(v[i]);
        }
      } else {
        float* dst = reinterpret_cast<float*>(p.c) + cm * p.ldc + n;
        if (p.c_vec_ok && n + 3 < p.N) {
          *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < p.N) dst[i] = v[i];
        }
      }
    }
  }
}

// LDS of the persistent grouped kernel: the largest tile body (256 x 128, 3 stages), then the four prefix tables
template <bool BLOCKSCALE>
constexpr int grouped_persist_table_offset() { return 3 * ((256 + 128) * 128 + (BLOCKSCALE ? 256 * 4 : 0)); }

template <bool BLOCKSCALE>
__global__ __launch_bounds__(512, 1) void gemm_grouped_persist_kernel(GemmArgs p_arg, int ctr_slot) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  constexpr int NTHREADS = 512, S_COLS = 8 * 64, TS = kGroupedMaxSlots + 1;
  const int tid = threadIdx.x;
  // prefix tables: row tiles of each kind in the slots before z (kinds 0 = L, 1 = M2, 2 = M1, 3 = S)
  int* tab = reinterpret_cast<int*>(smem + grouped_persist_table_offset<BLOCKSCALE>());
  // Everything a block keeps from tile to tile lives in LDS, and the arguments are read again from the kernel's
  // argument segment for every tile (a handful of scalar loads): values held in scalar registers across the tile
  // bodies would push the bodies' own loop values out of the register file.
  __shared__ int s_rt[4], s_ncol[4], s_step, s_sfirst, s_kind, s_t, s_xcd;
  {
    const GemmArgs& p = p_arg;
    const int na = p.num_active;
    // thread z counts slot z's row tiles of each kind; a block-wide exclusive scan makes the tables
    static_assert(kGroupedMaxSlots == NTHREADS, "one slot per thread");
    const int lane = tid & 63, wave = tid >> 6;
    int c[4] = {0, 0, 0, 0};
    if (tid < na) {
      const int rows = grouped_slot_count(p, tid);
      const int head = p.heads_elsewhere ? w4_grouped_head_rows(rows, p.w4_hot_rest, p.w4_cold_rows) : grouped_head_rows(p, rows), rest = rows - head;
      c[0] = p.heads_elsewhere ? 0 : head / 256;
      if (rest > 256) c[1] = (rest + 255) / 256;        // (slots below big_rows keep all their rows here)
      else if (rest > 128) c[1] = 1;
      else if (rest > p.small_rows) c[2] = 1;
      else if (rest > 0) c[3] = 1;
    }
    __shared__ int s_wsum[4][8];
    int incl[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      incl[k] = c[k];
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(incl[k], o, 64);
        if (lane >= o) incl[k] += up;
      }
      if (lane == 63) s_wsum[k][wave] = incl[k];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      int before = 0;
      for (int w = 0; w < wave; ++w) before += s_wsum[k][w];
      if (tid < na) tab[k * TS + tid] = before + incl[k] - c[k];
      if (tid == NTHREADS - 1) tab[k * TS + na] = before + incl[k];  // (threads past the last slot add nothing)
    }
    __syncthreads();
    if (tid == 0) {
      const int ncol[4] = {(p.N + 255) / 256, (p.N + 127) / 128, (p.N + 255) / 256, (p.N + S_COLS - 1) / S_COLS};
      int cnt[4];
      for (int k = 0; k < 4; ++k) {
        cnt[k] = tab[k * TS + na];
        s_rt[k] = cnt[k];
        s_ncol[k] = ncol[k];
      }
      // the share of the blocks that starts with the S tiles: their work / all work, in microseconds of one CU
      const float nslab = (float)((p.K + 127) / 128);
      const float w_mm = (float)(cnt[0] * ncol[0]) * (nslab * 1.63f + 11.4f) +
                         (float)(cnt[1] * ncol[1] + cnt[2] * ncol[2]) * (nslab * 0.92f + 9.0f);
      const float w_s = (float)(cnt[3] * ncol[3]) * (nslab * 2.6f + 6.0f) * p.share_bias;
      int first_s = cnt[3] > 0 ? (int)((float)gridDim.x * w_s / (w_mm + w_s + 1e-9f) + 0.5f) : 0;
      if (cnt[3] > 0 && first_s < 1) first_s = 1;
      s_sfirst = (int)blockIdx.x < first_s ? 1 : 0;
      s_step = 0;
    }
  }
  typedef const __attribute__((address_space(4))) GemmArgs* kernarg_ptr_t;
  kernarg_ptr_t pk = (kernarg_ptr_t)__builtin_amdgcn_kernarg_segment_ptr();  // (the argument block is the first argument)
  while (true) {
    __syncthreads();  // every wave is done with the last tile's LDS and with the claim; the first time: the tables are there
    if (tid < 64) {
      // Column tile c of every kind belongs to XCD c % 8 (blocks go to the XCDs round-robin): the weight tiles an XCD
      // works on stay in its L2 from one row tile to the next, and the eight XCDs read an activation row tile at about
      // the same time.  One counter per kind and XCD; a block whose own XCD has nothing left of a kind helps the others
      // before it moves on to the next kind.  `step` only grows: the 32 (kind, XCD) pairs come in this block's order.
      // A claim that comes back empty costs a trip to memory (the counters are shared by the eight L2s), and by the
      // end every pair is empty: after the first empty claim the wave reads all 32 counters at once, lane l that of
      // pair l, and goes straight to the next pair that still had tiles -- one trip instead of one per empty pair
      // (a launch of one L tile per CU spent 21 of its 45 us on the seven empty claims at its end).
      unsigned int* ctr = g_grouped_ctr + ctr_slot * kGroupedCtrStride;
      const int my_xcd = (int)(blockIdx.x & 7);
      const int sfirst = s_sfirst;
      auto pair_of = [&](int st, int& k, int& x, int& total) {
        k = sfirst ? 3 - (st >> 3) : (st >> 3);
        x = (my_xcd + (st & 7)) & 7;
        const int cols_x = x < s_ncol[k] ? (s_ncol[k] - x + 7) >> 3 : 0;
        total = s_rt[k] * cols_x;
      };
      int kind = -1, t = 0, xcd = 0, step = s_step;
      while (step < 32) {
        int k, x, total;
        pair_of(step, k, x, total);
        if (total > 0) {
          if (tid == 0) t = (int)atomicAdd(ctr + k * 8 + x, 1u);
          t = __builtin_amdgcn_readfirstlane(t);
          if (t < total) { kind = k; xcd = x; break; }
          int kl, xl, total_l, pair_l = tid & 31;
          asm volatile("" : "+v"(pair_l));  // (worked out here, where it is needed: not kept in registers across the tile bodies)
          pair_of(pair_l, kl, xl, total_l);
          unsigned int seen = 0xffffffffu;
          if (tid < 32 && tid > step && total_l > 0) seen = __hip_atomic_load(ctr + kl * 8 + xl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          const unsigned long long open = __ballot(seen < (unsigned int)total_l);
          step = open ? __builtin_ctzll(open) : 32;
        } else {
          ++step;
        }
      }
      if (tid == 0) { s_step = step; s_kind = kind; s_t = t; s_xcd = xcd; }
    }
    __syncthreads();
    const int kind = s_kind, t = s_t, xcd = s_xcd;
    if (kind < 0) {
      // nothing left for this block (nor, by then, for any block that arrives here): the last one cleans the counters
      if (tid == 0) {
        unsigned int* ctr = g_grouped_ctr + ctr_slot * kGroupedCtrStride;
        if (atomicAdd(ctr + 32, 1u) == gridDim.x - 1) {
          for (int i = 0; i < kGroupedCtrStride; ++i) atomicExch(ctr + i, 0u);
        }
      }
      break;
    }
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+s"(pk));
    GemmArgs p = *pk;
#else
    GemmArgs p = p_arg;  // (the host pass only parses this function)
#endif
    const int na = p.num_active;
    const int* tb = tab + kind * TS;
    const int cols_x = (s_ncol[kind] - xcd + 7) >> 3;
    const int rt = t / cols_x, col = xcd + 8 * (t - rt * cols_x);
    // the slot whose tiles hold row tile rt: the last z with tb[z] <= rt (slots without tiles of this kind repeat
    // their successor's value and are skipped by taking the last)
    int lo = 0, hi = na;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (tb[mid] <= rt) lo = mid; else hi = mid;
    }
    const int slot = lo, tile = rt - tb[lo];
    int64_t slot_begin, slot_end;
    grouped_slot_rows(p, slot, slot_begin, slot_end);
    const int head = p.heads_elsewhere ? w4_grouped_head_rows((int)(slot_end - slot_begin), p.w4_hot_rest, p.w4_cold_rows) : grouped_head_rows(p, (int)(slot_end - slot_begin));
    const int64_t row_begin = kind == 0 ? slot_begin + (int64_t)tile * 256 : slot_begin + head + (int64_t)tile * 256;
    const int64_t row_end = kind == 0 ? row_begin + 256 : slot_end;
    const int bn = kind == 1 ? 128 : (kind == 3 ? S_COLS : 256);
    const int n0 = col * bn;
    const int64_t left = row_end - row_begin;
    const int rows_here = (int)(left < 256 ? left : 256);
    const int e = p.expert_ids[slot];
    if (e < 0) {
      grouped_zero_tile<NTHREADS>(p, row_begin, rows_here, n0, bn);
      continue;
    }
    const uint8_t* bptr = p.b + (int64_t)e * p.b_expert_stride;
    const float* bs_ptr = p.b_scales + (int64_t)e * p.bs_expert_stride;
    if (kind == 0) {
      tile_body<256, 256, 2, 4, 2, BLOCKSCALE, true>(p, smem, row_begin, row_end, n0, bptr, bs_ptr);
    } else if (kind == 1) {
      // (a rest of at most 192 rows: three quarters of the MFMAs)
      // (a slot's rest is one row tile: its weights are read once, as the S tiles' are)
      if (rows_here <= 192) tile_body<192, 128, 2, 4, 3, BLOCKSCALE, true, false, kStreamOnce>(p, smem, row_begin, row_end, n0, bptr, bs_ptr);
      else tile_body<256, 128, 4, 2, 3, BLOCKSCALE, true, false, kStreamOnce>(p, smem, row_begin, row_end, n0, bptr, bs_ptr);
    } else if (kind == 2) {
      tile_body<128, 256, 2, 4, 3, BLOCKSCALE, true, false, kStreamOnce>(p, smem, row_begin, row_end, n0, bptr, bs_ptr);
    } else {
      if (rows_here <= 16) grouped_stream_body<1, 4, 2, BLOCKSCALE>(p, smem, row_begin, rows_here, n0, bptr, bs_ptr);
      else grouped_stream_body<2, 4, 2, BLOCKSCALE>(p, smem, row_begin, rows_here, n0, bptr, bs_ptr);
    }
  }
}

template <int BM, int BN, int NS, bool BLOCKSCALE>
constexpr int tile_lds_bytes() {
  return NS * ((BM + BN) * 128 + (BLOCKSCALE ? (BM < 64 ? 64 : BM) * 4 : 0));
}

template <typename Kern>
static int launch_with_lds(Kern kern, PerDeviceFlag& attr, int smem, int threads, const GemmArgs& p, dim3 grid, hipStream_t stream,
                           const char* name) {
  bool& attr_done = attr.here();
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", name, smem, hipGetErrorString(e));
    attr_done = true;
  }
  hipLaunchKernelGGL(kern, grid, dim3(threads), smem, stream, p);
  return launch_status(name);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int NS, bool BLOCKSCALE, bool KV = false>
static int launch_tiled(const GemmArgs& p, dim3 grid, hipStream_t stream, const char* name) {
  static PerDeviceFlag attr_done;
  // (fused QKV: 8 more bytes per tile row for the rows' cache offsets, after the 2 * BM * BN bytes of staged output)
  constexpr int stages = tile_lds_bytes<BM, BN, NS, BLOCKSCALE>(), kv = 2 * BM * BN + 8 * BM * WAVES_N;
  if constexpr (!KV) {
    // one row of tiles (and one matrix): every weight byte is read once
    if (p.M <= BM && grid.z == 1) {
      static PerDeviceFlag attr_done_stream;
      return launch_with_lds(gemm_tiled_kernel<BM, BN, WAVES_M, WAVES_N, NS, BLOCKSCALE, KV, true>, attr_done_stream, stages,
                             WAVES_M * WAVES_N * 64, p, grid, stream, name);
    }
  }
  return launch_with_lds(gemm_tiled_kernel<BM, BN, WAVES_M, WAVES_N, NS, BLOCKSCALE, KV>, attr_done,
                         KV && kv > stages ? kv : stages, WAVES_M * WAVES_N * 64, p, grid, stream, name);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int NS, int SBM, int SWAVES_M, int SWAVES_N, int SNS, bool BLOCKSCALE = true>
static int launch_grouped(const GemmArgs& p, dim3 grid, hipStream_t stream, const char* name) {
  static PerDeviceFlag attr_done;
  constexpr int big = tile_lds_bytes<BM, BN, NS, BLOCKSCALE>(), small = tile_lds_bytes<SBM, BN, SNS, BLOCKSCALE>();
  return launch_with_lds(gemm_grouped_kernel<BM, BN, WAVES_M, WAVES_N, NS, SBM, SWAVES_M, SWAVES_N, SNS, BLOCKSCALE>, attr_done,
                         big > small ? big : small, WAVES_M * WAVES_N * 64, p, grid, stream, name);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int NS, bool BLOCKSCALE = true>
static int launch_grouped_large(const GemmArgs& p, dim3 grid, hipStream_t stream, const char* name) {
  static PerDeviceFlag attr_done;
  return launch_with_lds(gemm_grouped_large_kernel<BM, BN, WAVES_M, WAVES_N, NS, BLOCKSCALE>, attr_done,
                         tile_lds_bytes<BM, BN, NS, BLOCKSCALE>(), WAVES_M * WAVES_N * 64, p, grid, stream, name);
}

int compute_units();
static bool stream_is_capturing(hipStream_t stream);
// One numbering of the launches for both scale modes: the two instantiations below share the counter sets (and, for the
// work-split kernel, the flags) in device memory, so a counter of their own each would hand the same set, and the same
// flag value, to a block-scaled and a row-scaled launch.
static unsigned int next_launch_number() {
  static std::atomic<unsigned int> seq{0};
  return seq.fetch_add(1, std::memory_order_relaxed);
}
template <bool BLOCKSCALE>
static int launch_grouped_persist(const GemmArgs& p, hipStream_t stream, const char* name) {
  static PerDeviceFlag attr_done;
  constexpr int bodies = grouped_persist_table_offset<BLOCKSCALE>();  // the largest of the four tile bodies; the tables sit behind it
  static_assert(bodies == tile_lds_bytes<256, 128, 3, BLOCKSCALE>(), "the 256 x 128 body's stages");
  static_assert(tile_lds_bytes<256, 256, 2, BLOCKSCALE>() <= bodies && tile_lds_bytes<128, 256, 3, BLOCKSCALE>() <= bodies && 8 * 16384 <= bodies,
                "the tables sit behind the largest tile");
  constexpr int lds = bodies + 4 * (kGroupedMaxSlots + 1) * 4;
  static_assert(lds + 64 <= 160 * 1024, "one block per CU");
  // A set of counters per launch in flight (64 sets: launches that follow each other on a stream could share one).
  // A launch recorded into a HIP graph keeps the set of the recording in every replay, and a replay may run beside
  // launches issued on another stream: recorded launches draw from sets of their own, which no eager launch ever
  // gets.  (Replays of one graph never overlap each other; two graphs share a set only when 64 launches were recorded
  // between theirs.)
  int slot = (int)(next_launch_number() % kGroupedCtrSlots);
  if (stream_is_capturing(stream)) {
    static std::atomic<unsigned int> recorded{0};
    slot = kGroupedCtrSlots + (int)(recorded.fetch_add(1, std::memory_order_relaxed) % (kGroupedCtrSlotsAll - kGroupedCtrSlots));
  }
  auto kern = gemm_grouped_persist_kernel<BLOCKSCALE>;
  bool& done = attr_done.here();
  if (!done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", name, lds, hipGetErrorString(e));
    done = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)compute_units()), dim3(512), lds, stream, p, slot);
  return launch_status(name);
}

// The persistent kernel takes matmuls of whole 256 x 256 tiles with 16-byte aligned bf16 rows of C, one launch,
// no K split, and operands whose byte offsets fit 31 bits (a tile's position rides in the copies' scalar offset).
// (The tuning switch `persist` turns it off for A/B runs.)
static bool persist_shape(int64_t M, int64_t N, int variant) {
  if (!tuning().persist) return false;
  return variant == 1 && M > 0 && N > 0 && M % 256 == 0 && N % 256 == 0;
}
static bool persist_ok(const GemmArgs& p, bool blockscale, dim3 grid) {
  if (!persist_shape(p.M, p.N, 1)) return false;
  if (p.kv_on || p.splits > 1 || grid.y != 1 || grid.z != 1) return false;
  if (p.c_dtype != MAXFP8_BF16 || !p.c_vec8_ok) return false;
  const int64_t lim = 0x7ff00000ll, nslab = ceil_div(p.K, 128);
  if ((int64_t)p.M * p.lda >= lim || (int64_t)p.N * p.ldb >= lim) return false;
  if (blockscale && (nslab * p.a_scales_ld + p.M) * 4 >= lim) return false;
  if ((int64_t)p.M * p.ldc * 2 >= lim) return false;
  return true;
}

// The four-wave kernel (gemm_w4.hip): 0 (no), or the sixteen-row groups per wave -- 5: tiles of 160 x 256, 6: 192 x 256.
bool gemm_w4_ok(const GemmArgs& p, bool blockscale);
bool gemm_w4_grouped_ok(const GemmArgs& p, bool blockscale);
int gemm_w4_grouped_launch(const GemmArgs& p, bool blockscale, hipStream_t stream);
int gemm_w4_launch(const GemmArgs& p, bool blockscale, int tm, bool split, hipStream_t stream);
W4Split gemm_w4_split(int64_t M, int64_t N, int64_t K, int tm);

int compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (!cached[dev]) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

template <bool BLOCKSCALE>
static int launch_persist(const GemmArgs& p, hipStream_t stream, const char* name) {
  static PerDeviceFlag attr_done;
  constexpr int lds = tile_lds_bytes<256, 256, 2, BLOCKSCALE>() + 8 * 2048;  // stages + a 2 KB side buffer per wave
  const int64_t tiles = (int64_t)(p.M / 256) * (p.N / 256);
  const int cus = compute_units();
  const dim3 grid((unsigned)(tiles < cus ? tiles : cus));
  return launch_with_lds(gemm_persist_kernel<256, 256, 2, 4, BLOCKSCALE>, attr_done, lds, 512, p, grid, stream, name);
}

// measurement aid: the persistent kernel's main loop on operands that stay in L2 (level 1) or in LDS (level 2), on every CU
template <bool BLOCKSCALE, int PROBE>
static int launch_persist_probe(const GemmArgs& p, hipStream_t stream) {
  static PerDeviceFlag attr_done;
  constexpr int lds = tile_lds_bytes<256, 256, 2, BLOCKSCALE>() + 8 * 2048;
  return launch_with_lds(gemm_persist_probe_kernel<256, 256, 2, 4, BLOCKSCALE, PROBE>, attr_done, lds, 512, p,
                         dim3((unsigned)compute_units()), stream, "gemm_persist_probe");
}
int gemm_persist_probe(const GemmArgs& p, bool blockscale, int level, hipStream_t stream) {
  if (level == 1) return blockscale ? launch_persist_probe<true, 1>(p, stream) : launch_persist_probe<false, 1>(p, stream);
  return blockscale ? launch_persist_probe<true, 2>(p, stream) : launch_persist_probe<false, 2>(p, stream);
}

// The work-split form: blocks = the CUs in whole rounds of the 8 XCDs; one workspace slot of 256 KB per block.
static int streamk_blocks() {
  const int g = (compute_units() / 8) * 8;
  return g > kStreamkMaxBlocks ? kStreamkMaxBlocks : g;
}
static size_t streamk_workspace_bytes() { return (size_t)streamk_blocks() * 256 * 256 * 4; }

template <bool BLOCKSCALE>
static int launch_streamk(const GemmArgs& p_in, hipStream_t stream, const char* name) {
  static PerDeviceFlag attr_done;
  constexpr int lds = tile_lds_bytes<256, 256, 2, BLOCKSCALE>() + 8 * 2048;
  GemmArgs p = p_in;
  // every launch gets a sequence number (never 0) as its flag value and one of 64 sets of flags: launches that
  // follow each other on a stream may reuse a set at once, and 64 matmuls of this size are never in flight together
  unsigned int n = next_launch_number() + 1;
  if (n == 0) n = next_launch_number() + 1;
  p.streamk_seq = n;
  p.streamk_slot = (int)(n % kStreamkSlots);
  return launch_with_lds(gemm_streamk_kernel<256, 256, 2, 4, BLOCKSCALE>, attr_done, lds, 512, p, dim3((unsigned)streamk_blocks()), stream, name);
}

// Hand-overs of the work-split kernel that a block stopped waiting for, on the current device since the library was
// loaded (0 unless a GPU stopped in the middle of a launch, or more launches of this kind were in flight at once than
// there are sets of flags).  Waits for the device's work to finish.
int gemm_streamk_gave_up(unsigned int* count) {
  hipError_t e = hipDeviceSynchronize();
  if (e == hipSuccess) e = hipMemcpyFromSymbol(count, HIP_SYMBOL(g_streamk_gave_up), sizeof(unsigned int));
  if (e != hipSuccess) MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "stream-K: cannot read the count of abandoned hand-overs: %s", hipGetErrorString(e));
  return MAXFP8_OK;
}

// Sums the split-K partial results in split order (deterministic), applies the row / tensor
// scales where the matmul has them, converts and stores.
template <bool BLOCKSCALE>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(GemmArgs p) {
  const int64_t total = (int64_t)p.M * p.N;
  const int64_t stride = (int64_t)gridDim.x * 256 * 4;
  const bool quads = (total & 3) == 0;
  // four consecutive elements sit in one row of C and may leave as one store
  const bool row_quads = quads && (p.N & 3) == 0 && p.c_vec_ok;
  for (int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4; i < total; i += stride) {
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    const int cnt = (total - i) < 4 ? (int)(total - i) : 4;
    if (cnt == 4 && quads) {
      // the shares are added in their order, whatever the number of loads in flight
      const float* src = p.workspace + i;
      int sp = 0;
      for (; sp + 4 <= p.splits; sp += 4) {
        float4 t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) t[u] = *reinterpret_cast<const float4*>(src + (int64_t)(sp + u) * total);
#pragma unroll
        for (int u = 0; u < 4; ++u) { v[0] += t[u].x; v[1] += t[u].y; v[2] += t[u].z; v[3] += t[u].w; }
      }
      for (; sp < p.splits; ++sp) {
        const float4 t = *reinterpret_cast<const float4*>(src + (int64_t)sp * total);
        v[0] += t.x; v[1] += t.y; v[2] += t.z; v[3] += t.w;
      }
    } else {
      for (int sp = 0; sp < p.splits; ++sp) {
        const float* src = p.workspace + (int64_t)sp * total + i;
        for (int j = 0; j < cnt; ++j) v[j] += src[j];
      }
    }
    if (row_quads) {
      const int64_t m = i / p.N;
      const int64_t n = i - m * p.N;
      if constexpr (!BLOCKSCALE) {
        const float a_s = scale_at(p.a_scales, m * p.a_scale_stride, p.scales_dtype);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float r = v[j] * a_s;
          v[j] = r * scale_at(p.b_scales, (n + j) * p.b_scale_stride, p.scales_dtype);
        }
      }
      if (p.c_dtype == MAXFP8_BF16)
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(p.c) + m * p.ldc + n) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
      else
        *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.c) + m * p.ldc + n) = make_float4(v[0], v[1], v[2], v[3]);
      continue;
    }
    for (int j = 0; j < cnt; ++j) {
      const int64_t m = (i + j) / p.N;
      const int64_t n = (i + j) - m * p.N;
      float r = v[j];
      if constexpr (!BLOCKSCALE) {
        r = r * scale_at(p.a_scales, m * p.a_scale_stride, p.scales_dtype);
        r = r * scale_at(p.b_scales, n * p.b_scale_stride, p.scales_dtype);
      }
      if (p.c_dtype == MAXFP8_BF16) reinterpret_cast<uint16_t*>(p.c)[m * p.ldc + n] = (uint16_t)f32_to_bf16_bits(r);
      else reinterpret_cast<float*>(p.c)[m * p.ldc + n] = r;
    }
  }
}

// ---- kernel selection ------------------------------------------------------------------------
// Three tile shapes.  A block spends t_slab microseconds per 128-byte K slab and t_tile on the
// rest of a tile (pipeline fill, the store burst at the end), both measured with the whole chip
// busy and weights coming from HBM; the cost of a shape is rounds * (slabs * t_slab + t_tile)
// with rounds = ceil(tiles / resident blocks).
struct TileShape { int bm, bn, slots; float t_slab_block, t_slab_row, t_tile; };
static int gemm_tiled_launch(const GemmArgs& p, bool blockscale, int variant, dim3 grid, hipStream_t stream);

static const TileShape kShapes[4] = {
    // (block scaling: 1.63 measured at K = 4096; on long K the chip settles lower -- 1.72 ... 1.74 at K = 7168 ... 18432 --
    // and the planner, reading the shape 5 % fast, kept it where the four-wave kernel measures ahead)
    {256, 256, 256, 1.70f, 1.40f, 11.4f},   // 8 waves, 2 stages
    {256, 128, 256, 0.92f, 0.82f, 9.0f},    // 8 waves, 3 stages
    {128, 128, 512, 0.96f, 0.86f, 11.4f},   // 4 waves, 2 stages, two blocks per CU
    {128, 128, 256, 0.74f, 0.66f, 9.0f},    // 4 waves, 3 stages, one block per CU: problems of at most one round of such tiles
};

// the tuning switch `tile` forces a shape (tuning runs and tests); 0 lets the cost model pick
static int tile_override() { return tuning().tile; }

// Split-K: when the tiles of a matmul cover only part of the chip, K is cut into `splits` shares
// (each at least 4 slabs) until the grid fills the resident-block slots.  Needs
// splits * M * N * 4 bytes of workspace; without workspace the matmul runs unsplit.
static int pick_splits(int64_t tiles, int slots, int nslab) {
  int splits = tuning().splitk;
  if (splits <= 0) {
    splits = 1;
    if (tiles * 2 <= slots) splits = (int)(slots / tiles);
    if (splits > 16) splits = 16;
  }
  if (splits > nslab / 4) splits = nslab / 4;
  if (splits < 1) splits = 1;
  const int per = (nslab + splits - 1) / splits;
  return (nslab + per - 1) / per;  // no empty share
}

// The per-tile overhead of shape i on an M x N region: the persistent kernel (whole 256 x 256 tiles, no K split)
// hides 3.5 of the 11.4 microseconds between two tiles (measured: 3.2 per round on q_b, 4.4 on kv_b).
static bool persist_shape(int64_t M, int64_t N, int variant);
static float tile_overhead(int64_t M, int64_t N, int i, int splits) {
  return kShapes[i].t_tile - ((splits == 1 && persist_shape(M, N, i + 1)) ? 3.5f : 0.f);
}

// cost of a shape (microseconds) = rounds of resident blocks * time of one tile
static int pick_shape(int64_t M, int64_t N, int nslab, bool blockscale, bool can_split, int64_t batch = 1) {
  int best = 0;
  float best_cost = 0.f;
  for (int i = 0; i < 4; ++i) {
    const TileShape& t = kShapes[i];
    const int64_t tiles = ceil_div(M, t.bm) * ceil_div(N, t.bn) * batch;
    const int sp = can_split ? pick_splits(tiles, t.slots, nslab) : 1;
    float cost = (float)ceil_div(tiles * sp, t.slots) *
                 ((float)ceil_div(nslab, sp) * (blockscale ? t.t_slab_block : t.t_slab_row) + tile_overhead(M, N, i, sp));
    // a split pays a second launch and one write + one read of sp * M * N f32 partial sums (~4 TB/s)
    if (sp > 1) cost += 5.0f + (float)sp * (float)M * (float)N * 8.0f / 4.0e6f;
    if (i == 0 || cost < best_cost) { best = i; best_cost = cost; }
  }
  return best + 1;
}

static bool streamk_shape(int64_t M, int64_t N, size_t workspace_bytes);
static bool streamk_planned(int64_t M, int64_t N, int64_t K, bool blockscale);
size_t gemm_tiled_plan_workspace_bytes(int64_t M, int64_t N, int64_t K, bool blockscale);
static size_t workspace_bytes_uncached(int64_t M, int64_t N, int64_t K);
// (callers ask before every matmul: the answers are kept, like the plans, keyed by the shape and the generation of the
// tuning switches)
size_t gemm_tiled_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  struct Entry { int64_t M, N, K; unsigned generation; bool valid; size_t bytes; };
  static Entry table[128];
  static std::mutex mu;
  const unsigned generation = (unsigned)tuning().generation;
  const uint64_t h = ((uint64_t)M * 0x9e3779b97f4a7c15ull) ^ ((uint64_t)N * 0xc2b2ae3d27d4eb4full) ^ ((uint64_t)K * 0x165667b19e3779f9ull);
  Entry& e = table[(h >> 32) % 128];
  {
    std::lock_guard<std::mutex> lock(mu);
    if (e.valid && e.M == M && e.N == N && e.K == K && e.generation == generation) return e.bytes;
  }
  const size_t bytes = workspace_bytes_uncached(M, N, K);
  std::lock_guard<std::mutex> lock(mu);
  e = Entry{M, N, K, generation, true, bytes};
  return bytes;
}
static size_t workspace_bytes_uncached(int64_t M, int64_t N, int64_t K) {
  // the largest split count any shape could choose for this problem
  size_t worst = 0;
  const int nslab = (int)ceil_div(K, 128);
  for (int i = 0; i < 4; ++i) {
    const TileShape& t = kShapes[i];
    const int64_t tiles = ceil_div(M, t.bm) * ceil_div(N, t.bn);
    const int sp = pick_splits(tiles, t.slots, nslab);
    if (sp > 1 && (size_t)sp > worst) worst = sp;
  }
  const size_t split_k = worst * (size_t)M * (size_t)N * 4;
  // the work-split persistent kernel: a slot per block for the accumulators a block hands to its successor, where the
  // planner would use it given the memory (in either scale mode: this size does not know which one is coming)
  size_t split_work = 0;
  if (streamk_shape(M, N, ~(size_t)0) && (streamk_planned(M, N, K, true) || streamk_planned(M, N, K, false)))
    split_work = streamk_workspace_bytes();
  // the four-wave kernel's tail cut: a slot per block for the sums of a piece of a tile
  for (int bs = 0; bs < 2; ++bs) {
    const size_t cut = gemm_tiled_plan_workspace_bytes(M, N, K, bs != 0);
    if (cut > split_work) split_work = cut;
  }
  return split_k > split_work ? split_k : split_work;
}

// cost (microseconds) of an unsplit M x N region in tiles of shape t
static float region_cost(int64_t M, int64_t N, int nslab, const TileShape& t, bool blockscale) {
  const int64_t tiles = ceil_div(M, t.bm) * ceil_div(N, t.bn);
  return (float)ceil_div(tiles, t.slots) *
         ((float)nslab * (blockscale ? t.t_slab_block : t.t_slab_row) + tile_overhead(M, N, (int)(&t - kShapes), 1));
}

// A matmul whose tiles fill the chip a whole number of times plus a small rest wastes most of its
// last round.  Such a problem is cut in two along N or M: a first region that the main shape
// covers in full rounds, and a rest that runs as a second launch in whatever shape fills the
// chip best (e.g. Llama-8B gate_up, M = 2048: 896 tiles of 256 x 256 are 3.5 rounds; 768 of
// them plus 256 tiles of 256 x 128 are 3 rounds and one short one).  The cost model decides.
struct TwoRegionPlan { int axis; int64_t cut; int v1, v2; float cost; };  // axis 0: none, 1: N, 2: M
static TwoRegionPlan pick_two_regions(int64_t M, int64_t N, int nslab, bool blockscale, float single_cost) {
  constexpr float kSecondLaunch = 4.0f;  // the second launch starts when the first has drained
  TwoRegionPlan best = {0, 0, 0, 0, single_cost - 4.0f};  // must beat the single launch by a margin
  for (int i = 0; i < 3; ++i) {
    for (int j = 0; j < 3; ++j) {
      const TileShape &a = kShapes[i], &b = kShapes[j];
      for (int64_t c = 1; c < ceil_div(N, a.bn); ++c) {
        const float t = region_cost(M, c * a.bn, nslab, a, blockscale) + region_cost(M, N - c * a.bn, nslab, b, blockscale) + kSecondLaunch;
        if (t < best.cost) best = {1, c * a.bn, i + 1, j + 1, t};
      }
      for (int64_t c = 1; c < ceil_div(M, a.bm); ++c) {
        const float t = region_cost(c * a.bm, N, nslab, a, blockscale) + region_cost(M - c * a.bm, N, nslab, b, blockscale) + kSecondLaunch;
        if (t < best.cost) best = {2, c * a.bm, i + 1, j + 1, t};
      }
    }
  }
  return best;
}

// What a tiled matmul will launch: one shape (possibly with K split), two regions, or the four-wave kernel (w4: 0, or
// its sixteen-row groups per wave).
struct TiledPlan { int variant; int splits; TwoRegionPlan two; bool streamk; int w4; bool w4_split; };

// One persistent launch of `tiles` tiles on `slots` CUs, a tile taking t microseconds with the chip full: whole rounds
// cost t each; a last round that fills only part of the chip is faster than a full one but not in proportion (fewer
// CUs share the clock budget, the L2s and the fabric; each tile still walks all of K) -- measured 0.76 ... 0.78 t at a
// fill of 3 ... 40 %, 0.98 ... 1.03 t at 75 ... 85 %.
static float persistent_cost(int64_t tiles, int slots, float t) {
  const int64_t full = tiles / slots, rest = tiles % slots;
  return (float)full * t + (rest ? t * (0.75f + 0.3f * (float)rest / (float)slots) : 0.f);
}

// Per-slab and per-tile times (microseconds, chip full, operands from HBM) of the four-wave kernel's three tile heights:
// index 0: 128 x 256, 1: 160 x 256, 2: 192 x 256.  Against the eight-wave persistent kernel's 1.63 / 1.40 per slab of a 256 x 256 tile
// that is 6 ... 9 % less per flop with block scaling and level with row scaling; what decides between the three is
// mostly how the tile count divides by the CUs.
static const float kW4SlabBlock[3] = {0.90f, 1.00f, 1.14f}, kW4SlabRow[3] = {0.93f, 0.88f, 1.00f}, kW4Tile = 5.5f;
// With the tail cut: whole rounds, then a piece per block and the hand-over: a piece's sums written through to memory,
// then read and added by the tile's last block, piece after piece (measured on 4096 x 7168 x 16384, 104 tiles in two
// pieces each behind two whole rounds, and on 2048 x 7168 x 18432, 52 tiles in four pieces behind one).
static const float kW4HandOver = 8.0f, kW4HandOverPiece = 7.0f;

// The shapes the four-wave kernel takes (see gemm_w4_ok; pointers and strides are checked at the launch).
static bool w4_shape(int64_t M, int64_t N, int64_t K) { return M > 0 && N > 0 && N % 8 == 0 && K >= 512 && K % 256 == 0; }

// Which four-wave tile height, if any, beats `other_cost` (microseconds, what the plan made of the eight-wave shapes
// costs) by at least 3 %, and whether with its tail cut (*split; the workspace has to hold the pieces).
//
// other_splits: the other plan is a K split (two launches, the shares' sums through memory).  Then the matmul is at most
// half a round of tiles, and the one candidate is the four-wave kernel with EVERY tile cut into pieces, the pieces
// exchanging their sums inside the one launch: measured ahead where the pieces fill three quarters of the chip and are at
// least 16 slabs long (512 x 7168 x 16384: 67 against 84 us; 1024 x 2112 x 7168: 30 against 35; 384 x 6144 x 8192: 35
// against 42; 768 x 2048 x 8192, 16 slabs: 27 against 32), behind with shorter pieces (8 slabs: 25 against 22) and with
// fewer blocks (128 x 4096 x 14336, 16 tiles in 64 pieces: 38 against 27; 512 x 2048 x 28672, 128 pieces: 64 against 51).
static int pick_w4(int64_t M, int64_t N, int64_t K, bool blockscale, float other_cost, bool other_splits, size_t workspace_bytes, bool* split) {
  const int forced = tuning().w4, cut = tuning().w4_split;
  *split = false;
  if (forced == 0 || !tuning().persist || !w4_shape(M, N, K)) return 0;
  const int nslab = (int)(K / 128), slots = compute_units();
  if (other_splits) {
    const int tm = forced > 0 ? forced : 4;
    const W4Split sp = gemm_w4_split(M, N, K, tm);
    if (cut == 0 || sp.unit <= 0 || sp.bytes > workspace_bytes) return 0;
    if (ceil_div(M, 32 * tm) * ceil_div(N, 256) * 2 > slots) return 0;  // (not the case meant here)
    // (more than four pieces only where they are long: 128 x 8192 x 28672 in eight pieces of 28 slabs 59 against 64 us,
    // 512 x 2048 x 28672 46 against 52; in eight of 16 slabs 128 x 8192 x 16384 47 against 41.  And only where the rows
    // fill three quarters of the 128-row tiles: 48 ... 64 rows on 8192 x 28672 took 56 against 48 ... 51.)
    const int64_t pieces = ceil_div(nslab, sp.unit), rows_padded = ceil_div(M, 32 * tm) * 32 * tm;
    if (forced <= 0 && cut != 1 &&
        (sp.unit < (pieces > 4 ? 24 : 16) || (int64_t)sp.blocks * 4 < (int64_t)slots * 3 || M * 4 < rows_padded * 3))
      return 0;
    *split = true;
    return tm;
  }
  int best = 0;
  float best_cost = forced > 0 ? 3.0e38f : 0.97f * other_cost;  // (a forced height is taken whatever it costs)
  for (int i = 0; i < 3; ++i) {
    const int tm = 4 + i;
    if (forced > 0 && tm != forced) continue;
    const float t_slab = blockscale ? kW4SlabBlock[i] : kW4SlabRow[i], t = (float)nslab * t_slab + kW4Tile;
    const int64_t tiles = ceil_div(M, 32 * tm) * ceil_div(N, 256);
    if (forced <= 0 && tiles * 4 < (int64_t)slots * 3) continue;  // (well under one round: more, smaller tiles and a K split are the better fit)
    const float whole = persistent_cost(tiles, slots, t);
    if (whole < best_cost) { best = tm; best_cost = whole; *split = false; }
    const W4Split sp = gemm_w4_split(M, N, K, tm);
    if (cut != 0 && sp.unit > 0 && sp.bytes <= workspace_bytes) {
      const float pieces = (float)ceil_div(nslab, sp.unit);
      float with_cut = (float)(tiles / sp.blocks) * t + (float)sp.unit * t_slab + kW4Tile + kW4HandOver + kW4HandOverPiece * (pieces - 1.f);
      if (cut == 1) with_cut *= 1.0e-3f;  // (switched on: wherever there is one)
      if (with_cut < best_cost) { best = tm; best_cost = with_cut; *split = true; }
    }
  }
  return best;
}


// The work-split persistent kernel takes matmuls of whole 256 x 256 tiles that are at least one tile per block (so a
// tile has at most two parts) and not a whole number of rounds (those have nothing to gain), when the caller's
// workspace holds a 256 KB slot per block.
static bool streamk_shape(int64_t M, int64_t N, size_t workspace_bytes) {
  if (!tuning().streamk || !persist_shape(M, N, 1)) return false;
  const int64_t tiles = (M / 256) * (N / 256), g = streamk_blocks();
  return g >= 8 && tiles >= g && tiles % g != 0 && workspace_bytes >= streamk_workspace_bytes();
}
static TiledPlan make_plan(int64_t M, int64_t N, int64_t K, bool blockscale, bool has_workspace, size_t workspace_bytes,
                           int64_t batch, bool kv_on) {
  TiledPlan plan = {0, 1, {0, 0, 0, 0, 0.f}, false, 0, false};
  const int nslab = (int)ceil_div(K, 128);
  plan.variant = tile_override();
  const bool free_choice = plan.variant == 0;
  if (!plan.variant) plan.variant = pick_shape(M, N, nslab, blockscale, has_workspace && batch == 1, batch);
  if (kv_on && plan.variant != 1) plan.variant = 3;  // the fused QKV kernels exist in the 256 x 256 and 128 x 128 shapes
  const TileShape& t = kShapes[plan.variant - 1];
  const int64_t tiles = ceil_div(M, t.bm) * ceil_div(N, t.bn);
  // (wants_split: the shape calls for a K split, whether or not this workspace holds its partial sums -- what the
  // four-wave kernel's choice below goes by, so that a caller who brings exactly that kernel's bytes gets the same plan
  // as one who brings more)
  bool wants_split = false;
  if (has_workspace && batch == 1 && !kv_on) {
    const int sp = pick_splits(tiles, t.slots, nslab);
    wants_split = sp > 1;
    if (sp > 1 && (size_t)sp * M * N * 4 <= workspace_bytes) plan.splits = sp;
  }
  if (free_choice && batch == 1 && !kv_on && plan.splits == 1 && !tuning().one_region)
    plan.two = pick_two_regions(M, N, nslab, blockscale, region_cost(M, N, nslab, t, blockscale));
  // Every block the same number of slabs instead of whole rounds of tiles.  Measured (block scaling, 300 to 900 tiles,
  // K = 384 ... 16384): 23 microseconds (the hand-over: one drain of the pipeline, 256 KB each way per block) plus
  // 1.9 per slab -- a sixth more per slab than the persistent kernel, whose blocks of an XCD walk K in step and
  // find each other's operands in L2, while here neighbouring blocks sit at different K offsets.  So the split only
  // pays where whole rounds would leave most of the last round empty and K is long (300 tiles, K = 4096: 87 against
  // 107 microseconds; 448 tiles, K = 16384: 437 against 427): it has to beat the other plan by a tenth.
  if (has_workspace && batch == 1 && !kv_on && plan.splits == 1 && (free_choice || plan.variant == 1) &&
      streamk_shape(M, N, workspace_bytes)) {
    const float tiles = (float)((M / 256) * (N / 256)), g = (float)streamk_blocks();
    const float per_slab = 1.9f * (blockscale ? 1.0f : kShapes[0].t_slab_row / kShapes[0].t_slab_block);
    const float cost = 23.0f + tiles / g * (float)nslab * per_slab;
    const float other = plan.two.axis ? plan.two.cost : region_cost(M, N, nslab, t, blockscale);
    plan.streamk = tuning().streamk == 2 || cost < 0.9f * other;
  }
  // the four-wave kernel against whatever the eight-wave shapes make of the matmul (one launch; a forced tile shape other
  // than 256 x 256, a K split, a batch or the fused QKV epilogue keep it out)
  if (batch == 1 && !kv_on && !plan.streamk && (free_choice || plan.variant == 1)) {
    float other = plan.two.axis ? plan.two.cost : region_cost(M, N, nslab, t, blockscale);
    if (!plan.two.axis && persist_shape(M, N, plan.variant))
      other = persistent_cost(tiles, t.slots, (float)nslab * (blockscale ? t.t_slab_block : t.t_slab_row) + tile_overhead(M, N, plan.variant - 1, 1));
    plan.w4 = pick_w4(M, N, K, blockscale, other, wants_split, has_workspace ? workspace_bytes : 0, &plan.w4_split);
    if (plan.w4) plan.splits = 1;
  }
  return plan;
}

static TiledPlan cached_plan(int64_t M, int64_t N, int64_t K, bool blockscale, bool has_workspace, size_t workspace_bytes, int64_t batch, bool kv_on);
static bool streamk_planned(int64_t M, int64_t N, int64_t K, bool blockscale) {
  return cached_plan(M, N, K, blockscale, true, ~(size_t)0, 1, false).streamk;
}

// The split-K scratch of the plan an unlimited workspace gets (0: that plan does not split).  A workspace of this size --
// or of gemm_tiled_workspace_bytes, which is never smaller -- leads to this same plan.
size_t gemm_tiled_plan_workspace_bytes(int64_t M, int64_t N, int64_t K, bool blockscale) {
  // (from the table of plans: the entry points ask this on every call of a matmul of at most 64 rows)
  const TiledPlan plan = cached_plan(M, N, K, blockscale, true, ~(size_t)0, 1, false);
  // (a plan that splits the work between blocks instead has splits == 1: without the 64 MB of slots it needs, the
  // planner falls back to the persistent kernel, which forms the same sums)
  if (plan.w4 && plan.w4_split) return gemm_w4_split(M, N, K, plan.w4).bytes;
  return plan.splits > 1 ? (size_t)plan.splits * (size_t)M * (size_t)N * 4 : 0;
}

// make_plan tries every cut of every pair of shapes: microseconds of host time, as much as a small matmul
// takes on the GPU.  Plans are kept in a small table, keyed by everything make_plan reads (the generation
// of the tuning switches included, since tests and tuning runs reload them between calls).
static TiledPlan cached_plan(int64_t M, int64_t N, int64_t K, bool blockscale, bool has_workspace, size_t workspace_bytes,
                             int64_t batch, bool kv_on) {
  struct Entry { int64_t M, N, K, batch; size_t ws; int flags; bool valid; TiledPlan plan; };
  static Entry table[128];
  static std::mutex mu;
  const int flags = (blockscale ? 1 : 0) | (has_workspace ? 2 : 0) | (kv_on ? 4 : 0) | (int)(tuning().generation << 3);
  // (every part of the key reaches the high bits that pick the slot: one shape is asked for with several workspace
  // sizes and scale modes in turn, and those must not push each other out)
  const uint64_t h = ((uint64_t)M * 0x9e3779b97f4a7c15ull) ^ ((uint64_t)N * 0xc2b2ae3d27d4eb4full) ^ ((uint64_t)K * 0x165667b19e3779f9ull) ^
                     ((uint64_t)batch * 0xd6e8feb86659fd93ull) ^ ((uint64_t)flags * 0xa0761d6478bd642full) ^
                     ((uint64_t)workspace_bytes * 0xe7037ed1a0b428dbull);
  Entry& e = table[(h >> 32) % 128];
  {
    std::lock_guard<std::mutex> lock(mu);
    if (e.valid && e.M == M && e.N == N && e.K == K && e.batch == batch && e.ws == workspace_bytes && e.flags == flags) return e.plan;
  }
  const TiledPlan plan = make_plan(M, N, K, blockscale, has_workspace, workspace_bytes, batch, kv_on);
  std::lock_guard<std::mutex> lock(mu);
  e = Entry{M, N, K, batch, workspace_bytes, flags, true, plan};
  return plan;
}

// "256x256 x896" / "256x256 x448, K split 2" / "256x256 x768 + columns from 24576: 256x128 x256"
int gemm_tiled_describe(int64_t M, int64_t N, int64_t K, bool blockscale, bool has_workspace, char* buf, size_t len) {
  const TiledPlan plan = make_plan(M, N, K, blockscale, has_workspace, has_workspace ? gemm_tiled_workspace_bytes(M, N, K) : 0, 1, false);
  auto count = [](int64_t m, int64_t n, const TileShape& t) { return (long long)(ceil_div(m, t.bm) * ceil_div(n, t.bn)); };
  // (what a bf16 result with 16-byte aligned rows gets)
  auto how = [](int64_t m, int64_t n, int variant) { return persist_shape(m, n, variant) ? " persistent" : (variant == 4 ? " three-stage" : ""); };
  if (plan.w4 && plan.w4_split) {
    const long long n_tiles = (long long)(ceil_div(M, 32 * plan.w4) * ceil_div(N, 256));
    const W4Split sp = gemm_w4_split(M, N, K, plan.w4);
    return snprintf(buf, len, "%dx256 x%lld persistent, four waves, %s cut in pieces of %d slabs", 32 * plan.w4, n_tiles,
                    n_tiles * 2 <= compute_units() ? "every tile" : "tail", sp.unit);
  }
  if (plan.w4)
    return snprintf(buf, len, "%dx256 x%lld persistent, four waves", 32 * plan.w4, (long long)(ceil_div(M, 32 * plan.w4) * ceil_div(N, 256)));
  if (plan.two.axis && !plan.streamk) {
    const TileShape &a = kShapes[plan.two.v1 - 1], &b = kShapes[plan.two.v2 - 1];
    const bool cols = plan.two.axis == 1;
    const int64_t m1 = cols ? M : plan.two.cut, n1 = cols ? plan.two.cut : N;
    const int64_t m2 = cols ? M : M - plan.two.cut, n2 = cols ? N - plan.two.cut : N;
    return snprintf(buf, len, "%dx%d x%lld%s + %s from %lld: %dx%d x%lld%s", a.bm, a.bn, count(m1, n1, a), how(m1, n1, plan.two.v1),
                    cols ? "columns" : "rows", (long long)plan.two.cut, b.bm, b.bn, count(m2, n2, b), how(m2, n2, plan.two.v2));
  }
  const TileShape& t = kShapes[plan.variant - 1];
  if (plan.streamk)
    return snprintf(buf, len, "256x256 x%lld persistent, stream-K: equal shares of slabs for %d blocks", count(M, N, kShapes[0]), streamk_blocks());
  if (plan.splits > 1) return snprintf(buf, len, "%dx%d x%lld, K split %d", t.bm, t.bn, count(M, N, t), plan.splits);
  return snprintf(buf, len, "%dx%d x%lld%s", t.bm, t.bn, count(M, N, t), how(M, N, plan.variant));
}

// A launch recorded into a HIP graph replays with the arguments of the recording.  The work-split kernel's flag value
// would then repeat: a replay would find the flags of the replay before it already set, and a block could take over
// accumulators its predecessor has not written yet.  Such a launch runs as the persistent kernel instead, which forms the
// same sums in the same order.  (The grouped kernel's counters are put back to zero by the launch itself and replay as they are.)
static bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}

int gemm_tiled_dispatch(const GemmArgs& p_in, bool blockscale, size_t workspace_bytes, int64_t batch, hipStream_t stream) {
  GemmArgs p = p_in;
  const TiledPlan plan = cached_plan(p.M, p.N, p.K, blockscale, p.workspace != nullptr, workspace_bytes, batch, p.kv_on != 0);
  if (plan.streamk && !stream_is_capturing(stream)) {
    p.splits = 1;
    // (the plan knows the shape; whether this call's pointers and strides suit the persistent kernels is checked here)
    if (persist_ok(p, blockscale, dim3(1, 1, 1)))
      return blockscale ? launch_streamk<true>(p, stream, "gemm_streamk_block_256x256") : launch_streamk<false>(p, stream, "gemm_streamk_row_256x256");
  }
  if (plan.w4) {
    p.splits = 1;
    // (the plan knows the shape; whether this call's pointers and strides suit the kernel is checked here)
    if (gemm_w4_ok(p, blockscale)) return gemm_w4_launch(p, blockscale, plan.w4, plan.w4_split && p.workspace != nullptr, stream);
  }
  if (plan.two.axis) {
    const TwoRegionPlan& two = plan.two;
    GemmArgs r1 = p, r2 = p;
    r1.splits = r2.splits = 1;
    const int64_t esz = p.c_dtype == MAXFP8_BF16 ? 2 : 4;
    const int64_t ssz = p.scales_dtype == MAXFP8_F32 ? 4 : 2;  // (row / tensor scales; block scales are f32)
    if (two.axis == 1) {  // columns [0, cut) and [cut, N): weight rows, their scales, C columns
      r1.N = (int)two.cut;
      r2.N = p.N - (int)two.cut;
      r2.b = p.b + two.cut * p.ldb;
      r2.c = reinterpret_cast<uint8_t*>(p.c) + two.cut * esz;
      r2.b_scales = blockscale ? p.b_scales + (two.cut / 128) * p.b_scales_ld
                               : reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(p.b_scales) + two.cut * p.b_scale_stride * ssz);
    } else {              // rows [0, cut) and [cut, M): activation rows, their scales, C rows
      r1.M = (int)two.cut;
      r2.M = p.M - (int)two.cut;
      r2.a = p.a + two.cut * p.lda;
      r2.c = reinterpret_cast<uint8_t*>(p.c) + two.cut * p.ldc * esz;
      r2.a_scales = blockscale ? p.a_scales + two.cut
                               : reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(p.a_scales) + two.cut * p.a_scale_stride * ssz);
    }
    const TileShape &ta = kShapes[two.v1 - 1], &tb = kShapes[two.v2 - 1];
    const dim3 g1((unsigned)(ceil_div(r1.M, ta.bm) * ceil_div(r1.N, ta.bn)), 1, 1);
    const dim3 g2((unsigned)(ceil_div(r2.M, tb.bm) * ceil_div(r2.N, tb.bn)), 1, 1);
    const int rc = gemm_tiled_launch(r1, blockscale, two.v1, g1, stream);
    if (rc != MAXFP8_OK) return rc;
    return gemm_tiled_launch(r2, blockscale, two.v2, g2, stream);
  }
  const int variant = plan.variant;
  const TileShape& t = kShapes[variant - 1];
  const int64_t tiles = ceil_div(p.M, t.bm) * ceil_div(p.N, t.bn);
  if (tiles >= ((int64_t)1 << 31)) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "tiled matmul: too many tiles");
  p.splits = plan.splits;
  const dim3 grid((unsigned)tiles, (unsigned)p.splits, (unsigned)batch);
  const int rc = gemm_tiled_launch(p, blockscale, variant, grid, stream);
  if (rc != MAXFP8_OK || p.splits == 1) return rc;
  const int64_t quads = ceil_div((int64_t)p.M * p.N, 4);
  const unsigned rblocks = (unsigned)(ceil_div(quads, 256) < 4096 ? ceil_div(quads, 256) : 4096);
  if (blockscale) hipLaunchKernelGGL(splitk_reduce_kernel<true>, dim3(rblocks), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL(splitk_reduce_kernel<false>, dim3(rblocks), dim3(256), 0, stream, p);
  return launch_status("splitk_reduce");
}

static int gemm_tiled_launch(const GemmArgs& p, bool blockscale, int variant, dim3 grid, hipStream_t stream) {
  if (p.kv_on) {  // fused QKV: the two larger shapes
    if (blockscale) {
      if (variant == 1) return launch_tiled<256, 256, 2, 4, 2, true, true>(p, grid, stream, "gemm_qkv_block_256x256");
      return launch_tiled<128, 128, 2, 2, 2, true, true>(p, grid, stream, "gemm_qkv_block_128x128");
    }
    if (variant == 1) return launch_tiled<256, 256, 2, 4, 2, false, true>(p, grid, stream, "gemm_qkv_row_256x256");
    return launch_tiled<128, 128, 2, 2, 2, false, true>(p, grid, stream, "gemm_qkv_row_128x128");
  }
  if (variant == 1 && persist_ok(p, blockscale, grid))
    return blockscale ? launch_persist<true>(p, stream, "gemm_persist_block_256x256") : launch_persist<false>(p, stream, "gemm_persist_row_256x256");
  if (blockscale) {
    if (variant == 1) return launch_tiled<256, 256, 2, 4, 2, true>(p, grid, stream, "gemm_tiled_block_256x256");
    if (variant == 2) return launch_tiled<256, 128, 4, 2, 3, true>(p, grid, stream, "gemm_tiled_block_256x128");
    if (variant == 4) return launch_tiled<128, 128, 2, 2, 3, true>(p, grid, stream, "gemm_tiled_block_128x128x3");
    return launch_tiled<128, 128, 2, 2, 2, true>(p, grid, stream, "gemm_tiled_block_128x128");
  }
  if (variant == 1) return launch_tiled<256, 256, 2, 4, 2, false>(p, grid, stream, "gemm_tiled_row_256x256");
  if (variant == 2) return launch_tiled<256, 128, 4, 2, 3, false>(p, grid, stream, "gemm_tiled_row_256x128");
  if (variant == 4) return launch_tiled<128, 128, 2, 2, 3, false>(p, grid, stream, "gemm_tiled_row_128x128x3");
  return launch_tiled<128, 128, 2, 2, 2, false>(p, grid, stream, "gemm_tiled_row_128x128");
}

// One extra stream and two events per device, made at the first use and kept until the process ends
// (default priority, like every stream this library touches).
struct SideStream { hipStream_t stream; hipEvent_t fork, join; std::mutex mu; bool made, ok; };
static SideStream* side_stream() {
  static SideStream table[64];
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  SideStream& s = table[dev];
  if (!s.made) {
    s.made = true;
    s.ok = hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking) == hipSuccess &&
           hipEventCreateWithFlags(&s.fork, hipEventDisableTiming) == hipSuccess &&
           hipEventCreateWithFlags(&s.join, hipEventDisableTiming) == hipSuccess;
    if (!s.ok) (void)hipGetLastError();
  }
  return s.ok ? &s : nullptr;
}

int gemm_grouped_dispatch(const GemmArgs& p_in, bool blockscale, int64_t T, int64_t max_tokens, hipStream_t stream) {
  GemmArgs p = p_in;
  // Slots with at least 1024 rows (the caller's bound on the largest slot says whether there can
  // be any) hand their full 256-row tiles to a launch with 256 x 256 tiles; everything else --
  // their last rows, the other slots -- runs in 128 x 128 tiles, and in 32 x 128 tiles with a
  // third LDS stage where at most 32 rows are left.
  // tuning switch `tile` = 2: 256-row tiles in one launch; 3: no small tiles; 4: no large-tile launch
  const int tune = tile_override();
  const bool big = tune == 2;
  const int bm = big ? 256 : 128;
  p.small_rows = tune == 3 ? 0 : (big ? 64 : 32);
  p.big_rows = 0;
  p.big_bm = 256;
  const int big_rows = tuning().big_rows;
  // The large-tile launch goes down a second stream, as a fixed set of blocks, so that its tiles (bound by the matrix
  // pipe) and the other launch's (mostly bound by HBM) share the chip instead of taking turns; the caller's stream
  // waits for both.  (The tuning switch `grouped_overlap` = 0 keeps the two launches in line on the caller's stream.)
  // One persistent launch that shares the chip out between its four kinds of tiles (the tuning switch
  // `grouped_persist` = 0 goes back to the two launches below).
  if (tuning().grouped_persist && !big && p.num_active <= kGroupedMaxSlots) {
    p.share_bias = tuning().grouped_share * 2.0f;
    // A slot of more than 128 rows possible, and enough rows for it to matter: every slot's full 192-row
    // tiles, and a rest of more than 128 rows, go to the four-wave kernel (a quarter faster per row than the L tiles
    // below on the matrix pipe, twice as fast as the M2 tiles), which is issued first on the caller's stream; the
    // persistent launch takes the rests of at most 128 rows down the second stream.  How the
    // CUs are shared is decided on the device, where the group sizes are (see gemm_w4.hip).
    if (tuning().grouped_w4 && tune != 4 && max_tokens > tuning().grouped_w4_cold_rows && T >= tuning().grouped_w4_rows && gemm_w4_grouped_ok(p, blockscale)) {
      SideStream* side = side_stream();
      if (side) {
        std::unique_lock<std::mutex> side_lock(side->mu);  // one fork / join at a time per device
        p.big_rows = 0;
        p.big_bm = 192;
        p.small_rows = 32;
        p.w4_hot_rest = tuning().grouped_w4_hot_rest;
        p.w4_cold_rows = tuning().grouped_w4_cold_rows;
        if (hipEventRecord(side->fork, stream) != hipSuccess || hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess)
          MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "grouped matmul: cannot order the second stream behind the caller's: %s", hipGetErrorString(hipGetLastError()));
        GemmArgs ph = p;
        ph.share_bias = tuning().grouped_w4_share < 0.f ? tuning().grouped_w4_share : p.share_bias * tuning().grouped_w4_share;
        int rc = gemm_w4_grouped_launch(ph, blockscale, stream);
        if (rc == MAXFP8_OK) {
          p.heads_elsewhere = 1;
          rc = blockscale ? launch_grouped_persist<true>(p, side->stream, "gemm_grouped_persist_block")
                          : launch_grouped_persist<false>(p, side->stream, "gemm_grouped_persist_row");
        }
        if ((hipEventRecord(side->join, side->stream) != hipSuccess || hipStreamWaitEvent(stream, side->join, 0) != hipSuccess) && rc == MAXFP8_OK)
          MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "grouped matmul: cannot join the second stream: %s", hipGetErrorString(hipGetLastError()));
        return rc;
      }
    }
    // (every slot's full 256-row tiles are L tiles here: one kernel, no second launch to fill)
    p.big_rows = tune != 4 ? 256 : 0;
    return blockscale ? launch_grouped_persist<true>(p, stream, "gemm_grouped_persist_block")
                      : launch_grouped_persist<false>(p, stream, "gemm_grouped_persist_row");
  }
  SideStream* side = nullptr;
  const bool large = !big && tune != 4 && max_tokens >= big_rows && T / 256 <= 65535;
  if (large && tuning().grouped_overlap) side = side_stream();
  std::unique_lock<std::mutex> side_lock;
  if (large) {
    p.big_rows = big_rows;
    GemmArgs pl = p;
    dim3 lgrid((unsigned)ceil_div(p.N, 256), (unsigned)(T / 256));
    if (side) {
      // The large-tile blocks must reach the CUs first (a CU that holds two blocks of the other launch has no room for
      // one of these until both are gone), so this launch stays on the caller's stream and the other one, a few
      // microseconds behind because it waits for the fork event, goes down the second stream.
      side_lock = std::unique_lock<std::mutex>(side->mu);  // one fork / join at a time per device
      if (hipEventRecord(side->fork, stream) != hipSuccess || hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess)
        MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "grouped matmul: cannot order the second stream behind the caller's: %s", hipGetErrorString(hipGetLastError()));
      pl.big_tile_rows = (int)(T / 256);
      pl.share_bias = tuning().grouped_share;  // (0.5 measured: the model overrates the other launch's need of CUs)
      const int64_t pairs = (int64_t)lgrid.x * lgrid.y;
      const int cus = compute_units();
      lgrid = dim3((unsigned)(pairs < cus ? pairs : cus));
    }
    const int rc = blockscale ? launch_grouped_large<256, 256, 2, 4, 2>(pl, lgrid, stream, "gemm_grouped_block_256x256")
                              : launch_grouped_large<256, 256, 2, 4, 2, false>(pl, lgrid, stream, "gemm_grouped_row_256x256");
    if (rc != MAXFP8_OK) return rc;
  }
  // (every return below this line goes through join(): the caller's stream must wait for the second one)
  auto join = [&](int rc) -> int {
    if (side && (hipEventRecord(side->join, side->stream) != hipSuccess || hipStreamWaitEvent(stream, side->join, 0) != hipSuccess) &&
        rc == MAXFP8_OK)
      MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "grouped matmul: cannot join the second stream: %s", hipGetErrorString(hipGetLastError()));
    return rc;
  };
  // a slot owns one small tile or ceil(rows / BM) tiles: their sum is <= T / BM + num_active
  const int64_t m_tiles = T / bm + p.num_active;
  if (m_tiles > 65535) {
    join(MAXFP8_OK);
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped matmul: %lld row tiles exceed the launch limit", (long long)m_tiles);
  }
  const dim3 grid((unsigned)ceil_div(p.N, 128), (unsigned)m_tiles);
  hipStream_t rest_stream = side ? side->stream : stream;
  if (!blockscale) {
    if (big) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped rowwise matmul: the 256 x 128 shape is not built");
    return join(launch_grouped<128, 128, 2, 2, 2, 32, 1, 4, 3, false>(p, grid, rest_stream, "gemm_grouped_row_128x128"));
  }
  if (big) return launch_grouped<256, 128, 4, 2, 3, 64, 2, 4, 3>(p, grid, stream, "gemm_grouped_block_256x128");
  return join(launch_grouped<128, 128, 2, 2, 2, 32, 1, 4, 3>(p, grid, rest_stream, "gemm_grouped_block_128x128"));
}

}  // namespace maxfp8
