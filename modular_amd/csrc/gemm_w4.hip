// Scaled FP8 matmul on gfx950 with FOUR waves per block, one wave per SIMD:  C[M,N] = A[M,K] . B[N,K]^T.
//
// The layout of max/kernels/src/linalg/matmul/gpu/amd/amd_4wave_matmul.mojo:13-33,415-419 (a 2 x 2 grid of waves, every
// wave alone on its SIMD with the SIMD's whole register file) built for the block-scaled sum of
// max/kernels/src/linalg/fp8_quantization.mojo:1576-1624, whose per-slab promotion acc += P * (a_s * b_s) needs the
// accumulators as VALU operands: a wave owns 96 x 128 of a 192 x 256 tile (192 accumulator registers, ordinary VGPRs),
// the products of the MFMAs in flight take 16 more, and the operand fragments live in the other half of the register
// file (AGPRs: ds_read_b128 writes them and v_mfma reads its A / B operands from them directly).  The file is compiled
// with the MFMA results forced into VGPRs (-amdgpu-mfma-vgpr-form): left to its own choice the compiler puts them into
// AGPRs as soon as a kernel uses any and copies every product back for the promotion.
//
// Against eight waves of 128 x 64 on a 256 x 256 tile: 0.58 instead of 0.75 fragment reads per MFMA, four instead of
// eight waves at the slab's barrier, and a wave that never shares its SIMD's issue slots.
//
// Pipeline of a block (persistent: one block per CU walks its share of the tiles, the slab stream never stops at a tile
// boundary).  The registers are a pipeline stage of their own: a wave holds TWO sets of fragment registers, multiplies
// slab s from one and reads ALL fragments of slab s + 1 from LDS into the other meanwhile, one fragment every third
// MFMA.  So at the barrier of slab s (the slab's first instruction) nobody reads slab s's LDS any more, and what the
// barrier publishes -- slab s + 1, copied during slab s - 1 -- is not needed by any MFMA before the next barrier: no
// wave waits for LDS behind a barrier.  LDS holds TWO stages of activation rows (+ the slab's activation scales) and
// THREE stages of weight rows: weight tiles are read by one XCD at a time and come from HBM, activation tiles are read
// by all eight at once and mostly come from the memory-side cache, so the third stage goes to the operand with the
// longer way.  Behind the barrier of slab s a wave issues, one copy every third MFMA, the activation rows (and scales)
// of slab s + 2 into the stage slab s has left, then the weight rows of slab s + 3 into the weight stage it has left.
//
// Vector memory operations of a wave complete in order: at barrier s the wave may still have the PER_B weight copies of
// slab s + 2 in flight (and, in front of a tile's first slab, the NSTORE stores of the tile before, which sit between
// them and the activation copies in issue order), so the waits are exact counts.
//
// Promotion: the MFMA of (16-row group mt, fragment nt) writes a fresh product, and the four FMAs that fold it into the
// accumulators are issued LAG MFMAs later, when the product has left the matrix pipe.
//
// Tiles: any M and any N that is a multiple of 8 (rows of either operand past the end read as zero through the buffer
// descriptors, stores of rows past M fall outside C's descriptor, lanes whose columns lie past N store nothing), K an
// even number (at least four) of whole 128-byte slabs (the two sets of fragment registers alternate).
// Sums are formed in the same order as by the eight-wave kernels (one product per slab, promoted in slab order):
// results are bit-equal to theirs.
//
// The last round.  Tiles are dealt out in whole rounds of the blocks; what is left for a last round is often a fraction
// of a round, and its tiles take as long as any.  Where the caller brings a workspace, the tiles beyond the last whole
// round are cut along K into two to four pieces, a block per piece (see the job list in w4_body): the blocks of a tile
// share its rows out between them, exchange the f32 sums of each other's rows through the workspace, and each adds up,
// converts and stores its own rows.  These sums are added in another order than the uncut kernel's: equal where every
// sum is exact, a bf16 step apart at most elsewhere; the same bits from launch to launch.
#include <stdlib.h>

#include <atomic>

#include "common.h"
#include "gemm_args.h"
#include "gemm_device.h"
#include "tuning.h"

namespace maxfp8 {

int compute_units();

// a scalar load (the address is the same in every lane): through the constant address space, so that it does not
// take a place in the wave's queue of vector memory operations, whose in-order completion the copy waits count on
__device__ __forceinline__ float scalar_load_f32(const float* ptr) {
  typedef __attribute__((address_space(4))) const float* const_ptr_t;
  return *(const_ptr_t)(uintptr_t)ptr;
}

// A fragment belongs in the accumulation registers: the load writes them, the MFMA reads them, nothing else touches it.
// (Without the hint the allocator fills the ordinary registers with fragments first and then spills accumulators.)
__device__ __forceinline__ v8i in_agprs(v8i f) {
  asm("" : "+a"(f));
  return f;
}

// x, as a value the optimiser cannot see through and that is the same in every lane (in a scalar register)
__device__ __forceinline__ int opaque_uniform(int x) {
  asm volatile("" : "+v"(x));
  return __builtin_amdgcn_readfirstlane(x);
}

// the lane's number, formed where it is asked for (from the execution mask) and opaque to the optimiser: a value that
// is wanted only behind the slab loop then occupies no register across it
__device__ __forceinline__ int lane_here() {
  int l = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  asm volatile("" : "+v"(l));
  return l;
}

// the immediate of s_waitcnt on gfx9: vmcnt in bits 3:0 and 15:14, expcnt (left at its maximum) in 6:4, lgkmcnt in 11:8
constexpr int waitcnt_imm(int vmcnt, int lgkmcnt) { return (vmcnt & 15) | ((vmcnt >> 4) << 14) | (7 << 4) | (lgkmcnt << 8); }

// Flags of the tail pieces: a set per launch in flight (handed out round-robin: the first half to ordinary launches,
// the second to launches recorded into a graph, which replay with the set of the recording), and in a set a word per
// block and reader (a tile has at most kW4MaxPieces pieces).  A flag is raised by the block that wrote its sums and put
// back to zero by the one block it is meant for, so a launch leaves its set as it found it.  And the count of pieces a
// block gave up waiting for.
constexpr int kW4FlagSets = 64, kW4MaxBlocks = 512, kW4MaxPieces = 8;
static __device__ unsigned int g_w4_flags[kW4FlagSets * kW4MaxBlocks * kW4MaxPieces];
static __device__ unsigned int g_w4_gave_up;

// PROBE (measurement aid, results meaningless): 0 the matmul; 1 the same loop with every copy reading tile (0, 0) and
// slabs 0..7 over and over, so that its operands stay in L2; 2 the same without copies, waits and barriers -- the
// MFMA loop on what the prologue left in LDS.
//
// GROUPED (the MoE matmul -- rows sorted by expert, slot z = rows [offsets[z], offsets[z + 1]) times the weights of expert
// expert_ids[z], zeros where that is -1: max/kernels/src/linalg/grouped_matmul_sm100_blockwise_fp8.mojo:2938-3105,
// grouped_matmul.mojo:1440-1713 for row scaling; BM = 192): the tiles are those of w4_grouped_head_rows of every slot -- its full
// BM-row tiles and one more for a rest of more than 128 rows, stored up to the slot's end --
// numbered through all slots as if they were the row tiles of one matrix: row tile v lies in the slot
// found by bisection in a prefix table that every block builds in LDS from the device-resident offsets, and its weights
// are that slot's expert's.  The other rows are another launch's, sent down a second stream at the same time: this
// launch is issued first with a block per CU, every block adds up what both launches have to do (tiles x the cost
// model's time per tile), and the blocks past this launch's share of the chip exit at once and leave their CUs to the
// other one.
constexpr int kW4GroupedSlots = 256;  // slots (active experts) the tables hold, one per thread
constexpr int kW4GroupedTableBytes = (16 + 4 * kW4GroupedSlots + 8) * 4 + 4 * 96 * 4;  // (and the index entries of a tile's 96 rows, per wave)

//
// GROUPED == 2: with a row index on C (row m of the result goes to row p.c_row_index[m]).  The index entries of a tile's
// rows are copied into LDS by two more copy instructions per wave, issued behind the stores of the tile before (in front
// of the first tile: in the prologue) -- not loaded into registers in the epilogue, where waiting for such a load would
// mean waiting for every weight copy in flight, in-order completion being what the copy waits rely on.
template <int TM, int TN, bool BLOCKSCALE, int PROBE, int GROUPED = 0>
__device__ __forceinline__ void w4_body(const GemmArgs& p, uint8_t* smem) {
  constexpr int WM = TM * 16, WN = TN * 16, BM = 2 * WM, BN = 2 * WN;
  constexpr int IA = BM / 32, IB = BN / 32;                  // copy instructions per wave and slab (8 rows each)
  constexpr int SCALE_BYTES = BLOCKSCALE ? 1024 : 0;         // 2 wave rows x 16 lane rows x 8 words
  constexpr int A_STAGE = BM * 128 + SCALE_BYTES, B_STAGE = BN * 128;
  constexpr int B_BASE = 2 * A_STAGE, SIDE_BASE = B_BASE + 3 * B_STAGE, SIDE_BYTES = 2048;
  constexpr int PER_A = IA + (BLOCKSCALE ? 1 : 0), PER_B = IB;
  constexpr int NSTORE = TM * TN / 2;                        // 16-byte stores per lane and tile
  // a product is folded in LAG MFMAs after its own (2: 4 ... 6 % slower, the FMAs then wait for the matrix pipe; 4: the same)
  constexpr int LAG = 3;
  static_assert(TN == 8 && TM >= 3 && TM <= 8, "wave tile");
  // Row tiles that share weight columns in the tile order: the 32 blocks of an XCD work on a patch of kGroupM row tiles
  // x 32 / kGroupM column tiles at a time, and what the XCD's L2 fetches for it is the patch's rows of both operands --
  // least for a square patch: 8 x 4 for 128-row tiles (q_b M = 1024: 47 -> 43 us against 4 x 8; o_proj M = 1024: 112 ->
  // 109), 4 x 8 for the taller ones (3, 6 and 8 row tiles measured within a per cent of 4 on the long-K shapes, 8 a seventh
  // slower on kv_b M = 4096).
  constexpr int kGroupM = TM == 4 ? 8 : 4;
  static_assert(PER_B + NSTORE < 64, "the count must fit the vmcnt field");
  static_assert(IB % 2 == 0, "the weight copies go out in two halves");

  static_assert(!GROUPED || PROBE == 0, "the probe runs the dense form");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int lm = lane & 15, lq = lane >> 4;
  const int nslab = p.K / 128;                               // whole slabs, an even number of them (the host's rule)

  // ---- grouped: the tables (behind the side buffers).  hdr[0] = row tiles of all slots, hdr[1] = the blocks that stay,
  // hdr[3] / hdr[4] = the other launch's row tiles (rests of more than small_rows rows / of fewer), hdr[8..11] = the
  // waves' sums of the scan; tab_tiles[z] = row tiles in the slots before z, tab_begin[z] / tab_end[z] = slot z's rows,
  // tab_expert[z] = its expert; then, per wave, the index entries of a tile's rows (GROUPED == 2).
  int* const hdr = reinterpret_cast<int*>(smem + SIDE_BASE + 4 * SIDE_BYTES);
  int* const tab_tiles = hdr + 16;                     // (kW4GroupedSlots + 1 entries: the last is the total)
  int* const tab_begin = tab_tiles + kW4GroupedSlots + 8;
  int* const tab_expert = tab_begin + kW4GroupedSlots;
  int* const tab_end = tab_expert + kW4GroupedSlots;
  constexpr bool SCATTER = GROUPED == 2;
  uint32_t* const idx_lds = reinterpret_cast<uint32_t*>(tab_end + kW4GroupedSlots) + wave * 96;  // this wave's rows' entries
  if constexpr (GROUPED) {
    static_assert(BM == 192, "w4_grouped_head_rows");
    const int na = p.num_active;
    if (tid < 16) hdr[tid] = 0;
    __syncthreads();
    int c = 0, begin = 0, end = 0, e = -1;
    if (tid < na) {
      // (rows held inside [0, M): a stale routing tensor must not turn into accesses outside the operands)
      const int64_t M = p.M;
      int64_t b64 = p.offsets[tid], e64 = p.offsets[tid + 1];
      if (b64 > M) b64 = M;
      if (e64 > M) e64 = M;
      if (e64 < b64) e64 = b64;
      const int rows = (int)(e64 - b64);
      const int head = w4_grouped_head_rows(rows, p.w4_hot_rest, p.w4_cold_rows), rest = rows - head;
      c = (head + BM - 1) / BM;
      begin = (int)b64;
      end = (int)e64;
      e = p.expert_ids[tid];
      // the other launch's tiles, for the shares: a rest of more than small_rows, of anything
      if (rest > p.small_rows) atomicAdd(&hdr[3], 1);
      else if (rest > 0) atomicAdd(&hdr[4], 1);
    }
    int incl = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    int* const s_wave_sum = hdr + 8;  // (no static LDS in this kernel: it would push the stages past the block's 160 KB)
    if (lane == 63) s_wave_sum[wave] = incl;
    __syncthreads();
    int before = 0;
    for (int w = 0; w < wave; ++w) before += s_wave_sum[w];
    tab_tiles[tid] = before + incl - c;
    if (tid == 255) tab_tiles[256] = before + incl;
    tab_begin[tid] = begin;
    tab_expert[tid] = e;
    tab_end[tid] = end;
    if (tid == 255) {
      const int R = before + incl;
      const float ns = (float)nslab;
      const int ncol = (p.N + BN - 1) / BN;
      // (microseconds of one CU: this launch's tiles; the other launch's 128 x 256 tiles and its weight-streaming tiles of
      // 512 columns, as its own blocks price them)
      // (row scaling: the same figure although its tiles are a seventh faster -- priced at 1.0 the launch kept fewer
      // blocks and the pair took 805 instead of 750 microseconds on the 7168 x 2048 shape)
      const float w_here = (float)(R * ncol) * (ns * 1.15f + 3.0f);
      const float w_there = (float)(hdr[3] * ((p.N + 255) / 256)) * (ns * 0.92f + 9.0f) +
                            (float)(hdr[4] * ((p.N + 511) / 512)) * (ns * 2.6f + 6.0f) * p.share_bias;
      const int G = (int)gridDim.x & ~7;
      int keep = (int)((float)G * w_here / (w_here + w_there + 1e-9f) + 4.0f) & ~7;
      if (p.share_bias < 0.f) keep = (int)(-p.share_bias) & ~7;  // (tuning runs: the number itself)
      if (keep < 8) keep = 8;
      if (keep > G) keep = G;
      if (keep > R * ncol) keep = (R * ncol + 7) & ~7;
      // (the tiles are dealt out in whole rounds of the blocks that stay: no more blocks than that number of rounds needs)
      if (p.share_bias >= 0.f && R > 0) {
        const int rounds = (R * ncol + keep - 1) / keep;
        keep = (((R * ncol + rounds - 1) / rounds) + 7) & ~7;
      }
      hdr[0] = R;
      hdr[1] = R > 0 ? keep : 0;
    }
    __syncthreads();
    if ((int)blockIdx.x >= hdr[1]) return;
  }
  auto grouped_hdr = [&](int i) { return __builtin_amdgcn_readfirstlane(hdr[i]); };

  // ---- this block's tiles: every nb-th tile of its XCD's contiguous run (blocks are dealt to the XCDs round-robin)
  const int tiles_m = GROUPED ? grouped_hdr(0) : (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN, total = tiles_m * tiles_n;
  const int bs_rows = (p.N + 127) / 128;  // rows of the weight scales: a wave whose columns all lie past N reads the last one
  // The tail (p.tail_units = u > 0; the host then launches a multiple of 8 blocks and no more than there are tiles): the
  // T tiles beyond the last whole round of the blocks are not dealt out whole.  Each is cut along K into pieces of u slabs
  // (P = ceil(slabs / u) of them, the same cuts in every tile; u and the slabs of a tile are multiples of 4, so every
  // piece is at least four slabs and an even number; T P is no more than the blocks), and block number c (blocks of an
  // XCD next to each other) takes piece c / T of tile c % T: the last round then takes the time of a piece, and the
  // blocks of an XCD walk the same slabs of neighbouring tiles in step, as they do in the whole rounds -- they find each
  // other's operands in their L2.
  //
  // A job: slabs [s0, s1) of a tile.  WHOLE: all of them, the tile is stored.  PIECE: one of the P pieces of a tail tile.
  // The P blocks of a tile share its rows out between them (step st of every wave's epilogue -- 16 rows x 64 columns -- belongs to piece st P / (2 TM)):
  // a block writes the sums of the other blocks' rows to its slot of the workspace, raises a flag for each of them, then
  // waits for theirs, adds their sums of its own rows to its own (own first, then the others in the order of their
  // slabs: the same order on every launch) and stores those rows of the tile.  Nobody waits before it has published, so
  // nobody waits for a block that waits; each block moves (P - 1) / P of a tile each way and converts 1 / P of it.
  //
  // (Jobs are worked out from the block's number every time one begins, behind a value the optimiser cannot see through:
  // kept in scalar registers across the slab loop, the block's bookkeeping pushed the loop's own values out.)
  enum { WHOLE = 0, PIECE = 1 };
  struct Job { int tile, s0, s1, kind; };
  struct Plan { int main_total, run_begin, nb, my, n_main, tail_c, tail_u; };
  auto plan_of = [&]() {
    const int bid = opaque_uniform((int)blockIdx.x), G = GROUPED ? grouped_hdr(1) : (int)gridDim.x;
    const int xcd = bid & 7, my = bid >> 3;
    const int tail_u = PROBE || GROUPED ? 0 : p.tail_units;
    const int main_total = tail_u > 0 ? (total / G) * G : total;
    const int run_begin = xcd * (main_total >> 3) + (xcd < (main_total & 7) ? xcd : (main_total & 7));
    const int run_len = (main_total >> 3) + (xcd < (main_total & 7) ? 1 : 0);
    const int nb = (G - xcd + 7) >> 3;
    const int n_main = PROBE ? 1 : (my < run_len ? (run_len - my + nb - 1) / nb : 0);
    return Plan{main_total, run_begin, nb, my, n_main, xcd * (G >> 3) + my, tail_u};
  };
  // job k of this block; k == n_main: its piece of the tail, if it has one; *count = the number of jobs
  auto job_of = [&](int k, int* count) {
    const Plan pl = plan_of();
    Job tail = {0, 0, 0, WHOLE};
    int n_tail = 0;
    if (pl.tail_u > 0) {
      const int T = total - pl.main_total, P = (nslab + pl.tail_u - 1) / pl.tail_u;
      if (pl.tail_c < T * P) {
        const int q = pl.tail_c / T, s0 = q * pl.tail_u, s1 = min(s0 + pl.tail_u, nslab);
        tail = Job{pl.main_total + (pl.tail_c - q * T), s0, s1, P > 1 ? PIECE : WHOLE};
        n_tail = 1;
      }
    }
    if (count) *count = pl.n_main + n_tail;
    if (k < pl.n_main) return Job{pl.run_begin + pl.my + k * pl.nb, 0, nslab, WHOLE};
    return tail;
  };
  int njobs = 0;
  Job job = job_of(0, &njobs);
  if (njobs <= 0) return;

  // ---- global -> LDS copy plan (LDS-DMA, 16 bytes per lane, 8 rows x 128 bytes per instruction; lane (r, p) fetches
  // the chunk p ^ f(row) of its row, so the bytes land swizzled for conflict-free fragment reads)
  const __amdgpu_buffer_rsrc_t a_rsrc = t2_rsrc(p.a, t2_clamp_u32((int64_t)(p.M - 1) * p.lda + p.K));
  const uint32_t b_range = t2_clamp_u32((int64_t)(p.N - 1) * p.ldb + p.K);
  const __amdgpu_buffer_rsrc_t b_rsrc = t2_rsrc(p.b, b_range);
  const int cr = lane >> 3, cp = lane & 7;
  const int cchunk = cp ^ cr;
  const int cchunk_b = cp ^ (((wave & 1) << 2) | (cr & 3));
  const uint32_t a_voff = (uint32_t)(wave * 8 + cr) * (uint32_t)p.lda + cchunk * 16;
  const uint32_t b_voff = (uint32_t)(wave * 8 + cr) * (uint32_t)p.ldb + cchunk_b * 16;
  const uint32_t a_istep = 32u * (uint32_t)p.lda, b_istep = 32u * (uint32_t)p.ldb;
  // the slab's activation scales: word wm * 128 + lm * 8 + mt of the scale area holds the scale of row wm * WM + mt * 16
  // + lm, so that a lane finds its TM scales in 32 consecutive bytes; wave w copies words [64 w, 64 w + 64)
  __amdgpu_buffer_rsrc_t s_rsrc = t2_rsrc(nullptr, 0);
  uint32_t s_voff = 0, s_slab_step = 0;
  if constexpr (BLOCKSCALE) {
    s_rsrc = t2_rsrc(p.a_scales, t2_clamp_u32(((int64_t)(nslab - 1) * p.a_scales_ld + p.M) * 4));
    const int word = wave * 64 + lane, mt_w = word & 7, lm_w = (word >> 3) & 15, wm_w = word >> 7;
    s_voff = (uint32_t)(wm_w * WM + mt_w * 16 + lm_w) * 4u;
    if (mt_w >= TM) s_voff = 0x80000000u;
    s_slab_step = (uint32_t)p.a_scales_ld * 4u;
  }
  // byte offsets of a tile's activation rows, weight rows and activation scales; its first row; grouped: its expert's
  // weights and the element of the weight scales where the expert's begin
  struct TileAt { uint32_t a, b, s; int row0, row_end; const uint8_t* bp; uint32_t bs0; };
  // (grouped: tm = the row tile's number among its slot's, slot = that slot)
  auto tile_at = [&](int tm, int tn, int slot) {
    if constexpr (PROBE != 0) return TileAt{0u, 0u, 0u, 0, 0, p.b, 0u};
    if constexpr (GROUPED) {
      const int lo = slot;
      const int row0 = __builtin_amdgcn_readfirstlane(tab_begin[lo]) + tm * BM;
      const int e = __builtin_amdgcn_readfirstlane(tab_expert[lo]), row_end = __builtin_amdgcn_readfirstlane(tab_end[lo]);
      // (no expert: the weight copies read out of range, i.e. zeros, and the tile is stored as zeros)
      const uint32_t none = e < 0 ? 0x80000000u : 0u;
      const int ee = e < 0 ? 0 : e;
      return TileAt{(uint32_t)row0 * (uint32_t)p.lda, ((uint32_t)(tn * BN) * (uint32_t)p.ldb) | none, (uint32_t)row0 * 4u, row0, row_end,
                    p.b + (int64_t)ee * p.b_expert_stride, (uint32_t)((int64_t)ee * p.bs_expert_stride)};
    }
    return TileAt{(uint32_t)(tm * BM) * (uint32_t)p.lda, (uint32_t)(tn * BN) * (uint32_t)p.ldb, (uint32_t)(tm * BM) * 4u, tm * BM, p.M, p.b, 0u};
  };
  // copy number idx (0 .. PER_A - 1) of a slab's activation rows and scales into activation stage `stage`
  // Where a slab's copies read: the scalar offsets of its first activation, weight and scale copy.  A slab of nothing
  // (behind the block's last tile) gets offsets past 2^31: the scalar offset takes part in the descriptor's range
  // check, so such copies write zeros.  (K is a whole number of slabs: no lane ever reads past a row's end.)
  struct SlabAt { uint32_t a, b, s; const uint8_t* bp; };
  auto slab_at = [&](const TileAt& at, int slab, uint32_t dead) {
    if constexpr (PROBE != 0) slab &= 7;
    const uint32_t koff = (uint32_t)slab * 128u;
    return SlabAt{(at.a + koff) | dead, (at.b + koff) | dead, (at.s + (uint32_t)slab * s_slab_step) | dead, at.bp};
  };
  // copy number idx (0 .. PER_A - 1) of a slab's activation rows and scales into activation stage `stage`
  auto dma_a = [&](const SlabAt& at, int stage, int idx) {
    uint8_t* sa = smem + stage * A_STAGE;
    if (idx < IA) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr_t)(sa + (idx * 4 + wave) * 1024), 16, a_voff, at.a + idx * a_istep, 0, 0);
    } else if constexpr (BLOCKSCALE) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(s_rsrc, (lds_ptr_t)(sa + BM * 128 + wave * 256), 4, s_voff, at.s, 0, 0);
    }
  };
  // copy number idx (0 .. PER_B - 1) of a slab's weight rows into weight stage `stage`
  auto dma_b = [&](const SlabAt& at, int stage, int idx) {
    uint8_t* sb = smem + B_BASE + stage * B_STAGE;
    // (grouped: the descriptor of the expert whose rows this slab's copies read)
    const __amdgpu_buffer_rsrc_t rsrc = GROUPED ? t2_rsrc(at.bp, b_range) : b_rsrc;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)(sb + (idx * 4 + wave) * 1024), 16, b_voff, at.b + idx * b_istep, 0, 0);
  };

  // ---- fragment read plan.  Activation fragment mt: rows mt * 16 + lm of the wave's rows.  Weight fragments come in
  // pairs over 32 weight rows, MFMA row i <-> weight row 8 * (i / 4) + i % 4 (+ 4 for the odd fragment), which leaves a
  // lane with 8 consecutive columns of C per pair.
  const int sw = lm & 7;
  const uint8_t* a_frag = smem + (uint32_t)(wm * WM) * 128 + lm * 128;
  const uint32_t a_lo = (uint32_t)((lq ^ sw) << 4), a_hi = (uint32_t)(((lq + 4) ^ sw) << 4);
  auto read_afrag = [&](int stage, int mt) -> v8i {
    const uint8_t* g = a_frag + stage * A_STAGE + mt * 2048;
    const v4i lo = *reinterpret_cast<const v4i*>(g + a_lo);
    const v4i hi = *reinterpret_cast<const v4i*>(g + a_hi);
    return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  const int wrow = 8 * (lm >> 2) + (lm & 3);
  const int wsw = (((wrow >> 3) & 1) << 2) | (wrow & 3);
  const uint8_t* b_frag = smem + B_BASE + (uint32_t)(wn * WN) * 128 + wrow * 128;
  const uint32_t b_lo = (uint32_t)((lq ^ wsw) << 4), b_hi = (uint32_t)(((lq + 4) ^ wsw) << 4);
  auto read_bfrag = [&](int stage, int t) -> v8i {
    const uint8_t* g = b_frag + stage * B_STAGE + (t >> 1) * 4096 + (t & 1) * 512;
    const v4i lo = *reinterpret_cast<const v4i*>(g + b_lo);
    const v4i hi = *reinterpret_cast<const v4i*>(g + b_hi);
    return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  struct Scales { float v[TM]; };
  const uint8_t* s_rd = smem + BM * 128 + (wm * 128 + lm * 8) * 4;
  auto read_scales = [&](int stage) -> Scales {
    Scales out;
    const v4f lo = *reinterpret_cast<const v4f*>(s_rd + stage * A_STAGE);
    out.v[0] = lo[0]; out.v[1] = lo[1]; out.v[2] = lo[2]; out.v[3] = lo[3];
    if constexpr (TM > 6) {
      const v4f hi = *reinterpret_cast<const v4f*>(s_rd + stage * A_STAGE + 16);
      out.v[4] = hi[0]; out.v[5] = hi[1]; out.v[6] = hi[2];
      if constexpr (TM > 7) out.v[7] = hi[3];
    } else if constexpr (TM > 5) {
      const v2f hi = *reinterpret_cast<const v2f*>(s_rd + stage * A_STAGE + 16);
      out.v[4] = hi[0]; out.v[5] = hi[1];
    } else if constexpr (TM > 4) {
      out.v[4] = *reinterpret_cast<const float*>(s_rd + stage * A_STAGE + 16);
    }
    return out;
  };

  // ---- where C goes: through a 2 KB side buffer per wave, 16 rows x 64 columns at a time, so that a store instruction
  // writes 8 rows x one whole 128-byte line
  uint8_t* wbuf = smem + SIDE_BASE + wave * SIDE_BYTES;
  const __amdgpu_buffer_rsrc_t c_rsrc = t2_rsrc(p.c, t2_clamp_u32(((int64_t)(p.M - 1) * p.ldc + p.N) * 2));
  const uint32_t c_row_bytes = (uint32_t)p.ldc * 2u;

  // Where tile number t lies.  Grouped: the tiles are numbered slot by slot, in a slot column by column, in a column
  // row tile by row tile (large slots: see below) -- the blocks of an XCD, which take neighbouring numbers, work on all row tiles of a few weight
  // columns of one expert at a time (each weight tile comes from memory once), and an XCD's run of the numbers is a run
  // of slots: the weights of an expert are read by one XCD or two.
  auto locate = [&](int t, int& tm, int& tn, int& slot) {
    slot = 0;
    if constexpr (GROUPED) {
      // the last z with tab_tiles[z] * tiles_n <= t (slots without tiles repeat their successor's value and are skipped
      // by taking the last)
      const int v = t / tiles_n;
      int lo = 0, hi = p.num_active;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (__builtin_amdgcn_readfirstlane(tab_tiles[mid]) <= v) lo = mid; else hi = mid;
      }
      const int first = __builtin_amdgcn_readfirstlane(tab_tiles[lo]), c = __builtin_amdgcn_readfirstlane(tab_tiles[lo + 1]) - first;
      const int rem = t - first * tiles_n;
      // (a slot of more than 24 row tiles: in groups of 12 row tiles, or every pass over a weight column would fetch all
      // of the slot's activation rows again -- one expert of 83 row tiles: 3.85 against 4.34 ms for the launch; up to 24
      // the one group measured level or a per cent ahead)
      if (c <= 24) {
        tn = rem / c;
        tm = rem - tn * c;
      } else {
        tile_coords<12>(rem, c, tiles_n, tm, tn);
      }
      slot = lo;
    } else {
      tile_coords<kGroupM>(t, tiles_m, tiles_n, tm, tn);
    }
  };
  // the index entries of the 96 rows of this wave in the tile that begins at row0: lane l copies entry l, and lanes 0 .. 31
  // entry 64 + l (entries past the end of the index read as zero: such rows are not stored).  Two vector memory
  // operations for every lane's count, whether or not the lane takes part in the second.
  auto dma_idx = [&](int row0) {
    if constexpr (SCATTER) {
      static_assert(!SCATTER || WM == 96, "two copies of 64 and 32 entries");
      const __amdgpu_buffer_rsrc_t i_rsrc = t2_rsrc(p.c_row_index, t2_clamp_u32((int64_t)p.M * 4));
      const int l = lane_here();
      const uint32_t at = (uint32_t)(row0 + wm * WM) * 4u;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(i_rsrc, (lds_ptr_t)idx_lds, 4, (uint32_t)l * 4u, at, 0, 0);
      // (under the execution mask: a lane whose offset is merely out of range would still write a zero, into the next
      // wave's entries)
      if (l < 32) __builtin_amdgcn_raw_ptr_buffer_load_lds(i_rsrc, (lds_ptr_t)(idx_lds + 64), 4, (uint32_t)l * 4u, at + 256u, 0, 0);
    }
  };
  // ---- prologue: slabs 0 and 1 of the first tile
  int tm, tn, slot;
  locate(job.tile, tm, tn, slot);
  if constexpr (PROBE != 0) tm = tn = 0;
  TileAt cur_at = tile_at(tm, tn, slot);
  dma_idx(cur_at.row0);
  {
    const SlabAt s0 = slab_at(cur_at, job.s0, 0u), s1 = slab_at(cur_at, job.s0 + 1, 0u), s2 = slab_at(cur_at, job.s0 + 2, 0u);
#pragma unroll
    for (int idx = 0; idx < PER_A; ++idx) dma_a(s0, 0, idx);
#pragma unroll
    for (int idx = 0; idx < PER_B; ++idx) dma_b(s0, 0, idx);
#pragma unroll
    for (int idx = 0; idx < PER_A; ++idx) dma_a(s1, 1, idx);
#pragma unroll
    for (int idx = 0; idx < PER_B; ++idx) dma_b(s1, 1, idx);
#pragma unroll
    for (int idx = 0; idx < PER_B; ++idx) dma_b(s2, 2, idx);
  }
  if constexpr (PROBE == 2) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PER_A + 2 * PER_B) : "memory");
  }
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

  // (BN = 256: two weight-scale blocks per tile, one per wave column)
  auto bs_block = [&](int tile_n) {
    if constexpr (PROBE != 0) return wn;
    const int blk = 2 * tile_n + wn;
    return blk < bs_rows ? blk : bs_rows - 1;
  };
  // The weight-block scale of a slab is element bs_cur of the weight scales: that of the slab to come is loaded a slab ahead.
  uint32_t bs_cur = cur_at.bs0 + (uint32_t)(bs_block(tn) * p.b_scales_ld + job.s0);
  float bs_nxt = 1.f;
  if constexpr (BLOCKSCALE) bs_nxt = scalar_load_f32(p.b_scales + bs_cur);

  // two sets of fragment registers: a slab is multiplied from one while the next slab's fragments arrive in the other
  v8i bf[2][TN], af[2][TM];
  Scales sraw[2];
#pragma unroll
  for (int t = 0; t < TN; ++t) bf[0][t] = read_bfrag(0, t);
#pragma unroll
  for (int mt = 0; mt < TM; ++mt) af[0][mt] = read_afrag(0, mt);
  if constexpr (BLOCKSCALE) sraw[0] = read_scales(0);
#pragma unroll
  for (int t = 0; t < TN; ++t) bf[0][t] = in_agprs(bf[0][t]);
#pragma unroll
  for (int mt = 0; mt < TM; ++mt) af[0][mt] = in_agprs(af[0][mt]);

  // (probe: the core clock's cycle counter and the constant 100 MHz counter, around the slab loop)
  [[maybe_unused]] uint64_t probe_c0 = 0, probe_r0 = 0;
  if constexpr (PROBE != 0) {
    probe_c0 = clock64();
    probe_r0 = wall_clock64();
  }

  int bst = 0;          // weight stage of the slab being multiplied
  bool stored = false;  // a tile's stores sit in front of the weight copies now in flight
  // Where the copies of the slab about to start read: the activation rows (and scales) of its slab + 2, the weight rows
  // of its slab + 3.  Running offsets, 128 bytes (one row of scales) further with every slab, set to the next tile's
  // first slab when they pass the end of K -- a handful of scalar instructions per slab; worked out from the slab number
  // every time they were two dozen, and a wave alone on its SIMD pays for every instruction it issues.
  SlabAt cur = slab_at(cur_at, job.s0 + 2, 0u);
  cur.b = slab_at(cur_at, job.s0 + 3, 0u).b;

  // the pieces of tail tiles travel through the workspace: slot c = the sum of block c's PART, 64 lanes x 16 bytes per
  // fragment; flags (one per block and launch in flight) say that a slot is written.  The hand-over crosses XCDs, whose L2s
  // are not coherent with each other: stores and loads of the slots carry the device-scope cache policy.
  constexpr int SLOT_BYTES = BM * BN * 4;
  constexpr int kDeviceScope = 17;  // sc0 | sc1

  for (int k = 0; k < njobs; ++k) {
    const bool has_next = k + 1 < njobs;
    const Job next_job = has_next ? job_of(k + 1, nullptr) : job;
    int tm2 = tm, tn2 = tn;
    int slot2 = slot;
    if (has_next) locate(next_job.tile, tm2, tn2, slot2);
    const TileAt next_at = tile_at(tm2, tn2, slot2);
    // the first slab of the next job (of nothing behind the block's last one: offsets past 2^31 read as zeros)
    const SlabAt next0 = slab_at(next_at, next_job.s0, has_next ? 0u : 0x80000000u);
    const uint32_t next_bs0 = next_at.bs0 + (uint32_t)(bs_block(tn2) * p.b_scales_ld + next_job.s0);
    const int job_end = job.s1;

    v4f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    // One slab.  PAR = its parity = its activation stage = the set of fragment registers it multiplies from.
    // AFTER_STORES: the tile before this one has just been stored -- only a tile's first slab can be that.  A template flag
    // and not a branch at the wait: a branch would cut the slab's straight-line code in two, and the compiler schedules
    // each part on its own -- it then issued forty MFMAs in a row and parked their products in AGPRs.
    auto slab_body = [&](auto PAR_C, auto AFTER_STORES_C, const int slab) {
      constexpr int PAR = decltype(PAR_C)::value;
      constexpr bool AFTER_STORES = decltype(AFTER_STORES_C)::value;
      constexpr int NSLOT = TM * TN;            // MFMAs of the slab
      constexpr int NREAD = TN + TM + (BLOCKSCALE ? 1 : 0);  // fragments (and the scales) of the next slab
      constexpr int NCOPY = PER_A + PER_B;
      const int bst1 = bst == 2 ? 0 : bst + 1;  // weight stage of slab s + 1

      // ---- the barrier of slab s: this wave's copies of slab s + 1 have landed (its weight copies of slab s + 2, and a
      // tile's stores, may stay in flight) and its reads of slab s, issued during slab s - 1, have returned
      if constexpr (PROBE != 2) {
        // (the waits are the builtin, not inline assembly: the compiler's own bookkeeping of outstanding loads reads it, and
        // knows from here on that every fragment register has its value -- behind an opaque wait it guards the first use of
        // each with a wait of its own, which, with a scalar load in flight, is a wait for ALL of the slab's new reads)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(PER_B + (AFTER_STORES ? NSTORE : 0), 0));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
      }
      const SlabAt my = cur;
      // (the offsets of the next slab's copies: K has at least four slabs, so each of them passes the end of K once a tile)
      if constexpr (PROBE != 0) {
        cur.a = (cur.a + 128u) & 1023u;
        cur.b = (cur.b + 128u) & 1023u;
        cur.s = cur.s + s_slab_step == 8u * s_slab_step ? 0u : cur.s + s_slab_step;
      } else {
        cur.a = slab + 3 == job_end ? next0.a : cur.a + 128u;
        cur.s = slab + 3 == job_end ? next0.s : cur.s + s_slab_step;
        cur.b = slab + 4 == job_end ? next0.b : cur.b + 128u;
      }

      float s_cur[TM];
      if constexpr (BLOCKSCALE) {
        const float bs = bs_nxt;
#pragma unroll
        for (int mt = 0; mt < TM; ++mt) s_cur[mt] = sraw[PAR].v[mt] * bs;
        // the weight-block scale of the next slab (of the next tile behind this tile's last slab)
        if constexpr (PROBE != 0) bs_cur = (bs_cur & ~7u) | ((bs_cur + 1u) & 7u);
        else bs_cur = slab + 1 == job_end ? next_bs0 : bs_cur + 1u;
        bs_nxt = scalar_load_f32(p.b_scales + bs_cur);
      }
      [[maybe_unused]] v4f part[LAG + 1];
      // Slot i = MFMA i of the slab, the four FMAs of the product that left the pipe LAG MFMAs ago, and at most one
      // piece of memory work: a fragment read of slab s + 1 (two 16-byte LDS reads) or one copy instruction -- spread
      // evenly, because a wave that issues several of them in a row stalls on the queue and its matrix pipe drains.
      static_for<NSLOT>([&](auto I) {
        constexpr int i = decltype(I)::value, mt = i / TN, nt = i % TN;
        if constexpr (BLOCKSCALE) {
          constexpr v4f zero = {0.f, 0.f, 0.f, 0.f};
          part[i % (LAG + 1)] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[PAR][nt], af[PAR][mt], zero, 0, 0, 0, 0, 0, 0);
          if constexpr (i >= LAG) {
            constexpr int j = i - LAG;
            acc[j / TN][j % TN] += part[j % (LAG + 1)] * s_cur[j / TN];
          }
        } else {
          acc[mt][nt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[PAR][nt], af[PAR][mt], acc[mt][nt], 0, 0, 0, 0, 0, 0);
        }
        // read item r goes to slot r * NSLOT / NREAD: the scales, the weight fragments, the activation fragments
        constexpr int r = (i * NREAD + NSLOT - 1) / NSLOT;  // the first item whose slot is >= i
        if constexpr (r < NREAD && r * NSLOT / NREAD == i) {
          constexpr int f = r - (BLOCKSCALE ? 1 : 0);
          if constexpr (f < 0) sraw[PAR ^ 1] = read_scales(PAR ^ 1);
          else if constexpr (f < TN) bf[PAR ^ 1][f] = read_bfrag(bst1, f);
          else af[PAR ^ 1][f - TN] = read_afrag(PAR ^ 1, f - TN);
        }
        // copy d goes to slot d * NSLOT / NCOPY + 1: the activation rows and scales of slab s + 2 into the stage this slab
        // has left, then the weight rows of slab s + 3 into the weight stage it has left
        if constexpr (PROBE != 2 && i >= 1) {
          constexpr int d = ((i - 1) * NCOPY + NSLOT - 1) / NSLOT;
          if constexpr (d < NCOPY && d * NSLOT / NCOPY == i - 1) {
            if constexpr (d < PER_A) dma_a(my, PAR, d);
            // (grouped: the expert of the weight copies changes with their offset, but at the slab's end, behind these copies:
            // they read through cur.bp, and the old value need not be kept beside the new one)
            else if constexpr (GROUPED) dma_b(SlabAt{my.a, my.b, my.s, cur.bp}, bst, d - PER_A);
            else dma_b(my, bst, d - PER_A);
          }
        }
        // (nothing moves from one slot to another: left to itself the scheduler folds a product in right behind its own
        // MFMA and fills the wait with idle cycles, or runs a dozen MFMAs ahead and parks their products)
        __builtin_amdgcn_sched_barrier(0);
      });
      // (the slab's last products: folding them in during the first MFMAs of the next slab instead measured 7 % slower)
      if constexpr (BLOCKSCALE) {
#pragma unroll
        for (int j = NSLOT - LAG; j < NSLOT; ++j) acc[j / TN][j % TN] += part[j % (LAG + 1)] * s_cur[j / TN];
      }
      // (the hint sits at the slab's end, where the whole set has arrived: right behind a read it would be a use of the
      // value, and the compiler would wait for the read on the spot)
#pragma unroll
      for (int t = 0; t < TN; ++t) bf[PAR ^ 1][t] = in_agprs(bf[PAR ^ 1][t]);
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) af[PAR ^ 1][mt] = in_agprs(af[PAR ^ 1][mt]);
      bst = bst1;
      if constexpr (GROUPED) cur.bp = slab + 4 == job_end ? next0.bp : cur.bp;
    };

    constexpr std::integral_constant<int, 0> EVEN{};
    constexpr std::integral_constant<int, 1> ODD{};
    // (a job begins at an even slab and has an even number of slabs, four at least)
    if (stored) slab_body(EVEN, std::true_type{}, job.s0);
    else slab_body(EVEN, std::false_type{}, job.s0);
    slab_body(ODD, std::false_type{}, job.s0 + 1);
    for (int slab = job.s0 + 2; slab < job_end; slab += 2) {
      slab_body(EVEN, std::false_type{}, slab);
      slab_body(ODD, std::false_type{}, slab + 1);
    }

    if constexpr (PROBE != 0) {
      if (p.workspace != nullptr && wave == 0 && lane_here() == 0) {
        uint64_t* out = reinterpret_cast<uint64_t*>(p.workspace) + 2 * blockIdx.x;
        out[0] = clock64() - probe_c0;
        out[1] = wall_clock64() - probe_r0;
      }
    }
    // the steps of the epilogue (16 rows x 64 columns of a wave's part: step = 2 * group of rows + half of the columns)
    // that this block converts and stores: all of them, or its share of a tile that is cut
    int st_lo = 0, st_hi = 2 * TM;
    if (!GROUPED && job.kind == PIECE) {
      const Plan pl = plan_of();
      const int tail_c = pl.tail_c, T = total - pl.main_total, P = (nslab + pl.tail_u - 1) / pl.tail_u;
      const int q = tail_c / T, t = tail_c - q * T;
      st_lo = q * (2 * TM) / P;
      st_hi = (q + 1) * (2 * TM) / P;
      const __amdgpu_buffer_rsrc_t w_rsrc = t2_rsrc(p.workspace, t2_clamp_u32((int64_t)gridDim.x * SLOT_BYTES));
      // (a flag per block and reader: the reader puts it down again)
      unsigned int* const flags = g_w4_flags + (size_t)p.streamk_slot * (kW4MaxBlocks * kW4MaxPieces);
      const int lane_p = lane_here();
      // ---- the other blocks' rows go to this block's slot; the flags follow once every wave's stores have completed
      {
        const uint32_t base = (uint32_t)tail_c * SLOT_BYTES + (uint32_t)wave * (SLOT_BYTES / 4);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            if (2 * i + j / 4 >= st_lo && 2 * i + j / 4 < st_hi) continue;
            const v4f a4 = acc[i][j];
            const v4u_t v = {__float_as_uint(a4[0]), __float_as_uint(a4[1]), __float_as_uint(a4[2]), __float_as_uint(a4[3])};
            buffer_store_b128_guarded<kDeviceScope>(v, w_rsrc, (uint32_t)lane_p * 16u, base + (uint32_t)(i * TN + j) * 1024u);
          }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        if (wave == 0 && lane_p < P && lane_p != q)
          __hip_atomic_store(flags + tail_c * kW4MaxPieces + lane_p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      // ---- the other blocks' sums of this block's rows
      for (int r = 0; r < P; ++r) {
        if (r == q) continue;
        const int c = t + r * T;
        // (in practice written by the time this block has published its own: the pieces are equally long.  Every lane
        // reads the same word; a block that gives up -- its partner never ran: a hung GPU -- poisons its rows with NaN
        // and counts the event)
        bool there = false;
        for (int spin = 0; spin < (1 << 22); ++spin) {
          // (one value for the wave, so that the loop's exit is the same for every lane)
          const unsigned int seen = __builtin_amdgcn_readfirstlane(
              __hip_atomic_load(flags + c * kW4MaxPieces + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
          if (seen != 0u) { there = true; break; }
          __builtin_amdgcn_s_sleep(16);
        }
        asm volatile("" ::: "memory");
        // (every wave has seen the flag: down it goes, for the next launch that uses this set)
        __builtin_amdgcn_s_barrier();
        if (wave == 0 && lane_p == 0) {
          if (there) __hip_atomic_store(flags + c * kW4MaxPieces + q, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          else atomicAdd(&g_w4_gave_up, 1u);
        }
        const uint32_t base = (uint32_t)c * SLOT_BYTES + (uint32_t)wave * (SLOT_BYTES / 4);
        const uint32_t poison = there ? 0u : 0x7fc00000u;
#pragma unroll
        for (int st = 0; st < 2 * TM; ++st) {
          if (st < st_lo || st >= st_hi) continue;
          const int i = st / 2, j0 = (st & 1) * 4;
          v4u_t v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j)
            v[j] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (uint32_t)lane_p * 16u, base + (uint32_t)(i * TN + j0 + j) * 1024u, kDeviceScope);
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i][j0 + j] += v4f{__uint_as_float(v[j].x | poison), __uint_as_float(v[j].y | poison), __uint_as_float(v[j].z | poison),
                                  __uint_as_float(v[j].w | poison)};
        }
      }
    }
    // ---- the tile leaves, 16 rows x 64 columns of the wave's part at a time
    // (row scaling: every scale of the tile is loaded before the first store, so that no later wait for a load also
    // waits for the stores in front of it)
    float b_s[TN / 2][8], a_s_all[TM];
    if constexpr (!BLOCKSCALE) {
#pragma unroll
      for (int q = 0; q < TN / 2; ++q)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          b_s[q][i] = scale_at(p.b_scales, (int64_t)cur_at.bs0 + (int64_t)min(tn * BN + wn * WN + q * 32 + lq * 8 + i, p.N - 1) * p.b_scale_stride,
                               p.scales_dtype);  // (grouped: bs0 = where the expert's scales begin)
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
        int64_t m = (int64_t)cur_at.row0 + wm * WM + mt * 16 + lm;
        if (m >= p.M) m = p.M - 1;
        a_s_all[mt] = scale_at(p.a_scales, m * p.a_scale_stride, p.scales_dtype);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    const uint32_t c_tile = ((uint32_t)(cur_at.row0 + wm * WM) * (uint32_t)p.ldc + (uint32_t)(tn * BN + wn * WN)) * 2u;
    // (the lane's offsets are formed here, out of sight of the optimiser: hoisted out of the tile loop they would sit in
    // vector registers all through the slab loop, which has none to spare)
    const int lane_e = lane_here();
    const int lm_e = lane_e & 15, lq_e = lane_e >> 4, rr = lane_e >> 3, cc = lane_e & 7;
    const uint32_t c_lane = (uint32_t)rr * c_row_bytes + (uint32_t)cc * 16u;
    // (the last column tile may reach past N, which is a multiple of 8: a lane whose eight columns lie there stores out of
    // the descriptor's range, i.e. nothing -- every store is still issued, so the counts of the waits stay exact)
    uint32_t c_lane_h[TN / 4];
#pragma unroll
    for (int h = 0; h < TN / 4; ++h) c_lane_h[h] = tn * BN + wn * WN + h * 64 + cc * 8 < p.N ? c_lane : 0x80000000u;
    // one step = 16 rows x 64 columns of the wave's part: two pairs of fragments converted and written to the side buffer ...
    auto stage = [&](int mt, int h) {
      float a_s = 1.f;
      if constexpr (!BLOCKSCALE) a_s = a_s_all[mt];
#pragma unroll
      for (int qq = 0; qq < 2; ++qq) {
        const int q = 2 * h + qq;
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
        *reinterpret_cast<v4u_t*>(wbuf + lm_e * 128 + (((qq * 4 + lq_e) ^ (lm_e & 7)) * 16)) =
            v4u_t{pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]), pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3])};
      }
    };
    // ... read back as 8 rows x one whole 128-byte line per instruction (a wave reads back only what it wrote itself, and
    // its LDS operations execute in order) ...
    // (with a row index: dst[i] = the byte offset in C of the row that receives row mt * 16 + i * 8 + rr of the wave's part,
    // past every range for a row behind the slot's end)
    auto read_back = [&](v4u_t (&v)[2], uint32_t (&dst)[2], int mt) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int r = i * 8 + rr;
        v[i] = *reinterpret_cast<const v4u_t*>(wbuf + r * 128 + ((cc ^ (r & 7)) * 16));
        dst[i] = 0u;
        if constexpr (SCATTER) {
          const int row = mt * 16 + r;
          dst[i] = cur_at.row0 + wm * WM + row < cur_at.row_end ? idx_lds[row] * c_row_bytes + (uint32_t)cc * 16u : 0x80000000u;
        }
      }
    };
    // ... and stored (non-temporal: C is not read again here, and its lines should not push the operands out of L2)
    // (grouped: C ends, for this tile, where the tile's slot ends -- the rows of a slot's last tile that lie past it are
    // the next slot's, and are not stored)
    const __amdgpu_buffer_rsrc_t c_rsrc_tile =
        GROUPED ? t2_rsrc(p.c, t2_clamp_u32(((int64_t)(cur_at.row_end - 1) * p.ldc + p.N) * 2)) : c_rsrc;
    auto store_step = [&](const v4u_t (&v)[2], const uint32_t (&dst)[2], int mt, int h) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if constexpr (SCATTER)
          buffer_store_b128_guarded<2>(v[i], c_rsrc, dst[i] | (c_lane_h[h] & 0x80000000u), (uint32_t)(tn * BN + wn * WN) * 2u + (uint32_t)h * 128u);
        else
          buffer_store_b128_guarded<2>(v[i], c_rsrc_tile, c_lane_h[h], c_tile + (uint32_t)(mt * 16 + i * 8) * c_row_bytes + (uint32_t)h * 128u);
      }
    };
    if (GROUPED || job.kind == WHOLE) {
      // The steps overlap: a step's two reads go out together, the next step is converted and written behind them (the
      // LDS executes a wave's operations in order, so those writes cannot overtake the reads), and only then are the
      // reads waited for and stored -- one LDS round trip per step, hidden behind the next step's conversions, instead of
      // two exposed ones (2.3 -> 1.x microseconds per 192 x 256 tile).
      constexpr int NSTEP = TM * (TN / 4);
      stage(0, 0);
      static_for<NSTEP>([&](auto S) {
        constexpr int st = decltype(S)::value, mt = st / (TN / 4), h = st % (TN / 4);
        v4u_t v[2];
        uint32_t dst[2];
        read_back(v, dst, mt);
        if constexpr (st + 1 < NSTEP) stage((st + 1) / (TN / 4), (st + 1) % (TN / 4));
        store_step(v, dst, mt, h);
      });
      // (the next tile's index entries, behind this tile's stores)
      if (has_next) dma_idx(next_at.row0);
    } else {
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
#pragma unroll
        for (int h = 0; h < TN / 4; ++h) {
          if (2 * mt + h < st_lo || 2 * mt + h >= st_hi) continue;   // (a piece of a cut tile: the other steps are another block's)
          stage(mt, h);
          v4u_t v[2];
          uint32_t dst[2];
          read_back(v, dst, mt);
          store_step(v, dst, mt, h);
        }
      }
    }
    stored = true;
    job = next_job;
    tm = tm2;
    tn = tn2;
    slot = slot2;
    cur_at = next_at;
  }
  // the last copies (of nothing: every lane out of range) still write zeros into the stages: they must have landed
  // before the block's LDS goes to another block
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <int TM, int TN, bool BLOCKSCALE, int PROBE>
__global__ __launch_bounds__(256, 1) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_w4_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  w4_body<TM, TN, BLOCKSCALE, PROBE>(p, smem);
}

template <int TM, int TN, bool BLOCKSCALE, bool SCATTER>
__global__ __launch_bounds__(256, 1) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_w4_grouped_kernel(GemmArgs p) {
  static_assert(BLOCKSCALE || !SCATTER, "the row index on C is the block-scaled MoE layer's");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  w4_body<TM, TN, BLOCKSCALE, 0, SCATTER ? 2 : 1>(p, smem);
}

template <int TM, int TN, bool BLOCKSCALE>
constexpr int w4_lds_bytes() {
  return 2 * (TM * 32 * 128 + (BLOCKSCALE ? 1024 : 0)) + 3 * (TN * 32 * 128) + 4 * 2048;
}

// The shapes this kernel takes: bf16 C with 16-byte aligned rows, N a multiple of 8, K a whole and even number of slabs,
// operands whose byte offsets fit 31 bits (a tile's position rides in the copies' scalar offset).
bool gemm_w4_ok(const GemmArgs& p, bool blockscale) {
  if (p.M <= 0 || p.N <= 0 || p.N % 8 != 0 || p.K < 512 || p.K % 256 != 0) return false;
  const int64_t nslab = p.K / 128;
  if (p.kv_on || p.splits > 1) return false;
  if (p.c_dtype != MAXFP8_BF16 || !p.c_vec8_ok) return false;
  const int64_t lim = 0x7ff00000ll;
  const int64_t rows = ceil_div(p.M, 192) * 192 + 192;
  if (rows * p.lda >= lim || (ceil_div(p.N, 256) * 256) * p.ldb >= lim) return false;
  if (blockscale && (nslab * p.a_scales_ld + rows) * 4 >= lim) return false;
  if (rows * p.ldc * 2 >= lim) return false;
  return true;
}

template <int TM, bool BLOCKSCALE, int PROBE>
static int launch_w4(const GemmArgs& p, unsigned blocks, hipStream_t stream, const char* name) {
  static PerDeviceFlag attr_done;
  constexpr int lds = w4_lds_bytes<TM, 8, BLOCKSCALE>();
  static_assert(lds <= 160 * 1024, "one block's LDS");
  auto kern = gemm_w4_kernel<TM, 8, BLOCKSCALE, PROBE>;
  bool& done = attr_done.here();
  if (!done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", name, lds, hipGetErrorString(e));
    done = true;
  }
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds, stream, p);
  return launch_status(name);
}

// The tail cut of an M x N x K matmul in tiles of 32 tm rows: the blocks it runs on, the slabs of a piece and the bytes
// of workspace (a slot of a tile's sums per block); unit == 0: this shape has no cut.  It takes more than one tile per
// block (what is cut is what lies beyond the last whole round), slabs in whole fours per tile, and a last round of at
// most half the blocks' number of tiles: every tile is cut into the same number of pieces, two to four, at the same
// slabs, and every piece is one block's work.
W4Split gemm_w4_split(int64_t M, int64_t N, int64_t K, int tm) {
  const W4Split none = {0, 0, 0};
  const int64_t tiles = ceil_div(M, 32 * tm) * ceil_div(N, 256), nslab = K / 128;
  int g = (compute_units() / 8) * 8;
  if (g > kW4MaxBlocks) g = kW4MaxBlocks;
  if (g < 8 || K % 512 != 0) return none;
  if (tiles * 2 <= g) {
    // fewer tiles than half the blocks: every tile is cut, into as many pieces (eight at most -- a piece owns at least
    // one of the 2 tm steps of the epilogue --, of four slabs at least) as there are blocks for
    int64_t pieces = g / tiles;
    if (pieces > kW4MaxPieces) pieces = kW4MaxPieces;
    if (pieces > nslab / 4) pieces = nslab / 4;
    if (pieces < 2) return none;
    const int64_t u = ceil_div(ceil_div(nslab, pieces), 4) * 4;
    if (u >= nslab) return none;
    const int64_t blocks = ceil_div(tiles * ceil_div(nslab, u), 8) * 8;
    return W4Split{(int)blocks, (int)u, (size_t)blocks * 32 * tm * 256 * 4};
  }
  if (tiles <= g || tiles % g == 0) return none;
  int64_t pieces = g / (tiles % g);
  if (pieces > 4) pieces = 4;
  if (pieces < 2) return none;
  const int64_t u = ceil_div(ceil_div(nslab, pieces), 4) * 4;
  if (u >= nslab) return none;
  return W4Split{g, (int)u, (size_t)g * 32 * tm * 256 * 4};
}

// rows of a tile: 32 * tm (tm = 4, 5 or 6 sixteen-row groups per wave); split: cut the tail (p.workspace holds what
// gemm_w4_split asks for)
int gemm_w4_launch(const GemmArgs& p_in, bool blockscale, int tm, bool split, hipStream_t stream) {
  GemmArgs p = p_in;
  const int64_t tiles = ceil_div(p.M, 32 * tm) * ceil_div(p.N, 256);
  const int cus = compute_units();
  unsigned blocks = (unsigned)(tiles < cus ? tiles : cus);
  p.tail_units = 0;
  if (split) {
    const W4Split sp = gemm_w4_split(p.M, p.N, p.K, tm);
    if (sp.unit > 0 && p.workspace != nullptr) {
      blocks = (unsigned)sp.blocks;
      p.tail_units = sp.unit;
      // a set of flags per launch in flight; a launch recorded into a graph keeps the set of the recording in every
      // replay, which may run beside launches of another stream: recorded launches draw from sets of their own
      static std::atomic<unsigned int> issued{0}, recorded{0};
      hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
      if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
        (void)hipGetLastError();
        status = hipStreamCaptureStatusNone;
      }
      p.streamk_slot = status == hipStreamCaptureStatusNone ? (int)(issued.fetch_add(1, std::memory_order_relaxed) % (kW4FlagSets / 2))
                                                            : kW4FlagSets / 2 + (int)(recorded.fetch_add(1, std::memory_order_relaxed) % (kW4FlagSets / 2));
    }
  }
  if (tm == 4)
    return blockscale ? launch_w4<4, true, 0>(p, blocks, stream, "gemm_w4_block_128x256") : launch_w4<4, false, 0>(p, blocks, stream, "gemm_w4_row_128x256");
  if (tm == 5)
    return blockscale ? launch_w4<5, true, 0>(p, blocks, stream, "gemm_w4_block_160x256") : launch_w4<5, false, 0>(p, blocks, stream, "gemm_w4_row_160x256");
  return blockscale ? launch_w4<6, true, 0>(p, blocks, stream, "gemm_w4_block_192x256") : launch_w4<6, false, 0>(p, blocks, stream, "gemm_w4_row_192x256");
}

// The grouped form takes: bf16 C with 16-byte aligned rows, N a multiple of 8, K a whole and even number of slabs, at most
// kW4GroupedSlots slots, operands whose byte offsets fit 31 bits (per expert, for the weights); row scaling: f32 scales,
// no row index on C.
bool gemm_w4_grouped_ok(const GemmArgs& p, bool blockscale) {
  if (!blockscale && (p.c_row_index != nullptr || p.scales_dtype != MAXFP8_F32)) return false;
  if (p.M < 192 || p.N <= 0 || p.N % 8 != 0 || p.K < 512 || p.K % 256 != 0) return false;
  if (p.num_active <= 0 || p.num_active > kW4GroupedSlots) return false;
  if (p.c_dtype != MAXFP8_BF16 || !p.c_vec8_ok) return false;
  const int64_t lim = 0x7ff00000ll, nslab = p.K / 128;
  const int64_t rows = (int64_t)p.M + 192;
  if (rows * p.lda >= lim || (ceil_div(p.N, 256) * 256) * p.ldb >= lim) return false;
  if (rows * p.ldc * 2 >= lim) return false;
  if (blockscale && (nslab * p.a_scales_ld + rows) * 4 >= lim) return false;
  // (the element of the weight scales where an expert's begin rides in 32 bits: fine for expert numbers below 2^16 with
  // fewer than 2^15 scales per expert)
  if (p.bs_expert_stride >= (1 << 15)) return false;
  return true;
}

// The full 192-row tiles of the slots with at least 192 rows (p.big_rows == p.big_bm == 192); the other launch takes the
// rest.  A block per CU: the blocks past this launch's share of the chip exit at once.
int gemm_w4_grouped_launch(const GemmArgs& p, bool blockscale, hipStream_t stream) {
  static PerDeviceFlag attr_done_plain, attr_done_scatter, attr_done_row;
  constexpr int lds = w4_lds_bytes<6, 8, true>() + kW4GroupedTableBytes;  // (the row-scaled kernel takes the same, for simplicity)
  static_assert(lds + 64 <= 160 * 1024, "one block's LDS");
  const bool scatter = p.c_row_index != nullptr;
  const char* name = !blockscale ? "gemm_w4_grouped_row_192x256" : (scatter ? "gemm_w4_grouped_block_192x256 (row index)" : "gemm_w4_grouped_block_192x256");
  auto kern = !blockscale ? gemm_w4_grouped_kernel<6, 8, false, false>
                          : (scatter ? gemm_w4_grouped_kernel<6, 8, true, true> : gemm_w4_grouped_kernel<6, 8, true, false>);
  bool& done = !blockscale ? attr_done_row.here() : (scatter ? attr_done_scatter.here() : attr_done_plain.here());
  if (!done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", name, lds, hipGetErrorString(e));
    done = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)((compute_units() / 8) * 8)), dim3(256), lds, stream, p);
  return launch_status(name);
}

// Pieces of a cut tail that a block stopped waiting for, on the current device since the library was loaded (0 unless
// a GPU hung in the middle of a launch; the tiles concerned hold NaN).  Waits for the device's work to finish.
int gemm_w4_gave_up(unsigned int* count) {
  hipError_t e = hipDeviceSynchronize();
  if (e == hipSuccess) e = hipMemcpyFromSymbol(count, HIP_SYMBOL(g_w4_gave_up), sizeof(unsigned int));
  if (e != hipSuccess) MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "tail cut: cannot read the count of abandoned pieces: %s", hipGetErrorString(e));
  return MAXFP8_OK;
}

// measurement aid: the kernel's main loop on operands that stay in L2 (level 1) or in LDS (level 2), on every CU
int gemm_w4_probe(const GemmArgs& p, bool blockscale, int level, int tm, hipStream_t stream) {
  const unsigned blocks = (unsigned)compute_units();
  const char* name = "gemm_w4_probe";
  if (tm == 4) {
    if (level == 1) return blockscale ? launch_w4<4, true, 1>(p, blocks, stream, name) : launch_w4<4, false, 1>(p, blocks, stream, name);
    return blockscale ? launch_w4<4, true, 2>(p, blocks, stream, name) : launch_w4<4, false, 2>(p, blocks, stream, name);
  }
  if (tm == 5) {
    if (level == 1) return blockscale ? launch_w4<5, true, 1>(p, blocks, stream, name) : launch_w4<5, false, 1>(p, blocks, stream, name);
    return blockscale ? launch_w4<5, true, 2>(p, blocks, stream, name) : launch_w4<5, false, 2>(p, blocks, stream, name);
  }
  if (level == 1) return blockscale ? launch_w4<6, true, 1>(p, blocks, stream, name) : launch_w4<6, false, 1>(p, blocks, stream, name);
  return blockscale ? launch_w4<6, true, 2>(p, blocks, stream, name) : launch_w4<6, false, 2>(p, blocks, stream, name);
}

}  // namespace maxfp8
