// Device helpers shared by the MFMA matmul kernels (gemm_tiled.hip, gemm_w4.hip).
#pragma once
#include <stdint.h>

#include <utility>
#include "common.h"

namespace maxfp8 {

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// Cache policy of copies whose bytes are read once per launch (the weights of experts with few rows): non-temporal.  The
// stream then does not displace what the memory-side cache and the L2 hold, and the chip reads 7.0 instead of 6.2 TB/s.
constexpr int kStreamOnce = 2;

// f(integral_constant<int, 0>{}) ... f(integral_constant<int, N - 1>{}): a loop whose index is a constant
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t t2_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
__device__ __forceinline__ uint32_t t2_clamp_u32(int64_t v) {
  return v > 0xfffffff0ll ? 0xfffffff0u : (v < 0 ? 0u : (uint32_t)v);
}

// A 16-byte buffer store whose scalar offset sits in a register.  The hardware reads the four data registers of such
// a store during the cycles AFTER it has issued, and a VALU instruction that follows at once and writes one of them
// changes what is stored; the compiler's hazard table has this case down as free of hazards (it pads only stores whose
// scalar offset is an immediate) and schedules the next values straight into the registers.  Seen on MI355X as a
// tile's bf16 pairs replaced, in some lanes, by the f32 products of the rows computed next.  The wait states are tied
// to the data registers, so that nothing that overwrites them can be scheduled between the store and the wait.
typedef unsigned int v4u_t __attribute__((ext_vector_type(4)));
template <int CACHE_POLICY>
__device__ __forceinline__ void buffer_store_b128_guarded(const v4u_t v, const __amdgpu_buffer_rsrc_t rsrc, uint32_t voffset, uint32_t soffset) {
  __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, voffset, soffset, CACHE_POLICY);
  asm volatile("s_nop 7" ::"v"(v));
}

// tile number -> (row tile, column tile): groups of GROUP_M row tiles share weight columns, walked column-major
template <int GROUP_M = 4>
__device__ __forceinline__ void tile_coords(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int per_group = GROUP_M * tiles_n;
  const int group = pid / per_group;
  const int first_m = group * GROUP_M;
  const int gsize = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_group = pid - group * per_group;
  tm = first_m + in_group % gsize;
  tn = in_group / gsize;
}

}  // namespace maxfp8
