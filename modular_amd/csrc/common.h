// Shared device/host helpers for the gfx950 FP8 linear kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/maxfp8.h"

namespace maxfp8 {

// ---- error reporting (host) -------------------------------------------------

void set_error(const char* fmt, ...);
int launch_status(const char* what);

// "done once per device" flags (a kernel's LDS attribute is a property of the device's copy of the kernel)
struct PerDeviceFlag {
  bool done[64] = {};
  // the flag of the current device (the last slot stands for every device past 62)
  bool& here() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev > 63) dev = 63;
    return done[dev];
  }
};
  // MAXFP8_OK or MAXFP8_ERR_LAUNCH after hipGetLastError

#define MAXFP8_FAIL(code, ...)        \
  do {                                \
    ::maxfp8::set_error(__VA_ARGS__); \
    return (code);                    \
  } while (0)

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- vector types -------------------------------------------------------------

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));


// ---- scalar conversions -------------------------------------------------------

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// f32 -> bf16 bits, round to nearest even; NaN keeps a quiet payload.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}
// two f32 -> two bf16 (a in the low half) with the hardware convert of gfx950, v_cvt_pk_bf16_f32:
// round to nearest even like f32_to_bf16_bits, one instruction instead of a dozen
typedef float v2f_t __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  const v2f_t f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, v2bf_t));
}
// f rounded to bf16 (nearest even) and widened back
__device__ __forceinline__ float bf16_round(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

__device__ __forceinline__ float clamp448(float v) {
  // fminf/fmaxf return the non-NaN operand; inputs are never NaN on this path.
  return fminf(fmaxf(v, -448.0f), 448.0f);
}

// Two f32 -> two e4m3fn bytes in the low (hi == false) or high half of `old`.
// v_cvt_pk_fp8_f32 on gfx950 is the OCP e4m3fn convert, round to nearest even.
__device__ __forceinline__ int cvt_pk_e4m3fn(float a, float b, int old, bool hi) {
  return hi ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, true)
            : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, false);
}

// e4m3fn byte -> f32 without the hardware convert (used by the naive kernels so
// they share nothing with the kernels they check).
__device__ __forceinline__ float e4m3fn_to_f32_sw(uint32_t b) {
  uint32_t s = (b & 0x80u) << 24, e = (b >> 3) & 15u, m = b & 7u;
  float v;
  if (e == 15u && m == 7u) return __uint_as_float(s | 0x7fc00000u);
  if (e == 0u) v = (float)m * 0.001953125f;                    // m * 2^-9
  else v = __uint_as_float(((e + 120u) << 23) | (m << 20));    // (1+m/8) * 2^(e-7)
  return __uint_as_float(__float_as_uint(v) | s);
}

// ---- cross-lane reductions ----------------------------------------------------

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

// max over each aligned group of 16 lanes; every lane of the group gets the result
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_mov<0xB1>(v));   // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp_mov<0x4E>(v));   // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp_mov<0x141>(v));  // row_half_mirror
  v = fmaxf(v, dpp_mov<0x140>(v));  // row_mirror
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
  v = row16_max(v);
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  v = fmaxf(v, __shfl_xor(v, 32, 64));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// scale = min(amax, ub) / 448 ; recip = guarded 1/scale.  Both divisions are the
// correctly rounded IEEE ones (no -ffast-math, no v_rcp approximation).
__device__ __forceinline__ void dynamic_scale_f32(float amax, float ub, float& scale, float& recip) {
  scale = fminf(amax, ub) / 448.0f;
  float r = 0.0f;
  if (scale != 0.0f) {
    r = 1.0f / scale;
    if (isinf(r) || isnan(r)) r = 0.0f;
  }
  recip = r;
}


}  // namespace maxfp8
