// C ABI of the library (include/maxfp8.h): argument checks, kernel selection, error text.
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "common.h"
#include "gemm_args.h"
#include "tuning.h"

namespace maxfp8 {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int launch_status(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return MAXFP8_OK;
}

// kernels (defined in the other translation units)
int quantize_dispatch(void*, void*, const void*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int, int,
                      float, int64_t, int64_t, int64_t, int64_t, const uint32_t*, uint32_t, hipStream_t);
int quantize_scatter_dispatch(void*, void*, const void*, int64_t, int64_t, int64_t, int64_t, int64_t, float, const uint32_t*, int64_t,
                              int64_t, hipStream_t);
int rmsnorm_quantize_dispatch(void*, void*, const void*, const void*, int64_t, int64_t, int64_t, int64_t, int, int, float,
                              float, float, hipStream_t);
int quantize_static_dispatch(void*, const void*, int64_t, int64_t, int64_t, int64_t, int, float, hipStream_t);
int quantize_tensor_dispatch(void*, void*, const void*, int64_t, int64_t, int64_t, int64_t, int, int, float, hipStream_t);
int moe_create_indices_dispatch(uint32_t*, uint32_t*, uint32_t*, int32_t*, uint32_t*, const int32_t*, int64_t, int64_t, hipStream_t);
int fused_silu_dispatch(void*, float*, const void*, const uint32_t*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int,
                        hipStream_t);
int cast_f32_to_e4m3fn_dispatch(void*, const float*, int64_t, hipStream_t);
int cast_e4m3fn_to_f32_dispatch(float*, const void*, int64_t, hipStream_t);
int cast_f32_to_bf16_dispatch(void*, const float*, int64_t, hipStream_t);
int copy_bytes_dispatch(void*, const void*, int64_t, hipStream_t);
int naive_blockwise_dispatch(void*, const void*, const void*, const void*, const void*, int64_t, int64_t, int64_t,
                             int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int, int64_t, int64_t,
                             int64_t, int64_t, int64_t, int64_t, hipStream_t);
int naive_rowwise_dispatch(void*, const void*, const void*, const void*, const void*, int64_t, int64_t, int64_t,
                           int64_t, int64_t, int64_t, int64_t, int64_t, int, int, hipStream_t);
int naive_grouped_dispatch(void*, const void*, const void*, const void*, const void*, const uint32_t*,
                           const int32_t*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int, hipStream_t);
int gemm_tiled_dispatch(const GemmArgs&, bool, size_t, int64_t, hipStream_t);
size_t gemm_tiled_workspace_bytes(int64_t, int64_t, int64_t);
size_t gemm_tiled_plan_workspace_bytes(int64_t, int64_t, int64_t, bool);
int gemm_tiled_describe(int64_t, int64_t, int64_t, bool, bool, char*, size_t);
int gemm_grouped_dispatch(const GemmArgs&, bool, int64_t, int64_t, hipStream_t);
int gemm_skinny_dispatch(const GemmArgs&, bool, int64_t, hipStream_t);
int gemm_skinny_max_m();
bool gemm_skinny_preferred(int64_t M, int64_t N, int64_t K);
int gemm_skinny_read_probe(const void* b, int64_t M, int64_t N, int64_t K, int64_t ldb, hipStream_t stream);
int gemm_persist_probe(const GemmArgs&, bool, int, hipStream_t);
int gemm_w4_probe(const GemmArgs&, bool, int, int, hipStream_t);
bool gemm_w4_ok(const GemmArgs&, bool);
int gemm_w4_gave_up(unsigned int*);
int gemm_streamk_gave_up(unsigned int*);

// v rounded to bf16 / f16 and widened back: how an op parameter of the input's dtype arrives
static float round_to_dtype(float v, int dtype) {
  if (dtype == MAXFP8_BF16) {
    uint32_t u;
    memcpy(&u, &v, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return v;
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    memcpy(&v, &u, 4);
    return v;
  }
  if (dtype == MAXFP8_F16) return (float)(_Float16)v;
  return v;
}

static bool is_aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// ---- the library's own scratch memory (maxfp8_matmul_dynamic_scaled_fp8_noalloc) ------------------
// A file-scope device array: every GPU the library runs on holds its own copy, at its own address, from the
// moment the code object is loaded there until the process ends.  In host code the array's NAME is only a handle
// for hipGetSymbolAddress -- it is not a device address and is never passed to a kernel or a memory call.  The
// address is looked up once per device, with that device current, and kept; kernels receive it as an argument,
// exactly like a caller's workspace.
constexpr size_t kScratchBytes = (size_t)48 << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
static void* g_scratch_ptr[64] = {};
static std::mutex g_scratch_mu;

static int scratch_of_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= 64)
    MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "matmul (no-alloc): no current device in 0..63: %s", hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      (void)hipGetLastError();
      MAXFP8_FAIL(MAXFP8_ERR_LAUNCH, "matmul (no-alloc): cannot resolve the scratch array on device %d: %s", dev, hipGetErrorString(e));
    }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MAXFP8_OK;
}

// The MFMA kernels address a tile's operands with 32-bit buffer offsets whose top bit marks lanes that are out of
// range: the rows of the tallest tile (256) times the row stride, and the activation scales of all slabs of a tile
// (ceil(K / 128) rows of a_scales_ld floats), must stay below 2^31 bytes.
static bool offsets_fit(int64_t K, int64_t lda, int64_t ldb, int64_t a_scales_ld, bool block) {
  const int64_t lim = (int64_t)1 << 31;
  if (256 * lda + K >= lim || 256 * ldb + K >= lim) return false;
  return !block || (ceil_div(K, 128) * a_scales_ld + 256) * 4 < lim;
}

// ---- tuning switches: one immutable snapshot of the environment, replaced as a whole by a reload ----
static std::atomic<const Tuning*> g_tuning{nullptr};
static std::mutex g_tuning_mu;

static const Tuning* read_tuning(unsigned generation) {
  Tuning* t = new Tuning();
  auto num = [](const char* name, int dflt) { const char* e = getenv(name); return e ? atoi(e) : dflt; };
  const int tile = num("MAXFP8_TILE", 0);
  t->tile = (tile >= 1 && tile <= 4) ? tile : 0;
  t->splitk = num("MAXFP8_SPLITK", 0);
  t->one_region = getenv("MAXFP8_ONE_REGION") != nullptr;
  t->persist = num("MAXFP8_PERSIST", 1) != 0;
  t->streamk = num("MAXFP8_STREAMK", 1);
  t->big_rows = num("MAXFP8_BIG_ROWS", 1024);
  t->grouped_overlap = num("MAXFP8_GROUPED_OVERLAP", 1) != 0;
  t->grouped_persist = num("MAXFP8_GROUPED_PERSIST", 1) != 0;
  const int w4 = num("MAXFP8_W4", -1);
  t->w4 = (w4 == 0 || w4 == 4 || w4 == 5 || w4 == 6) ? w4 : -1;
  const int w4_split = num("MAXFP8_W4_SPLIT", -1);
  t->w4_split = (w4_split == 0 || w4_split == 1) ? w4_split : -1;
  t->skinny_alds = num("MAXFP8_SKINNY_ALDS", 1) != 0;
  const char* sb = getenv("MAXFP8_GROUPED_SHARE");
  t->grouped_share = sb ? (float)atof(sb) : 0.5f;
  t->grouped_w4 = num("MAXFP8_GROUPED_W4", 1) != 0;
  t->grouped_w4_rows = num("MAXFP8_GROUPED_W4_ROWS", 4096);
  const char* sw = getenv("MAXFP8_GROUPED_W4_SHARE");
  t->grouped_w4_share = sw ? (float)atof(sw) : 0.6f;
  t->grouped_w4_hot_rest = num("MAXFP8_GROUPED_W4_HOT_REST", 32);
  t->grouped_w4_cold_rows = num("MAXFP8_GROUPED_W4_COLD_ROWS", 128);
  t->skinny = num("MAXFP8_SKINNY", 0);
  t->generation = generation;
  return t;
}

const Tuning& tuning() {
  const Tuning* t = g_tuning.load(std::memory_order_acquire);
  if (t) return *t;
  std::lock_guard<std::mutex> lock(g_tuning_mu);
  t = g_tuning.load(std::memory_order_acquire);
  if (!t) {
    t = read_tuning(0);
    g_tuning.store(t, std::memory_order_release);
  }
  return *t;
}

// (the old snapshot is left in place for threads that still read it: a few dozen bytes per reload)
void tuning_reload() {
  std::lock_guard<std::mutex> lock(g_tuning_mu);
  const Tuning* old = g_tuning.load(std::memory_order_acquire);
  g_tuning.store(read_tuning(old ? old->generation + 1 : 1), std::memory_order_release);
}

}  // namespace maxfp8

using namespace maxfp8;

extern "C" {

const char* maxfp8_last_error(void) { return g_error; }
const char* maxfp8_version(void) { return "maxfp8 0.2 (gfx950)"; }
void maxfp8_tuning_reload(void) { tuning_reload(); }

}  // extern "C"

static int quantize_common(void* out_fp8, void* out_scales, const void* in, const uint32_t* row_index, uint32_t index_div,
                           int64_t M, int64_t K, int64_t in_row_stride, int64_t out_row_stride, int64_t group_size,
                           int64_t scales_ld, int in_dtype, int scales_dtype, float scale_ub, void* stream) {
  if (in_dtype != MAXFP8_BF16 && in_dtype != MAXFP8_F16 && in_dtype != MAXFP8_F32)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "quantize: input dtype %d is not bf16, f16 or f32", in_dtype);
  if (scales_dtype != MAXFP8_F32 && scales_dtype != MAXFP8_BF16)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "quantize: scales dtype should be bfloat16 or float32 (got %d)", scales_dtype);
  if (M < 0 || K < 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize: negative size M=%lld K=%lld", (long long)M, (long long)K);
  if (M == 0 || K == 0) return MAXFP8_OK;  // fp8_quantization.mojo:428-429
  if (group_size == -1) group_size = K;
  if (group_size <= 0 || K % group_size != 0)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize: group size %lld must divide K = %lld", (long long)group_size, (long long)K);
  if (group_size % 4 != 0)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize: group size must be multiple of simd size (4), got %lld", (long long)group_size);
  if (in_row_stride < K || out_row_stride < K || scales_ld < M)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize: strides (in %lld, out %lld, scales %lld) smaller than the extents",
                (long long)in_row_stride, (long long)out_row_stride, (long long)scales_ld);
  if (!out_fp8 || !out_scales || !in) MAXFP8_FAIL(MAXFP8_ERR_NULL, "quantize: null pointer");
  return quantize_dispatch(out_fp8, out_scales, in, M, K, in_row_stride, out_row_stride, group_size, scales_ld,
                           in_dtype, scales_dtype, scale_ub, 1, 0, 0, 0, row_index, index_div, (hipStream_t)stream);
}

extern "C" {

int maxfp8_quantize_dynamic_scaled_fp8(void* out_fp8, void* out_scales, const void* in, int64_t M, int64_t K,
                                       int64_t in_row_stride, int64_t out_row_stride, int64_t group_size,
                                       int64_t scales_ld, int in_dtype, int scales_dtype, float scale_ub,
                                       void* stream) {
  return quantize_common(out_fp8, out_scales, in, nullptr, 1, M, K, in_row_stride, out_row_stride, group_size, scales_ld,
                         in_dtype, scales_dtype, scale_ub, stream);
}

int maxfp8_quantize_dynamic_scaled_fp8_gather(void* out_fp8, void* out_scales, const void* in, const uint32_t* row_index,
                                              int64_t index_div, int64_t M, int64_t K, int64_t in_row_stride,
                                              int64_t out_row_stride, int64_t group_size, int64_t scales_ld, int in_dtype,
                                              int scales_dtype, float scale_ub, void* stream) {
  if (M > 0 && K > 0 && !row_index) MAXFP8_FAIL(MAXFP8_ERR_NULL, "quantize (gather): null row index");
  if (index_div < 1 || index_div > 0xffffffffll) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize (gather): index_div must be at least 1");
  return quantize_common(out_fp8, out_scales, in, row_index, (uint32_t)index_div, M, K, in_row_stride, out_row_stride,
                         group_size, scales_ld, in_dtype, scales_dtype, scale_ub, stream);
}

int maxfp8_quantize_dynamic_scaled_fp8_scatter(void* out_fp8, void* out_scales, const void* in, const uint32_t* dst_index,
                                               int64_t copies, int64_t M, int64_t K, int64_t out_rows, int64_t in_row_stride,
                                               int64_t out_row_stride, int64_t group_size, int64_t scales_ld, int in_dtype,
                                               int scales_dtype, float scale_ub, void* stream) {
  if (M < 0 || K < 0 || out_rows < 0 || copies < 0)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize (scatter): negative size M=%lld K=%lld out_rows=%lld copies=%lld", (long long)M, (long long)K,
                (long long)out_rows, (long long)copies);
  if (M == 0 || K == 0 || copies == 0 || out_rows == 0) return MAXFP8_OK;
  if (in_dtype != MAXFP8_BF16 || scales_dtype != MAXFP8_F32 || group_size != 128)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "quantize (scatter): takes bfloat16 input, float32 scales and groups of 128 (got dtypes %d, %d, group %lld); "
                "the gather form takes the rest", in_dtype, scales_dtype, (long long)group_size);
  if (in_row_stride < K || out_row_stride < K || scales_ld < out_rows)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize (scatter): strides (in %lld, out %lld, scales %lld) smaller than the extents",
                (long long)in_row_stride, (long long)out_row_stride, (long long)scales_ld);
  if (!out_fp8 || !out_scales || !in || !dst_index) MAXFP8_FAIL(MAXFP8_ERR_NULL, "quantize (scatter): null pointer");
  const int rc = quantize_scatter_dispatch(out_fp8, out_scales, in, M, K, in_row_stride, out_row_stride, scales_ld, scale_ub, dst_index,
                                           copies, out_rows, (hipStream_t)stream);
  if (rc == -1)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize (scatter): rows must be 16-byte aligned and K a multiple of 128; the gather form takes the rest");
  return rc;
}

int maxfp8_batched_quantize_dynamic_scaled_fp8(void* out_fp8, void* out_scales, const void* in, int64_t B, int64_t M, int64_t K,
                                               int64_t in_batch_stride, int64_t in_row_stride, int64_t out_batch_stride,
                                               int64_t out_row_stride, int64_t group_size, int64_t scales_batch_stride,
                                               int64_t scales_ld, int in_dtype, int scales_dtype, float scale_ub,
                                               void* stream) {
  if (B < 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "batched quantize: negative batch");
  if (B == 0) return MAXFP8_OK;  // fp8_quantization.mojo:826-827
  if (B > 65535) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "batched quantize: batch %lld exceeds 65535", (long long)B);
  if (in_dtype != MAXFP8_BF16 && in_dtype != MAXFP8_F16 && in_dtype != MAXFP8_F32)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "quantize: input dtype %d is not bf16, f16 or f32", in_dtype);
  if (scales_dtype != MAXFP8_F32 && scales_dtype != MAXFP8_BF16)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "quantize: scales dtype should be bfloat16 or float32 (got %d)", scales_dtype);
  if (M < 0 || K < 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize: negative size M=%lld K=%lld", (long long)M, (long long)K);
  if (M == 0 || K == 0) return MAXFP8_OK;
  if (group_size == -1) group_size = K;
  if (group_size <= 0 || K % group_size != 0)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize: group size %lld must divide K = %lld", (long long)group_size, (long long)K);
  if (group_size % 4 != 0)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize: group size must be multiple of simd size (4), got %lld", (long long)group_size);
  if (in_row_stride < K || out_row_stride < K || scales_ld < M)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize: strides smaller than the extents");
  if (!out_fp8 || !out_scales || !in) MAXFP8_FAIL(MAXFP8_ERR_NULL, "quantize: null pointer");
  return quantize_dispatch(out_fp8, out_scales, in, M, K, in_row_stride, out_row_stride, group_size, scales_ld, in_dtype,
                           scales_dtype, scale_ub, B, in_batch_stride, out_batch_stride, scales_batch_stride, nullptr, 1,
                           (hipStream_t)stream);
}

int maxfp8_rms_norm_fused_quantize_dynamic_scaled_fp8(void* out_fp8, void* out_scales, const void* in, const void* gamma,
                                                      int64_t rows, int64_t K, int64_t in_row_stride,
                                                      int64_t out_row_stride, int in_dtype, int scales_dtype,
                                                      float epsilon, float weight_offset, float scale_ub, void* stream) {
  if (in_dtype != MAXFP8_BF16 && in_dtype != MAXFP8_F16 && in_dtype != MAXFP8_F32)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "rms_norm_fused_quantize: input dtype %d is not bf16, f16 or f32", in_dtype);
  if (scales_dtype != MAXFP8_F32 && scales_dtype != MAXFP8_BF16)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "rms_norm_fused_quantize: scales dtype should be bfloat16 or float32 (got %d)", scales_dtype);
  if (rows < 0 || K < 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "rms_norm_fused_quantize: negative size");
  if (rows == 0 || K == 0) return MAXFP8_OK;
  if (rows >= ((int64_t)1 << 31) || K >= ((int64_t)1 << 31)) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "rms_norm_fused_quantize: sizes must fit 31 bits");
  if (in_row_stride < K || out_row_stride < K)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "rms_norm_fused_quantize: row strides smaller than the row length");
  if (!out_fp8 || !out_scales || !in || !gamma) MAXFP8_FAIL(MAXFP8_ERR_NULL, "rms_norm_fused_quantize: null pointer");
  return rmsnorm_quantize_dispatch(out_fp8, out_scales, in, gamma, rows, K, in_row_stride, out_row_stride, in_dtype,
                                   scales_dtype, round_to_dtype(epsilon, in_dtype), round_to_dtype(weight_offset, in_dtype),
                                   scale_ub, (hipStream_t)stream);
}

int maxfp8_quantize_static_scaled_fp8(void* out_fp8, const void* in, int64_t M, int64_t K, int64_t in_row_stride,
                                      int64_t out_row_stride, int in_dtype, float scale, void* stream) {
  if (in_dtype != MAXFP8_BF16 && in_dtype != MAXFP8_F16 && in_dtype != MAXFP8_F32)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "quantize_static: expected input dtype to be float16, bfloat16, or float32 (got %d)", in_dtype);
  if (M < 0 || K < 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize_static: negative size");
  if (M == 0 || K == 0) return MAXFP8_OK;
  if (in_row_stride < K || out_row_stride < K) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize_static: row strides smaller than the row length");
  if (!out_fp8 || !in) MAXFP8_FAIL(MAXFP8_ERR_NULL, "quantize_static: null pointer");
  return quantize_static_dispatch(out_fp8, in, M, K, in_row_stride, out_row_stride, in_dtype, scale, (hipStream_t)stream);
}

int maxfp8_quantize_tensor_dynamic_scaled_fp8(void* out_fp8, void* out_scales, const void* in, int64_t M, int64_t K,
                                              int64_t in_row_stride, int64_t out_row_stride, int in_dtype, int scales_dtype,
                                              float scale_ub, void* stream) {
  if (in_dtype != MAXFP8_BF16 && in_dtype != MAXFP8_F16 && in_dtype != MAXFP8_F32)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "quantize_tensor: input dtype %d is not bf16, f16 or f32", in_dtype);
  if (scales_dtype != MAXFP8_F32 && scales_dtype != MAXFP8_BF16)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "quantize_tensor: scales dtype should be bfloat16 or float32 (got %d)", scales_dtype);
  if (M < 0 || K < 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize_tensor: negative size");
  if (M == 0 || K == 0) return MAXFP8_OK;  // fp8_quantization.mojo:296-297
  if (M >= ((int64_t)1 << 31)) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize_tensor: M must fit 31 bits");
  if (K % 4 != 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize_tensor: group size must be multiple of simd size (4), got %lld", (long long)K);
  if (in_row_stride < K || out_row_stride < K) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "quantize_tensor: row strides smaller than the row length");
  if (!out_fp8 || !out_scales || !in) MAXFP8_FAIL(MAXFP8_ERR_NULL, "quantize_tensor: null pointer");
  return quantize_tensor_dispatch(out_fp8, out_scales, in, M, K, in_row_stride, out_row_stride, in_dtype, scales_dtype,
                                  scale_ub, (hipStream_t)stream);
}

int maxfp8_moe_create_indices(uint32_t* token_expert_order, uint32_t* expert_start_indices, uint32_t* restore_token_order,
                              int32_t* expert_ids, uint32_t* expert_usage_stats, const void* topk_ids, int64_t n,
                              int64_t num_experts, void* stream) {
  if (n < 0 || num_experts < 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "moe_create_indices: negative size");
  if (n >= ((int64_t)1 << 31) || num_experts > 65535)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "moe_create_indices: %lld assignments / %lld experts exceed the limits", (long long)n,
                (long long)num_experts);
  if (!expert_usage_stats || !expert_start_indices) MAXFP8_FAIL(MAXFP8_ERR_NULL, "moe_create_indices: null pointer");
  if (num_experts == 0) return MAXFP8_OK;
  if (!expert_ids || (n > 0 && (!token_expert_order || !restore_token_order || !topk_ids)))
    MAXFP8_FAIL(MAXFP8_ERR_NULL, "moe_create_indices: null pointer");
  return moe_create_indices_dispatch(token_expert_order, expert_start_indices, restore_token_order, expert_ids,
                                     expert_usage_stats, (const int32_t*)topk_ids, n, num_experts, (hipStream_t)stream);
}

int maxfp8_fused_silu(void* out, void* out_scales, const void* in, const uint32_t* row_offsets, int64_t num_offsets,
                      int64_t max_rows, int64_t inter, int64_t in_row_stride, int64_t out_row_stride, int64_t scales_ld,
                      int in_dtype, int quantize, void* stream) {
  if (in_dtype != MAXFP8_BF16) MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "fused_silu: input dtype %d is not bf16", in_dtype);
  if (max_rows < 0 || inter < 0 || num_offsets < 1) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused_silu: bad sizes");
  if (max_rows == 0 || inter == 0) return MAXFP8_OK;
  if (inter % 128 != 0)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused_silu: the output width %lld must be a multiple of 128", (long long)inter);
  if (quantize < 0 || quantize > 2) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused_silu: quantize = %d is not 0, 1 or 2", quantize);
  const bool quant = quantize == 1;
  if (in_row_stride < 2 * inter || out_row_stride < inter || (quant && scales_ld < max_rows))
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused_silu: strides smaller than the extents");
  if (!out || !in || !row_offsets || (quant && !out_scales)) MAXFP8_FAIL(MAXFP8_ERR_NULL, "fused_silu: null pointer");
  if (!is_aligned(in, 16) || in_row_stride % 8 != 0 || !is_aligned(out, 16) || out_row_stride % 8 != 0)
    MAXFP8_FAIL(MAXFP8_ERR_ALIGN, "fused_silu: rows must be 16-byte aligned");
  return fused_silu_dispatch(out, (float*)out_scales, in, row_offsets, num_offsets, max_rows, inter, in_row_stride,
                             out_row_stride, scales_ld, quantize, (hipStream_t)stream);
}

size_t maxfp8_matmul_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || gemm_skinny_preferred(M, N, K)) return 0;
  return gemm_tiled_workspace_bytes(M, N, K);  // split-K partial sums; 0 when no split would be used
}

}  // extern "C"

namespace maxfp8 {
struct BatchStrides { int64_t n, a, b, c, a_scales, b_scales; };  // n batches; steps in elements

static int matmul_common(void* c, const void* a, const void* b, const void* a_scales, const void* b_scales, int64_t M,
                         int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int input_granularity,
                         int weight_granularity, int64_t gm, int64_t gn, int64_t gk, int64_t a_scales_ld,
                         int64_t b_scales_ld, int c_dtype, int scales_dtype, int algo, void* workspace,
                         size_t workspace_bytes, const BatchStrides& bt, void* stream) {
  if (c_dtype != MAXFP8_BF16 && c_dtype != MAXFP8_F32)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "matmul: output dtype %d is not bf16 or f32", c_dtype);
  if (M < 0 || N < 0 || K < 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "matmul: negative size");
  if (M == 0 || N == 0) return MAXFP8_OK;  // fp8_quantization.mojo:1103-1104
  if (M >= ((int64_t)1 << 31) || N >= ((int64_t)1 << 31) || K >= ((int64_t)1 << 31))
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "matmul: sizes must fit 31 bits");
  if (lda < K || ldb < K || ldc < N) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "matmul: leading dimension smaller than the row length");
  if (!c || !a || !b || !a_scales || !b_scales) MAXFP8_FAIL(MAXFP8_ERR_NULL, "matmul: null pointer");

  const bool block = input_granularity == MAXFP8_GRAN_BLOCK && weight_granularity == MAXFP8_GRAN_BLOCK;
  const bool row = input_granularity == MAXFP8_GRAN_COLWISE && weight_granularity == MAXFP8_GRAN_ROWWISE;
  const bool tensor = input_granularity == MAXFP8_GRAN_TENSOR && weight_granularity == MAXFP8_GRAN_TENSOR;
  if (!block && !row && !tensor) MAXFP8_FAIL(MAXFP8_ERR_GRANULARITY, "unsupported FP8 scaling granularity");
  hipStream_t st = (hipStream_t)stream;

  if (block) {
    if (scales_dtype != MAXFP8_F32) MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "a_scales and b_scales dtypes must be float32");
    if (gm <= 0 || gn <= 0 || gk <= 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "matmul: block granularities must be positive");
    if (a_scales_ld < ceil_div(M, gm) || b_scales_ld < ceil_div(K, gk))
      MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "matmul: scale leading dimensions too small");
  } else if (scales_dtype != MAXFP8_F32 && scales_dtype != MAXFP8_BF16 && scales_dtype != MAXFP8_F16) {
    // the three scale dtypes of the reference (fp8_quantization.mojo:996-1018)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "matmul: scales dtype %d is not f32, bf16 or f16", scales_dtype);
  }

  // Fast kernels: 16-byte aligned rows, K a multiple of 16, and for block scaling the
  // (1, 128, 128) granularity.  (Row / tensor scales of any dtype are widened in the epilogue.)
  const bool fast_layout = is_aligned(a, 16) && is_aligned(b, 16) && lda % 16 == 0 && ldb % 16 == 0 && K % 16 == 0 &&
                           K > 0 && (!block || (gm == 1 && gn == 128 && gk == 128)) &&
                           (bt.n == 1 || (bt.a % 16 == 0 && bt.b % 16 == 0)) && offsets_fit(K, lda, ldb, a_scales_ld, block);
  if (algo == MAXFP8_ALGO_AUTO) {
    if (!fast_layout) algo = MAXFP8_ALGO_NAIVE;
    else if (gemm_skinny_preferred(M, N, K)) algo = MAXFP8_ALGO_SKINNY;
    else algo = MAXFP8_ALGO_TILED;
    // 33 to 64 rows: the tiles win through their K split.  Without the workspace the split needs, a narrow weight
    // matrix would run on a fraction of the chip: the streaming kernel then.  (What this shape's own plan needs, not the
    // worst case over all tile shapes: a plan that does not split runs the same with and without a workspace.)
    if (algo == MAXFP8_ALGO_TILED && M <= gemm_skinny_max_m() && bt.n == 1 &&
        gemm_tiled_plan_workspace_bytes(M, N, K, block) > (workspace ? workspace_bytes : 0))
      algo = MAXFP8_ALGO_SKINNY;
  }
  if (algo == MAXFP8_ALGO_NAIVE) {
    if (block)
      return naive_blockwise_dispatch(c, a, b, a_scales, b_scales, M, N, K, lda, ldb, ldc, gm, gn, gk, a_scales_ld,
                                      b_scales_ld, c_dtype, bt.n, bt.a, bt.b, bt.c, bt.a_scales, bt.b_scales, st);
    if (bt.n != 1) MAXFP8_FAIL(MAXFP8_ERR_GRANULARITY, "batched matmul: only block scaling is supported");
    return naive_rowwise_dispatch(c, a, b, a_scales, b_scales, M, N, K, lda, ldb, ldc, tensor ? 0 : 1,
                                  tensor ? 0 : b_scales_ld, c_dtype, scales_dtype, st);
  }
  if (algo != MAXFP8_ALGO_TILED && algo != MAXFP8_ALGO_SKINNY) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "matmul: unknown algo %d", algo);
  if (!fast_layout)
    MAXFP8_FAIL(MAXFP8_ERR_ALIGN,
                "matmul: the MFMA kernels need 16-byte aligned rows, K %% 16 == 0, (1,128,128) blocks and "
                "row strides below 2^31 / 256 bytes");

  GemmArgs p;
  memset(&p, 0, sizeof(p));
  p.a = (const uint8_t*)a;
  p.b = (const uint8_t*)b;
  p.c = c;
  p.a_scales = (const float*)a_scales;
  p.b_scales = (const float*)b_scales;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.a_scales_ld = a_scales_ld;
  p.b_scales_ld = b_scales_ld;
  p.a_scale_stride = tensor ? 0 : 1;
  p.b_scale_stride = tensor ? 0 : b_scales_ld;
  p.c_dtype = c_dtype;
  p.scales_dtype = scales_dtype;  // (f32 for block scaling, checked above)
  p.c_vec_ok = (ldc % 4 == 0) && is_aligned(c, c_dtype == MAXFP8_BF16 ? 8 : 16);
  p.c_vec8_ok = (ldc % 8 == 0) && is_aligned(c, 16);
  if (bt.n != 1) {  // every batch's C must keep the alignment the vector stores assume
    p.c_vec_ok = p.c_vec_ok && bt.c % 4 == 0;
    p.c_vec8_ok = p.c_vec8_ok && bt.c % 8 == 0;
  }
  p.a_batch = bt.a; p.b_batch = bt.b; p.c_batch = bt.c;
  p.a_scales_batch = bt.a_scales; p.b_scales_batch = bt.b_scales;
  if (algo == MAXFP8_ALGO_SKINNY) return gemm_skinny_dispatch(p, block, bt.n, st);
  if (workspace && !is_aligned(workspace, 16)) MAXFP8_FAIL(MAXFP8_ERR_ALIGN, "matmul: workspace must be 16-byte aligned");
  p.workspace = (float*)workspace;
  return gemm_tiled_dispatch(p, block, workspace_bytes, bt.n, st);
}
}  // namespace maxfp8

extern "C" {

int maxfp8_matmul_describe(int64_t M, int64_t N, int64_t K, int block_scaling, int with_workspace, char* buf, size_t len) {
  if (!buf || len == 0) return 0;
  if (M <= 0 || N <= 0 || K <= 0) return snprintf(buf, len, "nothing to do");
  if (gemm_skinny_preferred(M, N, K)) return snprintf(buf, len, "skinny");
  if (M <= gemm_skinny_max_m() && !with_workspace && gemm_tiled_plan_workspace_bytes(M, N, K, block_scaling != 0) > 0)
    return snprintf(buf, len, "skinny");
  return gemm_tiled_describe(M, N, K, block_scaling != 0, with_workspace != 0, buf, len);
}

int maxfp8_matmul_dynamic_scaled_fp8(void* c, const void* a, const void* b, const void* a_scales,
                                     const void* b_scales, int64_t M, int64_t N, int64_t K, int64_t lda,
                                     int64_t ldb, int64_t ldc, int input_granularity, int weight_granularity,
                                     int64_t gm, int64_t gn, int64_t gk, int64_t a_scales_ld, int64_t b_scales_ld,
                                     int c_dtype, int scales_dtype, int algo, void* workspace,
                                     size_t workspace_bytes, void* stream) {
  const BatchStrides one = {1, 0, 0, 0, 0, 0};
  return matmul_common(c, a, b, a_scales, b_scales, M, N, K, lda, ldb, ldc, input_granularity, weight_granularity, gm, gn,
                       gk, a_scales_ld, b_scales_ld, c_dtype, scales_dtype, algo, workspace, workspace_bytes, one, stream);
}

size_t maxfp8_matmul_noalloc_max_scratch_bytes(void) { return kScratchBytes; }

int maxfp8_matmul_dynamic_scaled_fp8_noalloc(void* c, const void* a, const void* b, const void* a_scales,
                                             const void* b_scales, int64_t M, int64_t N, int64_t K, int64_t lda,
                                             int64_t ldb, int64_t ldc, int input_granularity, int weight_granularity,
                                             int64_t gm, int64_t gn, int64_t gk, int64_t a_scales_ld, int64_t b_scales_ld,
                                             int c_dtype, int scales_dtype, int algo, void* stream) {
  // The scratch of the K split this shape gets when its caller brings all the workspace
  // maxfp8_matmul_workspace_bytes asks for: with exactly that much the planner lands on the same plan, so both
  // entry points add the same partial sums in the same order.
  const bool block = input_granularity == MAXFP8_GRAN_BLOCK && weight_granularity == MAXFP8_GRAN_BLOCK;
  size_t need = 0;
  if (M > 0 && N > 0 && K > 0 && maxfp8_matmul_workspace_bytes(M, N, K) > 0) need = gemm_tiled_plan_workspace_bytes(M, N, K, block);
  if (need > kScratchBytes)
    MAXFP8_FAIL(MAXFP8_ERR_WORKSPACE,
                "matmul (no-alloc): the split of %lld x %lld x %lld uses %zu bytes of scratch, the library's static buffer holds "
                "%zu; call maxfp8_matmul_dynamic_scaled_fp8 with workspace = NULL (no split, no allocation) or with a workspace",
                (long long)M, (long long)N, (long long)K, need, kScratchBytes);
  void* ws = nullptr;
  if (need > 0 && M > 0 && N > 0) {
    const int rc = scratch_of_current_device(&ws);
    if (rc != MAXFP8_OK) return rc;
  }
  // (Nothing in the scratch has to start at zero: every partial tile a split writes is written in full before the
  // reduction reads it.  Its contents after the call are the last call's partial sums.)
  const BatchStrides one = {1, 0, 0, 0, 0, 0};
  return matmul_common(c, a, b, a_scales, b_scales, M, N, K, lda, ldb, ldc, input_granularity, weight_granularity, gm, gn,
                       gk, a_scales_ld, b_scales_ld, c_dtype, scales_dtype, algo, ws, ws ? need : 0, one, stream);
}

int maxfp8_batched_matmul_dynamic_scaled_fp8(void* c, const void* a, const void* b, const void* a_scales,
                                             const void* b_scales, int64_t B, int64_t M, int64_t N, int64_t K,
                                             int64_t a_batch_stride, int64_t lda, int64_t b_batch_stride, int64_t ldb,
                                             int64_t c_batch_stride, int64_t ldc, int64_t gm, int64_t gn, int64_t gk,
                                             int64_t a_scales_batch_stride, int64_t a_scales_ld,
                                             int64_t b_scales_batch_stride, int64_t b_scales_ld, int c_dtype,
                                             int scales_dtype, int algo, void* stream) {
  if (B < 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "batched matmul: negative batch");
  if (B == 0) return MAXFP8_OK;
  if (B > 65535) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "batched matmul: batch %lld exceeds 65535", (long long)B);
  const BatchStrides bt = {B, a_batch_stride, b_batch_stride, c_batch_stride, a_scales_batch_stride, b_scales_batch_stride};
  return matmul_common(c, a, b, a_scales, b_scales, M, N, K, lda, ldb, ldc, MAXFP8_GRAN_BLOCK, MAXFP8_GRAN_BLOCK, gm, gn, gk,
                       a_scales_ld, b_scales_ld, c_dtype, scales_dtype, algo, nullptr, 0, bt, stream);
}

int maxfp8_fused_qkv_matmul_ragged_paged_scale(void* output, const void* input, const uint32_t* input_row_offsets,
                                               const void* wqkv, const void* input_scale, const void* weight_scale,
                                               void* kv_blocks, const uint32_t* cache_lengths, const uint32_t* lookup_table,
                                               const void* bias, int64_t T, int64_t N, int64_t K, int64_t q_dim,
                                               int64_t batch_size, int64_t num_blocks, int64_t kv_dim, int64_t num_layers,
                                               int64_t layer_idx, int64_t page_size, int64_t num_kv_heads, int64_t head_dim,
                                               int64_t lut_ld, int64_t gm, int64_t gn, int64_t gk, int64_t input_scale_ld,
                                               int64_t weight_scale_ld, int scales_dtype, int algo, void* stream) {
  if (T < 0 || N < 0 || K < 0 || q_dim < 0 || batch_size < 0) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused qkv matmul: negative size");
  if (batch_size == 0 || T == 0 || N == 0) return MAXFP8_OK;  // kv_cache_ragged.mojo:1193-1194
  if (T >= ((int64_t)1 << 31) || N >= ((int64_t)1 << 31) || K >= ((int64_t)1 << 31) || batch_size >= ((int64_t)1 << 31))
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused qkv matmul: sizes must fit 31 bits");
  if (kv_dim != 1 && kv_dim != 2) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused qkv matmul: the cache holds 2 (K, V) or 1 (MLA) planes, got %lld", (long long)kv_dim);
  if (num_blocks <= 0 || num_layers <= 0 || layer_idx < 0 || layer_idx >= num_layers || page_size <= 0 || num_kv_heads <= 0 ||
      head_dim <= 0 || lut_ld <= 0)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused qkv matmul: bad cache geometry");
  const int64_t k_dim = num_kv_heads * head_dim;
  const int64_t rest = N - q_dim;
  if (rest != k_dim && !(rest == 2 * k_dim && kv_dim == 2))
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused qkv matmul: N = %lld is not q_dim %lld plus one or two times kv_heads * head_dim = %lld",
                (long long)N, (long long)q_dim, (long long)k_dim);
  if (!input || !wqkv || !input_scale || !weight_scale || !kv_blocks || !cache_lengths || !lookup_table || !input_row_offsets ||
      (q_dim > 0 && !output))
    MAXFP8_FAIL(MAXFP8_ERR_NULL, "fused qkv matmul: null pointer");
  if (scales_dtype != MAXFP8_F32) MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "fused qkv matmul: scales must be float32");
  const bool per_tensor = gm == -1 && gn == -1 && gk == -1;
  const bool per_channel = gm == 1 && gn == 1 && gk == -1;
  const bool block = !per_tensor && !per_channel;
  if (block && !(gm == 1 && gn == 128 && gk == 128))
    MAXFP8_FAIL(MAXFP8_ERR_GRANULARITY, "fused qkv matmul: block scaling needs the (1, 128, 128) granularity");
  if (block && (input_scale_ld < T || weight_scale_ld < ceil_div(K, 128)))
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused qkv matmul: scale leading dimensions too small");
  // the MFMA kernels' layout, and 8-element chunks that stay inside one of Q / K / V and one cache row
  if (!is_aligned(input, 16) || !is_aligned(wqkv, 16) || K % 16 != 0 || K <= 0)
    MAXFP8_FAIL(MAXFP8_ERR_ALIGN, "fused qkv matmul: needs 16-byte aligned rows and K %% 16 == 0");
  if (!offsets_fit(K, K, K, input_scale_ld, block))
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused qkv matmul: K = %lld is too long for the kernels' 32-bit tile offsets", (long long)K);
  if (q_dim % 8 != 0 || k_dim % 8 != 0 || !is_aligned(kv_blocks, 16) || (q_dim > 0 && !is_aligned(output, 16)))
    MAXFP8_FAIL(MAXFP8_ERR_ALIGN, "fused qkv matmul: q_dim and kv_heads * head_dim must be multiples of 8, buffers 16-byte aligned");

  GemmArgs p;
  memset(&p, 0, sizeof(p));
  p.a = (const uint8_t*)input;
  p.b = (const uint8_t*)wqkv;
  p.c = output;
  p.a_scales = (const float*)input_scale;
  p.b_scales = (const float*)weight_scale;
  p.M = (int)T; p.N = (int)N; p.K = (int)K;
  p.lda = K; p.ldb = K; p.ldc = q_dim;
  p.a_scales_ld = input_scale_ld;
  p.b_scales_ld = weight_scale_ld;
  p.a_scale_stride = per_tensor ? 0 : 1;
  p.b_scale_stride = per_tensor ? 0 : weight_scale_ld;
  p.c_dtype = MAXFP8_BF16;
  p.scales_dtype = MAXFP8_F32;
  p.c_vec_ok = 1;
  p.c_vec8_ok = 1;
  p.kv_on = 1;
  const int64_t plane = page_size * k_dim;  // one (block, K|V, layer) plane
  uint16_t* blocks = (uint16_t*)kv_blocks;
  p.kv.k_base = blocks + layer_idx * plane;
  p.kv.v_base = kv_dim == 2 ? blocks + (num_layers + layer_idx) * plane : nullptr;
  p.kv.lookup_table = lookup_table;
  p.kv.cache_lengths = cache_lengths;
  p.kv.row_offsets = input_row_offsets;
  p.kv.bias = (const uint16_t*)bias;
  p.kv.block_stride = kv_dim * num_layers * plane;
  p.kv.lut_ld = lut_ld;
  p.kv.num_blocks = num_blocks;
  p.kv.q_dim = (int)q_dim;
  p.kv.k_dim = (int)k_dim;
  p.kv.row_elems = (int)k_dim;
  p.kv.page_size = (int)page_size;
  p.kv.batch = (int)batch_size;
  p.kv.bf16_scaling = block ? 0 : 1;
  hipStream_t st = (hipStream_t)stream;
  if (algo == MAXFP8_ALGO_AUTO) algo = T <= gemm_skinny_max_m() ? MAXFP8_ALGO_SKINNY : MAXFP8_ALGO_TILED;
  if (algo == MAXFP8_ALGO_SKINNY) return gemm_skinny_dispatch(p, block, 1, st);
  if (algo != MAXFP8_ALGO_TILED) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "fused qkv matmul: algo %d is not available", algo);
  return gemm_tiled_dispatch(p, block, 0, 1, st);
}

}  // extern "C"

static int grouped_block_common(void* c, const uint32_t* c_row_index, const void* a, const void* b, const void* a_scales,
                                const void* b_scales, const uint32_t* expert_start_indices, const int32_t* expert_ids,
                                int64_t T, int64_t N, int64_t K, int64_t num_experts, int64_t max_num_tokens_per_expert,
                                int64_t num_active_experts, int64_t a_scales_ld, int c_dtype, int scales_dtype, int algo,
                                void* stream) {
  if (c_dtype != MAXFP8_BF16 && c_dtype != MAXFP8_F32)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "grouped matmul: output dtype %d is not bf16 or f32", c_dtype);
  if (scales_dtype != MAXFP8_F32)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "grouped matmul: scales must be float32");
  if (T < 0 || N < 0 || K < 0 || num_experts < 0 || max_num_tokens_per_expert < 0 || num_active_experts < 0)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped matmul: negative size");
  // grouped_matmul_sm100_blockwise_fp8.mojo:3016-3017
  if (max_num_tokens_per_expert == 0 || num_active_experts == 0 || T == 0 || N == 0) return MAXFP8_OK;
  if (num_active_experts > num_experts)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped matmul: %lld active slots but expert_ids holds %lld", (long long)num_active_experts,
                (long long)num_experts);
  if (T >= ((int64_t)1 << 31) || N >= ((int64_t)1 << 31) || K >= ((int64_t)1 << 31))
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped matmul: sizes must fit 31 bits");
  if (a_scales_ld < T) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped matmul: a_scales leading dimension %lld < T = %lld",
                                   (long long)a_scales_ld, (long long)T);
  if (!c || !a || !b || !a_scales || !b_scales || !expert_start_indices || !expert_ids)
    MAXFP8_FAIL(MAXFP8_ERR_NULL, "grouped matmul: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const bool fast_layout = is_aligned(a, 16) && is_aligned(b, 16) && K % 16 == 0 && K > 0 && offsets_fit(K, K, K, a_scales_ld, true);
  if (algo == MAXFP8_ALGO_AUTO) algo = fast_layout ? MAXFP8_ALGO_TILED : MAXFP8_ALGO_NAIVE;
  if (algo == MAXFP8_ALGO_NAIVE && c_row_index)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped matmul: the row scatter needs the MFMA kernel (16-byte aligned rows, K %% 16 == 0)");
  if (algo == MAXFP8_ALGO_NAIVE)
    return naive_grouped_dispatch(c, a, b, a_scales, b_scales, expert_start_indices, expert_ids, T, N, K,
                                  max_num_tokens_per_expert, num_active_experts, a_scales_ld, c_dtype, st);
  if (algo != MAXFP8_ALGO_TILED) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped matmul: unknown algo %d", algo);
  if (!fast_layout) MAXFP8_FAIL(MAXFP8_ERR_ALIGN, "grouped matmul: the MFMA kernel needs 16-byte aligned rows and K %% 16 == 0");

  GemmArgs p;
  memset(&p, 0, sizeof(p));
  p.a = (const uint8_t*)a;
  p.b = (const uint8_t*)b;
  p.c = c;
  p.a_scales = (const float*)a_scales;
  p.b_scales = (const float*)b_scales;
  p.M = (int)T; p.N = (int)N; p.K = (int)K;
  p.lda = K; p.ldb = K; p.ldc = N;
  p.a_scales_ld = a_scales_ld;
  p.b_scales_ld = ceil_div(K, 128);
  p.c_dtype = c_dtype;
  p.scales_dtype = MAXFP8_F32;
  p.c_vec_ok = (N % 4 == 0) && is_aligned(c, c_dtype == MAXFP8_BF16 ? 8 : 16);
  p.c_vec8_ok = (N % 8 == 0) && is_aligned(c, 16);
  p.offsets = expert_start_indices;
  p.expert_ids = expert_ids;
  p.num_active = (int)num_active_experts;
  p.b_expert_stride = N * K;
  p.bs_expert_stride = ceil_div(N, 128) * ceil_div(K, 128);
  p.c_row_index = c_row_index;
  return gemm_grouped_dispatch(p, true, T, max_num_tokens_per_expert, st);
}

extern "C" {

int maxfp8_grouped_matmul_dynamic_scaled_fp8(void* c, const void* a, const void* b, const void* a_scales,
                                             const void* b_scales, const uint32_t* expert_start_indices,
                                             const int32_t* expert_ids, int64_t T, int64_t N, int64_t K,
                                             int64_t num_experts, int64_t max_num_tokens_per_expert,
                                             int64_t num_active_experts, int64_t a_scales_ld, int c_dtype,
                                             int scales_dtype, int algo, void* stream) {
  return grouped_block_common(c, nullptr, a, b, a_scales, b_scales, expert_start_indices, expert_ids, T, N, K, num_experts,
                              max_num_tokens_per_expert, num_active_experts, a_scales_ld, c_dtype, scales_dtype, algo, stream);
}

int maxfp8_grouped_matmul_dynamic_scaled_fp8_scatter(void* c, const uint32_t* c_row_index, const void* a, const void* b,
                                                     const void* a_scales, const void* b_scales,
                                                     const uint32_t* expert_start_indices, const int32_t* expert_ids,
                                                     int64_t T, int64_t N, int64_t K, int64_t num_experts,
                                                     int64_t max_num_tokens_per_expert, int64_t num_active_experts,
                                                     int64_t a_scales_ld, int c_dtype, int scales_dtype, int algo,
                                                     void* stream) {
  if (T > 0 && N > 0 && !c_row_index) MAXFP8_FAIL(MAXFP8_ERR_NULL, "grouped matmul (scatter): null row index");
  return grouped_block_common(c, c_row_index, a, b, a_scales, b_scales, expert_start_indices, expert_ids, T, N, K, num_experts,
                              max_num_tokens_per_expert, num_active_experts, a_scales_ld, c_dtype, scales_dtype, algo, stream);
}

int maxfp8_grouped_matmul_rowwise_dynamic_scaled_fp8(void* c, const void* a, const void* b, const void* a_scales,
                                                     const void* b_scales, const uint32_t* expert_start_indices,
                                                     const int32_t* expert_ids, int64_t T, int64_t N, int64_t K,
                                                     int64_t num_experts, int64_t max_num_tokens_per_expert,
                                                     int64_t num_active_experts, int c_dtype, int scales_dtype, void* stream) {
  if (c_dtype != MAXFP8_BF16 && c_dtype != MAXFP8_F32)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "grouped rowwise matmul: output dtype %d is not bf16 or f32", c_dtype);
  if (scales_dtype != MAXFP8_F32)
    MAXFP8_FAIL(MAXFP8_ERR_DTYPE, "grouped rowwise matmul: A and B scales must be float32 for rowwise/per-token granularity");
  if (T < 0 || N < 0 || K < 0 || num_experts < 0 || max_num_tokens_per_expert < 0 || num_active_experts < 0)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped rowwise matmul: negative size");
  // grouped_matmul.mojo:1675-1676
  if (max_num_tokens_per_expert == 0 || num_active_experts == 0 || T == 0 || N == 0) return MAXFP8_OK;
  if (num_active_experts > num_experts)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped rowwise matmul: %lld active slots but expert_ids holds %lld",
                (long long)num_active_experts, (long long)num_experts);
  if (T >= ((int64_t)1 << 31) || N >= ((int64_t)1 << 31) || K >= ((int64_t)1 << 31))
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped rowwise matmul: sizes must fit 31 bits");
  if (!c || !a || !b || !a_scales || !b_scales || !expert_start_indices || !expert_ids)
    MAXFP8_FAIL(MAXFP8_ERR_NULL, "grouped rowwise matmul: null pointer");
  if (!(is_aligned(a, 16) && is_aligned(b, 16) && K % 16 == 0 && K > 0))
    MAXFP8_FAIL(MAXFP8_ERR_ALIGN, "grouped rowwise matmul: needs 16-byte aligned rows and K %% 16 == 0");
  if (!offsets_fit(K, K, K, 0, false))
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "grouped rowwise matmul: K = %lld is too long for the kernels' 32-bit tile offsets", (long long)K);
  GemmArgs p;
  memset(&p, 0, sizeof(p));
  p.a = (const uint8_t*)a;
  p.b = (const uint8_t*)b;
  p.c = c;
  p.a_scales = (const float*)a_scales;  // [T, 1]
  p.b_scales = (const float*)b_scales;  // [E, N, 1]
  p.M = (int)T; p.N = (int)N; p.K = (int)K;
  p.lda = K; p.ldb = K; p.ldc = N;
  p.a_scale_stride = 1;
  p.b_scale_stride = 1;
  p.c_dtype = c_dtype;
  p.scales_dtype = MAXFP8_F32;
  p.c_vec_ok = (N % 4 == 0) && is_aligned(c, c_dtype == MAXFP8_BF16 ? 8 : 16);
  p.c_vec8_ok = (N % 8 == 0) && is_aligned(c, 16);
  p.offsets = expert_start_indices;
  p.expert_ids = expert_ids;
  p.num_active = (int)num_active_experts;
  p.b_expert_stride = N * K;
  p.bs_expert_stride = N;
  return gemm_grouped_dispatch(p, false, T, max_num_tokens_per_expert, (hipStream_t)stream);
}

int maxfp8_cast_f32_to_e4m3fn(void* out_fp8, const float* in, int64_t n, void* stream) {
  if (n <= 0) return MAXFP8_OK;
  if (!out_fp8 || !in) MAXFP8_FAIL(MAXFP8_ERR_NULL, "cast: null pointer");
  return cast_f32_to_e4m3fn_dispatch(out_fp8, in, n, (hipStream_t)stream);
}

int maxfp8_cast_e4m3fn_to_f32(float* out, const void* in_fp8, int64_t n, void* stream) {
  if (n <= 0) return MAXFP8_OK;
  if (!out || !in_fp8) MAXFP8_FAIL(MAXFP8_ERR_NULL, "cast: null pointer");
  return cast_e4m3fn_to_f32_dispatch(out, in_fp8, n, (hipStream_t)stream);
}

int maxfp8_cast_f32_to_bf16(void* out_bf16, const float* in, int64_t n, void* stream) {
  if (n <= 0) return MAXFP8_OK;
  if (!out_bf16 || !in) MAXFP8_FAIL(MAXFP8_ERR_NULL, "cast: null pointer");
  return cast_f32_to_bf16_dispatch(out_bf16, in, n, (hipStream_t)stream);
}

int maxfp8_copy_bytes(void* dst, const void* src, int64_t n, void* stream) {
  if (n <= 0) return MAXFP8_OK;
  if (!dst || !src) MAXFP8_FAIL(MAXFP8_ERR_NULL, "copy: null pointer");
  if (n % 16 != 0 || !is_aligned(dst, 16) || !is_aligned(src, 16))
    MAXFP8_FAIL(MAXFP8_ERR_ALIGN, "copy: size and pointers must be multiples of 16 bytes");
  return copy_bytes_dispatch(dst, src, n, (hipStream_t)stream);
}

int maxfp8_decode_weight_read_probe(const void* b, int64_t M, int64_t N, int64_t K, int64_t ldb, void* stream) {
  if (!b) MAXFP8_FAIL(MAXFP8_ERR_NULL, "read probe: null pointer");
  if (M <= 0 || M > 16 || N <= 0 || K <= 0 || ldb < K)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "read probe: needs 1 <= M <= 16, N > 0, 0 < K <= ldb (got M %lld, N %lld, K %lld, ldb %lld)",
                (long long)M, (long long)N, (long long)K, (long long)ldb);
  if (!is_aligned(b, 16) || K % 16 != 0 || ldb % 16 != 0) MAXFP8_FAIL(MAXFP8_ERR_ALIGN, "read probe: needs 16-byte aligned rows and K %% 16 == 0");
  if (!offsets_fit(K, ldb, ldb, 0, false)) MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "read probe: rows too long for 32-bit tile offsets");
  return gemm_skinny_read_probe(b, M, N, K, ldb, (hipStream_t)stream);
}

long long maxfp8_handovers_given_up(void) {
  unsigned int pieces = 0, shares = 0;
  int rc = gemm_w4_gave_up(&pieces);
  if (rc == MAXFP8_OK) rc = gemm_streamk_gave_up(&shares);
  return rc == MAXFP8_OK ? (long long)pieces + (long long)shares : (long long)rc;
}

int maxfp8_mfma_issue_probe(int kernel, int blockscale, int level, int64_t slabs, const void* a, const void* b, const float* a_scales,
                            const float* b_scales, void* c, uint64_t* clocks, void* stream) {
  if (!a || !b || !c || !a_scales || !b_scales) MAXFP8_FAIL(MAXFP8_ERR_NULL, "issue probe: null pointer");
  if (clocks && !is_aligned(clocks, 8)) MAXFP8_FAIL(MAXFP8_ERR_ALIGN, "issue probe: clocks must be 8-byte aligned");
  if ((kernel != 0 && kernel != 4 && kernel != 5 && kernel != 6) || (level != 1 && level != 2) || slabs < 8 || slabs > (1 << 22) || slabs % 2 != 0)
    MAXFP8_FAIL(MAXFP8_ERR_SHAPE, "issue probe: kernel 0 / 4 / 5 / 6, level 1 / 2, an even number of slabs in [8, 2^22]");
  if (!is_aligned(a, 16) || !is_aligned(b, 16) || !is_aligned(c, 16)) MAXFP8_FAIL(MAXFP8_ERR_ALIGN, "issue probe: 16-byte aligned buffers");
  GemmArgs p;
  memset(&p, 0, sizeof(p));
  p.a = (const uint8_t*)a;
  p.b = (const uint8_t*)b;
  p.c = c;
  p.a_scales = a_scales;
  p.b_scales = b_scales;
  p.M = 256; p.N = 256; p.K = (int)(slabs * 128);
  p.lda = 1024; p.ldb = 1024; p.ldc = 256;
  p.a_scales_ld = 256; p.b_scales_ld = 8;
  p.a_scale_stride = 0; p.b_scale_stride = 0;  // (row mode: element 0 of each scale vector, in the epilogue)
  p.c_dtype = MAXFP8_BF16;
  p.scales_dtype = MAXFP8_F32;
  p.c_vec_ok = 1; p.c_vec8_ok = 1;
  p.splits = 1;
  p.workspace = reinterpret_cast<float*>(clocks);
  return kernel == 0 ? gemm_persist_probe(p, blockscale != 0, level, (hipStream_t)stream) : gemm_w4_probe(p, blockscale != 0, level, kernel, (hipStream_t)stream);
}

}  // extern "C"
