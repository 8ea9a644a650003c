/*
 * maxfp8.h -- C ABI of the MI355X (gfx950) FP8 linear hot path.
 *
 * The operators, named after the MAX custom ops they stand in for:
 *
 *   mo.quantize_dynamic_scaled_float8      -> maxfp8_quantize_dynamic_scaled_fp8
 *   mo.matmul_dynamic_scaled_fp8           -> maxfp8_matmul_dynamic_scaled_fp8
 *   mo.grouped.matmul.dynamic.scaled.fp8   -> maxfp8_grouped_matmul_dynamic_scaled_fp8
 *   mo.batched.matmul.dynamic.scaled.fp8   -> maxfp8_batched_matmul_dynamic_scaled_fp8
 *   mo.fused_qkv_matmul.ragged.paged.scale -> maxfp8_fused_qkv_matmul_ragged_paged_scale
 *
 * Conventions (the same as the reference's destination-passing custom-op ABI,
 * max/kernels/src/graph_compiler/extensibility/decorators.mojo:46-131):
 *   - every pointer is a DEVICE pointer owned by the caller; outputs are
 *     pre-allocated; the library never allocates or frees caller memory;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 *     null stream) and the call returns without synchronising;
 *   - zero-sized work is a silent no-op returning MAXFP8_OK;
 *   - the return value is MAXFP8_OK (0) or a negative maxfp8_status; the text of
 *     the last error on the calling thread is returned by maxfp8_last_error().
 */
#ifndef MAXFP8_H
#define MAXFP8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum maxfp8_status {
  MAXFP8_OK = 0,
  MAXFP8_ERR_DTYPE = -1,       /* unsupported element / scale dtype            */
  MAXFP8_ERR_SHAPE = -2,       /* inconsistent sizes, strides or group size    */
  MAXFP8_ERR_ALIGN = -3,       /* pointer or stride alignment not supported    */
  MAXFP8_ERR_GRANULARITY = -4, /* unsupported scaling granularity combination  */
  MAXFP8_ERR_LAUNCH = -5,      /* HIP reported an error at launch              */
  MAXFP8_ERR_NULL = -6,        /* required pointer was NULL                    */
  MAXFP8_ERR_WORKSPACE = -7    /* reserved: a missing or short workspace is not an
                                  error, the matmul then runs without split-K  */
} maxfp8_status;

typedef enum maxfp8_dtype {
  MAXFP8_BF16 = 0,
  MAXFP8_F16 = 1,
  MAXFP8_F32 = 2,
  MAXFP8_E4M3FN = 3
} maxfp8_dtype;

/* Scaling granularity names, verbatim from
 * max/python/max/nn/quant_config.py:26-46 (ScaleGranularity). */
typedef enum maxfp8_granularity {
  MAXFP8_GRAN_TENSOR = 0,
  MAXFP8_GRAN_ROWWISE = 1,
  MAXFP8_GRAN_COLWISE = 2,
  MAXFP8_GRAN_BLOCK = 3
} maxfp8_granularity;

/* Kernel selection for the dense matmul.  AUTO picks by shape. */
typedef enum maxfp8_algo {
  MAXFP8_ALGO_AUTO = 0,
  MAXFP8_ALGO_NAIVE = 1,  /* one thread per output, reference summation order */
  MAXFP8_ALGO_TILED = 2,  /* LDS-staged MFMA tiles                            */
  MAXFP8_ALGO_SKINNY = 3  /* weight-streaming kernel for M <= 64              */
} maxfp8_algo;

const char* maxfp8_last_error(void);
const char* maxfp8_version(void);

/*
 * The kernel selection reads its tuning switches (MAXFP8_TILE, MAXFP8_SPLITK, MAXFP8_SKINNY, ...;
 * the list is in modular_amd/csrc/tuning.h) from the environment once per process.  This call
 * reads them again: for tuning runs and tests that change a switch between calls.  No counterpart
 * in the reference.
 */
void maxfp8_tuning_reload(void);

/*
 * Dynamic activation quantisation.
 * Replaces QuantizeDynamicScaledFloat8.execute
 *   (max/kernels/src/graph_compiler/builtin_kernels/quantization.mojo:1363-1406)
 * -> quantize_dynamic_scaled_fp8 (max/kernels/src/linalg/fp8_quantization.mojo:369-463).
 *
 *   in          [M, K] row-major with row stride `in_row_stride` elements,
 *               dtype `in_dtype` (MAXFP8_BF16, MAXFP8_F16 or MAXFP8_F32)
 *   out_fp8     [M, K] e4m3fn bytes, row stride `out_row_stride` bytes
 *   out_scales  [K / group_size, scales_ld] of `scales_dtype` (MAXFP8_F32 or
 *               MAXFP8_BF16); element (g, r) = scale of row r, group g
 *               (TRANSPOSED, fp8_quantization.mojo:564-565); columns
 *               M..scales_ld-1 are never written
 *   group_size  128 for blockwise, K for per-token; must divide K and be a
 *               multiple of 4
 *   scale_ub    upper clamp on the group amax (1200.0 in every reference call,
 *               max/python/max/nn/kernels.py:6880)
 */
int maxfp8_quantize_dynamic_scaled_fp8(
    void* out_fp8, void* out_scales, const void* in,
    int64_t M, int64_t K, int64_t in_row_stride, int64_t out_row_stride,
    int64_t group_size, int64_t scales_ld,
    int in_dtype, int scales_dtype, float scale_ub, void* stream);

/*
 * The same with a row gather in front: output row r is quantised from input row
 * row_index[r] / index_div.  The FFI form of the fused input the reference's op takes
 * (FusedInputTensor, builtin_kernels/quantization.mojo:1376-1390): the MoE layer quantises
 * x gathered by token_expert_order / top_k (max/python/max/nn/moe/moe_fp8.py:525-560)
 * without materialising the gathered copy.  row_index is a device array of M uint32.
 */
int maxfp8_quantize_dynamic_scaled_fp8_gather(
    void* out_fp8, void* out_scales, const void* in, const uint32_t* row_index, int64_t index_div,
    int64_t M, int64_t K, int64_t in_row_stride, int64_t out_row_stride,
    int64_t group_size, int64_t scales_ld,
    int in_dtype, int scales_dtype, float scale_ub, void* stream);

/*
 * The same fused input seen from the other side, for a gather whose source rows repeat: input row r
 * is quantised once and written to the output rows dst_index[r * copies + j], j < copies (rows of
 * out_fp8, columns of out_scales; a destination >= out_rows is skipped).  With dst_index the inverse
 * of the gather's row_index it writes the same bytes as maxfp8_quantize_dynamic_scaled_fp8_gather:
 * the MoE layer (max/python/max/nn/moe/moe_fp8.py:525-560) quantises each token once and stores it
 * to its top_k sorted rows restore_token_order[token * top_k + j] instead of quantising it top_k
 * times.  bfloat16 input, float32 scales, group_size 128, 16-byte aligned rows; anything else is an
 * error that names the gather form.  dst_index is a device array of M * copies uint32.
 */
int maxfp8_quantize_dynamic_scaled_fp8_scatter(
    void* out_fp8, void* out_scales, const void* in, const uint32_t* dst_index, int64_t copies,
    int64_t M, int64_t K, int64_t out_rows, int64_t in_row_stride, int64_t out_row_stride,
    int64_t group_size, int64_t scales_ld,
    int in_dtype, int scales_dtype, float scale_ub, void* stream);

/*
 * Batched dynamic activation quantisation: B independent [M, K] problems in one
 * launch.  Replaces batched_quantize_dynamic_scaled_fp8
 *   (max/kernels/src/linalg/fp8_quantization.mojo:779-954), which the MLA
 * graph calls on a [row, batch, col] view of its activations
 *   (max/kernels/src/nn/attention/gpu/mla_graph.mojo:1010-1033): hence the free
 * batch and row strides of the input.
 *
 *   in          element (b, m, k) at in + b * in_batch_stride + m * in_row_stride + k
 *   out_fp8     [B, M, K]: byte (b, m, k) at b * out_batch_stride + m * out_row_stride + k
 *   out_scales  [B, K / group_size, scales_ld]: element (b, g, m) at
 *               b * scales_batch_stride + g * scales_ld + m
 *   B           at most 65535; B == 0 is a no-op (fp8_quantization.mojo:826-827)
 * Everything else as in maxfp8_quantize_dynamic_scaled_fp8; each batch gets
 * exactly that function's result.
 */
int maxfp8_batched_quantize_dynamic_scaled_fp8(
    void* out_fp8, void* out_scales, const void* in,
    int64_t B, int64_t M, int64_t K,
    int64_t in_batch_stride, int64_t in_row_stride,
    int64_t out_batch_stride, int64_t out_row_stride,
    int64_t group_size, int64_t scales_batch_stride, int64_t scales_ld,
    int in_dtype, int scales_dtype, float scale_ub, void* stream);

/*
 * Scaled FP8 matmul, C = A . B^T with B stored [N, K] ("transpose_b").
 * Replaces MatmulDynamicScaledFloat8.execute
 *   (max/kernels/src/graph_compiler/builtin_kernels/linalg.mojo:1677-1720)
 * -> matmul_dynamic_scaled_fp8 (max/kernels/src/linalg/fp8_quantization.mojo:963-1334).
 *
 *   a  [M, K] e4m3fn, row stride lda bytes     b  [N, K] e4m3fn, row stride ldb bytes
 *   c  [M, N] of c_dtype (MAXFP8_BF16 or MAXFP8_F32), row stride ldc elements
 *
 *   input/weight granularity BLOCK/BLOCK with (gm, gn, gk) = (1, 128, 128):
 *       a_scales [ceil(K/128), a_scales_ld] f32, element (k/128, m)
 *       b_scales [ceil(N/128), b_scales_ld] f32, element (n/128, k/128)
 *       C[m,n] = sum_k A[m,k] B[n,k] a_scales[k/128,m] b_scales[n/128,k/128]
 *   input COLWISE, weight ROWWISE (per-token / per-output-channel):
 *       a_scales [1, M], b_scales [N, 1] (b_scales_ld = element stride between
 *       rows of b_scales, normally 1)
 *       C[m,n] = (sum_k A[m,k] B[n,k]) * a_scales[m] * b_scales[n]
 *   input TENSOR, weight TENSOR: a_scales[0], b_scales[0].
 *
 *   scales_dtype MAXFP8_F32 (block requires it), or MAXFP8_BF16 / MAXFP8_F16 for rowwise / tensor scales
 *               (the reference's three scale dtypes, fp8_quantization.mojo:996-1018): widened to f32
 *               when the epilogue loads them, on every kernel.
 *   algo        a maxfp8_algo value.
 *   workspace   optional device scratch for partial sums (a split of K, a
 *               last round of tiles computed in pieces), 16-byte aligned, of
 *               workspace_bytes bytes (maxfp8_matmul_workspace_bytes gives the
 *               size that allows every split the library would choose).  NULL
 *               or too small: the matmul runs unsplit (with at most 64 rows:
 *               on the weight-streaming kernel), which is slower only when
 *               its tiles, or those of its last round, cover a small part of
 *               the chip.  The f32 sums of a split are added in another order
 *               than those of the unsplit matmul: results with and without a
 *               workspace may differ in the last bit of a bf16 element.  The
 *               contents are scratch: overwritten by the call, meaningless
 *               afterwards; calls that overlap in time need a workspace each.
 */
int maxfp8_matmul_dynamic_scaled_fp8(
    void* c, const void* a, const void* b,
    const void* a_scales, const void* b_scales,
    int64_t M, int64_t N, int64_t K,
    int64_t lda, int64_t ldb, int64_t ldc,
    int input_granularity, int weight_granularity,
    int64_t gm, int64_t gn, int64_t gk,
    int64_t a_scales_ld, int64_t b_scales_ld,
    int c_dtype, int scales_dtype, int algo,
    void* workspace, size_t workspace_bytes, void* stream);

/*
 * maxfp8_matmul_dynamic_scaled_fp8 for callers that cannot allocate device memory -- code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc -- and therefore cannot bring a
 * workspace.  No counterpart in the reference (its matmul takes temporaries from the device context's
 * caching allocator).  Same arguments without workspace / workspace_bytes, same result: the partial
 * sums of a K split, or of the pieces a cut last round of tiles is computed in, go to a static device
 * array of the library, maxfp8_matmul_noalloc_max_scratch_bytes() = 48 MiB per GPU, held from the first
 * use of the library on that GPU until the process ends.  The call allocates and frees nothing, on the
 * device or through any library.  A shape whose K split needs more than the array holds (splits x M x N
 * x 4 bytes; the large-M, narrow-N shapes) is refused with MAXFP8_ERR_WORKSPACE and a message that says
 * so: for those, maxfp8_matmul_dynamic_scaled_fp8 with workspace = NULL runs unsplit and allocates
 * nothing either.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (two
 * streams, two threads) race on it; calls in stream order are safe, and nothing in the array needs
 * clearing between them.
 */
int maxfp8_matmul_dynamic_scaled_fp8_noalloc(
    void* c, const void* a, const void* b,
    const void* a_scales, const void* b_scales,
    int64_t M, int64_t N, int64_t K,
    int64_t lda, int64_t ldb, int64_t ldc,
    int input_granularity, int weight_granularity,
    int64_t gm, int64_t gn, int64_t gk,
    int64_t a_scales_ld, int64_t b_scales_ld,
    int c_dtype, int scales_dtype, int algo, void* stream);

/* Size of the static scratch array behind maxfp8_matmul_dynamic_scaled_fp8_noalloc. */
size_t maxfp8_matmul_noalloc_max_scratch_bytes(void);

/*
 * Batched blockwise-scaled FP8 matmul: C[b] = A[b] . B[b]^T for b < B in one
 * launch.  Replaces Struct_batched_matmul_dynamic_scaled_fp8.execute
 *   (max/kernels/src/graph_compiler/builtin_kernels/linalg.mojo:1041-1090)
 * -> batched_matmul_dynamic_scaled_fp8 (max/kernels/src/linalg/bmm.mojo:1561-1660;
 * its portable form loops the 2-D blockwise kernel over the batch, bmm.mojo:1430-1558).
 * Block scaling only, as in the reference (max/python/max/nn/kernels.py:6693-6724).
 *
 *   a         [B, M, K] e4m3fn: batch stride a_batch_stride, row stride lda (bytes)
 *   b         [B, N, K] e4m3fn: batch stride b_batch_stride, row stride ldb (bytes)
 *   c         [B, M, N] of c_dtype: batch stride c_batch_stride, row stride ldc (elements)
 *   a_scales  [B, ceil(K/128), a_scales_ld] f32, batch stride a_scales_batch_stride
 *   b_scales  [B, ceil(N/128), b_scales_ld] f32, batch stride b_scales_batch_stride
 *   B         at most 65535; B == 0 is a no-op
 * (gm, gn, gk), c_dtype, scales_dtype and algo as in
 * maxfp8_matmul_dynamic_scaled_fp8; each batch gets that function's result up to
 * the order of the f32 sums (the tile shape is chosen for the whole batch and K is
 * never split).  The MFMA kernels additionally need batch strides
 * of a and b that are multiples of 16; AUTO falls back to the naive kernel otherwise.
 */
int maxfp8_batched_matmul_dynamic_scaled_fp8(
    void* c, const void* a, const void* b,
    const void* a_scales, const void* b_scales,
    int64_t B, int64_t M, int64_t N, int64_t K,
    int64_t a_batch_stride, int64_t lda,
    int64_t b_batch_stride, int64_t ldb,
    int64_t c_batch_stride, int64_t ldc,
    int64_t gm, int64_t gn, int64_t gk,
    int64_t a_scales_batch_stride, int64_t a_scales_ld,
    int64_t b_scales_batch_stride, int64_t b_scales_ld,
    int c_dtype, int scales_dtype, int algo, void* stream);

/*
 * Diagnostic: which launches MAXFP8_ALGO_AUTO makes for a fast-layout M x N x K matmul, as text
 * ("256x256 x768 + columns from 24576: 256x128 x256", "256x128 x112, K split 4", "skinny").
 * Returns the length snprintf would have written.  No counterpart in the reference.
 */
int maxfp8_matmul_describe(int64_t M, int64_t N, int64_t K, int block_scaling, int with_workspace,
                           char* buf, size_t len);

/* Bytes of workspace that lets AUTO use every kernel for this shape. */
size_t maxfp8_matmul_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * Diagnostic with no counterpart in the reference.  Two kernels hand f32 sums from block to block inside one launch
 * (the four-wave kernel that computes its last round of tiles in pieces; the eight-wave kernel's work split along K,
 * MAXFP8_STREAMK).  A block that waits for such a hand-over does so for a bounded time (seconds: a GPU that stopped in
 * the middle of a launch gets there, and so would more such launches in flight at once on different streams than
 * there are sets of flags: 32 and 64), then fills its tile with NaN and counts the event: the call that launched it
 * has long returned MAXFP8_OK.  Returns that count for the current device since the library was loaded (0 in a
 * healthy process), or a negative maxfp8 error code.  Waits for the device's outstanding work.
 */
long long maxfp8_handovers_given_up(void);

/*
 * Fused QKV projection with the K / V columns stored straight into a paged KV cache.
 * Replaces Struct_fused_qkv_matmul_ragged_paged_scale (".bias" with a non-null bias)
 *   (max/kernels/src/graph_compiler/builtin_kernels/attention.mojo:1043-1107)
 * -> _fused_qkv_matmul_kv_cache_ragged_impl_scale (max/kernels/src/nn/kv_cache_ragged.mojo:1122-1307)
 * and, with q_dim = 0 and N = kv_heads * head_dim, mo.k_matmul.ragged.paged.scale
 *   (k_matmul_ragged_paged_scale, kv_cache_ragged.mojo:3025-3224).
 *
 *   input       [T, K] e4m3fn, contiguous; row t is token t of the ragged batch
 *   wqkv        [N, K] e4m3fn, contiguous; N = q_dim + k_dim (K only, also the MLA layout)
 *               or q_dim + 2 * k_dim (K then V), k_dim = num_kv_heads * head_dim
 *   output      [T, q_dim] bf16, receives columns [0, q_dim) (may be NULL when q_dim == 0)
 *   kv_blocks   [num_blocks, kv_dim, num_layers, page_size, num_kv_heads, head_dim] bf16,
 *               kv_dim = 2 (K, V) or 1 (MLA); column q_dim + h * head_dim + d of row t goes to
 *               kv_blocks[lookup_table[b, p / page_size], 0 (K) or 1 (V), layer_idx,
 *                         p % page_size, h, d]
 *               with b the sequence that owns row t (input_row_offsets[b] <= t <
 *               input_row_offsets[b + 1]) and p = t - input_row_offsets[b] + cache_lengths[b]
 *               (max/kernels/src/kv_cache/types.mojo:2274-2296).  A row whose page index is
 *               outside the lookup table, or whose block index is >= num_blocks, stores nothing.
 *   input_row_offsets [batch_size + 1], cache_lengths [batch_size], lookup_table [batch_size, lut_ld]: u32
 *   bias        [N] bf16 or NULL
 *   (gm, gn, gk)  the op's scales_granularity_mnk: (-1, -1, -1) per tensor (input_scale[0],
 *               weight_scale[0]); (1, 1, -1) per token / per channel (input_scale [1, T],
 *               weight_scale [N, 1] with element stride weight_scale_ld); otherwise block
 *               scaling, of which (1, 128, 128) is built: input_scale [K/128, input_scale_ld],
 *               weight_scale [N/128, weight_scale_ld].  scales_dtype must be MAXFP8_F32.
 * Values take the reference's roundings: the f32 accumulator (block: with its scales applied) is
 * rounded to bf16; per tensor / per channel that value is multiplied in bf16 by
 * bf16(bf16(input_scale) * bf16(weight_scale)); the bias is added in bf16.
 * The MFMA kernels need K % 16 == 0, 16-byte aligned buffers and q_dim, k_dim multiples of 8.
 */
int maxfp8_fused_qkv_matmul_ragged_paged_scale(
    void* output, const void* input, const uint32_t* input_row_offsets,
    const void* wqkv, const void* input_scale, const void* weight_scale,
    void* kv_blocks, const uint32_t* cache_lengths, const uint32_t* lookup_table,
    const void* bias,
    int64_t T, int64_t N, int64_t K, int64_t q_dim, int64_t batch_size,
    int64_t num_blocks, int64_t kv_dim, int64_t num_layers, int64_t layer_idx,
    int64_t page_size, int64_t num_kv_heads, int64_t head_dim, int64_t lut_ld,
    int64_t gm, int64_t gn, int64_t gk,
    int64_t input_scale_ld, int64_t weight_scale_ld,
    int scales_dtype, int algo, void* stream);

/*
 * Grouped (MoE) blockwise-scaled FP8 matmul over token rows sorted by expert.
 * Replaces Struct_grouped_matmul_dynamic_scaled_fp8.execute
 *   (max/kernels/src/graph_compiler/builtin_kernels/linalg.mojo:702-757)
 * -> grouped_matmul_dynamic_scaled_fp8
 *   (max/kernels/src/linalg/grouped_matmul_sm100_blockwise_fp8.mojo:2938-3105).
 *
 *   a  [T, K] e4m3fn (row stride K)            b  [E, N, K] e4m3fn (contiguous)
 *   c  [T, N] c_dtype (row stride N)
 *   a_scales [ceil(K/128), a_scales_ld] f32    b_scales [E, ceil(N/128), ceil(K/128)] f32
 *   expert_start_indices  uint32[num_active_experts + 1], device
 *   expert_ids            int32[num_active_experts], device; -1 => the slot's
 *                         rows of C are written with zeros
 *   max_num_tokens_per_expert, num_active_experts: host scalars; either == 0
 *                         => no-op.  max_num_tokens_per_expert is an upper bound
 *                         used only to bound the launch.
 *
 * Enqueued on `stream`; a large matmul (T >= 4096, bf16 c) runs as two launches side by side,
 * one of them on a stream the library keeps per device, ordered behind `stream` by an event
 * and joined to it by another before the call returns: work enqueued on `stream` afterwards
 * sees all of c.  Nothing is allocated per call; the call records into a HIP graph.
 */
int maxfp8_grouped_matmul_dynamic_scaled_fp8(
    void* c, const void* a, const void* b,
    const void* a_scales, const void* b_scales,
    const uint32_t* expert_start_indices, const int32_t* expert_ids,
    int64_t T, int64_t N, int64_t K, int64_t num_experts,
    int64_t max_num_tokens_per_expert, int64_t num_active_experts,
    int64_t a_scales_ld, int c_dtype, int scales_dtype, int algo, void* stream);

/*
 * maxfp8_grouped_matmul_dynamic_scaled_fp8 with a row scatter behind it: row m of the result
 * is stored at row c_row_index[m] of c (a device array of T uint32, every row of c written at
 * most once).  The FFI form of the op's output lambda: the MoE layer puts the rows of the down
 * projection back into (token, k) order -- c_row_index = token_expert_order --
 * (moe_fp8.py:614-616) without a second pass.  MFMA kernel only.
 */
int maxfp8_grouped_matmul_dynamic_scaled_fp8_scatter(
    void* c, const uint32_t* c_row_index, const void* a, const void* b,
    const void* a_scales, const void* b_scales,
    const uint32_t* expert_start_indices, const int32_t* expert_ids,
    int64_t T, int64_t N, int64_t K, int64_t num_experts,
    int64_t max_num_tokens_per_expert, int64_t num_active_experts,
    int64_t a_scales_ld, int c_dtype, int scales_dtype, int algo, void* stream);

/*
 * Grouped (MoE) FP8 matmul with per-token activation scales and per-output-channel weight
 * scales.  Replaces mo.grouped.matmul.rowwise.dynamic.scaled.fp8
 *   (wrapper max/python/max/nn/kernels.py:6490-6640)
 * -> grouped_matmul_rowwise_dynamic_scaled_fp8 (max/kernels/src/linalg/grouped_matmul.mojo:1440-1713):
 *   C[t, n] = (sum_k A[t, k] B[expert_ids[z], n, k]) * a_scales[t] * b_scales[expert_ids[z], n]
 * for the rows t of slot z; slots with expert id -1 give zeros.
 *   a [T, K], b [num_experts, N, K] e4m3fn contiguous; a_scales [T, 1], b_scales [num_experts, N, 1] f32;
 *   expert_start_indices, expert_ids, max_num_tokens_per_expert, num_active_experts as in
 *   maxfp8_grouped_matmul_dynamic_scaled_fp8.  Needs K % 16 == 0 and 16-byte aligned a, b.
 * Launches as that entry point does (a large matmul: two launches side by side, joined on `stream`).
 */
int maxfp8_grouped_matmul_rowwise_dynamic_scaled_fp8(
    void* c, const void* a, const void* b, const void* a_scales, const void* b_scales,
    const uint32_t* expert_start_indices, const int32_t* expert_ids,
    int64_t T, int64_t N, int64_t K, int64_t num_experts,
    int64_t max_num_tokens_per_expert, int64_t num_active_experts,
    int c_dtype, int scales_dtype, void* stream);

/*
 * mo.composite.rms_norm_fused_quantize_dynamic_scaled_fp8
 *   (op registration: max/kernels/src/graph_compiler/builtin_kernels/quantization.mojo:112-237;
 *    kernel: max/kernels/src/nn/normalization.mojo:3996-4175)
 * RMSNorm over the last axis fused with the per-row (per-token) dynamic quantisation:
 *   inv_rms = 1/sqrt(sum_c x[r,c]^2 / K + epsilon),  g'[c] = gamma[c] + weight_offset
 *   scales[r] = min(max_c |x*g'| * inv_rms, scale_ub) / 448
 *   out[r,c]  = e4m3fn(clamp(((x * inv_rms) * g'[c]) / scales[r]))   (as x * (1/scale))
 * in [rows, K] and gamma [K] share in_dtype; out [rows, K] e4m3fn; out_scales [rows]
 * (the op's [1, rows] tensor).  epsilon and weight_offset are rounded to in_dtype first,
 * as the registration does (quantization.mojo:205-213).  Higher-rank inputs are passed
 * flattened to [rows, K].
 */
int maxfp8_rms_norm_fused_quantize_dynamic_scaled_fp8(
    void* out_fp8, void* out_scales, const void* in, const void* gamma,
    int64_t rows, int64_t K, int64_t in_row_stride, int64_t out_row_stride,
    int in_dtype, int scales_dtype, float epsilon, float weight_offset,
    float scale_ub, void* stream);

/*
 * mo.quantize_static_scaled_float8  (wrapper: max/python/max/nn/kernels.py:6753-6801;
 * registration: builtin_kernels/quantization.mojo:1268-1315; kernel:
 * max/kernels/src/linalg/fp8_quantization.mojo:89-141)
 *   out[m,k] = e4m3fn(clamp(f32(in[m,k]) * (1 / scale), -448, 448))
 * with the per-tensor scale a host scalar.  (The op's scale_is_inverted parameter has no
 * effect in the reference -- it always multiplies by 1 / scale -- and has none here.)
 */
int maxfp8_quantize_static_scaled_fp8(
    void* out_fp8, const void* in, int64_t M, int64_t K,
    int64_t in_row_stride, int64_t out_row_stride, int in_dtype, float scale, void* stream);

/*
 * Dynamic per-tensor quantisation: one scale for the whole [M, K] tensor.
 * Replaces QuantizeTensorDynamicScaledFloat8.execute
 *   (max/kernels/src/graph_compiler/builtin_kernels/quantization.mojo:1318-1360)
 * -> quantize_tensor_dynamic_scaled_fp8 (max/kernels/src/linalg/fp8_quantization.mojo:209-360).
 *
 *   out_scales  [1, M] of scales_dtype: EVERY element receives the tensor's scale
 *               min(max |x|, scale_ub) / 448 (the reference guarantees it only for
 *               element 0, which is what its callers read, quant_ops.py:451).  The
 *               buffer doubles as the scratch of the row maxima during the call.
 *   out_fp8     e4m3fn(clamp(x * (1 / scale))) with the guarded reciprocal of
 *               maxfp8_quantize_dynamic_scaled_fp8
 *   K           a multiple of 4 (the reference's smallest vector width)
 */
int maxfp8_quantize_tensor_dynamic_scaled_fp8(
    void* out_fp8, void* out_scales, const void* in,
    int64_t M, int64_t K, int64_t in_row_stride, int64_t out_row_stride,
    int in_dtype, int scales_dtype, float scale_ub, void* stream);

/*
 * mo.moe.create.indices  (wrapper: max/python/max/nn/kernels.py:4980-5060; kernel:
 * max/kernels/src/nn/moe.mojo:435-720).  Groups the n = tokens * top_k expert assignments
 * topk_ids[i] (int32 / uint32, values in [0, num_experts)) by expert:
 *   token_expert_order[n]   assignment indices grouped by expert slot
 *   expert_start_indices[num_experts + 1]  slot z owns token_expert_order[start[z] .. start[z+1])
 *   restore_token_order[n]  position of assignment i in token_expert_order
 *   expert_ids[num_experts] expert of slot z
 *   expert_usage_stats[2]   {most assignments on one expert, number of slots = num_experts}
 * The reference assigns slots in the order its blocks reach a lock, so any permutation of the
 * experts is a valid expert_ids; this library always returns slot z = expert z with the
 * assignments of a slot in increasing order (deterministic).  No outputs need initialising.
 */
int maxfp8_moe_create_indices(
    uint32_t* token_expert_order, uint32_t* expert_start_indices, uint32_t* restore_token_order,
    int32_t* expert_ids, uint32_t* expert_usage_stats, const void* topk_ids,
    int64_t n, int64_t num_experts, void* stream);

/*
 * ep.fused_silu  (wrapper: max/python/max/nn/comm/ep/ep_kernels.py:1121-1165 and 1168-1290;
 * kernels: max/kernels/src/shmem/ep_comm.mojo:4409-4500, 4505-4624).
 * in [max_rows, 2 * inter]: out[m, k] = silu(in[m, k]) * in[m, inter + k] for the
 * rows m < row_offsets[num_offsets - 1] (read on the device; the other rows are not written).
 * quantize == 0: out has in_dtype.  quantize == 1: out is e4m3fn with one f32 scale per 128
 * outputs, out_scales[k / 128, m] (row stride scales_ld), scale = max(amax, 1e-4) / 448 and
 * out = clamp(value / scale) -- this op's own recipe.  inter % 128 == 0.
 * quantize == 2: like 0, with silu(in[m, k]) rounded to in_dtype before the product -- the arithmetic of
 * the dense gated MLP, where silu and the multiplication are two operations on bf16 tensors
 * (max/python/max/nn/linear.py:1072); out_scales is not used.
 */
int maxfp8_fused_silu(
    void* out, void* out_scales, const void* in, const uint32_t* row_offsets,
    int64_t num_offsets, int64_t max_rows, int64_t inter, int64_t in_row_stride,
    int64_t out_row_stride, int64_t scales_ld, int in_dtype, int quantize, void* stream);

/*
 * Elementwise f32 -> e4m3fn (clamp to +-448, round to nearest even), the cast
 * inside fp8_quantize (max/kernels/src/internal_utils/fp8_utils.mojo:96-143).
 * Exposed so the hardware convert can be checked exhaustively.
 */
int maxfp8_cast_f32_to_e4m3fn(void* out_fp8, const float* in, int64_t n, void* stream);

/*
 * Elementwise f32 -> bf16 (round to nearest even) with the hardware convert the
 * matmul epilogues use, exposed so it can be checked against the software rounding.
 */
int maxfp8_cast_f32_to_bf16(void* out_bf16, const float* in, int64_t n, void* stream);

/* Elementwise e4m3fn -> f32 (mojo/stdlib/std/builtin/simd.mojo:3690-3749). */
int maxfp8_cast_e4m3fn_to_f32(float* out, const void* in_fp8, int64_t n, void* stream);

/* Plain device copy kernel of n bytes (n % 16 == 0); the calibration unit for
 * hardware byte counters. */
int maxfp8_copy_bytes(void* dst, const void* src, int64_t n, void* stream);

/*
 * Measurement aid with no counterpart in the reference: streams the weight matrix b[N, K] (row stride ldb bytes)
 * through the weight-streaming (decode) matmul's own grid, LDS ring and DMA instructions -- the shape MAXFP8_ALGO_AUTO
 * would pick for (M, N, K) with row scaling; that kernel takes up to 64 rows, the probe models it for M <= 16 -- and
 * does nothing else: no activations, no MFMA, no stores.  Its
 * time is the ceiling the weight-streaming matmul is measured against.
 */
int maxfp8_decode_weight_read_probe(const void* b, int64_t M, int64_t N, int64_t K, int64_t ldb, void* stream);

/*
 * Measurement aid with no counterpart in the reference: the main loop of a dense block- or row-scaled matmul kernel
 * (kernel 0: eight waves, 256 x 256 tiles; kernel 4 / 5 / 6: four waves, 128 x 256 / 160 x 256 / 192 x 256 tiles) run for `slabs` K slabs of 128 bytes
 * by one block on every compute unit, all blocks on the same tile:
 *   level 2: the MFMA loop alone (block scaling: with its promotions), fragments read from what one copy left in LDS;
 *   level 1: the whole loop -- LDS-DMA copies, waits, barriers -- with operands that stay in L2 (slabs 0..7 of tile
 *            (0, 0) over and over).
 * a, b: 256 rows x 1024 bytes of e4m3fn each; a_scales: 8 x 256 floats, b_scales: 2 x 8 floats; c: 256 x 256 bf16, written
 * once at the end with meaningless values; clocks: null, or two 64-bit words per compute unit, which receive what the
 * block's first wave counted around its slab loop -- cycles of the core clock and ticks of the constant 100 MHz clock --
 * so that the clock the chip held under the load can be read off.  The kernel's time over slabs * 256 * 256 * 128 * 2 flops per block (four waves:
 * 160 or 192 rows) is the issue ceiling the matmul kernels are measured against.
 */
int maxfp8_mfma_issue_probe(int kernel, int blockscale, int level, int64_t slabs, const void* a, const void* b, const float* a_scales,
                            const float* b_scales, void* c, uint64_t* clocks, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MAXFP8_H */
