/*
 * C ABI of the MI355X (gfx950) quantized-inference operator library, libmi355_quant.so.
 *
 * These entry points are what a torch_npu-style operator adapter binds instead of the
 * aclnn* functions that the reference resolves from CANN's libopapi.so by dlsym and
 * calls through typed function pointers returning an int status, 0 = success
 * (torch_npu/csrc/core/npu/interface/OpInterface.cpp:8-17,28-56;
 *  torch_npu/csrc/core/npu/register/FunctionLoader.h:86-96).
 *
 * Conventions (all entry points)
 *   - plain pointers and sizes only; every pointer is DEVICE memory owned by the caller;
 *   - the launcher never allocates, never synchronises and never throws: it validates its
 *     arguments on the host, enqueues kernels on `stream` (a hipStream_t passed as void*,
 *     NULL = the default stream) and returns;
 *   - return value: MI355_OK (0) or a negative mi355_status; mi355_status_string() names it;
 *   - launches are re-entrant and keep no state between calls, with three documented exceptions: the planner knobs of
 *     mi355_set_tuning() are process-wide, mi355_quant_matmul_noalloc() works on one scratch array per GPU, and
 *     mi355_workspace_status() is a query that synchronises the stream it is given.
 *   - strides ("ld*", "*_stride") are in ELEMENTS of the respective array.
 */
#ifndef MI355_QUANT_H
#define MI355_QUANT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum mi355_status {
    MI355_OK = 0,
    MI355_ERR_BAD_ARGUMENT = -1,   /* null pointer, negative size, bad enum value          */
    MI355_ERR_UNSUPPORTED = -2,    /* valid request outside what the kernels implement     */
    MI355_ERR_ALIGNMENT = -3,      /* pointer / stride alignment the kernels cannot handle */
    MI355_ERR_WORKSPACE = -4,      /* workspace missing or smaller than *_workspace() says */
    MI355_ERR_LAUNCH = -5,         /* hipGetLastError() != hipSuccess after the launch     */
    MI355_ERR_DEVICE = -6          /* a kernel reported a failure through the workspace's status word (mi355_workspace_status) */
} mi355_status;

/* 16-bit floating-point element formats of activations. */
#define MI355_DTYPE_BF16 0
#define MI355_DTYPE_FP16 1
#define MI355_DTYPE_FP32 2   /* accepted where a function's comment says so */
#define MI355_DTYPE_INT32 3  /* likewise */

/* Output formats of mi355_quant_matmul. */
#define MI355_OUT_BF16 0
#define MI355_OUT_INT32 1   /* int32 accumulators (plus an int32 bias if given); scales are ignored */
#define MI355_OUT_FP16 2
#define MI355_OUT_INT8 3    /* re-quantised output; only mi355_quant_matmul_qparam produces it */

/* bias element types of mi355_quant_matmul */
#define MI355_BIAS_NONE 0
#define MI355_BIAS_BF16 1   /* added after both scales */
#define MI355_BIAS_INT32 2  /* added to the int32 accumulator before dequantisation (wraps like the accumulator) */
#define MI355_BIAS_FP32 3   /* added after both scales */

const char *mi355_status_string(int status);

/* Library/ABI version: major * 1000 + minor. */
int mi355_quant_abi_version(void);

/*
 * npu_dynamic_quant, per-token symmetric int8.
 * Replaces the aclnn DynamicQuant call behind torch_npu.npu_dynamic_quant
 * (signature and output shapes: test/test_fake_tensor.py:1670-1687,
 *  torch_npu/onnx/wrapper_onnx_ops.py:740-759).
 *
 *   x      [rows, cols] in_dtype, row r starts at x + r * x_row_stride
 *   smooth NULL, or [cols] in_dtype: x is multiplied by it (in float32) before quantisation
 *   y      [rows, cols] int8, contiguous
 *   scale  [rows] float32:  scale = max_j |x| / 127,  y = rint_half_even(x / scale) in [-127, 127]
 * A row of zeros yields scale 0 and y 0.  rows == 0 or cols == 0 is a no-op.
 */
int mi355_dynamic_quant(const void *x, int in_dtype, const void *smooth,
                        int8_t *y, float *scale,
                        int64_t rows, int64_t cols, int64_t x_row_stride, void *stream);

/*
 * npu_dynamic_quant with per-expert smooth scales (the `group_index` argument of torch_npu.npu_dynamic_quant,
 * signature test/test_fake_tensor.py:1670-1687, test/torch_npu_schema.json:2144-2146; the reference tree holds no call
 * that passes it, the meaning is the operator's published one).
 *   smooth       [groups, cols] in_dtype, contiguous
 *   group_index  [groups] int32 on the device, non-decreasing running totals of the rows of each expert: row r is
 *                multiplied by smooth[e] for the first e with r < group_index[e]; rows past the last total take the
 *                last expert.  NULL: as mi355_dynamic_quant (smooth is then [cols] or NULL)
 * Everything else as mi355_dynamic_quant.
 */
int mi355_dynamic_quant_grouped(const void *x, int in_dtype, const void *smooth, const int32_t *group_index,
                                int64_t groups, int8_t *y, float *scale,
                                int64_t rows, int64_t cols, int64_t x_row_stride, void *stream);

/*
 * npu_dynamic_quant with dst_type=torch.quint4x2: per-token symmetric int4 (the `dst_type` argument of the operator's
 * signature, test/test_fake_tensor.py:1670-1687; the reference tree holds no call or golden for it, the meaning is the
 * operator's published one: an int32 result whose last dimension is an eighth of the input's).
 *   y_words  [rows, cols / 8] int32, contiguous; word j of a row holds the codes of columns 8j .. 8j+7, column 8j in
 *            bits 0-3 (the nibble order of mi355_unpack_int4); cols must be a multiple of 8
 *   scale    [rows] float32:  scale = max_j |x| / 7,  code = rint_half_even(x / scale) in [-7, 7]
 * x, smooth, group_index, groups, rows, cols, x_row_stride as in mi355_dynamic_quant_grouped (group_index may be NULL).
 */
int mi355_dynamic_quant_int4(const void *x, int in_dtype, const void *smooth, const int32_t *group_index,
                             int64_t groups, void *y_words, float *scale,
                             int64_t rows, int64_t cols, int64_t x_row_stride, void *stream);

/*
 * npu_dynamic_quant_asymmetric, per-token asymmetric int8.
 * Replaces the aclnn DynamicQuantV2 call behind torch_npu.npu_dynamic_quant_asymmetric (signature and output
 * shapes: test/test_fake_tensor.py:1689-1709, test/torch_npu_schema.json:2147-2149).  The arithmetic is not in the
 * reference tree; it follows the operator's published description:
 *   scale  = (row_max - row_min) / 255          offset = 127 - row_max / scale
 *   y      = rint_half_even(x / scale + offset) in [-128, 127]   (row_max -> 127, row_min -> -128)
 * every operation rounded to float32 on its own.  x, smooth, y, rows, cols, x_row_stride as in mi355_dynamic_quant;
 * scale and offset are float32 [rows].  A row whose elements are all equal yields scale 0, offset 0 and y 0
 * (this library's choice).  cols == 0 leaves scale and offset unwritten.
 */
int mi355_dynamic_quant_asymmetric(const void *x, int in_dtype, const void *smooth,
                                   int8_t *y, float *scale, float *offset,
                                   int64_t rows, int64_t cols, int64_t x_row_stride, void *stream);

/*
 * npu_dynamic_quant_asymmetric with per-expert smooth scales (`group_index`): smooth [groups, cols], group_index as in
 * mi355_dynamic_quant_grouped (NULL: as mi355_dynamic_quant_asymmetric); everything else as mi355_dynamic_quant_asymmetric.
 */
int mi355_dynamic_quant_asymmetric_grouped(const void *x, int in_dtype, const void *smooth, const int32_t *group_index,
                                           int64_t groups, int8_t *y, float *scale, float *offset,
                                           int64_t rows, int64_t cols, int64_t x_row_stride, void *stream);

/*
 * npu_quant_matmul, W8A8 with int32 accumulation and fused dequantisation.
 * Replaces the aclnn QuantMatmul call behind torch_npu.npu_quant_matmul
 * (callers: torch_npu/contrib/module/linear_quant.py:96-112, linear_a8w8_quant.py:87-120;
 *  shapes/dtypes: test/test_fake_tensor.py:1883-1925).
 *
 *   a   int8 [M, K], element (m,k) at a[m*lda + k]
 *   b   int8 logical [K, N], element (k,n) at b[k*ldb_k + n*ldb_n]; one of ldb_k, ldb_n must be 1
 *       (ldb_n == 1: contiguous [K,N]; ldb_k == 1: the transposed view of an [N,K] weight)
 *   pertoken_scale  float32 [M] or NULL;   scale float32 [scale_len], scale_len in {1, N}
 *   bias            [N] of bias_dtype (MI355_BIAS_*) or NULL with MI355_BIAS_NONE.  LinearQuant's default bias is
 *                   int32 (linear_quant.py:92), the bf16-output configuration uses bf16.
 *   out_dtype MI355_OUT_BF16 / MI355_OUT_FP16:
 *                 out[m*ldc+n] = round(((float(acc + bias_i32[n]) * pertoken_scale[m]) * scale[n]) + float(bias[n]))
 *                 (each bias term only for its type), rounded once to bf16 / fp16
 *             MI355_OUT_INT32: out[m*ldc+n] = acc + bias_i32[n] (scales are ignored and may be NULL; other bias
 *                 types are rejected)
 *   workspace: at least mi355_quant_matmul_workspace(...) bytes (may be NULL when that is 0), 16-byte aligned.
 *              It holds a transposed copy of a contiguous [K,N] weight and, for narrow outputs with a long K,
 *              the partial sums and arrival counters of a split over K.  The first MI355_WORKSPACE_ZERO_BYTES of
 *              every workspace of this library (arrival counters, then a zone for exchanges that recognise data by
 *              its being non-zero) must be zero before the first launch that uses the buffer; every launch leaves
 *              them zero and keeps everything else behind them, so one zero-initialised buffer can serve all later
 *              launches of all operators on the same stream.
 */
#define MI355_WORKSPACE_ZERO_BYTES ((size_t)16 * 1024 * 1024 + 16384)
/* The same number as a query, for hosts that bind the library without this header. */
size_t mi355_workspace_zero_bytes(void);

/*
 * Device-side failures.  The reference reports a failed device task to the caller at the next synchronisation
 * (torch_npu/csrc/framework/OpParamMaker.cpp:541-571); here the only failure a kernel can detect is a bounded wait
 * running out: the int4 kernels of mi355_weight_quant_matmul exchange split-K partial sums through the workspace's
 * zero zone, and the workgroup that collects them polls a bounded number of times.  When the bound is hit the kernel
 * writes NaN where the missing sums would have gone and stores a non-zero code in the workspace's sticky status word
 * (4 bytes at MI355_WORKSPACE_STATUS_OFFSET, inside the zero area); later stores of the late producers may leave
 * non-zero words in the zone, so the zone must be cleared before the workspace is used again.
 *
 * mi355_workspace_status waits for `stream`, reads the status word and returns MI355_OK when it is zero, MI355_ERR_DEVICE
 * otherwise.  With `reset` non-zero a failed workspace is made usable again: its whole zero area, the status word
 * included, is cleared on `stream` before the call returns.  Unlike the launchers this call synchronises; call it where
 * the caller synchronises anyway, or before a workspace is retired.
 */
#define MI355_WORKSPACE_STATUS_OFFSET ((size_t)16384 - 16)
int mi355_workspace_status(void *workspace, size_t workspace_bytes, int reset, void *stream);

size_t mi355_quant_matmul_workspace(int64_t M, int64_t N, int64_t K, int64_t ldb_k, int64_t ldb_n);

int mi355_quant_matmul(const int8_t *a, const int8_t *b,
                       const float *pertoken_scale, const float *scale, int64_t scale_len,
                       const void *bias, int bias_dtype, void *out, int out_dtype,
                       int64_t M, int64_t N, int64_t K,
                       int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                       void *workspace, size_t workspace_bytes, void *stream);

/*
 * npu_trans_quant_param: packs a float32 scale (and optional float32 offset) per channel into the 64-bit quantisation
 * parameter that npu_quant_matmul takes as an int64 `scale`.
 * Replaces the aclnn TransQuantParam call behind torch_npu.npu_trans_quant_param(scale, offset=None)
 * (caller torch_npu/contrib/module/linear_quant.py:104-108; shapes and the int64 result type
 * test/test_fake_tensor.py:1929-1943).  The bit layout is not in the reference tree; it follows the operator's
 * published description:
 *   bits 0-31   the float32 bit pattern of scale[i]
 *   bits 37-45  clamp(rint(offset[i]), -256, 255) as a 9-bit two's-complement integer (zero without an offset)
 *   bit 46      set
 * scale_len and offset_len are n or 1 (broadcast); out receives n words.
 */
int mi355_trans_quant_param(const float *scale, int64_t scale_len, const float *offset, int64_t offset_len,
                            uint64_t *out, int64_t n, void *stream);

/*
 * npu_quant_matmul with the packed 64-bit parameters of mi355_trans_quant_param in place of the float32 scale
 * (the int64 `scale` of torch_npu.npu_quant_matmul, which LinearQuant passes whenever its scale is float32, there is
 * no pertoken_scale and the output is int8 or float16: torch_npu/contrib/module/linear_quant.py:104-112).
 *   qparam    [qparam_len], qparam_len in {1, N}
 *   bias      int32 [N] (added to the accumulator) or NULL; for the floating-point outputs also float32 / bf16 as in
 *             mi355_quant_matmul
 *   out_dtype MI355_OUT_INT8:  out[m*ldc+n] = clamp(rint(float(acc + bias[n]) * scale[n] + offset[n]), -128, 127) as
 *                              int8 (scale and offset decoded from qparam[n], each operation rounded to float32,
 *                              rint = round half to even)
 *             MI355_OUT_FP16 / MI355_OUT_BF16: as mi355_quant_matmul with scale[n] decoded from qparam[n] and no
 *                              pertoken_scale (the packed offset is ignored)
 * a, b, strides, M, N, K, workspace: as mi355_quant_matmul (the same mi355_quant_matmul_workspace() query).
 */
int mi355_quant_matmul_qparam(const int8_t *a, const int8_t *b, const uint64_t *qparam, int64_t qparam_len,
                              const void *bias, int bias_dtype, void *out, int out_dtype,
                              int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                              void *workspace, size_t workspace_bytes, void *stream);

/*
 * One-time weight pre-layout for mi355_quant_matmul: src int8 [K,N] (rows ld_src bytes apart) -> dst int8 [N,K]
 * contiguous, the K-major storage the GEMM reads directly (ldb_k = 1, ldb_n = K); a [K,N] weight passed as it is gets
 * transposed into the workspace on every call instead.  The counterpart of casting a weight to the device's private
 * format before deployment (the reference's modules rely on such a cast, e.g.
 * torch_npu/optim/npu_fused_optim_base.py:49); weights are static, so this runs once per weight.
 */
int mi355_transpose_int8(const int8_t *src, int8_t *dst, int64_t K, int64_t N, int64_t ld_src, void *stream);

/*
 * mi355_quant_matmul without a workspace argument and without any allocation.  It has no counterpart in the
 * reference (there the adapter allocates a workspace per call, torch_npu/csrc/framework/utils/OpPreparation.h:130-132);
 * it exists for callers that cannot allocate or carry a workspace: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  Arguments and results are those of mi355_quant_matmul (bit-identical outputs).
 * The arrival counters, split-K partial sums and the transposed copy of a contiguous [K,N] weight live in a fixed
 * device array of MI355_NOALLOC_SCRATCH_BYTES inside the library, one copy per GPU, held until the process ends.
 *   - the array is private to this operator, so it holds only 16 KiB of counters plus what the problem needs behind
 *     them.  A split of K is planned so that its partial sums fit (mi355_quant_matmul may prefer a split with more of
 *     them; integer sums make the results identical); returns MI355_ERR_WORKSPACE when the transposed copy of a
 *     weight stored [K,N] does not fit (store it [N,K], or use mi355_quant_matmul);
 *   - calls no hipMalloc / hipFree and no allocating library routine; the first call on a device resolves the
 *     array's address and clears its counters with a small kernel on `stream` (recorded again by every capturing call
 *     until a call outside a capture has enqueued it);
 *   - the array belongs to the current device: `stream` must be NULL or a stream of the current device
 *     (MI355_ERR_BAD_ARGUMENT otherwise);
 *   - all calls on one GPU share that GPU's array: calls that may overlap in time (different streams without an
 *     ordering between them, several host threads) race on it and must be serialised by the caller.
 */
#define MI355_NOALLOC_SCRATCH_BYTES ((size_t)16 * 1024 * 1024 + 16384)
int mi355_quant_matmul_noalloc(const int8_t *a, const int8_t *b, const float *pertoken_scale,
                               const float *scale, int64_t scale_len, const void *bias, int bias_dtype,
                               void *out, int out_dtype, int64_t M, int64_t N, int64_t K,
                               int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc, void *stream);

/*
 * npu_weight_quant_batchmatmul, W8A16 per channel and W4A16 per group.
 * Replaces the aclnn WeightQuantBatchMatmulV2 call behind torch_npu.npu_weight_quant_batchmatmul
 * (caller: torch_npu/contrib/module/linear_weight_quant.py:98-109; CPU golden:
 *  test/contrib/test_linear_weight_quant.py:20-28; int4 nibble order:
 *  test/custom_ops/test_npu_anti_quant.py:12-24).
 *
 *   x       [M, K] of act_dtype (MI355_DTYPE_BF16 or MI355_DTYPE_FP16, the dtype of the reference's own test,
 *           test/contrib/test_linear_weight_quant.py:57-62), element (m,k) at x[m*ldx + k]; scale, offset and out
 *           have the same element type
 *   w       w_bits == 8: int8 logical [K, N], element (k,n) at w[k*ldw_k + n*ldw_n], one stride == 1
 *           w_bits == 4: int32 words of eight two's-complement int4 values, element i in bits [4i, 4i+3], either
 *             ldw_n == 1: [K, N/8], rows ldw_k words apart; word j of row k holds n = 8j..8j+7, or
 *             ldw_k == 1 (and ldw_n != 1): [N, K/8], columns ldw_n words apart; word j of column n holds
 *                        k = 8j..8j+7 - the transposed view the contrib module passes (linear_weight_quant.py:71,106)
 *   scale   element (g, n) at scale[g*ld_param_g + n*ld_param_n], G = 1 when group_size == 0 else K / group_size;
 *           row-major [G, N] is (N, 1); the module's transposed view of [N, G] is (1, G)
 *           (linear_weight_quant.py:98-105).  Only the kernel for words along K reads strided parameters at full
 *           speed; every other layout falls back to a slow one-thread-per-output kernel unless they are row-major.
 *   offset  same strides as scale, or NULL;  bias [N] or NULL (the module's optional bias, linear_weight_quant.py:89-92)
 *   out[m*ldo+n] = round( sum_k float(x[m,k]) * ((float(w[k,n]) + float(offset[g,n])) * float(scale[g,n])) + float(bias[n]) )
 *   group_size: 0 (per channel) or a multiple of 32 that divides K
 *   workspace: at least mi355_weight_quant_matmul_workspace(...) bytes (may be NULL when that is 0), 16-byte aligned.
 *              It holds the arrival counters and partial sums of a split over K; its first
 *              MI355_WORKSPACE_ZERO_BYTES must be zero before the first launch that uses the buffer and are left
 *              zero by every launch (see mi355_quant_matmul), so one zero-initialised buffer can serve all later
 *              launches on the same stream.
 *   One kernel launch per call: weight-streaming kernels for M <= 32 (for int4 words along N a barrier-free one whose
 *   workgroups exchange their partial sums through the workspace's zero zone) and a tiled GEMM above that; int4
 *   words along K take a kernel of their own in which a wavefront owns 16 output columns for all of K (no split of
 *   K at decode shapes); from 256 rows up they are first rewritten into the workspace with their words along N (the
 *   tiled GEMM for that layout is faster by more than the rewrite costs: three small launches in front of it), which
 *   is what the workspace query asks room for at those sizes.
 */
size_t mi355_weight_quant_matmul_workspace(int64_t M, int64_t N, int64_t K, int w_bits, int64_t group_size);

int mi355_weight_quant_matmul(const void *x, int act_dtype, const void *w, int w_bits,
                              const void *scale, const void *offset, const void *bias, void *out,
                              int64_t M, int64_t N, int64_t K, int64_t group_size,
                              int64_t ld_param_g, int64_t ld_param_n,
                              int64_t ldx, int64_t ldw_k, int64_t ldw_n, int64_t ldo,
                              void *workspace, size_t workspace_bytes, void *stream);

/*
 * npu_swiglu on the last dimension: out = silu(x[:, :half]) * x[:, half:], bf16 arithmetic
 * (silu rounded to bf16, then the product rounded to bf16).
 * Formula: torch_npu/_inductor/decomposition.py:186-188.
 *   x bf16 [rows, 2*half] with row stride ldx; out bf16 [rows, half] contiguous.
 */
int mi355_swiglu(const void *x_bf16, void *out_bf16, int64_t rows, int64_t half, int64_t ldx, void *stream);

/*
 * Fused SwiGLU + per-token dynamic quantisation: y, scale = dynamic_quant(swiglu(x)) without the bf16
 * intermediate in memory; bit-identical to mi355_swiglu followed by mi355_dynamic_quant.
 * Stands for the aclnn SwiGluQuant call behind torch_npu.npu_swiglu_quant in its dynamic mode (the operator is
 * only named in the reference tree, docs/zh/release_notes.md:303; its fused relative
 * npu_grouped_matmul_swiglu_quant_v2 appears in torch_npu/profiler/_flops_formulas.py:161-183).
 *
 *   x  bf16 [rows, 2*half], row pitch x_row_stride elements
 *   activate_left != 0: silu(x[:, :half]) * x[:, half:]  (the orientation of npu_swiglu,
 *                       torch_npu/_inductor/decomposition.py:186-188);  0: silu(x[:, half:]) * x[:, :half]
 *   y  int8 [rows, half] contiguous;  scale float32 [rows]
 */
int mi355_swiglu_quant(const void *x_bf16, int activate_left, int8_t *y, float *scale,
                       int64_t rows, int64_t half, int64_t x_row_stride, void *stream);

/*
 * The same with smooth scales (the smooth_scales argument of torch_npu.npu_swiglu_quant, named in
 * docs/zh/release_notes.md:303 only): y, scale = dynamic_quant(swiglu(x), smooth) as mi355_dynamic_quant defines it,
 * i.e. the bf16 SwiGLU value times smooth[j] in float32 before the row maximum and the quantisation.
 *   smooth_bf16  bf16 [half]
 */
int mi355_swiglu_quant_smooth(const void *x_bf16, int activate_left, const void *smooth_bf16, int8_t *y, float *scale,
                              int64_t rows, int64_t half, int64_t x_row_stride, void *stream);

/*
 * The same with per-expert smooth scales (the `group_index` argument of torch_npu.npu_swiglu_quant; the operator is only
 * named in the reference tree, the meaning is the vendor's published one): smooth_bf16 [groups, half], group_index
 * [groups] int32 on the device, running totals of the rows of each expert as in mi355_dynamic_quant_grouped.
 */
int mi355_swiglu_quant_grouped(const void *x_bf16, int activate_left, const void *smooth_bf16, const int32_t *group_index,
                               int64_t groups, int8_t *y, float *scale, int64_t rows, int64_t half, int64_t x_row_stride,
                               void *stream);

/*
 * npu_anti_quant: the standalone antiquantisation out = cast((float(x) + offset) * scale).
 * Replaces the aclnn AscendAntiQuant call behind torch_npu.npu_anti_quant (signature test/torch_npu_schema.json:2117-2119,
 * wrapper torch_npu/onnx/wrapper_onnx_ops.py:824-828; CPU golden test/custom_ops/test_npu_anti_quant.py:29-42, int4
 * unpacking :12-24).
 *
 *   x       x_bits == 8: int8 [rows, cols], row pitch ldx bytes
 *           x_bits == 4: int32 [rows, cols/8], row pitch ldx words; word j of a row holds columns 8j..8j+7,
 *                        element i in bits [4i, 4i+3], two's complement (cols must be a multiple of 8)
 *   scale   float32 [scale_len], scale_len == cols or 1;  offset float32 [offset_len] likewise, or NULL (zero)
 *   out     [rows, cols] of out_dtype (MI355_DTYPE_BF16 or MI355_DTYPE_FP16), row pitch ldo elements:
 *           out[r,c] = round((float(x[r,c]) + offset[c]) * scale[c]), the sum and the product each rounded to float32
 */
int mi355_anti_quant(const void *x, int x_bits, const float *scale, int64_t scale_len, const float *offset,
                     int64_t offset_len, void *out, int out_dtype, int64_t rows, int64_t cols, int64_t ldx, int64_t ldo,
                     void *stream);

/*
 * npu_quantize: static quantisation with given scales and zero points along one axis.
 * Replaces the aclnn Quantize / AscendQuant call behind torch_npu.npu_quantize(inputs, scales, zero_points, dtype, axis,
 * div_mode=True) (signature test/torch_npu_schema.json:2273-2275, wrapper torch_npu/onnx/wrapper_onnx_ops.py:855-877
 * and :1278-1279, whose dtype codes name the three output types; the reference tree holds no golden for it, the
 * formula is the operator's published one).
 *
 *   x          contiguous [outer, channels, inner] of in_dtype (MI355_DTYPE_BF16 / FP16 / FP32); channels is the
 *              size of the quantisation axis, outer / inner the products of the dimensions before / after it
 *   scale      float32 [scale_len], scale_len == channels or 1;  zero_point [zero_point_len] likewise, of
 *              zero_point_dtype MI355_DTYPE_FP32 or MI355_DTYPE_INT32 (converted to float32), or NULL
 *   out        contiguous, same shape, of out_dtype: MI355_Q_INT8 [-128,127], MI355_Q_UINT8 [0,255], MI355_Q_INT32
 *   div_mode != 0: out = clamp(rint(x / scale[c] + zero_point[c]));  0: out = clamp(rint(x * scale[c] + zero_point[c]))
 *              every operation rounded to float32, rint = round half to even, NaN -> 0
 */
#define MI355_Q_INT8 0
#define MI355_Q_UINT8 1
#define MI355_Q_INT32 2
int mi355_quantize(const void *x, int in_dtype, const float *scale, int64_t scale_len, const void *zero_point,
                   int zero_point_dtype, int64_t zero_point_len, void *out, int out_dtype, int64_t outer, int64_t channels,
                   int64_t inner, int div_mode, void *stream);

/*
 * Packed int4 -> int8: widens the A4W4 operands of npu_quant_matmul (both inputs int32, eight int4 values per word:
 * test/test_fake_tensor.py:1917-1923, torch_npu/contrib/module/linear_quant.py:40-50 and :98-102) so that
 * mi355_quant_matmul can multiply them; the int32 accumulators of the widened operands are those of the int4
 * product.  Nibble order as in mi355_anti_quant (test/custom_ops/test_npu_anti_quant.py:12-24).
 *
 *   x    int32 [rows, cols/8], row pitch ldx words; word j of a row holds columns 8j..8j+7, element i in bits
 *        [4i, 4i+3], two's complement (cols must be a multiple of 8)
 *   out  int8 [rows, cols], row pitch ldo bytes, values in [-8, 7]
 */
int mi355_unpack_int4(const void *x, int8_t *out, int64_t rows, int64_t cols, int64_t ldx, int64_t ldo, void *stream);

/*
 * Planner knobs for tuning and for tests that must force a particular plan (a given split of K, a tile shape).
 * No counterpart in the reference: aclnn chooses its tiling inside the closed kernels.  `name` is one of the
 * names listed in pytorch_amd/csrc/tuning.hip (e.g. "MI355_WQ_SPLIT"); value 0 restores the automatic choice.
 * A knob's initial value is read once, at load time, from the environment variable of the same name; no launch
 * reads the environment.  Returns MI355_ERR_BAD_ARGUMENT for an unknown name.  Process-wide, not thread-scoped.
 */
int mi355_set_tuning(const char *name, int value);

/*
 * Identifier of the HIP graph capture that `stream` is part of, 0 when the stream is not capturing.  No counterpart in
 * the reference (aclnn workspaces are allocated per call by the adapter, OpPreparation.h:130-132); a host layer that
 * caches zeroed workspaces uses it to give every capture a workspace of its own.
 */
int mi355_stream_capture_id(void *stream, unsigned long long *id);

/*
 * Measurement aid, no counterpart in the reference: keeps `workgroups` x 8 wavefronts issuing dependent int8 MFMAs for
 * `iters` x 4 instructions each and writes, per workgroup, the elapsed shader-clock cycles and the elapsed ticks of
 * the constant 100 MHz counter into out[2*w], out[2*w+1]: cycles / ticks x 100 is the clock in MHz that the chip
 * sustains under matrix-core load.
 */
int mi355_probe_clock(unsigned long long *out, int workgroups, int iters, void *stream);

/* Measurement aid: a kernel that does nothing, `workgroups` x 256 threads (the per-launch floor inside a captured graph). */
int mi355_probe_empty_launch(int workgroups, void *stream);

/* Peak engine clock (kHz) and compute-unit count of the current device from the HIP runtime; either pointer may be NULL. */
int mi355_device_info(int *clock_khz, int *compute_units);

#ifdef __cplusplus
}
#endif
#endif /* MI355_QUANT_H */
