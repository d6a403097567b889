/*
 * CPU oracle for the quantized-inference operator path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may link, import or
 * call this file; it exists so that tests, the smoke check and the benchmark's
 * CPU-baseline leg have an independent statement of the arithmetic to compare
 * the HIP kernels with.
 *
 * The reference tree (Ascend/pytorch) does not contain the arithmetic of these
 * operators: it lives in the un-vendored third_party/op-plugin submodule
 * (.gitmodules:1-4, pinned commit not recoverable) and in closed CANN binaries.
 * Every function below therefore restates the closed-form "CPU golden formula"
 * of the benchmark configuration and cites the in-tree material that fixes the
 * part of it that *is* in the tree.
 *
 * Pinning status (what checks the restatement, see tests/test_oracle_*.py):
 *   orc_unpack_int4         pinned: nibble order of test/custom_ops/test_npu_anti_quant.py:12-24,
 *                           hand-typed known answers, pack/unpack round trip.
 *   orc_antiquant           pinned: (x+offset)*scale of test/custom_ops/test_npu_anti_quant.py:29-42,
 *                           torch fp32 evaluation, hand-typed known answers.
 *   orc_weight_quant_matmul pinned: CPU golden of test/contrib/test_linear_weight_quant.py:20-28
 *                           evaluated with torch fp32 and numpy float64; special cases
 *                           (offset 0 & scale 1 => plain matmul, group = K => per channel, M = 1).
 *   orc_int8_gemm           pinned: torch._int_mm, float64 matmul (exact below 2^53), closed forms.
 *   orc_quant_matmul_epilogue  formula of the benchmark configuration, checked against torch fp32
 *                           elementwise evaluation and special cases; behaviour of the Ascend
 *                           kernel itself: PARITY UNPINNED (no in-tree result test).
 *   orc_dynamic_quant       formula of the benchmark configuration, checked against torch fp32 /
 *                           numpy evaluation, hand-typed round-half-even cases and invariants;
 *                           behaviour of the Ascend kernel itself: PARITY UNPINNED.
 *   orc_dynamic_quant_asymmetric  the operator's published description (scale = (max - min) / 255,
 *                           offset = 127 - max / scale), checked against numpy float32 evaluation and
 *                           hand-computed rows; behaviour of the Ascend kernel itself: PARITY UNPINNED.
 *   orc_swiglu              torch_npu/_inductor/decomposition.py:186-188 (silu(a)*b), checked against
 *                           torch CPU bf16 evaluation.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off; no fast-math, so every
 * float operation below is a separately rounded IEEE-754 binary32 operation).
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <math.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ helpers */

static inline float bf16_to_f32(uint16_t h)
{
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* binary32 -> bfloat16, round to nearest even; NaN stays NaN (quiet). */
static inline uint16_t f32_to_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u)
        return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

static inline float fp16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3ffu;
            u = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

void orc_set_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

int orc_get_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_bf16_to_f32(const uint16_t *src, float *dst, int64_t n)
{
    for (int64_t i = 0; i < n; i++) dst[i] = bf16_to_f32(src[i]);
}

void orc_f32_to_bf16(const float *src, uint16_t *dst, int64_t n)
{
    for (int64_t i = 0; i < n; i++) dst[i] = f32_to_bf16(src[i]);
}

/* ------------------------------------------------------- npu_dynamic_quant */
/*
 * Per-token symmetric int8 quantisation.
 *   xf    = float32(x)                      (exact for bf16 / fp16 input)
 *   amax  = max_j |xf[j]|
 *   scale = amax / 127                      (one binary32 division)
 *   y[j]  = clamp(rint(xf[j] / scale), -127, 127)   (binary32 division, round half to even)
 * A row whose amax is 0 gets scale 0 and y 0 (the closed form is 0/0 there; this
 * is the convention chosen for this build).
 * Shapes: signature and output shapes follow test/test_fake_tensor.py:1670-1687
 * (y has the shape of the input, scale drops the last dimension, float32).
 * in_dtype: 0 = bfloat16, 1 = float16 (both passed as raw 16-bit patterns).
 * smooth: optional [cols] vector in the input dtype; when given, xf = float32(x) * float32(smooth)
 * rounded once to binary32 before everything else (SmoothQuant pre-multiply).
 */
void orc_dynamic_quant(const uint16_t *x, int in_dtype, const uint16_t *smooth,
                       int64_t rows, int64_t cols, int64_t row_stride,
                       int8_t *y, float *scale)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const uint16_t *xr = x + r * row_stride;
        int8_t *yr = y + r * cols;
        float amax = 0.0f;
        for (int64_t j = 0; j < cols; j++) {
            float v = in_dtype ? fp16_to_f32(xr[j]) : bf16_to_f32(xr[j]);
            if (smooth) v = v * (in_dtype ? fp16_to_f32(smooth[j]) : bf16_to_f32(smooth[j]));
            float a = fabsf(v);
            if (a > amax) amax = a;
        }
        float s = amax / 127.0f;
        scale[r] = s;
        if (!(amax > 0.0f)) {
            for (int64_t j = 0; j < cols; j++) yr[j] = 0;
            continue;
        }
        for (int64_t j = 0; j < cols; j++) {
            float v = in_dtype ? fp16_to_f32(xr[j]) : bf16_to_f32(xr[j]);
            if (smooth) v = v * (in_dtype ? fp16_to_f32(smooth[j]) : bf16_to_f32(smooth[j]));
            float q = v / s;
            float rq = rintf(q); /* default rounding mode: to nearest, ties to even */
            if (rq > 127.0f) rq = 127.0f;
            if (rq < -127.0f) rq = -127.0f;
            yr[j] = (int8_t)rq;
        }
    }
}

/*
 * npu_dynamic_quant_asymmetric (signature and shapes: test/test_fake_tensor.py:1689-1709).  The arithmetic is not
 * in the reference tree: this restates the operator's published description,
 *   scale = (row_max - row_min) / 255,  offset = 127 - row_max / scale,  y = rint(x / scale + offset) in [-128, 127],
 * one binary32 operation at a time.  A row of equal elements: scale 0, offset 0, y 0.  PARITY UNPINNED against the
 * Ascend kernel; the function itself is checked against a numpy float32 evaluation and hand-computed rows.
 */
void orc_dynamic_quant_asymmetric(const uint16_t *x, int in_dtype, const uint16_t *smooth,
                                  int64_t rows, int64_t cols, int64_t row_stride,
                                  int8_t *y, float *scale, float *offset)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const uint16_t *xr = x + r * row_stride;
        int8_t *yr = y + r * cols;
        float mx = -INFINITY, mn = INFINITY;
        for (int64_t j = 0; j < cols; j++) {
            float v = in_dtype ? fp16_to_f32(xr[j]) : bf16_to_f32(xr[j]);
            if (smooth) v = v * (in_dtype ? fp16_to_f32(smooth[j]) : bf16_to_f32(smooth[j]));
            if (v > mx) mx = v;
            if (v < mn) mn = v;
        }
        if (!(mx > mn)) {
            scale[r] = 0.0f;
            offset[r] = 0.0f;
            for (int64_t j = 0; j < cols; j++) yr[j] = 0;
            continue;
        }
        float s = (mx - mn) / 255.0f;
        float o = 127.0f - mx / s;
        scale[r] = s;
        offset[r] = o;
        for (int64_t j = 0; j < cols; j++) {
            float v = in_dtype ? fp16_to_f32(xr[j]) : bf16_to_f32(xr[j]);
            if (smooth) v = v * (in_dtype ? fp16_to_f32(smooth[j]) : bf16_to_f32(smooth[j]));
            float q = v / s;
            q = q + o;
            float rq = rintf(q);
            if (rq > 127.0f) rq = 127.0f;
            if (rq < -128.0f) rq = -128.0f;
            yr[j] = (int8_t)rq;
        }
    }
}

/* ---------------------------------------------------------- npu_quant_matmul */
/*
 * acc[m,n] = sum_k int32(a[m,k]) * int32(b[k,n]), exact in int32.
 * b is addressed as b[k*ldb_k + n*ldb_n], which covers both the contiguous [K,N]
 * layout and the [N,K]-stored transpose view that
 * torch_npu/contrib/module/linear_quant.py:110-112 passes.
 */
void orc_int8_gemm(const int8_t *a, int64_t lda, const int8_t *b, int64_t ldb_k, int64_t ldb_n,
                   int64_t M, int64_t N, int64_t K, int32_t *acc)
{
    /* Repack b as [N][K] so the inner loop is a contiguous dot product. */
    int8_t *bt = (int8_t *)malloc((size_t)N * (size_t)K);
    if (!bt) return;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++)
        for (int64_t k = 0; k < K; k++)
            bt[n * K + k] = b[k * ldb_k + n * ldb_n];
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            const int8_t *ar = a + m * lda;
            const int8_t *br = bt + n * K;
            int32_t s = 0;
            for (int64_t k = 0; k < K; k++) s += (int32_t)ar[k] * (int32_t)br[k];
            acc[m * N + n] = s;
        }
    }
    free(bt);
}

/*
 * Dequantising epilogue of the W8A8 path, bf16 output:
 *   out[m,n] = bf16( (float32(acc[m,n]) * pertoken_scale[m]) * scale[n] + float32(bias[n]) )
 * evaluated left to right, every operation rounded to binary32, final RNE to bf16.
 * pertoken_scale may be NULL (treated as absent: out = float(acc) * scale[n] (+ bias)).
 * bias is bf16 [N] or NULL.  scale_len is N or 1 (a single per-tensor scale is broadcast,
 * as in test/test_fake_tensor.py:1886-1894).
 * Callers: torch_npu/contrib/module/linear_quant.py:96-112.
 */
void orc_quant_matmul_epilogue(const int32_t *acc, const float *pertoken_scale, const float *scale,
                               int64_t scale_len, const uint16_t *bias_bf16,
                               int64_t M, int64_t N, uint16_t *out_bf16)
{
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            float f = (float)acc[m * N + n];
            if (pertoken_scale) f = f * pertoken_scale[m];
            f = f * scale[scale_len == 1 ? 0 : n];
            if (bias_bf16) f = f + bf16_to_f32(bias_bf16[n]);
            out_bf16[m * N + n] = f32_to_bf16(f);
        }
    }
}

/* binary32 -> binary16, round to nearest even (overflow to infinity, gradual underflow). */
static inline uint16_t f32_to_f16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);              /* NaN */
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);             /* >= 65536 (or inf): infinity; 65520..65535.99 round below */
    if (a < 0x33000000u) return sign;                                    /* < 2^-25: rounds to zero */
    int e = (int)(a >> 23) - 127;                                        /* unbiased exponent */
    uint32_t mant = (a & 0x7fffffu) | 0x800000u;                         /* 24-bit significand */
    int shift = e < -14 ? 13 + (-14 - e) : 13;                           /* bits dropped */
    uint32_t kept = mant >> shift, rest = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rest > half || (rest == half && (kept & 1u))) kept++;
    /* normal: kept has bit 10 set (or 11 after a carry); subnormal: kept < 1024 */
    uint32_t h = e < -14 ? kept : ((uint32_t)(e + 15) << 10) + (kept - 1024u);
    return (uint16_t)(sign | (h > 0x7c00u ? 0x7c00u : h));
}

/*
 * The wider signature surface of npu_quant_matmul (shapes and dtypes: test/test_fake_tensor.py:1886-1915;
 * LinearQuant's default int32 bias: torch_npu/contrib/module/linear_quant.py:92):
 *   bias_kind 0 none, 1 bf16 (added after both scales), 2 int32 (added to the int32 accumulator before
 *   dequantisation, wrapping like the accumulator), 3 float32 (added after both scales);
 *   out_kind 0 bf16, 1 fp16, 2 int32 (accumulator plus int32 bias, no scaling).
 * Results on Ascend silicon: PARITY UNPINNED (no in-tree result test); the formula is the benchmark
 * configuration's with the bias moved where its type puts it.
 */
void orc_quant_matmul_epilogue_ex(const int32_t *acc, const float *pertoken_scale, const float *scale,
                                  int64_t scale_len, const void *bias, int bias_kind, int out_kind,
                                  int64_t M, int64_t N, void *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            int32_t a = acc[m * N + n];
            if (bias_kind == 2) a = (int32_t)((uint32_t)a + (uint32_t)((const int32_t *)bias)[n]);
            if (out_kind == 2) {
                ((int32_t *)out)[m * N + n] = a;
                continue;
            }
            float f = (float)a;
            if (pertoken_scale) f = f * pertoken_scale[m];
            f = f * scale[scale_len == 1 ? 0 : n];
            if (bias_kind == 1) f = f + bf16_to_f32(((const uint16_t *)bias)[n]);
            if (bias_kind == 3) f = f + ((const float *)bias)[n];
            ((uint16_t *)out)[m * N + n] = out_kind == 1 ? f32_to_f16(f) : f32_to_bf16(f);
        }
    }
}

/* ------------------------------------------------ int4 packing / antiquant */
/*
 * int32 word j of a row holds logical elements 8j..8j+7; element i sits in bits
 * [4i, 4i+3] (low nibble of the lowest-addressed byte first), two's complement.
 * Follows unpack_int4 in test/custom_ops/test_npu_anti_quant.py:12-24.
 */
void orc_unpack_int4(const int32_t *packed, int64_t n_words, int8_t *out)
{
    for (int64_t j = 0; j < n_words; j++) {
        uint32_t w = (uint32_t)packed[j];
        for (int i = 0; i < 8; i++) {
            int v = (int)((w >> (4 * i)) & 0xfu);
            out[j * 8 + i] = (int8_t)((v ^ 8) - 8);
        }
    }
}

void orc_pack_int4(const int8_t *vals, int64_t n_words, int32_t *packed)
{
    for (int64_t j = 0; j < n_words; j++) {
        uint32_t w = 0;
        for (int i = 0; i < 8; i++) w |= ((uint32_t)(vals[j * 8 + i] & 0xf)) << (4 * i);
        packed[j] = (int32_t)w;
    }
}

/*
 * Antiquant of one element: (float32(w) + offset) * scale, two binary32 roundings.
 * Follows custom_op_exec in test/custom_ops/test_npu_anti_quant.py:29-42 and the
 * weight golden in test/contrib/test_linear_weight_quant.py:20-28 (add offset, then
 * multiply by scale).
 */
void orc_antiquant(const int8_t *w, const float *scale, const float *offset,
                   int64_t rows, int64_t cols, float *out)
{
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++) {
            float t = (float)w[r * cols + c];
            if (offset) t = t + offset[c];
            out[r * cols + c] = t * scale[c];
        }
}

/* ------------------------------------------- npu_weight_quant_batchmatmul */
/*
 * out[m,n] = bf16( sum_k float32(x[m,k]) * wf[k,n] ),
 * wf[k,n]  = (float32(w[k,n]) + float32(off[g,n])) * float32(scale[g,n]),  g = k / group_size
 * (group_size 0 = per channel: g = 0).  Follows cpu_linear_weight_quant in
 * test/contrib/test_linear_weight_quant.py:20-28 with bf16 parameters and float32 arithmetic.
 * That test evaluates w + offset and * scale in the tensors' own type (float16 there), i.e. it
 * rounds the antiquantised weight twice before its float32 matmul; the benchmark's gate is stated
 * against the float32 formula, which is what this function restates.  The difference between the
 * two on the reference test's own data is measured by
 * tests/test_gpu_ops.py::test_linear_weight_quant_reference_test_shape.
 *
 * w_bits 8: w is int8 addressed as w[k*ldw_k + n*ldw_n].
 * w_bits 4: w is int32 [K, N/8] row-major, packed as described at orc_unpack_int4.
 * scale/off: bf16 [G, N] row-major (off may be NULL).
 * accum: 0 = binary32 accumulator, k ascending (the float32 golden);
 *        1 = binary64 accumulator over the same binary32 wf (error-budget reference).
 * out_f32 (optional) receives the unrounded accumulator as float32 (accum 0) or the
 * double rounded to float32 (accum 1).
 */
static void weight_quant_matmul_impl(const uint16_t *x_bf16, int64_t ldx,
                             const void *w, int w_bits, int64_t ldw_k, int64_t ldw_n,
                             const uint16_t *scale_bf16, const uint16_t *off_bf16,
                             int64_t M, int64_t N, int64_t K, int64_t group_size, int accum,
                             uint16_t *out_bf16, float *out_f32, int f16, const uint16_t *bias)
{
    /* f16: activations, parameters and output are IEEE binary16 (the dtype of the reference's own test,
     * test/contrib/test_linear_weight_quant.py:57-62) instead of bfloat16; nothing else changes */
#define ACT_TO_F32(h) (f16 ? fp16_to_f32(h) : bf16_to_f32(h))
    int64_t gs = group_size > 0 ? group_size : K;
    float *wf = (float *)malloc(sizeof(float) * (size_t)K * (size_t)N); /* [N][K] */
    float *xf = (float *)malloc(sizeof(float) * (size_t)M * (size_t)K);
    if (!wf || !xf) { free(wf); free(xf); return; }
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
        for (int64_t k = 0; k < K; k++) {
            int64_t g = k / gs;
            float wv;
            if (w_bits == 8) {
                wv = (float)((const int8_t *)w)[k * ldw_k + n * ldw_n];
            } else {
                uint32_t word = (uint32_t)((const int32_t *)w)[k * (N / 8) + n / 8];
                int v = (int)((word >> (4 * (n % 8))) & 0xfu);
                wv = (float)((v ^ 8) - 8);
            }
            if (off_bf16) wv = wv + ACT_TO_F32(off_bf16[g * N + n]);
            wf[n * K + k] = wv * ACT_TO_F32(scale_bf16[g * N + n]);
        }
    }
    for (int64_t m = 0; m < M; m++)
        for (int64_t k = 0; k < K; k++) xf[m * K + k] = ACT_TO_F32(x_bf16[m * ldx + k]);
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            const float *xr = xf + m * K;
            const float *wr = wf + n * K;
            float r;
            if (accum == 0) {
                float s = 0.0f;
                for (int64_t k = 0; k < K; k++) s = s + xr[k] * wr[k];
                r = s;
            } else {
                double s = 0.0;
                for (int64_t k = 0; k < K; k++) s += (double)xr[k] * (double)wr[k];
                r = (float)s;
            }
            if (bias) r = r + ACT_TO_F32(bias[n]);   /* the module's optional bias: added to the float32 sum (results on Ascend: parity unpinned) */
            if (out_bf16) out_bf16[m * N + n] = f16 ? f32_to_f16(r) : f32_to_bf16(r);
            if (out_f32) out_f32[m * N + n] = r;
        }
    }
    free(wf);
    free(xf);
}
#undef ACT_TO_F32

void orc_weight_quant_matmul(const uint16_t *x_bf16, int64_t ldx,
                             const void *w, int w_bits, int64_t ldw_k, int64_t ldw_n,
                             const uint16_t *scale_bf16, const uint16_t *off_bf16,
                             int64_t M, int64_t N, int64_t K, int64_t group_size, int accum,
                             uint16_t *out_bf16, float *out_f32)
{
    weight_quant_matmul_impl(x_bf16, ldx, w, w_bits, ldw_k, ldw_n, scale_bf16, off_bf16, M, N, K, group_size, accum,
                             out_bf16, out_f32, 0, NULL);
}

/* dtype: 0 bfloat16, 1 float16; bias: [N] of that type or NULL */
void orc_weight_quant_matmul_bias(const uint16_t *x, int64_t ldx, const void *w, int w_bits, int64_t ldw_k, int64_t ldw_n,
                                  const uint16_t *scale, const uint16_t *off, const uint16_t *bias, int dtype,
                                  int64_t M, int64_t N, int64_t K, int64_t group_size, int accum,
                                  uint16_t *out, float *out_f32)
{
    weight_quant_matmul_impl(x, ldx, w, w_bits, ldw_k, ldw_n, scale, off, M, N, K, group_size, accum, out, out_f32, dtype, bias);
}

void orc_weight_quant_matmul_f16(const uint16_t *x_f16, int64_t ldx,
                                 const void *w, int w_bits, int64_t ldw_k, int64_t ldw_n,
                                 const uint16_t *scale_f16, const uint16_t *off_f16,
                                 int64_t M, int64_t N, int64_t K, int64_t group_size, int accum,
                                 uint16_t *out_f16, float *out_f32)
{
    weight_quant_matmul_impl(x_f16, ldx, w, w_bits, ldw_k, ldw_n, scale_f16, off_f16, M, N, K, group_size, accum,
                             out_f16, out_f32, 1, NULL);
}

/* ----------------------------------------------------------------- npu_swiglu */
/*
 * x bf16 [rows, 2*half]: a = x[:, :half], b = x[:, half:]; out = silu(a) * b in the
 * input dtype: s = bf16(a / (1 + exp(-a))) evaluated in binary32, out = bf16(float(s) * float(b)).
 * Follows torch_npu/_inductor/decomposition.py:186-188 (silu(chunk0) * chunk1) as
 * eager bf16 tensor arithmetic evaluates it (each tensor op rounds to bf16).
 */
void orc_swiglu(const uint16_t *x_bf16, int64_t rows, int64_t half, uint16_t *out_bf16)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const uint16_t *a = x_bf16 + r * 2 * half;
        const uint16_t *b = a + half;
        for (int64_t j = 0; j < half; j++) {
            float av = bf16_to_f32(a[j]);
            float s = av / (1.0f + expf(-av));
            float sb = bf16_to_f32(f32_to_bf16(s));
            out_bf16[r * half + j] = f32_to_bf16(sb * bf16_to_f32(b[j]));
        }
    }
}
