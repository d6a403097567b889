// npu_dynamic_quant for gfx950: per-token symmetric int8 quantisation.
//
// One pass over HBM: every row is read once (16-byte loads), kept in registers while the
// row maximum is reduced, then quantised and written as packed int8 (8-byte stores).
// Algorithmic traffic per row: cols * 2 bytes in, cols bytes + 4 bytes out.
//
// Bit-exactness.  The contract is y = rint_half_even(fl(x / fl(amax / 127))) with IEEE
// binary32 divisions.  A division per element is ~11 VALU operations; instead the row's
// reciprocal r = fl(1 / scale) is formed once (correctly rounded division) and each element
// uses  q0 = x * r;  e = fma(-scale, q0, x);  q = fma(e, r, q0).
// For x and amax taken from bf16 or fp16 (8 / 11 significant bits) this sequence returns
// exactly the correctly rounded quotient: verified exhaustively over every pair of
// significands and every exponent distance that can produce a non-zero result.  Rows whose
// scale lies outside [2^-60, 2^60], and rows pre-multiplied by smooth scales (arbitrary
// binary32 significands), take the plain IEEE division instead.
//
// Rounding to int8 uses the add-magic-constant trick: q + 1.5 * 2^23 is rounded by the adder
// to the nearest integer (ties to even, unit = 1 in that binade) and the low byte of the sum's
// bit pattern is the two's-complement result.  |q| <= 127 * (1 + 2^-23), so no clamp is needed
// on the fast path.
#include "common.h"

namespace mi355 {
namespace {

constexpr int kBlock = 256;
// At most this many rows (one workgroup per CU or fewer) of more than 4096 elements: the time is that of one row, so a row
// takes 1024 threads instead of 256 (16 rows x 14336: SwiGLU + quantisation 9.7 -> 5.9 us, plain quantisation 3.4 -> 3.05;
// from about 400 rows on the 256-thread blocks win again).
constexpr int kFewRows = 256;

template <bool FP16>
__device__ __forceinline__ void unpack2(uint32_t u, float &lo, float &hi)
{
    if constexpr (FP16) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 v = __builtin_bit_cast(h2, u);
        lo = (float)v[0];
        hi = (float)v[1];
    } else {
        lo = bf16_lo(u);
        hi = bf16_hi(u);
    }
}

template <bool FP16>
__device__ __forceinline__ float cvt1(uint16_t h)
{
    if constexpr (FP16) {
        return (float)__builtin_bit_cast(_Float16, h);
    } else {
        return bf16_1(h);
    }
}

// Maximum over a wavefront of 64 lanes (all lanes receive it).
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        uint32_t o = (uint32_t)__shfl_xor((int)v, off, 64);
        v = v > o ? v : o;
    }
    return v;
}

__device__ __forceinline__ uint32_t quant_fast(float x, float scale, float r)
{
    float q0 = x * r;
    float e = __builtin_fmaf(-scale, q0, x);
    float q = __builtin_fmaf(e, r, q0);
    return __float_as_uint(q + 12582912.0f);
}

__device__ __forceinline__ uint32_t quant_exact(float x, float scale)
{
    float q = x / scale;
    q = __builtin_rintf(q);
    q = q > 127.0f ? 127.0f : q;
    q = q < -127.0f ? -127.0f : q; // NaN falls through both tests and converts to 0
    return (uint32_t)(int)q;
}


// TPR threads cooperate on one row (64 = one wavefront, no barrier; more = the whole block of BLOCK threads);
// each thread holds ITERS vectors of 8 elements.
// SWIGLU: the input row holds two halves of `cols` elements each and the quantised row is
// bf16(silu(act half)) * other half (rounded to bf16 like the stand-alone SwiGLU kernel): the fused
// SwiGLU + dynamic_quant of an MLP, which saves writing and re-reading the bf16 activation.
template <int TPR, int ITERS, bool FP16, bool SWIGLU = false, int BLOCK = kBlock>
__global__ __launch_bounds__(BLOCK) void dq_rows_kernel(const uint16_t *__restrict__ x, int8_t *__restrict__ y,
                                                         float *__restrict__ scale_out, int64_t rows, int cols,
                                                         int64_t row_stride, int act_offset = 0, int mul_offset = 0)
{
    constexpr int RPB = BLOCK / TPR;
    const int t = threadIdx.x % TPR;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;
    const bool live = row < rows;
    const int nvec = cols >> 3;
    const u32x4 *xr = reinterpret_cast<const u32x4 *>(x + (live ? row : 0) * row_stride);

    u32x4 v[ITERS];
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < ITERS; i++) {
        const int idx = t + i * TPR;
        if (live && idx < nvec) {
            if constexpr (SWIGLU) {
                // act_offset / mul_offset: position (in 16-byte vectors) of the activated and of the other half
                const u32x4 a = __builtin_nontemporal_load(xr + act_offset + idx);
                const u32x4 b = __builtin_nontemporal_load(xr + mul_offset + idx);
                v[i] = u32x4{swiglu2(a.x, b.x), swiglu2(a.y, b.y), swiglu2(a.z, b.z), swiglu2(a.w, b.w)};
            } else {
                v[i] = __builtin_nontemporal_load(xr + idx);
            }
        } else {
            v[i] = u32x4{0, 0, 0, 0};
        }
        // |x| compared on the bit patterns: two 16-bit lanes per dword
        typedef uint16_t us2 __attribute__((ext_vector_type(2)));
        us2 mm = __builtin_bit_cast(us2, m);
        mm = __builtin_elementwise_max(mm, __builtin_bit_cast(us2, v[i].x & 0x7fff7fffu));
        mm = __builtin_elementwise_max(mm, __builtin_bit_cast(us2, v[i].y & 0x7fff7fffu));
        mm = __builtin_elementwise_max(mm, __builtin_bit_cast(us2, v[i].z & 0x7fff7fffu));
        mm = __builtin_elementwise_max(mm, __builtin_bit_cast(us2, v[i].w & 0x7fff7fffu));
        m = __builtin_bit_cast(uint32_t, mm);
    }
    uint32_t m16 = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
    m16 = wave_max_u32(m16);
    if constexpr (TPR > 64) {
        __shared__ uint32_t part[BLOCK / 64];
        if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m16;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < BLOCK / 64; w++) m16 = part[w] > m16 ? part[w] : m16;
    }
    if (!live) return;

    const float amax = cvt1<FP16>((uint16_t)m16);
    const float scale = amax / 127.0f;
    if (t == 0) scale_out[row] = scale;
    u32x2 *yr = reinterpret_cast<u32x2 *>(y + row * (int64_t)cols);

    if (!(amax > 0.0f)) { // zero row (or NaN maximum): codes are all zero
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const int idx = t + i * TPR;
            if (idx < nvec) yr[idx] = u32x2{0, 0};
        }
        return;
    }
    const bool fast = scale >= 0x1p-60f && scale <= 0x1p60f;
    if (fast) {
        const float r = 1.0f / scale;
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const int idx = t + i * TPR;
            float f0, f1, f2, f3, f4, f5, f6, f7;
            unpack2<FP16>(v[i].x, f0, f1);
            unpack2<FP16>(v[i].y, f2, f3);
            unpack2<FP16>(v[i].z, f4, f5);
            unpack2<FP16>(v[i].w, f6, f7);
            u32x2 o;
            o.x = pack4(quant_fast(f0, scale, r), quant_fast(f1, scale, r), quant_fast(f2, scale, r),
                        quant_fast(f3, scale, r));
            o.y = pack4(quant_fast(f4, scale, r), quant_fast(f5, scale, r), quant_fast(f6, scale, r),
                        quant_fast(f7, scale, r));
            if (idx < nvec) __builtin_nontemporal_store(o, yr + idx);
        }
    } else {
#pragma unroll
        for (int i = 0; i < ITERS; i++) {
            const int idx = t + i * TPR;
            float f0, f1, f2, f3, f4, f5, f6, f7;
            unpack2<FP16>(v[i].x, f0, f1);
            unpack2<FP16>(v[i].y, f2, f3);
            unpack2<FP16>(v[i].z, f4, f5);
            unpack2<FP16>(v[i].w, f6, f7);
            u32x2 o;
            o.x = pack4(quant_exact(f0, scale), quant_exact(f1, scale), quant_exact(f2, scale),
                        quant_exact(f3, scale));
            o.y = pack4(quant_exact(f4, scale), quant_exact(f5, scale), quant_exact(f6, scale),
                        quant_exact(f7, scale));
            if (idx < nvec) yr[idx] = o;
        }
    }
}

// Any shape, stride and alignment; optional smooth scales.  One block per row, two passes
// over the row (the second one hits in cache), IEEE division per element.
template <bool FP16>
__global__ __launch_bounds__(kBlock) void dq_generic_kernel(const uint16_t *__restrict__ x,
                                                            const uint16_t *__restrict__ smooth,
                                                            int8_t *__restrict__ y, float *__restrict__ scale_out,
                                                            int64_t cols, int64_t row_stride,
                                                            const int32_t *__restrict__ group_index = nullptr, int groups = 0)
{
    const int64_t row = blockIdx.x;
    const uint16_t *xr = x + row * row_stride;
    if (smooth) smooth = expert_scales(smooth, group_index, groups, row, cols);
    float amax = 0.0f;
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) {
        float v = cvt1<FP16>(xr[j]);
        if (smooth) v = v * cvt1<FP16>(smooth[j]);
        amax = fmaxf(amax, fabsf(v));
    }
    uint32_t mb = wave_max_u32(__float_as_uint(amax)); // non-negative floats order like their bit patterns
    __shared__ uint32_t part[kBlock / 64];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = mb;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kBlock / 64; w++) mb = part[w] > mb ? part[w] : mb;
    amax = __uint_as_float(mb);
    const float scale = amax / 127.0f;
    if (threadIdx.x == 0) scale_out[row] = scale;
    int8_t *yr = y + row * cols;
    const bool zero = !(amax > 0.0f);
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) {
        float v = cvt1<FP16>(xr[j]);
        if (smooth) v = v * cvt1<FP16>(smooth[j]);
        yr[j] = zero ? (int8_t)0 : (int8_t)quant_exact(v, scale);
    }
}

// int4 output (dst_type torch.quint4x2): scale = max|x| / 7, codes rint(x / scale) in [-7, 7], eight codes per int32
// word with the first column in the low nibble (the order of mi355_unpack_int4 and mi355_anti_quant).  One block per
// row, two passes like dq_generic_kernel; cols is a multiple of 8 and a thread packs whole words.
template <bool FP16>
__global__ __launch_bounds__(kBlock) void dq_int4_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ smooth,
                                                         uint32_t *__restrict__ y, float *__restrict__ scale_out,
                                                         int64_t cols, int64_t row_stride,
                                                         const int32_t *__restrict__ group_index, int groups)
{
    const int64_t row = blockIdx.x;
    const uint16_t *xr = x + row * row_stride;
    if (smooth) smooth = expert_scales(smooth, group_index, groups, row, cols);
    float amax = 0.0f;
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) {
        float v = cvt1<FP16>(xr[j]);
        if (smooth) v = v * cvt1<FP16>(smooth[j]);
        amax = fmaxf(amax, fabsf(v));
    }
    uint32_t mb = wave_max_u32(__float_as_uint(amax));
    __shared__ uint32_t part[kBlock / 64];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = mb;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kBlock / 64; w++) mb = part[w] > mb ? part[w] : mb;
    amax = __uint_as_float(mb);
    const float scale = amax / 7.0f;
    if (threadIdx.x == 0) scale_out[row] = scale;
    uint32_t *yr = y + row * (cols >> 3);
    const bool zero = !(amax > 0.0f);
    for (int64_t w = threadIdx.x; w < (cols >> 3); w += kBlock) {
        uint32_t word = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float v = cvt1<FP16>(xr[8 * w + i]);
            if (smooth) v = v * cvt1<FP16>(smooth[8 * w + i]);
            float q = __builtin_rintf(v / scale);
            q = q > 7.0f ? 7.0f : q;
            q = q < -7.0f ? -7.0f : q;                       // NaN falls through both tests and converts to 0
            word |= ((uint32_t)(int)q & 0xfu) << (4 * i);
        }
        yr[w] = zero ? 0u : word;
    }
}

// Rows pre-multiplied by smooth scales, cols % 8 == 0 and at most 8 * BLOCK * MAXV, 16-byte aligned rows and smooth scales: one
// block per row, the products (arbitrary float32 significands) stay in registers between the maximum and the
// quantisation.  x / scale uses the row's refined reciprocal with the operation sequence of the compiler's own
// float32 division (quotient and two residual corrections) when the scale lies within [2^-60, 2^60]: that sequence's
// range scaling and fix-up are then the identity for every numerator that matters.  |x| <= 127 * scale, so nothing
// overflows; a numerator small enough for a residual to leave the normal range has a quotient below 2^-40, which
// rounds to zero either way; a NaN numerator becomes code 0 on both paths; an infinite one makes the scale infinite.
// Rows with a scale outside the range divide the ordinary way.
// SWIGLU (bf16): the row holds two halves of `cols` elements and the value that is smoothed and quantised is
// bf16(silu(act half)) * other half, rounded to bf16 like the stand-alone SwiGLU kernel; act_offset / mul_offset are
// the positions of the two halves in 16-byte vectors.
template <bool FP16, bool SWIGLU = false, int MAXV = 4, int BLOCK = kBlock>
__global__ __launch_bounds__(BLOCK) void dq_smooth_rows_kernel(const uint16_t *__restrict__ x,
                                                                const uint16_t *__restrict__ smooth,
                                                                int8_t *__restrict__ y, float *__restrict__ scale_out,
                                                                int cols, int64_t row_stride, int act_offset = 0,
                                                                int mul_offset = 0,
                                                                const int32_t *__restrict__ group_index = nullptr, int groups = 0)
{
    const int64_t row = blockIdx.x;
    const int t = threadIdx.x, nvec = cols >> 3;
    const u32x4 *xr = reinterpret_cast<const u32x4 *>(x + row * row_stride);
    const u32x4 *sr = reinterpret_cast<const u32x4 *>(expert_scales(smooth, group_index, groups, row, cols));
    float f[MAXV][8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < MAXV; i++) {
        const int idx = t + i * BLOCK;
        u32x4 a{0, 0, 0, 0}, b{0, 0, 0, 0};
        if (idx < nvec) {
            if constexpr (SWIGLU) {
                const u32x4 g = __builtin_nontemporal_load(xr + act_offset + idx);
                const u32x4 m = __builtin_nontemporal_load(xr + mul_offset + idx);
                a = u32x4{swiglu2(g.x, m.x), swiglu2(g.y, m.y), swiglu2(g.z, m.z), swiglu2(g.w, m.w)};
            } else {
                a = __builtin_nontemporal_load(xr + idx);
            }
            b = sr[idx];
        }
        float s8[8];
        unpack2<FP16>(a.x, f[i][0], f[i][1]);
        unpack2<FP16>(a.y, f[i][2], f[i][3]);
        unpack2<FP16>(a.z, f[i][4], f[i][5]);
        unpack2<FP16>(a.w, f[i][6], f[i][7]);
        unpack2<FP16>(b.x, s8[0], s8[1]);
        unpack2<FP16>(b.y, s8[2], s8[3]);
        unpack2<FP16>(b.z, s8[4], s8[5]);
        unpack2<FP16>(b.w, s8[6], s8[7]);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            f[i][k] = f[i][k] * s8[k];
            amax = fmaxf(amax, fabsf(f[i][k]));
        }
    }
    uint32_t mb = wave_max_u32(__float_as_uint(amax));        // non-negative floats order like their bit patterns
    __shared__ uint32_t part[BLOCK / 64];
    if ((t & 63) == 0) part[t >> 6] = mb;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < BLOCK / 64; w++) mb = part[w] > mb ? part[w] : mb;
    amax = __uint_as_float(mb);
    const float scale = amax / 127.0f;
    if (t == 0) scale_out[row] = scale;
    u32x2 *yr = reinterpret_cast<u32x2 *>(y + row * (int64_t)cols);
    const bool zero = !(amax > 0.0f);
    const bool scale_safe = scale >= 0x1p-60f && scale <= 0x1p60f;
    float r = __builtin_amdgcn_rcpf(scale);
    r = __builtin_fmaf(__builtin_fmaf(-scale, r, 1.0f), r, r);
#pragma unroll
    for (int i = 0; i < MAXV; i++) {
        const int idx = t + i * BLOCK;
        uint32_t q[8];
        if (zero) {
#pragma unroll
            for (int k = 0; k < 8; k++) q[k] = 0u;
        } else if (scale_safe) {                              // the same for the whole row
#pragma unroll
            for (int k = 0; k < 8; k++) {
                float v = f[i][k] * r;
                v = __builtin_fmaf(__builtin_fmaf(-scale, v, f[i][k]), r, v);
                v = __builtin_fmaf(__builtin_fmaf(-scale, v, f[i][k]), r, v);
                // |v| <= 127 (1 + 2^-22) because |x| <= amax: adding 1.5 * 2^23 rounds to the integer (ties to even) and
                // leaves it in the low byte; a NaN stays a quiet NaN, whose low byte is 0
                q[k] = __float_as_uint(v + 12582912.0f);
            }
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) q[k] = quant_exact(f[i][k], scale);
        }
        if (idx < nvec) __builtin_nontemporal_store(u32x2{pack4(q[0], q[1], q[2], q[3]), pack4(q[4], q[5], q[6], q[7])}, yr + idx);
    }
}

template <int TPR, int ITERS, int BLOCK = kBlock>
void launch_rows(bool fp16, const uint16_t *x, int8_t *y, float *scale, int64_t rows, int cols, int64_t stride,
                 hipStream_t s)
{
    constexpr int RPB = BLOCK / TPR;
    const unsigned grid = (unsigned)((rows + RPB - 1) / RPB);
    if (fp16)
        hipLaunchKernelGGL((dq_rows_kernel<TPR, ITERS, true, false, BLOCK>), dim3(grid), dim3(BLOCK), 0, s, x, y, scale, rows,
                           cols, stride);
    else
        hipLaunchKernelGGL((dq_rows_kernel<TPR, ITERS, false, false, BLOCK>), dim3(grid), dim3(BLOCK), 0, s, x, y, scale, rows,
                           cols, stride);
}

template <int TPR, int ITERS, int BLOCK = kBlock>
void launch_swiglu_rows(const uint16_t *x, int8_t *y, float *scale, int64_t rows, int cols, int64_t stride, int act_off,
                        int mul_off, hipStream_t s)
{
    constexpr int RPB = BLOCK / TPR;
    const unsigned grid = (unsigned)((rows + RPB - 1) / RPB);
    hipLaunchKernelGGL((dq_rows_kernel<TPR, ITERS, false, true, BLOCK>), dim3(grid), dim3(BLOCK), 0, s, x, y, scale, rows, cols,
                       stride, act_off, mul_off);
}

// Any shape and alignment: one block per row, SwiGLU recomputed in the second pass.
__global__ __launch_bounds__(kBlock) void swiglu_dq_generic_kernel(const uint16_t *__restrict__ x, int8_t *__restrict__ y,
                                                                  float *__restrict__ scale_out, int64_t half,
                                                                  int64_t row_stride, int64_t act_off, int64_t mul_off,
                                                                  const uint16_t *__restrict__ smooth = nullptr,
                                                                  const int32_t *__restrict__ group_index = nullptr, int groups = 0)
{
    const int64_t row = blockIdx.x;
    const uint16_t *xr = x + row * row_stride;
    if (smooth) smooth = expert_scales(smooth, group_index, groups, row, half);
    auto value = [&](int64_t j) {
        const float sl = silu_bf16(bf16_1(xr[act_off + j]));
        const float v = bf16_1(f32_to_bf16(sl * bf16_1(xr[mul_off + j])));
        return smooth ? v * bf16_1(smooth[j]) : v;
    };
    float amax = 0.0f;
    for (int64_t j = threadIdx.x; j < half; j += kBlock) amax = fmaxf(amax, fabsf(value(j)));
    uint32_t mb = wave_max_u32(__float_as_uint(amax));
    __shared__ uint32_t part[kBlock / 64];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = mb;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kBlock / 64; w++) mb = part[w] > mb ? part[w] : mb;
    amax = __uint_as_float(mb);
    const float scale = amax / 127.0f;
    if (threadIdx.x == 0) scale_out[row] = scale;
    const bool zero = !(amax > 0.0f);
    for (int64_t j = threadIdx.x; j < half; j += kBlock) y[row * half + j] = zero ? (int8_t)0 : (int8_t)quant_exact(value(j), scale);
}

} // namespace
} // namespace mi355

namespace mi355 {
namespace {
int run_swiglu_quant(const void *x_bf16, int activate_left, const void *smooth, int8_t *y, float *scale, int64_t rows,
                     int64_t half, int64_t x_row_stride, void *stream, const int32_t *group_index = nullptr, int64_t groups = 0)
{
    if (rows < 0 || half < 0) return MI355_ERR_BAD_ARGUMENT;
    if (group_index && (!smooth || groups < 1 || groups > 0x7fffffff)) return MI355_ERR_BAD_ARGUMENT;
    if (group_index && !aligned(group_index, 4)) return MI355_ERR_ALIGNMENT;
    const int ng = group_index ? (int)groups : 0;
    if (rows == 0) return MI355_OK;
    if (!scale) return MI355_ERR_BAD_ARGUMENT;
    if (half > 0 && (!x_bf16 || !y || x_row_stride < 2 * half)) return MI355_ERR_BAD_ARGUMENT;
    if (rows > 0x7fffffff) return MI355_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint16_t *xp = static_cast<const uint16_t *>(x_bf16);
    const int64_t act = activate_left ? 0 : half, mul = activate_left ? half : 0;
    const int64_t nvec = half >> 3;
    const bool vec_ok = half > 0 && (half & 7) == 0 && (x_row_stride & 7) == 0 && aligned(xp, 16) && aligned(y, 8) &&
                        nvec <= 1024 * 8;       // halves of up to 16384 elements on 256 threads, up to 65536 on 1024
    const uint16_t *sm = static_cast<const uint16_t *>(smooth);
    if (sm) {
        if (!aligned(sm, 2)) return MI355_ERR_ALIGNMENT;
        if (vec_ok && aligned(sm, 16)) {
            const int c = (int)half, ao = (int)(act >> 3), mo = (int)(mul >> 3);
            if (rows <= kFewRows && nvec > 1024 && nvec <= 1024 * 4)      // measured: no gain up to 8192 elements
                hipLaunchKernelGGL((dq_smooth_rows_kernel<false, true, 4, 1024>), dim3((unsigned)rows), dim3(1024), 0, s, xp, sm,
                                   y, scale, c, x_row_stride, ao, mo, group_index, ng);
            else if (nvec <= kBlock * 4)
                hipLaunchKernelGGL((dq_smooth_rows_kernel<false, true, 4>), dim3((unsigned)rows), dim3(kBlock), 0, s, xp, sm, y,
                                   scale, c, x_row_stride, ao, mo, group_index, ng);
            else if (nvec <= kBlock * 8)
                hipLaunchKernelGGL((dq_smooth_rows_kernel<false, true, 8>), dim3((unsigned)rows), dim3(kBlock), 0, s, xp, sm, y,
                                   scale, c, x_row_stride, ao, mo, group_index, ng);
            else if (nvec <= 1024 * 4)
                hipLaunchKernelGGL((dq_smooth_rows_kernel<false, true, 4, 1024>), dim3((unsigned)rows), dim3(1024), 0, s, xp, sm,
                                   y, scale, c, x_row_stride, ao, mo, group_index, ng);
            else
                hipLaunchKernelGGL((dq_smooth_rows_kernel<false, true, 8, 1024>), dim3((unsigned)rows), dim3(1024), 0, s, xp, sm,
                                   y, scale, c, x_row_stride, ao, mo, group_index, ng);
        } else {
            hipLaunchKernelGGL(swiglu_dq_generic_kernel, dim3((unsigned)rows), dim3(kBlock), 0, s, xp, y, scale, half,
                               x_row_stride, act, mul, sm, group_index, ng);
        }
        return check_launch();
    }
    if (vec_ok) {
        const int c = (int)half, ao = (int)(act >> 3), mo = (int)(mul >> 3);
        // few long rows (a decode batch): a row takes 1024 threads instead of 256, the row is the critical path
        if (rows <= kFewRows && nvec > 256 * 2 && nvec <= 1024 * 2) launch_swiglu_rows<1024, 2, 1024>(xp, y, scale, rows, c, x_row_stride, ao, mo, s);
        else if (nvec <= 64 * 1) launch_swiglu_rows<64, 1>(xp, y, scale, rows, c, x_row_stride, ao, mo, s);
        else if (nvec <= 64 * 2) launch_swiglu_rows<64, 2>(xp, y, scale, rows, c, x_row_stride, ao, mo, s);
        else if (nvec <= 64 * 4) launch_swiglu_rows<64, 4>(xp, y, scale, rows, c, x_row_stride, ao, mo, s);
        else if (nvec <= 256 * 2) launch_swiglu_rows<256, 2>(xp, y, scale, rows, c, x_row_stride, ao, mo, s);
        else if (nvec <= 256 * 4) launch_swiglu_rows<256, 4>(xp, y, scale, rows, c, x_row_stride, ao, mo, s);
        else if (nvec <= 256 * 8) launch_swiglu_rows<256, 8>(xp, y, scale, rows, c, x_row_stride, ao, mo, s);
        else if (nvec <= 1024 * 4) launch_swiglu_rows<1024, 4, 1024>(xp, y, scale, rows, c, x_row_stride, ao, mo, s);
        else launch_swiglu_rows<1024, 8, 1024>(xp, y, scale, rows, c, x_row_stride, ao, mo, s);
    } else {
        hipLaunchKernelGGL(swiglu_dq_generic_kernel, dim3((unsigned)rows), dim3(kBlock), 0, s, xp, y, scale, half, x_row_stride,
                           act, mul);
    }
    return check_launch();
}

} // namespace
} // namespace mi355

extern "C" int mi355_swiglu_quant(const void *x_bf16, int activate_left, int8_t *y, float *scale, int64_t rows, int64_t half,
                                  int64_t x_row_stride, void *stream)
{
    return mi355::run_swiglu_quant(x_bf16, activate_left, nullptr, y, scale, rows, half, x_row_stride, stream);
}

extern "C" int mi355_swiglu_quant_smooth(const void *x_bf16, int activate_left, const void *smooth_bf16, int8_t *y, float *scale,
                                         int64_t rows, int64_t half, int64_t x_row_stride, void *stream)
{
    if (!smooth_bf16 && rows > 0 && half > 0) return MI355_ERR_BAD_ARGUMENT;
    return mi355::run_swiglu_quant(x_bf16, activate_left, smooth_bf16, y, scale, rows, half, x_row_stride, stream);
}

extern "C" int mi355_swiglu_quant_grouped(const void *x_bf16, int activate_left, const void *smooth_bf16, const int32_t *group_index,
                                          int64_t groups, int8_t *y, float *scale, int64_t rows, int64_t half,
                                          int64_t x_row_stride, void *stream)
{
    if ((!smooth_bf16 || !group_index) && rows > 0 && half > 0) return MI355_ERR_BAD_ARGUMENT;
    return mi355::run_swiglu_quant(x_bf16, activate_left, smooth_bf16, y, scale, rows, half, x_row_stride, stream, group_index, groups);
}

extern "C" int mi355_dynamic_quant(const void *x, int in_dtype, const void *smooth, int8_t *y, float *scale,
                                   int64_t rows, int64_t cols, int64_t x_row_stride, void *stream)
{
    return mi355_dynamic_quant_grouped(x, in_dtype, smooth, nullptr, 0, y, scale, rows, cols, x_row_stride, stream);
}

extern "C" int mi355_dynamic_quant_int4(const void *x, int in_dtype, const void *smooth, const int32_t *group_index,
                                        int64_t groups, void *y_words, float *scale, int64_t rows, int64_t cols,
                                        int64_t x_row_stride, void *stream)
{
    using namespace mi355;
    if (rows < 0 || cols < 0 || (cols & 7) != 0) return MI355_ERR_BAD_ARGUMENT;
    if (in_dtype != MI355_DTYPE_BF16 && in_dtype != MI355_DTYPE_FP16) return MI355_ERR_BAD_ARGUMENT;
    if (group_index && (!smooth || groups < 1 || groups > 0x7fffffff)) return MI355_ERR_BAD_ARGUMENT;
    if (group_index && !aligned(group_index, 4)) return MI355_ERR_ALIGNMENT;
    if (rows == 0) return MI355_OK;
    if (!scale) return MI355_ERR_BAD_ARGUMENT;
    if (cols > 0 && (!x || !y_words || x_row_stride < cols)) return MI355_ERR_BAD_ARGUMENT;
    if (y_words && !aligned(y_words, 4)) return MI355_ERR_ALIGNMENT;
    if (rows > 0x7fffffff) return MI355_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint16_t *xp = static_cast<const uint16_t *>(x), *sm = static_cast<const uint16_t *>(smooth);
    const int ng = group_index ? (int)groups : 0;
    if (in_dtype == MI355_DTYPE_FP16)
        hipLaunchKernelGGL((dq_int4_kernel<true>), dim3((unsigned)rows), dim3(kBlock), 0, s, xp, sm, static_cast<uint32_t *>(y_words),
                           scale, cols, x_row_stride, group_index, ng);
    else
        hipLaunchKernelGGL((dq_int4_kernel<false>), dim3((unsigned)rows), dim3(kBlock), 0, s, xp, sm, static_cast<uint32_t *>(y_words),
                           scale, cols, x_row_stride, group_index, ng);
    return check_launch();
}

extern "C" int mi355_dynamic_quant_grouped(const void *x, int in_dtype, const void *smooth, const int32_t *group_index,
                                           int64_t groups, int8_t *y, float *scale, int64_t rows, int64_t cols,
                                           int64_t x_row_stride, void *stream)
{
    using namespace mi355;
    if (rows < 0 || cols < 0) return MI355_ERR_BAD_ARGUMENT;
    if (group_index && (!smooth || groups < 1 || groups > 0x7fffffff)) return MI355_ERR_BAD_ARGUMENT;
    if (group_index && !aligned(group_index, 4)) return MI355_ERR_ALIGNMENT;
    const int ng = group_index ? (int)groups : 0;
    if (in_dtype != MI355_DTYPE_BF16 && in_dtype != MI355_DTYPE_FP16) return MI355_ERR_BAD_ARGUMENT;
    if (rows == 0) return MI355_OK;
    if (!scale) return MI355_ERR_BAD_ARGUMENT;
    if (cols > 0 && (!x || !y || x_row_stride < cols)) return MI355_ERR_BAD_ARGUMENT;
    if (rows > 0x7fffffff) return MI355_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool fp16 = in_dtype == MI355_DTYPE_FP16;
    const uint16_t *xp = static_cast<const uint16_t *>(x);

    const int64_t nvec = cols >> 3;
    // rows of up to 16384 elements on 256 threads, up to 65536 on 1024 (eight 16-byte vectors per thread at most)
    const bool vec_ok = !smooth && cols > 0 && (cols & 7) == 0 && (x_row_stride & 7) == 0 && aligned(x, 16) &&
                        aligned(y, 8) && nvec <= 1024 * 8;
    if (vec_ok) {
        const int c = (int)cols;
        if (rows <= kFewRows && nvec > 256 * 2 && nvec <= 1024 * 2) launch_rows<1024, 2, 1024>(fp16, xp, y, scale, rows, c, x_row_stride, s);
        else if (nvec <= 64 * 1) launch_rows<64, 1>(fp16, xp, y, scale, rows, c, x_row_stride, s);
        else if (nvec <= 64 * 2) launch_rows<64, 2>(fp16, xp, y, scale, rows, c, x_row_stride, s);
        else if (nvec <= 64 * 4) launch_rows<64, 4>(fp16, xp, y, scale, rows, c, x_row_stride, s);
        else if (nvec <= 256 * 2) launch_rows<256, 2>(fp16, xp, y, scale, rows, c, x_row_stride, s);
        else if (nvec <= 256 * 4) launch_rows<256, 4>(fp16, xp, y, scale, rows, c, x_row_stride, s);
        else if (nvec <= 256 * 8) launch_rows<256, 8>(fp16, xp, y, scale, rows, c, x_row_stride, s);
        else if (nvec <= 1024 * 4) launch_rows<1024, 4, 1024>(fp16, xp, y, scale, rows, c, x_row_stride, s);
        else launch_rows<1024, 8, 1024>(fp16, xp, y, scale, rows, c, x_row_stride, s);
    } else if (smooth && cols > 0 && (cols & 7) == 0 && (x_row_stride & 7) == 0 && aligned(x, 16) && aligned(smooth, 16) &&
               aligned(y, 8) && nvec <= 1024 * 8) {
        const uint16_t *sm = static_cast<const uint16_t *>(smooth);
#define MI355_DQS_LAUNCH(F, V, B) \
    hipLaunchKernelGGL((dq_smooth_rows_kernel<F, false, V, B>), dim3((unsigned)rows), dim3(B), 0, s, xp, sm, y, scale, (int)cols, \
                       x_row_stride, 0, 0, group_index, ng)
        if (nvec <= kBlock * 4) {
            if (fp16) MI355_DQS_LAUNCH(true, 4, kBlock);
            else MI355_DQS_LAUNCH(false, 4, kBlock);
        } else if (nvec <= kBlock * 8) {
            if (fp16) MI355_DQS_LAUNCH(true, 8, kBlock);
            else MI355_DQS_LAUNCH(false, 8, kBlock);
        } else if (nvec <= 1024 * 4) {
            if (fp16) MI355_DQS_LAUNCH(true, 4, 1024);
            else MI355_DQS_LAUNCH(false, 4, 1024);
        } else {
            if (fp16) MI355_DQS_LAUNCH(true, 8, 1024);
            else MI355_DQS_LAUNCH(false, 8, 1024);
        }
#undef MI355_DQS_LAUNCH
    } else {
        const uint16_t *sm = static_cast<const uint16_t *>(smooth);
        if (fp16)
            hipLaunchKernelGGL((dq_generic_kernel<true>), dim3((unsigned)rows), dim3(kBlock), 0, s, xp, sm, y, scale,
                               cols, x_row_stride, group_index, ng);
        else
            hipLaunchKernelGGL((dq_generic_kernel<false>), dim3((unsigned)rows), dim3(kBlock), 0, s, xp, sm, y, scale,
                               cols, x_row_stride, group_index, ng);
    }
    return check_launch();
}
