// npu_quantize for gfx950: static quantisation with given per-channel (or single) scales and zero points,
//   div_mode:  q = clamp(rint(x / scale[c] + zero_point[c]))      otherwise  q = clamp(rint(x * scale[c] + zero_point[c]))
// x is bf16 / fp16 / float32 viewed as [outer, channels, inner] (channels = the quantisation axis), q is int8, uint8 or
// int32.  Bandwidth-bound elementwise kernel; every operation is rounded separately in float32 (IEEE division, no
// contraction), so results equal a float32 evaluation of the formula element by element.
#include "common.h"
#include <algorithm>

namespace mi355 {
namespace {

struct QzArgs {
    const void *x;
    const float *scale;           // [channels] or [1]
    const void *zp;               // float32 or int32 (zp_int), [channels] or [1]; may be null (zero)
    int zp_int;
    void *out;
    int64_t total;                // outer * channels * inner
    int64_t channels, inner;
    int scale_one, zp_one, div_mode;
    float qmin, qmax;
};

template <int IN>                 // 0 bf16, 1 fp16, 2 float32
__device__ __forceinline__ float load1(const void *x, int64_t e)
{
    if constexpr (IN == 0) return bf16_1(static_cast<const uint16_t *>(x)[e]);
    else if constexpr (IN == 1) return (float)static_cast<const _Float16 *>(x)[e];
    else return static_cast<const float *>(x)[e];
}

// After the quotient (or product): add the zero point, round half to even, clamp.
__device__ __forceinline__ float finish1(float v, float zp, float qmin, float qmax)
{
    v = v + zp;
    v = rintf(v);                                     // ties to even
    v = v == v ? v : 0.0f;                            // NaN quantises to 0
    return fminf(fmaxf(v, qmin), qmax);               // (int32: qmax is 2^31 as a float, see to_i32)
}

template <bool DIV>
__device__ __forceinline__ float quant1(float x, float sc, float zp, float qmin, float qmax)
{
    return finish1(DIV ? x / sc : x * sc, zp, qmin, qmax);
}

// Division by a channel's scale with the reciprocal formed once per channel: the operation sequence of the compiler's
// own float32 division (reciprocal refined once, quotient, two residual corrections with fused multiply-adds) without
// its range scaling and special-case fix-up, which are the identity while no intermediate leaves the normal range.
// Used for a group of elements only when every lane of the wavefront has its scales within [2^-60, 2^60] and
// numerators of at most 2^60 (so nothing overflows; a numerator small enough for a residual to leave the normal
// range has a quotient below 2^-40, which the zero point absorbs or which rounds to zero either way); otherwise the
// whole wavefront takes the ordinary division, so there is one scalar branch per group and never both computations.
__device__ __forceinline__ bool safe_range(float v)
{
    const float a = __builtin_fabsf(v);
    return a >= 0x1p-60f && a <= 0x1p60f;
}
__device__ __forceinline__ float refined_rcp(float d)
{
    const float r = __builtin_amdgcn_rcpf(d);
    return __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
}
__device__ __forceinline__ float div_by_rcp(float x, float d, float r)
{
    float q = x * r;
    q = __builtin_fmaf(__builtin_fmaf(-d, q, x), r, q);
    q = __builtin_fmaf(__builtin_fmaf(-d, q, x), r, q);
    return q;
}

// q[i] = quantised x[i] for eight elements with per-element scale sc[i], reciprocal rc[i] and zero point zp[i]
template <bool DIV>
__device__ __forceinline__ void quant8(const float (&x)[8], const float (&sc)[8], const float (&rc)[8], bool scales_safe,
                                       const float (&zp)[8], float qmin, float qmax, float (&q)[8])
{
    if constexpr (DIV) {
        bool ok = scales_safe;
#pragma unroll
        for (int i = 0; i < 8; i++) ok = ok && __builtin_fabsf(x[i]) <= 0x1p60f;   // false for NaN and infinity too
        if (__builtin_amdgcn_ballot_w64(!ok) == 0) {          // uniform over the wavefront
#pragma unroll
            for (int i = 0; i < 8; i++) q[i] = finish1(div_by_rcp(x[i], sc[i], rc[i]), zp[i], qmin, qmax);
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) q[i] = quant1<DIV>(x[i], sc[i], zp[i], qmin, qmax);
}

__device__ __forceinline__ float zp_at(const QzArgs &p, int64_t i)
{
    return p.zp_int ? (float)static_cast<const int32_t *>(p.zp)[i] : static_cast<const float *>(p.zp)[i];
}

// float32 cannot hold 2^31 - 1: everything from 2^31 up saturates to it
__device__ __forceinline__ int32_t to_i32(float v) { return v >= 2147483648.0f ? 2147483647 : (int32_t)v; }

template <int OUT>                // 0 int8, 1 uint8, 2 int32
__device__ __forceinline__ void store1(void *out, int64_t e, float v)
{
    if constexpr (OUT == 0) static_cast<int8_t *>(out)[e] = (int8_t)(int)v;
    else if constexpr (OUT == 1) static_cast<uint8_t *>(out)[e] = (uint8_t)(int)v;
    else static_cast<int32_t *>(out)[e] = to_i32(v);
}

template <int IN>
__device__ __forceinline__ void load8(const void *x, int64_t e, float (&v)[8])
{
    if constexpr (IN == 2) {
        const f32x4 a = *reinterpret_cast<const f32x4 *>(static_cast<const float *>(x) + e);
        const f32x4 b = *reinterpret_cast<const f32x4 *>(static_cast<const float *>(x) + e + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = a[i], v[4 + i] = b[i];
    } else {
        const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(static_cast<const uint16_t *>(x) + e));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t u = w[i];
            if constexpr (IN == 0) {
                v[2 * i] = bf16_lo(u);
                v[2 * i + 1] = bf16_hi(u);
            } else {
                v[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u & 0xffffu));
                v[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u >> 16));
            }
        }
    }
}

template <int OUT>
__device__ __forceinline__ void store8(void *out, int64_t e, const float (&q)[8])
{
    if constexpr (OUT == 2) {
        i32x4 a, b;
#pragma unroll
        for (int i = 0; i < 4; i++) a[i] = to_i32(q[i]), b[i] = to_i32(q[4 + i]);
        *reinterpret_cast<i32x4 *>(static_cast<int32_t *>(out) + e) = a;
        *reinterpret_cast<i32x4 *>(static_cast<int32_t *>(out) + e + 4) = b;
    } else {
        u32x2 o{0u, 0u};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            o.x |= ((uint32_t)(int)q[i] & 0xffu) << (8 * i);
            o.y |= ((uint32_t)(int)q[4 + i] & 0xffu) << (8 * i);
        }
        __builtin_nontemporal_store(o, reinterpret_cast<u32x2 *>(static_cast<uint8_t *>(out) + e));
    }
}

// Eight consecutive elements per thread that share a channel (inner % 8 == 0, or a single scale and zero point).
template <int IN, int OUT, bool DIV>
__global__ __launch_bounds__(256) void quantize_vec_kernel(const QzArgs p)
{
    const int64_t groups = p.total / 8;
    const bool single = p.scale_one && (!p.zp || p.zp_one);
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
        const int64_t e = g * 8;
        float x[8], q[8];
        load8<IN>(p.x, e, x);
        const int64_t c = single ? 0 : (e / p.inner) % p.channels;
        const float sc = p.scale[p.scale_one ? 0 : c];
        const float zp = p.zp ? zp_at(p, p.zp_one ? 0 : c) : 0.0f;
        const float r = DIV ? refined_rcp(sc) : 0.0f;
        const float sc8[8] = {sc, sc, sc, sc, sc, sc, sc, sc}, rc8[8] = {r, r, r, r, r, r, r, r};
        const float zp8[8] = {zp, zp, zp, zp, zp, zp, zp, zp};
        quant8<DIV>(x, sc8, rc8, safe_range(sc), zp8, p.qmin, p.qmax, q);
        store8<OUT>(p.out, e, q);
    }
}

// The axis is the innermost dimension and channels % 8 == 0: x is [rows, channels]; a thread keeps the scales and zero
// points of its eight channels in registers and walks down the rows (blockIdx.y strides over them, four rows in
// flight per step).
template <int IN, int OUT, bool DIV>
__global__ __launch_bounds__(256) void quantize_cols_kernel(const QzArgs p)
{
    const int64_t c = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (c >= p.channels) return;
    float sc[8], zp[8];
    if (p.scale_one) {
#pragma unroll
        for (int i = 0; i < 8; i++) sc[i] = p.scale[0];
    } else {                                                   // 32-byte aligned: c is a multiple of 8
        const f32x4 a = *reinterpret_cast<const f32x4 *>(p.scale + c), b = *reinterpret_cast<const f32x4 *>(p.scale + c + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) sc[i] = a[i], sc[4 + i] = b[i];
    }
    if (!p.zp || p.zp_one) {
#pragma unroll
        for (int i = 0; i < 8; i++) zp[i] = p.zp ? zp_at(p, 0) : 0.0f;
    } else {
        const u32x4 a = *reinterpret_cast<const u32x4 *>(static_cast<const uint32_t *>(p.zp) + c);
        const u32x4 b = *reinterpret_cast<const u32x4 *>(static_cast<const uint32_t *>(p.zp) + c + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            zp[i] = p.zp_int ? (float)(int32_t)a[i] : __uint_as_float(a[i]);
            zp[4 + i] = p.zp_int ? (float)(int32_t)b[i] : __uint_as_float(b[i]);
        }
    }
    float rc[8];
    bool scales_safe = true;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        rc[i] = DIV ? refined_rcp(sc[i]) : 0.0f;
        scales_safe = scales_safe && safe_range(sc[i]);
    }
    const int64_t rows = p.total / p.channels;
    constexpr int RU = 4;
    for (int64_t r0 = (int64_t)blockIdx.y * RU; r0 < rows; r0 += (int64_t)gridDim.y * RU) {
        float x[RU][8];
#pragma unroll
        for (int u = 0; u < RU; u++) load8<IN>(p.x, min(r0 + u, rows - 1) * p.channels + c, x[u]);
#pragma unroll
        for (int u = 0; u < RU; u++) {
            if (r0 + u >= rows) break;
            float q[8];
            quant8<DIV>(x[u], sc, rc, scales_safe, zp, p.qmin, p.qmax, q);
            store8<OUT>(p.out, (r0 + u) * p.channels + c, q);
        }
    }
}

// any shape and alignment: one element per thread and step
template <int IN, int OUT, bool DIV>
__global__ __launch_bounds__(256) void quantize_scalar_kernel(const QzArgs p)
{
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < p.total; e += (int64_t)gridDim.x * 256) {
        const int64_t c = (e / p.inner) % p.channels;
        const float sc = p.scale[p.scale_one ? 0 : c];
        const float zp = p.zp ? zp_at(p, p.zp_one ? 0 : c) : 0.0f;
        store1<OUT>(p.out, e, quant1<DIV>(load1<IN>(p.x, e), sc, zp, p.qmin, p.qmax));
    }
}

template <int IN, int OUT, bool DIV>
int launch_quantize_mode(const QzArgs &p, int vec_mode, hipStream_t s)
{
    int64_t blocks = ((vec_mode ? p.total / 8 : p.total) + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;                 // grid-stride beyond that
    if (blocks < 1) blocks = 1;
    if (vec_mode == 1) {
        hipLaunchKernelGGL((quantize_vec_kernel<IN, OUT, DIV>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    } else if (vec_mode == 2) {
        const int64_t rows = p.total / p.channels;
        const int64_t bx = (p.channels / 8 + 255) / 256;
        // a block loads its parameters once: give it at least 8 rows (two steps) where that still leaves two
        // blocks per CU, and never more blocks than fill the chip several times over
        int64_t by = (rows + 7) / 8;
        const int64_t fill = (512 + bx - 1) / bx, cap = (256 * 16 + bx - 1) / bx;
        if (by < fill) by = std::min<int64_t>(fill, (rows + 3) / 4);
        if (by > cap) by = cap;
        if (bx > 0x7fffffff) return MI355_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((quantize_cols_kernel<IN, OUT, DIV>), dim3((unsigned)bx, (unsigned)by), dim3(256), 0, s, p);
    } else {
        hipLaunchKernelGGL((quantize_scalar_kernel<IN, OUT, DIV>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    }
    return check_launch();
}

template <int IN, int OUT>
int launch_quantize(const QzArgs &p, int vec_mode, hipStream_t s)
{
    return p.div_mode ? launch_quantize_mode<IN, OUT, true>(p, vec_mode, s) : launch_quantize_mode<IN, OUT, false>(p, vec_mode, s);
}

template <int IN>
int launch_quantize_out(const QzArgs &p, int out_dtype, int vec_mode, hipStream_t s)
{
    if (out_dtype == MI355_Q_INT8) return launch_quantize<IN, 0>(p, vec_mode, s);
    if (out_dtype == MI355_Q_UINT8) return launch_quantize<IN, 1>(p, vec_mode, s);
    return launch_quantize<IN, 2>(p, vec_mode, s);
}

} // namespace
} // namespace mi355

extern "C" int mi355_quantize(const void *x, int in_dtype, const float *scale, int64_t scale_len, const void *zero_point,
                              int zero_point_dtype, int64_t zero_point_len, void *out, int out_dtype, int64_t outer,
                              int64_t channels, int64_t inner, int div_mode, void *stream)
{
    using namespace mi355;
    if (outer < 0 || channels < 0 || inner < 0) return MI355_ERR_BAD_ARGUMENT;
    if (in_dtype != MI355_DTYPE_BF16 && in_dtype != MI355_DTYPE_FP16 && in_dtype != MI355_DTYPE_FP32) return MI355_ERR_BAD_ARGUMENT;
    if (out_dtype != MI355_Q_INT8 && out_dtype != MI355_Q_UINT8 && out_dtype != MI355_Q_INT32) return MI355_ERR_BAD_ARGUMENT;
    if (outer == 0 || channels == 0 || inner == 0) return MI355_OK;
    if (!x || !out || !scale) return MI355_ERR_BAD_ARGUMENT;
    if (scale_len != 1 && scale_len != channels) return MI355_ERR_BAD_ARGUMENT;
    if (zero_point && zero_point_len != 1 && zero_point_len != channels) return MI355_ERR_BAD_ARGUMENT;
    if (zero_point && zero_point_dtype != MI355_DTYPE_FP32 && zero_point_dtype != MI355_DTYPE_INT32) return MI355_ERR_BAD_ARGUMENT;
    const int in_size = in_dtype == MI355_DTYPE_FP32 ? 4 : 2, out_size = out_dtype == MI355_Q_INT32 ? 4 : 1;
    if (!aligned(x, in_size) || !aligned(out, out_size) || !aligned(scale, 4) || (zero_point && !aligned(zero_point, 4)))
        return MI355_ERR_ALIGNMENT;
    // total elements must fit the index arithmetic
    if (outer > (int64_t)1 << 40 || channels > (int64_t)1 << 40 || inner > (int64_t)1 << 40) return MI355_ERR_UNSUPPORTED;
    const __int128 total128 = (__int128)outer * channels * inner;
    if (total128 > ((__int128)1 << 46)) return MI355_ERR_UNSUPPORTED;

    QzArgs p;
    p.x = x;
    p.scale = scale;
    p.zp = zero_point;
    p.zp_int = zero_point_dtype == MI355_DTYPE_INT32;
    p.out = out;
    p.total = (int64_t)total128;
    p.channels = channels;
    p.inner = inner;
    p.scale_one = scale_len == 1;
    p.zp_one = zero_point_len == 1;
    p.div_mode = div_mode != 0;
    p.qmin = out_dtype == MI355_Q_INT8 ? -128.0f : out_dtype == MI355_Q_UINT8 ? 0.0f : -2147483648.0f;
    p.qmax = out_dtype == MI355_Q_INT8 ? 127.0f : out_dtype == MI355_Q_UINT8 ? 255.0f : 2147483648.0f;
    // eight elements per thread when loads and stores are whole and aligned
    int vec_mode = 0;
    const bool single = p.scale_one && (!zero_point || p.zp_one);
    if (p.total % 8 == 0 && aligned(x, 16) && aligned(out, out_size == 4 ? 16 : 8)) {
        if (single || inner % 8 == 0) vec_mode = 1;
        else if (inner == 1 && channels % 8 == 0 && aligned(scale, 16) && (!zero_point || aligned(zero_point, 16))) vec_mode = 2;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (in_dtype == MI355_DTYPE_BF16) return launch_quantize_out<0>(p, out_dtype, vec_mode, s);
    if (in_dtype == MI355_DTYPE_FP16) return launch_quantize_out<1>(p, out_dtype, vec_mode, s);
    return launch_quantize_out<2>(p, out_dtype, vec_mode, s);
}
