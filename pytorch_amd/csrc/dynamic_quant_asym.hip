// npu_dynamic_quant_asymmetric for gfx950: per-token asymmetric int8 quantisation,
//     scale = (row_max - row_min) / 255,   offset = 127 - row_max / scale,   y = rint_half_even(x / scale + offset)
// with every operation a separately rounded IEEE binary32 operation (the compile flags keep multiply-adds apart).
// A row whose elements are all equal has scale 0, offset 0 and y 0.
//
// One 256-thread block per row, two passes over the row: the first reduces the minimum and the maximum, the second
// divides, adds the offset and stores packed int8; rows of up to 8192 elements stay in registers between the passes,
// longer ones are re-read (they are in cache by then: HBM sees them once).
// The division is IEEE-correct (about a dozen instructions per element), which at [2048, 4096] costs about as much
// as the memory traffic.
#include "common.h"
#include <math.h>

namespace mi355 {
namespace {

template <bool FP16>
__device__ __forceinline__ float to_f32(uint16_t h)
{
    if constexpr (FP16) return (float)__builtin_bit_cast(_Float16, h);
    else return bf16_1(h);
}

__device__ __forceinline__ uint32_t finish1(float q, float offset)
{
    q = q + offset;
    q = __builtin_rintf(q);
    q = q > 127.0f ? 127.0f : q;
    q = q < -128.0f ? -128.0f : q;
    return (uint32_t)(int)q & 0xffu;
}

__device__ __forceinline__ uint32_t quant1(float x, float scale, float offset) { return finish1(x / scale, offset); }

// x / scale through the row's refined reciprocal `r`: the operation sequence of the compiler's own float32 division
// (quotient, two residual corrections with fused multiply-adds) without its range scaling and special-case fix-up.
// Those are the identity when the scale lies within [2^-60, 2^60] and no element of the row exceeds 2^60 (nothing
// overflows; a numerator small enough for a residual to leave the normal range has a quotient below 2^-40, which the
// offset absorbs or which rounds to zero either way; NaN becomes code 0 on both paths).  Rows outside that range
// divide the ordinary way; the choice is the same for a whole row.
__device__ __forceinline__ uint32_t quant1_rcp(float x, float scale, float r, float offset)
{
    float q = x * r;
    q = __builtin_fmaf(__builtin_fmaf(-scale, q, x), r, q);
    q = __builtin_fmaf(__builtin_fmaf(-scale, q, x), r, q);
    return finish1(q, offset);
}

// The same for a row without a NaN: rounding by the addition of 1.5 * 2^23 (ties to even in the adder; the integer is then
// the distance of the bit pattern from that constant's), clamped as an integer.  Sums beyond the range in which the
// addition rounds to an integer leave a pattern that is far above or below the constant's on the same side, so the clamp
// gives what clamping the rounded sum gives; a NaN would clamp to 127 instead of becoming 0, which is why rows with one
// keep to quant1_rcp.
__device__ __forceinline__ uint32_t quant1_rcp_nonan(float x, float scale, float r, float offset)
{
    float q = x * r;
    q = __builtin_fmaf(__builtin_fmaf(-scale, q, x), r, q);
    q = __builtin_fmaf(__builtin_fmaf(-scale, q, x), r, q);
    const float t = (q + offset) + 12582912.0f;
    const int k = (int)__float_as_uint(t) - 0x4b400000;
    return (uint32_t)min(max(k, -128), 127);
}

// VEC: cols % 8 == 0, rows (and smooth) 16-byte aligned, y rows 8-byte aligned
// REG (with VEC): cols <= 8192, the row stays in registers between the two passes (four 16-byte vectors per thread)
template <bool FP16, bool VEC, bool REG = false>
__global__ __launch_bounds__(256) void dq_asym_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ smooth,
                                                      int8_t *__restrict__ y, float *__restrict__ scale_out,
                                                      float *__restrict__ offset_out, int64_t rows, int cols, int64_t row_stride,
                                                      const int32_t *__restrict__ group_index = nullptr, int groups = 0)
{
    __shared__ float red[2][4];
    const int t = threadIdx.x;
    const uint16_t *const smooth_all = smooth;
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        if (smooth_all) smooth = expert_scales(smooth_all, group_index, groups, row, cols);   // per-expert scales: this row's vector
        const uint16_t *xr = x + row * row_stride;
        int8_t *yr = y + row * (int64_t)cols;
        float mx = -INFINITY, mn = INFINITY;
        bool has_nan = false;                             // maximum and minimum skip a NaN: noted apart
        u32x4 kept[REG ? 4 : 1];
        if constexpr (REG) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int v = t + 256 * i;
                kept[i] = v < cols / 8 ? __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(xr) + v) : u32x4{0, 0, 0, 0};
            }
        }
        if constexpr (VEC) {
            for (int v = t, it = 0; v < cols / 8; v += 256, it++) {
                u32x4 a;
                if constexpr (REG) a = it == 0 ? kept[0] : it == 1 ? kept[1] : it == 2 ? kept[2] : kept[3];
                else a = reinterpret_cast<const u32x4 *>(xr)[v];
                u32x4 s = u32x4{0, 0, 0, 0};
                if (smooth) s = reinterpret_cast<const u32x4 *>(smooth)[v];
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    float f = to_f32<FP16>((uint16_t)(a[i / 2] >> (16 * (i & 1))));
                    if (smooth) f = f * to_f32<FP16>((uint16_t)(s[i / 2] >> (16 * (i & 1))));
                    mx = fmaxf(mx, f);
                    mn = fminf(mn, f);
                    has_nan = has_nan || f != f;
                }
            }
        } else {
            for (int j = t; j < cols; j += 256) {
                float f = to_f32<FP16>(xr[j]);
                if (smooth) f = f * to_f32<FP16>(smooth[j]);
                mx = fmaxf(mx, f);
                mn = fminf(mn, f);
            }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            mx = fmaxf(mx, __shfl_xor(mx, off, 64));
            mn = fminf(mn, __shfl_xor(mn, off, 64));
        }
        __syncthreads();                                  // the previous row's readers are done with `red`
        if ((t & 63) == 0) red[0][t >> 6] = mx, red[1][t >> 6] = mn;
        __syncthreads();
        mx = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
        mn = fminf(fminf(red[1][0], red[1][1]), fminf(red[1][2], red[1][3]));
        float scale = (mx - mn) / 255.0f;
        float offset = 127.0f - mx / scale;
        const bool flat = !(mx > mn);                     // all elements equal (or no finite ordering): zeros
        if (flat) scale = 0.0f, offset = 0.0f;
        if (t == 0) scale_out[row] = scale, offset_out[row] = offset;
        float rcp = __builtin_amdgcn_rcpf(scale);
        rcp = __builtin_fmaf(__builtin_fmaf(-scale, rcp, 1.0f), rcp, rcp);
        const bool fast = __builtin_amdgcn_readfirstlane(
                              (int)(scale >= 0x1p-60f && scale <= 0x1p60f && fmaxf(fabsf(mx), fabsf(mn)) <= 0x1p60f)) != 0;
        const bool no_nan = __builtin_amdgcn_ballot_w64(has_nan) == 0;          // for this wavefront's elements
        if constexpr (VEC) {
            for (int v = t, it = 0; v < cols / 8; v += 256, it++) {
                u32x4 a;
                if constexpr (REG) a = it == 0 ? kept[0] : it == 1 ? kept[1] : it == 2 ? kept[2] : kept[3];
                else a = reinterpret_cast<const u32x4 *>(xr)[v];
                u32x4 s = u32x4{0, 0, 0, 0};
                if (smooth) s = reinterpret_cast<const u32x4 *>(smooth)[v];
                uint32_t q[8];
                float f8[8];
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    f8[i] = to_f32<FP16>((uint16_t)(a[i / 2] >> (16 * (i & 1))));
                    if (smooth) f8[i] = f8[i] * to_f32<FP16>((uint16_t)(s[i / 2] >> (16 * (i & 1))));
                }
                if (flat) {
#pragma unroll
                    for (int i = 0; i < 8; i++) q[i] = 0u;
                } else if (fast && no_nan) {                  // one branch: never both divisions
#pragma unroll
                    for (int i = 0; i < 8; i++) q[i] = quant1_rcp_nonan(f8[i], scale, rcp, offset);
                } else if (fast) {
#pragma unroll
                    for (int i = 0; i < 8; i++) q[i] = quant1_rcp(f8[i], scale, rcp, offset);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; i++) q[i] = quant1(f8[i], scale, offset);
                }
                u32x2 o;
                o.x = pack4(q[0], q[1], q[2], q[3]);
                o.y = pack4(q[4], q[5], q[6], q[7]);
                __builtin_nontemporal_store(o, reinterpret_cast<u32x2 *>(yr) + v);
            }
        } else {
            for (int j = t; j < cols; j += 256) {
                float f = to_f32<FP16>(xr[j]);
                if (smooth) f = f * to_f32<FP16>(smooth[j]);
                yr[j] = (int8_t)(flat ? 0u : fast ? quant1_rcp(f, scale, rcp, offset) : quant1(f, scale, offset));
            }
        }
    }
}

} // namespace
} // namespace mi355

extern "C" int mi355_dynamic_quant_asymmetric(const void *x, int in_dtype, const void *smooth, int8_t *y, float *scale,
                                              float *offset, int64_t rows, int64_t cols, int64_t x_row_stride, void *stream)
{
    return mi355_dynamic_quant_asymmetric_grouped(x, in_dtype, smooth, nullptr, 0, y, scale, offset, rows, cols, x_row_stride, stream);
}

extern "C" int mi355_dynamic_quant_asymmetric_grouped(const void *x, int in_dtype, const void *smooth, const int32_t *group_index,
                                                      int64_t groups, int8_t *y, float *scale, float *offset, int64_t rows,
                                                      int64_t cols, int64_t x_row_stride, void *stream)
{
    using namespace mi355;
    if (rows < 0 || cols < 0) return MI355_ERR_BAD_ARGUMENT;
    if (group_index && (!smooth || groups < 1 || groups > 0x7fffffff)) return MI355_ERR_BAD_ARGUMENT;
    if (group_index && !aligned(group_index, 4)) return MI355_ERR_ALIGNMENT;
    const int ng = group_index ? (int)groups : 0;
    if (in_dtype != MI355_DTYPE_BF16 && in_dtype != MI355_DTYPE_FP16) return MI355_ERR_BAD_ARGUMENT;
    if (rows == 0) return MI355_OK;
    if (!scale || !offset) return MI355_ERR_BAD_ARGUMENT;
    if (cols > 0 && (!x || !y || x_row_stride < cols)) return MI355_ERR_BAD_ARGUMENT;
    if (cols > 0x7fffffff) return MI355_ERR_UNSUPPORTED;
    if (!aligned(x, 2) || (smooth && !aligned(smooth, 2)) || !aligned(scale, 4) || !aligned(offset, 4)) return MI355_ERR_ALIGNMENT;
    const bool vec = cols % 8 == 0 && x_row_stride % 8 == 0 && aligned(x, 16) && (!smooth || aligned(smooth, 16)) && aligned(y, 8);
    const uint16_t *xp = static_cast<const uint16_t *>(x), *sp = static_cast<const uint16_t *>(smooth);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned blocks = (unsigned)(rows < 256 * 64 ? rows : 256 * 64);
    const bool f16 = in_dtype == MI355_DTYPE_FP16;
#define MI355_DQA_LAUNCH(F, V, R) \
    hipLaunchKernelGGL((dq_asym_kernel<F, V, R>), dim3(blocks), dim3(256), 0, s, xp, sp, y, scale, offset, rows, (int)cols, x_row_stride, \
                       group_index, ng)
    const bool reg = vec && cols <= 8192;
    if (f16 && reg) MI355_DQA_LAUNCH(true, true, true);
    else if (f16 && vec) MI355_DQA_LAUNCH(true, true, false);
    else if (f16) MI355_DQA_LAUNCH(true, false, false);
    else if (reg) MI355_DQA_LAUNCH(false, true, true);
    else if (vec) MI355_DQA_LAUNCH(false, true, false);
    else MI355_DQA_LAUNCH(false, false, false);
#undef MI355_DQA_LAUNCH
    return check_launch();
}
