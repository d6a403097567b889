// npu_anti_quant for gfx950: out = cast((float(x) + offset) * scale) for int8 or packed-int4 x, float32 per-column
// (or single) scale / offset, float16 or bfloat16 output.  Bandwidth-bound elementwise kernel: a thread produces
// eight consecutive outputs of one row (8 bytes of int8 or one int32 word of nibbles in, 16 bytes out), each
// operation rounded separately in float32 as the golden formula does.
#include "common.h"

namespace mi355 {
namespace {

struct AqArgs {
    const void *x;
    const float *scale, *offset;   // [cols] or [1]; offset may be null
    uint16_t *out;
    int64_t rows, cols;            // output elements
    int64_t ldx;                   // input row pitch in input elements (int8 bytes or int32 words)
    int64_t ldo;
    int scale_one, offset_one;     // parameter has a single element
};

template <int OUT_F16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi)
{
    if constexpr (OUT_F16) return pack_f16x2(lo, hi);
    else return pack_bf16x2(lo, hi);
}

// The product must exist as a float32 before it is rounded to the output type (two roundings, as the golden
// formula has them); the empty asm keeps the compiler from merging multiply and conversion into one mixed-precision
// instruction that rounds once.
__device__ __forceinline__ float antiquant1(int v, float off, float sc)
{
    float f = ((float)v + off) * sc;
    asm volatile("" : "+v"(f));
    return f;
}

// cols % 8 == 0, 16-byte aligned output rows, 8-byte (int8) / 4-byte (int4 words) aligned input rows,
// 16-byte aligned per-column parameters.  A thread keeps the parameters of its eight columns in registers and walks
// down the rows (blockIdx.y strides over them, four rows in flight per step).
template <int BITS, int OUT_F16>
__global__ __launch_bounds__(256) void anti_quant_vec_kernel(const AqArgs p)
{
    const int64_t c = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (c >= p.cols) return;
    float sc[8], of[8];
    if (p.scale_one) {
#pragma unroll
        for (int i = 0; i < 8; i++) sc[i] = p.scale[0];
    } else {
        const f32x4 s0 = *reinterpret_cast<const f32x4 *>(p.scale + c), s1 = *reinterpret_cast<const f32x4 *>(p.scale + c + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) sc[i] = s0[i], sc[4 + i] = s1[i];
    }
    if (!p.offset) {
#pragma unroll
        for (int i = 0; i < 8; i++) of[i] = 0.0f;
    } else if (p.offset_one) {
#pragma unroll
        for (int i = 0; i < 8; i++) of[i] = p.offset[0];
    } else {
        const f32x4 o0 = *reinterpret_cast<const f32x4 *>(p.offset + c), o1 = *reinterpret_cast<const f32x4 *>(p.offset + c + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) of[i] = o0[i], of[4 + i] = o1[i];
    }
    constexpr int RU = 4;
    for (int64_t r0 = (int64_t)blockIdx.y * RU; r0 < p.rows; r0 += (int64_t)gridDim.y * RU) {
        u32x2 w[RU];
#pragma unroll
        for (int u = 0; u < RU; u++) {
            const int64_t r = min(r0 + u, p.rows - 1);
            if constexpr (BITS == 8) {
                w[u] = *reinterpret_cast<const u32x2 *>(static_cast<const int8_t *>(p.x) + r * p.ldx + c);
            } else {
                w[u].x = static_cast<const uint32_t *>(p.x)[r * p.ldx + c / 8];
                w[u].y = 0;
            }
        }
#pragma unroll
        for (int u = 0; u < RU; u++) {
            if (r0 + u >= p.rows) break;
            int v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if constexpr (BITS == 8) v[i] = (int)(int8_t)((i < 4 ? w[u].x >> (8 * i) : w[u].y >> (8 * (i - 4))) & 0xffu);
                else v[i] = (int)(((w[u].x >> (4 * i)) & 0xfu) ^ 8u) - 8;           // nibble i, two's complement
            }
            u32x4 o;
            o.x = pack2<OUT_F16>(antiquant1(v[0], of[0], sc[0]), antiquant1(v[1], of[1], sc[1]));
            o.y = pack2<OUT_F16>(antiquant1(v[2], of[2], sc[2]), antiquant1(v[3], of[3], sc[3]));
            o.z = pack2<OUT_F16>(antiquant1(v[4], of[4], sc[4]), antiquant1(v[5], of[5], sc[5]));
            o.w = pack2<OUT_F16>(antiquant1(v[6], of[6], sc[6]), antiquant1(v[7], of[7], sc[7]));
            __builtin_nontemporal_store(o, reinterpret_cast<u32x4 *>(p.out + (r0 + u) * p.ldo + c));
        }
    }
}

// any shape and alignment: one output element per thread
template <int BITS, int OUT_F16>
__global__ __launch_bounds__(256) void anti_quant_scalar_kernel(const AqArgs p)
{
    const int64_t total = p.rows * p.cols;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
        const int64_t r = e / p.cols, c = e % p.cols;
        int v;
        if constexpr (BITS == 8) {
            v = static_cast<const int8_t *>(p.x)[r * p.ldx + c];
        } else {
            const uint32_t w = static_cast<const uint32_t *>(p.x)[r * p.ldx + c / 8];
            v = (int)(((w >> (4 * (c & 7))) & 0xfu) ^ 8u) - 8;
        }
        const float sc = p.scale[p.scale_one ? 0 : c];
        const float of = p.offset ? p.offset[p.offset_one ? 0 : c] : 0.0f;
        p.out[r * p.ldo + c] = (uint16_t)pack2<OUT_F16>(antiquant1(v, of, sc), 0.0f);
    }
}

template <int BITS, int OUT_F16>
int launch_anti_quant(const AqArgs &p, bool vec, hipStream_t s)
{
    if (vec) {
        const int64_t bx = (p.cols / 8 + 255) / 256;
        int64_t by = (p.rows + 3) / 4;                         // four rows per step of a block
        const int64_t cap = (256 * 16 + bx - 1) / bx;          // enough blocks to fill the chip several times over
        if (by > cap) by = cap;
        if (bx > 0x7fffffff) return MI355_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((anti_quant_vec_kernel<BITS, OUT_F16>), dim3((unsigned)bx, (unsigned)by), dim3(256), 0, s, p);
    } else {
        int64_t blocks = (p.rows * p.cols + 255) / 256;
        if (blocks > 256 * 32) blocks = 256 * 32;
        hipLaunchKernelGGL((anti_quant_scalar_kernel<BITS, OUT_F16>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    }
    return check_launch();
}

} // namespace
} // namespace mi355

extern "C" int mi355_anti_quant(const void *x, int x_bits, const float *scale, int64_t scale_len, const float *offset,
                                int64_t offset_len, void *out, int out_dtype, int64_t rows, int64_t cols, int64_t ldx,
                                int64_t ldo, void *stream)
{
    using namespace mi355;
    if (rows < 0 || cols < 0) return MI355_ERR_BAD_ARGUMENT;
    if (x_bits != 8 && x_bits != 4) return MI355_ERR_BAD_ARGUMENT;
    if (out_dtype != MI355_DTYPE_BF16 && out_dtype != MI355_DTYPE_FP16) return MI355_ERR_BAD_ARGUMENT;
    if (rows == 0 || cols == 0) return MI355_OK;
    if (!x || !scale || !out) return MI355_ERR_BAD_ARGUMENT;
    if (x_bits == 4 && cols % 8 != 0) return MI355_ERR_BAD_ARGUMENT;
    if ((scale_len != 1 && scale_len != cols) || (offset && offset_len != 1 && offset_len != cols)) return MI355_ERR_BAD_ARGUMENT;
    if (ldo < cols || ldx < (x_bits == 4 ? cols / 8 : cols)) return MI355_ERR_BAD_ARGUMENT;
    if (!aligned(scale, 4) || (offset && !aligned(offset, 4)) || !aligned(out, 2) || (x_bits == 4 && !aligned(x, 4)))
        return MI355_ERR_ALIGNMENT;
    AqArgs p;
    p.x = x;
    p.scale = scale;
    p.offset = offset;
    p.out = static_cast<uint16_t *>(out);
    p.rows = rows;
    p.cols = cols;
    p.ldx = ldx;
    p.ldo = ldo;
    p.scale_one = scale_len == 1;
    p.offset_one = offset_len == 1;
    const bool vec = cols % 8 == 0 && ldo % 8 == 0 && aligned(out, 16) && (x_bits == 4 || (ldx % 8 == 0 && aligned(x, 8))) &&
                     (p.scale_one || aligned(scale, 16)) && (!offset || p.offset_one || aligned(offset, 16));
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool f16 = out_dtype == MI355_DTYPE_FP16;
    if (x_bits == 8) return f16 ? launch_anti_quant<8, 1>(p, vec, s) : launch_anti_quant<8, 0>(p, vec, s);
    return f16 ? launch_anti_quant<4, 1>(p, vec, s) : launch_anti_quant<4, 0>(p, vec, s);
}
