// Packed int4 -> int8 for gfx950: the A4W4 operands of npu_quant_matmul arrive as int32 words of eight
// two's-complement nibbles (element i of a word in bits [4i, 4i+3]); gfx950 has no int4 matrix instruction, so the
// operands are widened to int8 once and the int8 GEMM runs on the result (the products and sums are the same
// integers).  Bandwidth-bound: a thread turns two words (8 bytes) into 16 bytes.
#include "common.h"

namespace mi355 {
namespace {

struct UnpackArgs {
    const uint32_t *x;
    int8_t *out;
    int64_t rows, words;    // words per row
    int64_t ldx, ldo;       // row pitch: input words, output bytes
};

// eight nibbles of `w` -> eight int8 in two words (elements 0..3, 4..7)
__device__ __forceinline__ u32x2 widen8(uint32_t w)
{
    // even elements in the bytes of e, odd ones in o; (v ^ 8) - 8 sign-extends a nibble, done on four bytes at once
    // (bit 7 set before the subtraction keeps borrows inside a byte)
    uint32_t e = (w & 0x0f0f0f0fu) ^ 0x08080808u, o = ((w >> 4) & 0x0f0f0f0fu) ^ 0x08080808u;
    e = ((e | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
    o = ((o | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
    u32x2 r;
    r.x = (e & 0xffu) | ((o & 0xffu) << 8) | ((e & 0xff00u) << 8) | ((o & 0xff00u) << 16);
    r.y = ((e >> 16) & 0xffu) | (((o >> 16) & 0xffu) << 8) | ((e >> 24) << 16) | ((o >> 24) << 24);
    return r;
}

// WPT words per thread: 2 (8-byte loads, 16-byte stores), 1 (8-byte stores) or 0 (one word, byte stores: any
// output alignment)
template <int WPT>
__global__ __launch_bounds__(256) void unpack_int4_kernel(const UnpackArgs p)
{
    constexpr int W = WPT ? WPT : 1;
    const int64_t per_row = p.words / W, total = p.rows * per_row;
    for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < total; u += (int64_t)gridDim.x * 256) {
        const int64_t r = u / per_row, c = (u % per_row) * W;
        const uint32_t *src = p.x + r * p.ldx + c;
        int8_t *dst = p.out + r * p.ldo + c * 8;
        if constexpr (WPT == 2) {
            const u32x2 w = *reinterpret_cast<const u32x2 *>(src);
            const u32x2 a = widen8(w.x), b = widen8(w.y);
            u32x4 o;
            o.x = a.x, o.y = a.y, o.z = b.x, o.w = b.y;
            *reinterpret_cast<u32x4 *>(dst) = o;
        } else if constexpr (WPT == 1) {
            *reinterpret_cast<u32x2 *>(dst) = widen8(*src);
        } else {
            const u32x2 a = widen8(*src);
#pragma unroll
            for (int i = 0; i < 4; i++) dst[i] = (int8_t)(a.x >> (8 * i)), dst[4 + i] = (int8_t)(a.y >> (8 * i));
        }
    }
}

} // namespace
} // namespace mi355

extern "C" int mi355_unpack_int4(const void *x, int8_t *out, int64_t rows, int64_t cols, int64_t ldx, int64_t ldo,
                                 void *stream)
{
    using namespace mi355;
    if (rows < 0 || cols < 0 || cols % 8 != 0) return MI355_ERR_BAD_ARGUMENT;
    if (rows == 0 || cols == 0) return MI355_OK;
    if (!x || !out || ldx < cols / 8 || ldo < cols) return MI355_ERR_BAD_ARGUMENT;
    if (!aligned(x, 4)) return MI355_ERR_ALIGNMENT;
    UnpackArgs p;
    p.x = static_cast<const uint32_t *>(x);
    p.out = out;
    p.rows = rows;
    p.words = cols / 8;
    p.ldx = ldx;
    p.ldo = ldo;
    const int wpt = (p.words % 2 == 0 && ldx % 2 == 0 && aligned(x, 8) && ldo % 16 == 0 && aligned(out, 16)) ? 2
                    : (ldo % 8 == 0 && aligned(out, 8)) ? 1 : 0;
    const int64_t units = rows * (p.words / (wpt ? wpt : 1));
    int64_t blocks = (units + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;               // grid-stride beyond a few waves per CU
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (wpt == 2) hipLaunchKernelGGL(unpack_int4_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, s, p);
    else if (wpt == 1) hipLaunchKernelGGL(unpack_int4_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, s, p);
    else hipLaunchKernelGGL(unpack_int4_kernel<0>, dim3((unsigned)blocks), dim3(256), 0, s, p);
    return check_launch();
}
