// npu_swiglu for gfx950 (last dimension): out = silu(a) * b with a, b the two halves of a row.
// Bandwidth-bound elementwise kernel; bf16 arithmetic as eager bf16 tensor ops evaluate it:
// s = bf16(a / (1 + exp(-a))) in float32, out = bf16(float(s) * float(b)).
#include "common.h"

namespace mi355 {
namespace {

// vectorised: half % 8 == 0, 16-byte aligned rows
__global__ __launch_bounds__(256) void swiglu_vec_kernel(const uint16_t *__restrict__ x, uint16_t *__restrict__ out,
                                                         int64_t rows, int half_vec, int64_t ldx)
{
    const int64_t total = rows * half_vec;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
        const int64_t r = e / half_vec;
        const int v = (int)(e % half_vec);
        const u32x4 *a = reinterpret_cast<const u32x4 *>(x + r * ldx) + v;
        const u32x4 av = __builtin_nontemporal_load(a), bv = __builtin_nontemporal_load(a + half_vec);
        u32x4 o;
        o.x = swiglu2(av.x, bv.x);
        o.y = swiglu2(av.y, bv.y);
        o.z = swiglu2(av.z, bv.z);
        o.w = swiglu2(av.w, bv.w);
        __builtin_nontemporal_store(o, reinterpret_cast<u32x4 *>(out) + e);
    }
}

__global__ __launch_bounds__(256) void swiglu_scalar_kernel(const uint16_t *__restrict__ x, uint16_t *__restrict__ out,
                                                            int64_t rows, int64_t half, int64_t ldx)
{
    const int64_t total = rows * half;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
        const int64_t r = e / half, j = e % half;
        const float a = bf16_1(x[r * ldx + j]), b = bf16_1(x[r * ldx + half + j]);
        const float s = silu_bf16(a);
        out[e] = f32_to_bf16(s * b);
    }
}

} // namespace
} // namespace mi355

extern "C" int mi355_swiglu(const void *x_bf16, void *out_bf16, int64_t rows, int64_t half, int64_t ldx, void *stream)
{
    using namespace mi355;
    if (rows < 0 || half < 0) return MI355_ERR_BAD_ARGUMENT;
    if (rows == 0 || half == 0) return MI355_OK;
    if (!x_bf16 || !out_bf16 || ldx < 2 * half) return MI355_ERR_BAD_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint16_t *x = static_cast<const uint16_t *>(x_bf16);
    uint16_t *o = static_cast<uint16_t *>(out_bf16);
    const bool vec = half % 8 == 0 && ldx % 8 == 0 && aligned(x, 16) && aligned(o, 16);
    const int64_t work = vec ? rows * (half / 8) : rows * half;
    int64_t blocks = (work + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    if (vec)
        hipLaunchKernelGGL(swiglu_vec_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, o, rows, (int)(half / 8), ldx);
    else
        hipLaunchKernelGGL(swiglu_scalar_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, o, rows, half, ldx);
    return check_launch();
}

extern "C" const char *mi355_status_string(int status)
{
    switch (status) {
    case MI355_OK: return "ok";
    case MI355_ERR_BAD_ARGUMENT: return "bad argument (null pointer, negative size or invalid enum)";
    case MI355_ERR_UNSUPPORTED: return "request outside what the gfx950 kernels implement";
    case MI355_ERR_ALIGNMENT: return "pointer or stride alignment not supported";
    case MI355_ERR_WORKSPACE: return "workspace missing or too small";
    case MI355_ERR_LAUNCH: return "kernel launch failed";
    case MI355_ERR_DEVICE: return "a kernel reported a failure through the workspace status word (a bounded wait for partial sums ran out)";
    default: return "unknown status";
    }
}

extern "C" int mi355_quant_abi_version(void) { return 3001; }
