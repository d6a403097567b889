// Device helpers shared by the npu_weight_quant_batchmatmul kernels: 16-bit activation encodings, the exact
// integer weight images and their expansion, buffer descriptors and wait counters.
#pragma once
#include "common.h"
#include <stdlib.h>

namespace mi355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) void lds_void;

constexpr int kNumCU = 256;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding: vmcnt in bits 3:0 and 15:14).
template <int VM>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(VM >= 0 && VM < 64, "vmcnt range");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(VM) : "memory");
}

__device__ __forceinline__ void wait_lgkmcnt0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// B fragments of the two MFMAs that share byte position jb of the dword (int4) / of MFMA #i (int8).
// w holds this lane's dword from its 8 k rows; fragment VGPR v pairs rows (2v, 2v+1).
// Activation / scale / output element type: ACT = 0 bfloat16, 1 float16.  Everything below is the same for both
// except the 16-bit encodings: conversions, the MFMA variant and the bit positions of the int4 image.
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

template <int ACT>
__device__ __forceinline__ float act_lo(uint32_t u)
{
    if constexpr (ACT == 0) return bf16_lo(u);
    else return (float)__builtin_bit_cast(_Float16, (uint16_t)(u & 0xffffu));
}
template <int ACT>
__device__ __forceinline__ float act_hi(uint32_t u)
{
    if constexpr (ACT == 0) return bf16_hi(u);
    else return (float)__builtin_bit_cast(_Float16, (uint16_t)(u >> 16));
}
template <int ACT>
__device__ __forceinline__ float act_1(uint16_t h)
{
    if constexpr (ACT == 0) return bf16_1(h);
    else return (float)__builtin_bit_cast(_Float16, h);
}
template <int ACT>
__device__ __forceinline__ uint32_t pack_act2(float lo, float hi)
{
    if constexpr (ACT == 0) return pack_bf16x2(lo, hi);
    else return pack_f16x2(lo, hi);
}
template <int ACT>
__device__ __forceinline__ f32x4 mfma_act(u32x4 a, u32x4 b, f32x4 c)
{
    if constexpr (ACT == 0)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}
template <int ACT>
constexpr uint32_t kOnes2 = ACT == 0 ? 0x3f803f80u : 0x3c003c00u;      // two ones
// int4 image: the nibble u = w + 8 goes into the top four mantissa bits of 8.0 (bf16: 8 + u/2 = (w + 24) / 2) or of
// 16.0 (fp16: 16 + u = w + 24)
template <int ACT>
constexpr uint32_t kInt4Magic = ACT == 0 ? 0x41004100u : 0x4c004c00u;
template <int WBITS, int ACT>
constexpr float kImageMul = (WBITS == 4 && ACT == 0) ? 2.0f : 1.0f;    // weight = kImageMul * image - kImageBias
template <int WBITS>
constexpr float kImageBias = WBITS == 4 ? 24.0f : 128.0f;

template <int WBITS, int ACT>
__device__ __forceinline__ void expand_pair(const uint32_t (&w)[8], int jb, uint32_t magic, u32x4 &b0, u32x4 &b1)
{
    if constexpr (WBITS == 4) {
        // `magic` (kInt4Magic) lives in a VGPR so that (x & mask) | magic is one v_and_or_b32 (mask from an SGPR)
        const uint32_t sel = 0x0c000c00u | ((4u + jb) << 16) | (uint32_t)jb;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const uint32_t t = __builtin_amdgcn_perm(w[2 * v + 1], w[2 * v], sel); // [byte jb of row 2v, 0, byte jb of row 2v+1, 0]
            if constexpr (ACT == 0) {
                b0[v] = ((t << 3) & 0x00780078u) | magic;                          // low nibble  -> element 2*jb
                b1[v] = ((t >> 1) & 0x00780078u) | magic;                          // high nibble -> element 2*jb+1
            } else {
                b0[v] = ((t << 6) & 0x03c003c0u) | magic;
                b1[v] = ((t << 2) & 0x03c003c0u) | magic;
            }
        }
    } else {
        (void)magic;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            b0[v] = pack_act2<ACT>((float)((w[2 * v] >> (16 * jb)) & 0xffu), (float)((w[2 * v + 1] >> (16 * jb)) & 0xffu));
            b1[v] = pack_act2<ACT>((float)((w[2 * v] >> (16 * jb + 8)) & 0xffu),
                                (float)((w[2 * v + 1] >> (16 * jb + 8)) & 0xffu));
        }
    }
}

constexpr uint32_t kOutOfRange = 0x80000000u;   // lane offset beyond every buffer size: the load returns zero, no traffic
constexpr int kNonTemporal = 2;                 // cache-policy bit for data that is read once

inline int env_int(const char *name)
{
    const char *e = getenv(name);
    return e ? atoi(e) : 0;
}

} // namespace
} // namespace mi355
