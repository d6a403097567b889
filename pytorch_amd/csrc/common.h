// Shared device/host helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include "../../include/mi355_quant.h"

namespace mi355 {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// 16-byte buffer store.  The store reads its data registers a few cycles after it issues, and the compiler keeps the wait
// states this needs only for stores whose scalar offset is an immediate: with the offset in a register, an instruction that
// reuses the data registers may follow at once (seen: a lane group's last word replaced by the next value written to the
// register, on launches in which the store unit was slow).  The empty wait below has the data as an operand, so the
// registers stay allocated until two wait states have passed.
template <int AUX>
__device__ __forceinline__ void buffer_store_b128(u32x4 data, __amdgpu_buffer_rsrc_t rsrc, uint32_t lane_offset, uint32_t scalar_offset)
{
    __builtin_amdgcn_raw_buffer_store_b128(data, rsrc, lane_offset, scalar_offset, AUX);
    asm volatile("s_nop 1" ::"v"(data) : "memory");
}

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
__device__ __forceinline__ float bf16_1(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// float32 -> bf16, round to nearest even (hardware v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint16_t f32_to_bf16(float f)
{
    __bf16 b = (__bf16)f;
    return __builtin_bit_cast(uint16_t, b);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    bf2 v;
    v[0] = (__bf16)lo;
    v[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, v);
}

// low bytes of a, b, c, d -> one dword (a lowest)
__device__ __forceinline__ uint32_t pack4(uint32_t a, uint32_t b, uint32_t c, uint32_t d)
{
    uint32_t ab = __builtin_amdgcn_perm(b, a, 0x0c0c0400u);
    uint32_t cd = __builtin_amdgcn_perm(d, c, 0x0c0c0400u);
    return __builtin_amdgcn_perm(cd, ab, 0x05040100u);
}

// SwiGLU on two packed bf16 pairs the way eager bf16 tensor ops evaluate it: s = bf16(a / (1 + exp(-a))) in
// float32, result = bf16(float(s) * float(b)).
__device__ __forceinline__ float silu_f32(float a) { return a / (1.0f + expf(-a)); }

// bf16(silu(a)) for an `a` that is itself a bf16 value, returned as a float.  Exponential and division through the
// hardware's exp2 and reciprocal are a few units in the last place of binary32 off, which changes the bf16 result only
// when the value lies next to a rounding boundary of bf16: those (lower 16 bits within 16 of 0x8000: one value in 2048),
// arguments beyond +-80 (where the exponential or the reciprocal leaves the normal range) and NaN take the exact formula.
// log2(e) is split into a head of 16 significant bits, whose product with the 8 significant bits of `a` is exact, and a
// tail applied to the exponential as a factor 1 + a * tail * ln(2): the rounding of a * log2(e) would otherwise grow
// with |a| (2^-18 of the result at a = -60) and send every argument below -8 - common among real gate activations - to
// the exact formula.  There are only 65536 arguments: tests compare all of them with the exact formula and with the oracle.
__device__ __forceinline__ float silu_bf16(float a)
{
    const float e0 = __builtin_amdgcn_exp2f(a * -1.44268798828125f);                  // head: 0x3fb8aa00
    const float e = __builtin_fmaf(e0, a * -4.888495152129525e-06f, e0);              // tail 7.0526077e-06 * ln(2)
    float s = a * __builtin_amdgcn_rcpf(1.0f + e);
    const uint32_t lo = __float_as_uint(s) & 0xffffu;
    if (__builtin_expect((lo - 0x7ff0u) < 0x20u || !(fabsf(a) <= 80.0f), 0)) s = silu_f32(a);
    return bf16_1(f32_to_bf16(s));
}

__device__ __forceinline__ uint32_t swiglu2(uint32_t a2, uint32_t b2)
{
    const float s0 = silu_bf16(bf16_lo(a2));
    const float s1 = silu_bf16(bf16_hi(a2));
    return pack_bf16x2(s0 * bf16_lo(b2), s1 * bf16_hi(b2));
}

// Per-expert smooth scales (npu_dynamic_quant with group_index): `group_index` holds the running totals of the rows of
// each expert, so row r belongs to the first expert e with r < group_index[e] (rows past the last total take the last
// expert); returns the first element of that expert's scales.
__device__ __forceinline__ const uint16_t *expert_scales(const uint16_t *smooth, const int32_t *group_index, int groups, int64_t row,
                                                         int64_t cols)
{
    if (!group_index) return smooth;
    int e = 0;
    while (e < groups - 1 && row >= (int64_t)group_index[e]) e++;
    return smooth + (int64_t)e * cols;
}

// Every workspace of this library starts with a zero area: kWorkspaceCounterCapacity bytes of arrival counters followed
// by kWorkspaceZoneBytes for exchanges that recognise data by its being non-zero (weight_quant_decode.hip).  The area
// is zero before the first launch and every launch leaves it zero; whatever else a launch keeps in the workspace
// (split-K partial sums, a transposed weight) lies behind it and needs no initialisation, so one zero-initialised
// buffer can be shared by all launches of a stream.
constexpr size_t kWorkspaceCounterCapacity = 16384;
// The last 16 bytes of the counter part are not counters: the first word of them is the workspace's sticky status word
// (MI355_WORKSPACE_STATUS_OFFSET).  A kernel whose bounded wait for another workgroup's partial sums ran out stores a
// non-zero code there (and NaNs where its sums should be); mi355_workspace_status() reads and clears it.
constexpr size_t kWorkspaceStatusOffset = kWorkspaceCounterCapacity - 16;
constexpr size_t kWorkspaceCounterBytes = kWorkspaceStatusOffset;      // what planners may fill with arrival counters
constexpr uint32_t kStatusExchangeTimeout = 1;
constexpr size_t kWorkspaceZoneBytes = (size_t)16 << 20;
constexpr size_t kWorkspaceZeroBytes = kWorkspaceCounterCapacity + kWorkspaceZoneBytes;

__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi)
{
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 v;
    v[0] = (_Float16)lo;        // round to nearest even
    v[1] = (_Float16)hi;
    return __builtin_bit_cast(uint32_t, v);
}

// Planner tuning knobs (tuning.hip): 0 = automatic.  Read with knob(); set through mi355_set_tuning() or, once at
// load time, through the environment variable of the same name.
// MI355_WQ_GEMM4_OFF / MI355_WQ_DECODE_OFF: 1 = the register-expanding int4 GEMM / the int4 decode kernel is not used;
// 2 = its K-split exchange always writes through to memory.
// MI355_QMM_DECODE_OFF: 1 = quant_matmul with at most 64 rows takes the tiled kernel instead of the decode kernel.
// MI355_WQ_MAX_POLLS: bound of the int4 kernels' wait for the other workgroups' partial sums (0 = 2^20 polls);
// MI355_WQ_ONLY_CHUNK: c + 1 = only the workgroups of K chunk c do anything, -1 = only the collecting chunk (with a small MI355_WQ_MAX_POLLS this drives
// a collector into its give-up path from the host, every kernel still ending normally: tests of the error reporting).
enum Knob { kKnobWqSplit, kKnobWqW, kKnobWqgSplit, kKnobWqgBm, kKnobWqGemmOff, kKnobWqkMt, kKnobWqkNw, kKnobWqkKs,
            kKnobQmmSplit, kKnobQmmTile /* bm * 1000 + bn */, kKnobWqDecodeOff, kKnobQmmDeepOff, kKnobWqGemm4Off, kKnobQmmDecodeOff,
            kKnobQmmLoop, kKnobWqMaxPolls, kKnobWqOnlyChunk, kKnobQmmStreamOut, kKnobCount };
int knob(Knob k);

inline int check_launch()
{
    return hipGetLastError() == hipSuccess ? MI355_OK : MI355_ERR_LAUNCH;
}

__device__ __forceinline__ bool aligned_dev(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

} // namespace mi355
