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
// int8 image: the weight itself (every integer up to 256 is a bf16 / fp16 number).  Byte i of a word is converted with its
// sign in one instruction (v_cvt_f32_i32 with a sign-extending byte select), so no bias has to be removed afterwards: an
// image w + 128 made the sum of products 128 X + sum(x w) and its float32 rounding, 2^-24 of 128 X, the error floor of
// small outputs.
template <int WBITS>
constexpr float kImageBias = WBITS == 4 ? 24.0f : 0.0f;
__device__ __forceinline__ float sbyte_f32(uint32_t w, int i) { return (float)(int8_t)((w >> (8 * i)) & 0xffu); }

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
            b0[v] = pack_act2<ACT>(sbyte_f32(w[2 * v], 2 * jb), sbyte_f32(w[2 * v + 1], 2 * jb));
            b1[v] = pack_act2<ACT>(sbyte_f32(w[2 * v], 2 * jb + 1), sbyte_f32(w[2 * v + 1], 2 * jb + 1));
        }
    }
}

// Second expansion of int4 bytes, one instruction shorter per fragment register and without the separate sign flip.
// t = [byte of row 2v, 0, byte of row 2v + 1, 0] straight from the packed words.  out = mask ? (t ^ c) : c is a single
// three-input bitwise instruction: c carries the image's exponent bits outside the mask and, inside it, the bit that
// turns the two's-complement nibble into u = w + 8.  bf16: the low nibble stays where it is, as the low mantissa bits
// of 128.0 (image 128 + u), the high nibble moves down one bit into the top mantissa bits of 8.0 (image 8 + u / 2);
// fp16: both go to the top mantissa bits of 16.0 (image 16 + u).  weight = mul * image - bias per nibble position.
__device__ __forceinline__ uint32_t bit_blend(uint32_t t, uint32_t mask, uint32_t c)
{
    return __builtin_amdgcn_bitop3_b32(t, mask, c, 0x6a);   // truth table of (mask & (t ^ c)) | (~mask & c), t the high index bit
}
template <int ACT>
__device__ __forceinline__ void expand_byte(uint32_t t, uint32_t mask_lo, uint32_t c_lo, uint32_t mask_hi, uint32_t c_hi, uint32_t &lo, uint32_t &hi)
{
    if constexpr (ACT == 0) {
        lo = bit_blend(t, mask_lo, c_lo);
        hi = bit_blend(t >> 1, mask_hi, c_hi);
    } else {
        lo = bit_blend(t << 6, mask_hi, c_hi);
        hi = bit_blend(t << 2, mask_hi, c_hi);
    }
}
template <int ACT> constexpr uint32_t kMaskLo4 = 0x000f000fu;
template <int ACT> constexpr uint32_t kBlendLo4 = 0x43004300u | 0x00080008u;
template <int ACT> constexpr uint32_t kMaskHi4 = ACT == 0 ? 0x00780078u : 0x03c003c0u;
template <int ACT> constexpr uint32_t kBlendHi4 = ACT == 0 ? (0x41004100u | 0x00400040u) : (0x4c004c00u | 0x02000200u);
template <int ACT> constexpr float kMulLo4 = 1.0f;
template <int ACT> constexpr float kBiasLo4 = ACT == 0 ? 136.0f : 24.0f;
template <int ACT> constexpr float kMulHi4 = kImageMul<4, ACT>;
template <int ACT> constexpr float kBiasHi4 = kImageBias<4>;
// the blend operands, opaque to the optimiser (which would otherwise split the blend into two instructions again)
struct BlendRegs {
    uint32_t mask_lo, c_lo, mask_hi, c_hi;
};
template <int ACT>
__device__ __forceinline__ BlendRegs blend_regs()
{
    BlendRegs r;
    asm volatile("s_mov_b32 %0, %1" : "=s"(r.mask_lo) : "n"(kMaskLo4<ACT>));
    asm volatile("s_mov_b32 %0, %1" : "=s"(r.mask_hi) : "n"(kMaskHi4<ACT>));
    asm volatile("v_mov_b32 %0, %1" : "=v"(r.c_lo) : "n"(kBlendLo4<ACT>));
    asm volatile("v_mov_b32 %0, %1" : "=v"(r.c_hi) : "n"(kBlendHi4<ACT>));
    return r;
}
// B fragments of the two MFMA column tiles that share byte position jb (low nibble -> b0, high nibble -> b1); w holds
// this lane's dword of its 8 k rows, unmodified
template <int ACT>
__device__ __forceinline__ void expand_pair_blend(const uint32_t (&w)[8], int jb, const BlendRegs &r, u32x4 &b0, u32x4 &b1)
{
    const uint32_t sel = 0x0c000c00u | ((4u + jb) << 16) | (uint32_t)jb;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const uint32_t t = __builtin_amdgcn_perm(w[2 * v + 1], w[2 * v], sel);
        uint32_t lo, hi;
        expand_byte<ACT>(t, r.mask_lo, r.c_lo, r.mask_hi, r.c_hi, lo, hi);
        b0[v] = lo;
        b1[v] = hi;
    }
}

constexpr uint32_t kOutOfRange = 0x80000000u;   // lane offset beyond every buffer size: the load returns zero, no traffic
// s_getreg operand for the four-bit id of the XCD (accelerator die with its own L2) the wavefront runs on: register 20
// (XCC_ID), offset 0, width 4
constexpr int kHwRegXccId = (3 << 11) | (0 << 6) | 20;
constexpr int kNonTemporal = 2;                 // cache-policy bit for data that is read once


struct WqArgs {
    const uint16_t *x;              // bf16 [M, K]
    const void *w;                  // weight rows, contiguous along N
    const uint16_t *scale;          // bf16 [G, N]
    const uint16_t *offset;         // bf16 [G, N] or null
    const uint16_t *bias;           // [N] or null: added to the float32 sum before the final rounding
    uint16_t *out;                  // bf16 [M, N]
    float *partial;                 // workspace [S][M][N] float32 (S > 1)
    uint32_t *counter;              // workspace [mchunks][sgroups], zero on entry, left zero
    int64_t ldx, ldo;
    uint32_t ldw_bytes;             // bytes between weight rows
    uint32_t row_bytes;             // valid bytes of a weight row
    int M, N, K;
    int unit_steps;                 // 32-row steps per unit of K: a scale group, or one loop body per channel
    int n_units;                    // K / (32 * unit_steps)
    int grouped;                    // 0: one scale row for all K
    int strips;                     // 128-byte strips of a weight row
    int sgroups;                    // workgroup tiles along N: groups of W adjacent strips
    int S;                          // workgroups that share the K range of a tile
    // K-packed int4 kernel only
    int unit_sub;                   // sub-steps of 128 k per scale group
    int64_t ld_param_g, ld_param_n; // element strides of scale / offset: element (group, column)
};

// Output side of a workgroup tile of NBW columns whose partial sums lie in LDS as red[slice][16 rows][NBW].
// Every thread owns quads of 4 consecutive columns; N must be a multiple of 4 (every planner that uses this requires it),
// so a quad is either wholly inside the row or skipped.  Without a split over K the sums go straight to the output.
// With K split over S workgroups every workgroup publishes its partial and the last arrival adds them in chunk
// order: the exchange uses agent-scope (sc1) write-through stores and cache-bypassing loads, ordered by the
// wavefronts' own store counters, the workgroup barrier and a relaxed agent-scope counter; a full release/acquire
// fence would write back and invalidate the whole L2 of the XCD, which costs far more than the kernel itself.
template <int NBW, int KS, int THREADS, int ACT>
struct TileOut {
    static constexpr int QPR = NBW / 4;
    static constexpr int SC1 = 16;            // cache-policy bit: agent scope
    const WqArgs &p;
    char *lds;
    const int m_base, n0, chunk;
    const bool out_vec;
    const uint32_t chunk_bytes;
    const __amdgpu_buffer_rsrc_t rsrc_p;

    __device__ TileOut(const WqArgs &p_, char *lds_, int m_base_, int n0_, int chunk_)
        : p(p_), lds(lds_), m_base(m_base_), n0(n0_), chunk(chunk_), out_vec((p_.ldo & 3) == 0 && aligned_dev(p_.out, 8)),
          chunk_bytes((uint32_t)p_.M * (uint32_t)p_.N * 4u),
          rsrc_p(make_rsrc(p_.partial, p_.S > 1 ? (uint32_t)p_.M * (uint32_t)p_.N * 4u * (uint32_t)p_.S : 0u))
    {
    }

    __device__ __forceinline__ void store_out(int row, int nl, f32x4 v) const
    {
        if (p.bias) {
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = v[i] + act_1<ACT>(p.bias[min(n0 + nl + i, p.N - 1)]);
        }
        uint16_t *o = p.out + (int64_t)(m_base + row) * p.ldo + n0 + nl;
        if (out_vec) {
            u32x2 pk;
            pk.x = pack_act2<ACT>(v[0], v[1]);
            pk.y = pack_act2<ACT>(v[2], v[3]);
            *reinterpret_cast<u32x2 *>(o) = pk;
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = (uint16_t)pack_act2<ACT>(v[i], 0.0f);
        }
    }

    __device__ __forceinline__ uint32_t partial_off(int row, int nl) const { return (uint32_t)(((m_base + row) * p.N + n0 + nl) * 4); }

    // rows row0 .. row0+rows_mt-1 of the tile: add the slices, then store or publish
    __device__ __forceinline__ void emit_mtile(const float *red, int row0, int rows_mt) const
    {
        for (int qd = threadIdx.x; qd < rows_mt * QPR; qd += THREADS) {
            const int row = qd / QPR, nl = (qd % QPR) * 4;
            if (n0 + nl >= p.N) continue;
            f32x4 acc = *reinterpret_cast<const f32x4 *>(red + (size_t)row * NBW + nl);
#pragma unroll
            for (int ks = 1; ks < KS; ks++) acc += *reinterpret_cast<const f32x4 *>(red + ((size_t)ks * 16 + row) * NBW + nl);
            if (p.S == 1)
                store_out(row0 + row, nl, acc);
            else
                buffer_store_b128<SC1>(__builtin_bit_cast(u32x4, acc), rsrc_p, partial_off(row0 + row, nl),
                                                       (uint32_t)chunk * chunk_bytes);
        }
    }

    // after every m tile has been emitted: meet the other K chunks of the tile
    __device__ __forceinline__ void finish(int rows_valid, int tile) const
    {
        if (p.S == 1) return;
        int &is_last = *reinterpret_cast<int *>(lds);
        wait_vmcnt<0>();                      // this wavefront's partial sums have reached the coherence point
        __syncthreads();
        uint32_t *cnt = p.counter + (size_t)blockIdx.y * p.sgroups + tile;
        if (threadIdx.x == 0) {
            const uint32_t old = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = old == (uint32_t)(p.S - 1);
        }
        __syncthreads();
        if (!is_last) return;
        for (int qd = threadIdx.x; qd < rows_valid * QPR; qd += THREADS) {
            const int row = qd / QPR, nl = (qd % QPR) * 4;
            if (n0 + nl >= p.N) continue;
            const uint32_t off = partial_off(row, nl);
            f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int ch = 0; ch < p.S; ch += 8) {
                f32x4 v[8];                   // eight loads in flight
#pragma unroll
                for (int i = 0; i < 8; i++)
                    v[i] = ch + i < p.S ? __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                              rsrc_p, off, (uint32_t)(ch + i) * chunk_bytes, SC1))
                                        : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < 8; i++) acc += v[i];
            }
            store_out(row, nl, acc);
        }
        if (threadIdx.x == 0) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // ready for the next launch
    }
};

} // namespace
} // namespace mi355
