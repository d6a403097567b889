// K loop of npu_quant_matmul for the widest tiles: 256 x (32 * WTN) outputs per workgroup, eight wavefronts arranged
// 4 x 2, each owning 64 rows x 16 * WTN columns (4 x WTN accumulators of v_mfma_i32_16x16x64_i8).
//
// What differs from the generic tiled loop in quant_matmul.hip:
//
//  * Loader roles.  Wavefront (wm, 0) refills the 64 activation rows that it and (wm, 1) multiply (eight direct-to-LDS
//    loads of 1 KiB per K step); wavefront (wm, 1) refills a quarter of the weight rows.  Loads retire in order per
//    wavefront, so the activations, which come from cache, no longer queue behind weights that come from HBM.
//  * Activation slots are released without a workgroup barrier.  Only two wavefronts read a given activation row, and
//    both read the fragments of a whole K step (both 64-byte halves) right after the step's barrier; (wm, 1) then
//    publishes the step number in an LDS flag and (wm, 0) refills the slot as soon as it sees it.  With two slots the
//    refill gets ~1.8 K steps to land instead of exactly one.
//  * Weight slots (three) are released by the one barrier per K step, as before: two steps of lead.
//  * Addresses: slot offsets live in scalar registers, fragment addresses are two vector registers per operand, and a
//    K step past the end moves no bytes because its scalar offset is out of range, so the loop carries four vector
//    ALU instructions per step besides the MFMAs.
#pragma once
#include "common.h"
#include <utility>

#ifndef MI355_WIDE_ABL
#define MI355_WIDE_ABL 0       // compile-time ablations for timing experiments (wrong results): 1 no refill traffic, 2 no fragment reads, 4 no MFMAs, 8 no handshake, 16 no barrier, 32 / 64 all tiles read the first tile's activation rows / weight columns
#endif

namespace mi355 {
namespace wide {

typedef int32_t i32x4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;

constexpr int BK = 128;
constexpr uint32_t kPastEnd = 0x80000000u;     // scalar offset beyond every buffer: the load moves no bytes
constexpr int A_BYTES = 32768;                 // one activation slot: 256 rows x 128 bytes
constexpr int LAW = 8;                         // activation refills per loader wavefront and K step

template <int WTN>
struct Geometry {
    static constexpr int LBW = WTN;                          // weight units (8 rows x 128 B) per loader wavefront: 4 * WTN / 4
    static constexpr int B_BYTES = LBW * 4 * 1024;           // one weight slot
    static constexpr int B_BASE = 2 * A_BYTES;
    static constexpr int FLAG_BASE = B_BASE + 3 * B_BYTES;   // four flag words, one per pair of wavefronts
    static constexpr int PARAM_BASE = FLAG_BASE + 64;        // epilogue parameters (filled during the prologue): 2.5 KiB
    static constexpr int LDS_BYTES = PARAM_BASE + 3072;
};

// s_waitcnt vmcnt(VM) lgkmcnt(0) as the builtin, so that the compiler's own bookkeeping of outstanding LDS reads sees it
// (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4 left at "no wait", lgkmcnt 11:8)
template <int VM>
__device__ __forceinline__ void wait_vmcnt_lgkm0()
{
    static_assert(VM >= 0 && VM < 64, "vmcnt range");
    __builtin_amdgcn_s_waitcnt((VM & 15) | (7 << 4) | (0 << 8) | ((VM >> 4) << 14));
}
template <int VM>
__device__ __forceinline__ void wait_vmcnt_only()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(VM) : "memory");
}
template <int LG>
__device__ __forceinline__ void wait_lgkmcnt()
{
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(LG) : "memory");
}

struct LoopState {
    // loader side
    __amdgpu_buffer_rsrc_t rsrc;       // operand rows this wavefront refills
    uint32_t voff0, voff1;             // lane offsets for the even / odd units of its run
    uint32_t unit_stride;              // bytes between units (8 rows)
    uint32_t sbase;                    // scalar offset of its first unit at the first K step of the workgroup
    uint32_t dst0;                     // LDS byte offset of its first unit inside a slot
    // reader side
    uint32_t va0, va1, vb0, vb1;       // LDS byte offsets of the lane's fragment rows (first / second 64 bytes of a K step)
    uint32_t flag;                     // LDS byte offset of the pair's flag word
    int KT;                            // K steps of this workgroup
#ifdef MI355_QMM_TS
    unsigned long long *ts;
#endif
};

#ifdef MI355_QMM_TS
#define MI355_WIDE_TS(IDX) if (st.ts && (threadIdx.x & 63) == 0 && (IDX) < 128) st.ts[(IDX)] = __builtin_readcyclecounter();
#else
#define MI355_WIDE_TS(IDX)
#endif

// ---------------------------------------------------------------------------------------------------------------
// Instruction order.  A part of a K step is written as a string, one character per instruction, and emitted in exactly
// that order (every instruction is pinned by a scheduling group of its own):
//   M  the next MFMA of the half step (activation fragment outer, weight fragment inner)
//   a  the next activation fragment read (first the four fragments of the first 64 bytes of K, then the second four)
//   b  the next weight fragment read
//   D  the next refill (1 KiB direct-to-LDS load) of this wavefront
// Every wavefront issues, per K step, the second half "S" (behind the barrier in the middle of the step; split into the
// part before the release of the activation slot, S1, and the part after it, S2) and the first half "F" of the next step.
// The refills of one stage may be spread over S2 and the following F: they all precede the next barrier, so the number
// of loads that may be outstanding there does not change.
template <int V, int WTN, int ROLE, int PART>
struct Order {
    static constexpr const char *str()
    {
        if constexpr (WTN == 6) {
            if constexpr (V == 0) {
                if constexpr (PART == 0) return "aMaMaMaMaMaMaMaMbMbMbMbMbMbM";
                if constexpr (PART == 1) return ROLE == 0 ? "DMDMDMDMDMDMDMDMMM" : "DMDMDMDMDMDMMMMM";
                if constexpr (PART == 2) return "bMMbMMbMMbMMbMMbMMMMMMMMMMMMMM";
            }
            if constexpr (V == 1) {
                if constexpr (PART == 0) return "aMaMaMaMaMaMaMaMbMbMbMbMbMbM";
                if constexpr (PART == 1) return "DMMMDMMMDMMMM";
                if constexpr (PART == 2) return ROLE == 0 ? "bMMDMbMMMbDMMMbMDMMbMMDMbMMMDMMMMMM" : "bMMMbMDMMbMMMbMDMMbMMMbMDMMMMMMMM";
            }
        } else if constexpr (WTN == 7) {
            if constexpr (V == 0) {
                if constexpr (PART == 0) return "aMaMaMaMaMaMaMaMbMbMbMbMbMbMbM";
                if constexpr (PART == 1) return ROLE == 0 ? "DMDMDMDMDMDMDMDMMMMMM" : "DMDMDMDMDMDMDMMMMMMM";
                if constexpr (PART == 2) return "bMMbMMbMMbMMbMMbMMbMMMMMMMMMMMMMMMM";
            }
            if constexpr (V == 1) {
                if constexpr (PART == 0) return "aMaMaMaMaMaMaMaMbMbMbMbMbMbMbM";
                if constexpr (PART == 1) return "DMMMDMMMDMMMMMMM";
                if constexpr (PART == 2) return ROLE == 0 ? "bMMDMbMMMbDMMMbMDMMbMMDMbMMMbDMMMMMMMMMM" : "bMMMbMDMMbMMMbMDMMbMMMbMDMMbMMMMDMMMMMM";
            }
        }
        return "";
    }
    static constexpr int length()
    {
        int n = 0;
        while (str()[n]) n++;
        return n;
    }
    static constexpr char at(int i) { return str()[i]; }
    static constexpr int count(char c, int upto = length())
    {
        int n = 0;
        for (int i = 0; i < upto; i++) n += str()[i] == c;
        return n;
    }
    // weight fragment reads behind the last activation fragment read (what may still be in flight when the slot is released)
    static constexpr int b_after_last_a()
    {
        int n = 0;
        for (int i = 0; i < length(); i++) {
            if (str()[i] == 'a') n = 0;
            if (str()[i] == 'b') n++;
        }
        return n;
    }
};

// refill number i of a stage: 1 KiB, eight rows of 128 bytes
__device__ __forceinline__ void issue_unit(const LoopState &st, char *lds, uint32_t dst, uint32_t soff, int i)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(st.rsrc, (lds_void *)(lds + dst + i * 1024), 16, (i & 1) ? st.voff1 : st.voff0,
                                             soff + (uint32_t)i * st.unit_stride, 0, 0);
}

template <int WTN>
struct PartCtx {
    i32x4v (&acc)[4][WTN];
    const i32x4v (&ma)[4];             // MFMA operands of this part
    const i32x4v (&mb)[WTN];
    i32x4v (&ra0)[4];                  // destinations of the fragment reads
    i32x4v (&ra1)[4];
    i32x4v (&rb)[WTN];
    char *lds;
    uint32_t a0, a1, b;                // LDS byte offsets the fragments are read from
    const LoopState &st;
    uint32_t dst, soff;                // refills: LDS byte offset and scalar offset of the wavefront's first unit
};

template <char C, int IDX, int M0, int A0, int B0, int D0, int WTN>
__device__ __forceinline__ void emit_one(PartCtx<WTN> &c)
{
    if constexpr (C == 'M') {
        constexpr int t = M0 + IDX, i = t / WTN, j = t % WTN;
        if constexpr (MI355_WIDE_ABL & 4) asm volatile("" ::"v"(c.mb[j]), "v"(c.ma[i]));
        else c.acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(c.mb[j], c.ma[i], c.acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    } else if constexpr (C == 'a') {
        constexpr int r = A0 + IDX;
        if constexpr (!(MI355_WIDE_ABL & 2)) {
            if constexpr (r < 4) c.ra0[r] = *reinterpret_cast<const i32x4v *>(c.lds + c.a0 + r * 2048);
            else c.ra1[r - 4] = *reinterpret_cast<const i32x4v *>(c.lds + c.a1 + (r - 4) * 2048);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    } else if constexpr (C == 'b') {
        constexpr int r = B0 + IDX;
        if constexpr (!(MI355_WIDE_ABL & 2)) {
            c.rb[r] = *reinterpret_cast<const i32x4v *>(c.lds + c.b + r * 2048);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    } else {
        static_assert(C == 'D', "unknown instruction class");
        issue_unit(c.st, c.lds, c.dst, c.soff, D0 + IDX);
        __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
    }
}

// emits the instructions of Order O; M0 / A0 / B0 / D0: how many of each class the earlier parts of the half step held
template <class O, int M0, int A0, int B0, int D0, int WTN, int... I>
__device__ __forceinline__ void emit_part(PartCtx<WTN> &c, std::integer_sequence<int, I...>)
{
    (emit_one<O::at(I), O::count(O::at(I), I), M0, A0, B0, D0, WTN>(c), ...);
}

template <int NL>
__device__ __forceinline__ void issue_units(const LoopState &st, char *lds, uint32_t dst, uint32_t soff)
{
#pragma unroll
    for (int i = 0; i < NL; i++) issue_unit(st, lds, dst, soff, i);
}

// ROLE 0: refills activations (two slots); ROLE 1: refills weights (three slots).  V: instruction order (Order).
template <int WTN, int ROLE, int V>
__device__ __forceinline__ void k_loop(i32x4v (&acc)[4][WTN], char *lds, const LoopState st)
{
    using G = Geometry<WTN>;
    constexpr int LBW = G::LBW, B_BYTES = G::B_BYTES, B_BASE = G::B_BASE;
    constexpr int NL = ROLE == 0 ? LAW : LBW;                  // refills of this wavefront per stage
    constexpr int HALF = 4 * WTN;                              // MFMAs per half step
    using S1 = Order<V, WTN, ROLE, 0>;
    using S2 = Order<V, WTN, ROLE, 1>;
    using F = Order<V, WTN, ROLE, 2>;
    constexpr int DS1 = S1::count('D'), DS = DS1 + S2::count('D');   // refills issued in S; the rest follow in F
    static_assert(S1::count('M') + S2::count('M') == HALF && F::count('M') == HALF, "MFMAs per half step");
    static_assert(S1::count('a') == 8 && S2::count('a') == 0 && F::count('a') == 0, "activation fragments are read before the release");
    static_assert(S1::count('b') + S2::count('b') == WTN && F::count('b') == WTN, "weight fragment reads");
    static_assert(DS + F::count('D') == NL, "refills per stage");
    static_assert(ROLE == 1 || DS1 == 0, "activation refills follow the release");
    const int KT = st.KT;
    auto k_off = [&](int stage) { return stage < KT && !(MI355_WIDE_ABL & 1) ? st.sbase + (uint32_t)stage * BK : kPastEnd; };
    typedef __attribute__((address_space(3))) volatile uint32_t lds_flag_t;
    lds_flag_t *flag = (lds_flag_t *)(lds + st.flag);

    i32x4v ap[4], aq0[4], aq1[4], bf0[WTN], bf1[WTN];

    // release of the activation slot just read: the reader publishes the step, the loader waits for it
#define MI355_WIDE_PUBLISH(VAL_)                                                                                     \
    if constexpr (!(MI355_WIDE_ABL & 8)) {                                                                           \
        /* LDS reads return in order: at most the weight fragment reads behind the last activation read may be     \
           outstanding; one lane stores the flag */                                                                 \
        asm volatile("s_waitcnt lgkmcnt(%2)\n\ts_mov_b64 exec, 1\n\tds_write_b32 %0, %1\n\ts_mov_b64 exec, -1"           \
                     ::"v"(st.flag), "v"((uint32_t)(VAL_)), "n"(S1::b_after_last_a()) : "memory");                   \
    }
#define MI355_WIDE_AWAIT(VAL_)                                                                                       \
    if constexpr (!(MI355_WIDE_ABL & 8)) {                                                                           \
        /* like the barrier, this wait ends because the other wavefront of the pair runs the same steps */          \
        uint32_t f_;                                                                                                 \
        do {                                                                                                         \
            f_ = __builtin_amdgcn_readfirstlane(*flag);                                                              \
        } while (f_ < (VAL_));                                                                                       \
    }
    // the second half of step KT_ (KT_ = -1: what precedes the loop): fragments of stage KT_ + 1, refills of stage KT_ + 3
#define MI355_WIDE_SECOND(KT_, Q_, QN_, ASLOT_, MFMA_)                                                               \
    {                                                                                                                \
        PartCtx<WTN> c_{acc, Q_, bf1, ap, QN_, bf0, lds, st.va0 + (ASLOT_) * A_BYTES, st.va1 + (ASLOT_) * A_BYTES,   \
                        st.vb0 + sb_rd, st, ROLE == 0 ? st.dst0 + (ASLOT_) * A_BYTES : B_BASE + st.dst0 + sb_wr,     \
                        k_off((KT_) + 3)};                                                   \
        emit_part<S1, 0, 0, 0, 0>(c_, std::make_integer_sequence<int, S1::length()>{});                              \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
        if constexpr (ROLE == 1) { MI355_WIDE_PUBLISH((uint32_t)((KT_) + 2)) } else { MI355_WIDE_AWAIT((uint32_t)((KT_) + 2)) } \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
        emit_part<S2, S1::count('M'), 8, S1::count('b'), DS1>(c_, std::make_integer_sequence<int, S2::length()>{});  \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
    }

    // prologue: stages 0 and 1 are requested, stage 0 has landed behind the barrier
    if constexpr (ROLE == 0) {
        issue_units<NL>(st, lds, st.dst0, k_off(0));
        issue_units<NL>(st, lds, st.dst0 + A_BYTES, k_off(1));
    } else {
        issue_units<NL>(st, lds, B_BASE + st.dst0, k_off(0));
        issue_units<NL>(st, lds, B_BASE + st.dst0 + B_BYTES, k_off(1));
    }
    wait_vmcnt_lgkm0<NL>();                  // stage 0 (also the caller's LDS stores: the cleared flags)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    MI355_WIDE_TS(1)

    uint32_t sb_rd = 0;                      // byte offset of the weight slot that is read
    uint32_t sb_wr = 2 * B_BYTES;            // ... of the weight slot being refilled
    {
        // what precedes the loop is the second half of "step -1" without MFMAs: fragments of stage 0, release of its
        // activation slot, the first refills of stage 2
#pragma unroll
        for (int i = 0; i < 4; i++) ap[i] = *reinterpret_cast<const i32x4v *>(lds + st.va0 + i * 2048);
#pragma unroll
        for (int i = 0; i < 4; i++) aq0[i] = *reinterpret_cast<const i32x4v *>(lds + st.va1 + i * 2048);
        __builtin_amdgcn_sched_barrier(0);   // the order of the reads matters to the publishing wait
#pragma unroll
        for (int j = 0; j < WTN; j++) bf0[j] = *reinterpret_cast<const i32x4v *>(lds + st.vb0 + j * 2048);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (ROLE == 1) { MI355_WIDE_PUBLISH(1u) } else { MI355_WIDE_AWAIT(1u) }
        __builtin_amdgcn_sched_barrier(0);
        issue_units<DS>(st, lds, ROLE == 0 ? st.dst0 : B_BASE + st.dst0 + sb_wr, k_off(2));
        __builtin_amdgcn_sched_barrier(0);
    }

    // One K step.  Q_ holds the activation fragments of the second half of this step, QN_ receives those of the next
    // step; ASLOT_ is the activation slot of the next step (compile time: the loop is unrolled by two).
#define MI355_WIDE_STEP(KT_, Q_, QN_, ASLOT_)                                                                        \
    {                                                                                                                \
        /* first half: the weights of the second 64 bytes of K arrive while the first 64 are multiplied; the      \
           remaining refills of stage KT_ + 2 */                                                                    \
        {                                                                                                            \
            PartCtx<WTN> c_{acc, ap, bf0, ap, ap, bf1, lds, 0u, 0u, st.vb1 + sb_rd, st,                              \
                            ROLE == 0 ? st.dst0 + (1 - (ASLOT_)) * A_BYTES : B_BASE + st.dst0 + sb_wr, k_off((KT_) + 2)}; \
            emit_part<F, 0, 0, 0, DS>(c_, std::make_integer_sequence<int, F::length()>{});                           \
        }                                                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
        /* stage KT_ + 1 has landed (only this wavefront's newest refill may be in flight) and this wavefront is   \
           done reading the weights of stage KT_ */                                                                 \
        MI355_WIDE_TS(8 + 2 * (KT_))                                                                                 \
        wait_vmcnt_lgkm0<NL>();                                                                                      \
        MI355_WIDE_TS(9 + 2 * (KT_))                                                                                 \
        if constexpr (!(MI355_WIDE_ABL & 16)) __builtin_amdgcn_s_barrier();                                          \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
        sb_rd = sb_rd == 2 * B_BYTES ? 0u : sb_rd + B_BYTES;                                                         \
        sb_wr = sb_wr == 2 * B_BYTES ? 0u : sb_wr + B_BYTES;                                                         \
        MI355_WIDE_SECOND(KT_, Q_, QN_, ASLOT_, 1)                                                                   \
    }

    for (int kt = 0; kt < KT; kt += 2) {
        MI355_WIDE_STEP(kt, aq0, aq1, 1)
        if (kt + 1 >= KT) break;
        MI355_WIDE_STEP(kt + 1, aq1, aq0, 0)
    }
#undef MI355_WIDE_STEP
#undef MI355_WIDE_SECOND
#undef MI355_WIDE_PUBLISH
#undef MI355_WIDE_AWAIT
    wait_vmcnt_only<0>();                    // the refills past the end must not land in the epilogue's LDS
}


// ---------------------------------------------------------------------------------------------------------------
// Epilogue for the common cases: per-token scales or none, one float32 scale per column or one for all, optional bf16 bias,
// bf16 / fp16 output
// with 16-byte aligned rows.  The three parameter vectors of the tile were requested into LDS (PARAM_BASE) before the
// first K step, so nothing here waits for global memory.  Per block of 16 rows a wavefront converts its WTN accumulator
// tiles, stages them in its own LDS rows and stores whole rows of the wavefront tile (16 bytes per lane) right away, so
// the stores of one block leave while the next block is converted.
//   ((float(acc) * pertoken[m]) * scale[n]) + bias[n], every operation rounded to binary32, one rounding to 16 bits.
struct EpilogueArgs {
    void *out;
    int64_t ldc;
    int M, N;
    int m0, n0;                        // first row / column of the workgroup tile
    int has_bias, out_f16;             // has_bias: the MI355_BIAS_* code of the 16-bit epilogue, 0 / 1 for the int8 one
    int stream_out;                    // store the rows with non-temporal stores (see the launcher's choice)
    int wm, wn;                        // position of the wavefront's 64 x 16 * WTN share in the workgroup tile
    int packed_scale;                  // 16-bit output: the column scales come from the packed 64-bit parameter words
    int param_base;                    // LDS byte offset of the parameter vectors
};

constexpr int PARAM_PS = 0, PARAM_SCALE = 1024, PARAM_BIAS = 2048;

// issued by one wavefront in front of its first stage requests (loads retire in order, so they have landed when
// stage 0 has); rows / columns past the matrix read as zero
// (no per-token scales: the vector is filled with 1.0f, by which the epilogue's multiplication changes nothing; a single
// scale for all columns is spread over the vector)
__device__ __forceinline__ void request_params(char *lds, int param_base, const float *pertoken, const float *scale, bool one_scale,
                                                const void *bias, int bias_size, int m0, int n0, int rows, int cols, int lane)
{
    if (pertoken) {
        const __amdgpu_buffer_rsrc_t r_ps = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(pertoken + m0), 0, rows * 4, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r_ps, (lds_void *)(lds + param_base + PARAM_PS), 16, (uint32_t)lane * 16u, 0, 0, 0);
    } else {
        *reinterpret_cast<f32x4 *>(lds + param_base + PARAM_PS + lane * 16) = f32x4{1.0f, 1.0f, 1.0f, 1.0f};
    }
    if (!one_scale) {
        const __amdgpu_buffer_rsrc_t r_sc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(scale + n0), 0, cols * 4, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r_sc, (lds_void *)(lds + param_base + PARAM_SCALE), 16, (uint32_t)lane * 16u, 0, 0, 0);
    } else {
        const float s1 = scale[0];
        *reinterpret_cast<f32x4 *>(lds + param_base + PARAM_SCALE + lane * 16) = f32x4{s1, s1, s1, s1};
    }
    if (bias) {                                               // bias_size bytes per column: bf16, or int32 / float32
        const __amdgpu_buffer_rsrc_t r_b = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char *>(static_cast<const char *>(bias) + (size_t)n0 * bias_size), 0, cols * bias_size, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r_b, (lds_void *)(lds + param_base + PARAM_BIAS), 16, (uint32_t)lane * 16u, 0, 0, 0);
    }
}

// BIAS: 0 none, 1 bf16 (added last), 2 int32 (added to the accumulator, wrapping like it), 3 float32 (added last)
// QP: the column scales are the low words of the packed 64-bit parameters (request_params_i8's layout) and there are no
// per-token scales
template <int WTN, bool F16, int BIAS, bool NT, bool QP = false>
__device__ __forceinline__ void epilogue_rows(i32x4v (&acc)[4][WTN], char *lds, const EpilogueArgs &e, int wave, int lane)
{
    constexpr int ROWB = WTN * 32 + 16;                       // padded pitch of a staged row: spreads rows over the banks
    constexpr int CHUNKS = WTN * 2;                           // 16-byte chunks per row of the wavefront tile
    const int wm = e.wm, wn = e.wn;
    const int mrow = lane & 15, nquad = (lane >> 4) * 4;
    const char *par = lds + e.param_base;
    float ps[4];
#pragma unroll
    for (int i = 0; i < 4; i++) ps[i] = QP ? 1.0f : *reinterpret_cast<const float *>(par + PARAM_PS + (wm * 64 + i * 16 + mrow) * 4);
    f32x4 sc[WTN], bs[WTN];
#pragma unroll
    for (int j = 0; j < WTN; j++) {
        const int c = wn * WTN * 16 + j * 16 + nquad;
        if constexpr (QP) {
            const u32x4 q01 = *reinterpret_cast<const u32x4 *>(par + c * 8);       // low, high words of columns c, c + 1
            const u32x4 q23 = *reinterpret_cast<const u32x4 *>(par + c * 8 + 16);
            sc[j] = f32x4{__uint_as_float(q01.x), __uint_as_float(q01.z), __uint_as_float(q23.x), __uint_as_float(q23.z)};
        } else {
            sc[j] = *reinterpret_cast<const f32x4 *>(par + PARAM_SCALE + c * 4);
        }
        if constexpr (BIAS == 1) {
            const u32x2 b2 = *reinterpret_cast<const u32x2 *>(par + PARAM_BIAS + c * 2);
            bs[j] = f32x4{bf16_lo(b2.x), bf16_hi(b2.x), bf16_lo(b2.y), bf16_hi(b2.y)};
        } else if constexpr (BIAS >= 2) {
            bs[j] = *reinterpret_cast<const f32x4 *>(par + PARAM_BIAS + c * 4);       // int32: its bit patterns
        }
    }
    char *stg = lds + wave * (16 * ROWB);
    const int mw = e.m0 + wm * 64, nw = e.n0 + wn * WTN * 16;
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            float f[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float v = BIAS == 2 ? (float)(int32_t)((uint32_t)acc[i][j][r] + __float_as_uint(bs[j][r])) : (float)acc[i][j][r];
                v = v * ps[i];
                v = v * sc[j][r];
                if constexpr (BIAS == 1 || BIAS == 3) v = v + bs[j][r];
                f[r] = v;
            }
            u32x2 pk;
            pk.x = F16 ? pack_f16x2(f[0], f[1]) : pack_bf16x2(f[0], f[1]);
            pk.y = F16 ? pack_f16x2(f[2], f[3]) : pack_bf16x2(f[2], f[3]);
            *reinterpret_cast<u32x2 *>(stg + mrow * ROWB + (j * 16 + nquad) * 2) = pk;
        }
#pragma unroll
        for (int q0 = 0; q0 < 16 * CHUNKS; q0 += 64) {
            const int q = q0 + lane;
            const int row = q / CHUNKS, ch = q % CHUNKS;
            if ((16 * CHUNKS) % 64 != 0 && row >= 16) continue;
            const int m = mw + i * 16 + row, n = nw + ch * 8;
            if (m >= e.M || n >= e.N) continue;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(stg + row * ROWB + ch * 16);
            uint16_t *o = static_cast<uint16_t *>(e.out) + (int64_t)m * e.ldc + n;
            if (n + 7 < e.N) {
                if constexpr (NT) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(o));
                else *reinterpret_cast<u32x4 *>(o) = v;
            } else {
                for (int r = 0; r < 8; r++)
                    if (n + r < e.N) o[r] = (uint16_t)(v[r >> 1] >> ((r & 1) * 16));
            }
        }
    }
}

// EPI: the variants a kernel of the widest tile holds (0: float32 scales with no bias or a bf16 one; 1: float32 scales with
// an int32 or float32 bias; 2: packed parameter words with no bias or an int32 one); the narrower tiles hold them all.
template <int WTN, int EPI = 0>
__device__ __forceinline__ void epilogue_fast(i32x4v (&acc)[4][WTN], char *lds, const EpilogueArgs &e, int wave, int lane)
{
    // output type, kind of bias and kind of store are resolved once per wavefront
    auto go = [&](auto f16, auto bias) {
        constexpr bool H = decltype(f16)::value;
        constexpr int B = decltype(bias)::value;
        constexpr bool LEAN = WTN >= 7;
        constexpr bool PLAIN = !LEAN || (EPI == 0 && B < 2) || (EPI == 1 && B >= 2);   // variants with float32 scales
        constexpr bool PACKED = !LEAN || (EPI == 2 && (B == 0 || B == 2));             // ... with packed parameter words
        if constexpr (PACKED) {
            if (LEAN || e.packed_scale) {
                if (e.stream_out) epilogue_rows<WTN, H, B, true, true>(acc, lds, e, wave, lane);
                else epilogue_rows<WTN, H, B, false, true>(acc, lds, e, wave, lane);
                return;
            }
        }
        if constexpr (PLAIN) {
            if (e.stream_out) epilogue_rows<WTN, H, B, true>(acc, lds, e, wave, lane);
            else epilogue_rows<WTN, H, B, false>(acc, lds, e, wave, lane);
        }
    };
    using T = std::true_type;
    using F = std::false_type;
    auto by_bias = [&](auto f16) {
        switch (e.has_bias) {                 // the MI355_BIAS_* code
        case 1: go(f16, std::integral_constant<int, 1>{}); break;
        case 2: go(f16, std::integral_constant<int, 2>{}); break;
        case 3: go(f16, std::integral_constant<int, 3>{}); break;
        default: go(f16, std::integral_constant<int, 0>{}); break;
        }
    };
    if (e.out_f16) by_bias(T{});
    else by_bias(F{});
}

// ---- the same for the re-quantised int8 output: clamp(rint(float(acc + int32 bias) * scale + offset)), scale and the
// 9-bit offset from the packed 64-bit parameter words, each operation rounded to binary32.  The parameter words of the
// tile's columns (2 KiB) and the int32 bias (1 KiB) are requested into LDS in front of the first K step; a wavefront
// stages its whole tile (a lane owns one 32-bit word of four columns per 16x16 tile) and stores 16 bytes per lane.
constexpr int PARAM_QP = 0, PARAM_BIAS32 = 2048;

__device__ __forceinline__ void request_params_i8(char *lds, int param_base, const uint64_t *qparam, const void *bias, int n0,
                                                   int cols, int lane, int bias_size = 4)
{
    const __amdgpu_buffer_rsrc_t r_q = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint64_t *>(qparam + n0), 0, cols * 8, 0x00020000);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r_q, (lds_void *)(lds + param_base + PARAM_QP), 16, (uint32_t)lane * 16u, 0, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r_q, (lds_void *)(lds + param_base + PARAM_QP + 1024), 16, (uint32_t)lane * 16u, 1024, 0, 0);
    if (bias) {                                               // int32 for the int8 output; any kind for the 16-bit ones
        const __amdgpu_buffer_rsrc_t r_b = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char *>(static_cast<const char *>(bias) + (size_t)n0 * bias_size), 0, cols * bias_size, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r_b, (lds_void *)(lds + param_base + PARAM_BIAS32), 16, (uint32_t)lane * 16u, 0, 0, 0);
    }
}

template <int WTN, bool BIAS, bool NT>
__device__ __forceinline__ void epilogue_rows_i8(i32x4v (&acc)[4][WTN], char *lds, const EpilogueArgs &e, int wave, int lane)
{
    constexpr int ROWQ = WTN * 16 + 16;                       // padded pitch of a staged row of the wavefront tile
    constexpr int CHQ = WTN;                                  // 16-byte chunks per row
    const int wm = e.wm, wn = e.wn;
    const int mrow = lane & 15, nquad = (lane >> 4) * 4;
    const char *par = lds + e.param_base;
    char *stq = lds + wave * (64 * ROWQ);
#pragma unroll
    for (int j = 0; j < WTN; j++) {
        const int c = wn * WTN * 16 + j * 16 + nquad;
        const u32x4 q01 = *reinterpret_cast<const u32x4 *>(par + PARAM_QP + c * 8);        // low, high words of columns c, c + 1
        const u32x4 q23 = *reinterpret_cast<const u32x4 *>(par + PARAM_QP + c * 8 + 16);
        const uint32_t lo[4] = {q01.x, q01.z, q23.x, q23.z}, hi[4] = {q01.y, q01.w, q23.y, q23.w};
        i32x4v bi = i32x4v{0, 0, 0, 0};
        if constexpr (BIAS) bi = *reinterpret_cast<const i32x4v *>(par + PARAM_BIAS32 + c * 4);
        float sc[4], of[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            sc[r] = __uint_as_float(lo[r]);
            of[r] = (float)(((int32_t)((hi[r] >> 5) << 23)) >> 23);                        // bits 37-45 of the 64: a 9-bit integer
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t w = 0;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float v = (float)(int32_t)((uint32_t)acc[i][j][r] + (uint32_t)bi[r]);      // wraps like the accumulator
                v = v * sc[r];
                v = v + of[r];
                v = fminf(fmaxf(rintf(v), -128.0f), 127.0f);
                w |= ((uint32_t)(int32_t)v & 0xffu) << (8 * r);
            }
            *reinterpret_cast<uint32_t *>(stq + (i * 16 + mrow) * ROWQ + j * 16 + nquad) = w;
        }
    }
    const int mw = e.m0 + wm * 64, nw = e.n0 + wn * WTN * 16;
#pragma unroll
    for (int q0 = 0; q0 < 64 * CHQ; q0 += 64) {
        const int q = q0 + lane;
        const int row = q / CHQ, ch = q % CHQ;
        const int m = mw + row, n = nw + ch * 16;
        if (m >= e.M || n >= e.N) continue;
        const u32x4 v = *reinterpret_cast<const u32x4 *>(stq + row * ROWQ + ch * 16);
        int8_t *o = static_cast<int8_t *>(e.out) + (int64_t)m * e.ldc + n;
        if (n + 15 < e.N) {
            if constexpr (NT) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(o));
            else *reinterpret_cast<u32x4 *>(o) = v;
        } else {
            for (int r = 0; r < 16; r++)
                if (n + r < e.N) o[r] = (int8_t)(v[r >> 2] >> ((r & 3) * 8));
        }
    }
}

template <int WTN>
__device__ __forceinline__ void epilogue_fast_i8(i32x4v (&acc)[4][WTN], char *lds, const EpilogueArgs &e, int wave, int lane)
{
    if (e.has_bias) {
        if (e.stream_out) epilogue_rows_i8<WTN, true, true>(acc, lds, e, wave, lane);
        else epilogue_rows_i8<WTN, true, false>(acc, lds, e, wave, lane);
    } else {
        if (e.stream_out) epilogue_rows_i8<WTN, false, true>(acc, lds, e, wave, lane);
        else epilogue_rows_i8<WTN, false, false>(acc, lds, e, wave, lane);
    }
}

} // namespace wide
} // namespace mi355
