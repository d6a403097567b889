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
    static constexpr int PARAM_BASE = FLAG_BASE + 64;        // epilogue parameters (filled during the prologue)
    static constexpr int LDS_BYTES = PARAM_BASE + 4096;
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

// MFMAs FROM .. TO-1 of a half step (activation fragment outer, weight fragment inner).  The weight fragment is the
// first operand: a lane ends up with four consecutive output columns of one row.
template <int WTN, int FROM, int TO>
__device__ __forceinline__ void mfma_range(i32x4v (&acc)[4][WTN], const i32x4v (&af)[4], const i32x4v (&bf)[WTN])
{
#pragma unroll
    for (int t = FROM; t < TO; t++) {
        const int i = t / WTN, j = t % WTN;
        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bf[j], af[i], acc[i][j], 0, 0, 0);
    }
}

// N groups of (one instruction of class MASK, then PER MFMAs) for the scheduler
template <int MASK, int N, int PER>
__device__ __forceinline__ void interleave()
{
#pragma unroll
    for (int q = 0; q < N; q++) {
        __builtin_amdgcn_sched_group_barrier(MASK, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
    }
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
};

template <int NL>
__device__ __forceinline__ void issue_units(const LoopState &st, char *lds, uint32_t dst, uint32_t soff)
{
#pragma unroll
    for (int i = 0; i < NL; i++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(st.rsrc, (lds_void *)(lds + dst + i * 1024), 16, (i & 1) ? st.voff1 : st.voff0,
                                                 soff + (uint32_t)i * st.unit_stride, 0, 0);
}

// ROLE 0: refills activations (two slots); ROLE 1: refills weights (three slots).
// BPOS 0: weights are requested right behind the barrier that releases their slot (two steps of lead);
// BPOS 1: half a step later, in the first half of the next step, so that the two roles' requests alternate.
template <int WTN, int ROLE, int BPOS>
__device__ __forceinline__ void k_loop(i32x4v (&acc)[4][WTN], char *lds, const LoopState st)
{
    using G = Geometry<WTN>;
    constexpr int LBW = G::LBW, B_BYTES = G::B_BYTES, B_BASE = G::B_BASE;
    constexpr int NL = ROLE == 0 ? LAW : LBW;                  // refills of this wavefront per stage
    constexpr int HALF = 4 * WTN;                              // MFMAs per half step
    static_assert(HALF - 8 - WTN >= (ROLE == 0 ? LAW : (BPOS == 0 ? LBW : 0)), "refills need MFMAs to hide behind");
    const int KT = st.KT;
    auto k_off = [&](int stage) { return stage < KT ? st.sbase + (uint32_t)stage * BK : kPastEnd; };
    typedef __attribute__((address_space(3))) volatile uint32_t lds_flag_t;
    lds_flag_t *flag = (lds_flag_t *)(lds + st.flag);

    i32x4v ap[4], aq0[4], aq1[4], bf0[WTN], bf1[WTN];

#define MI355_WIDE_READ_A(P_, Q_, SLOT_)                                                                             \
    _Pragma("unroll") for (int i = 0; i < 4; i++)                                                                    \
        P_[i] = *reinterpret_cast<const i32x4v *>(lds + st.va0 + (SLOT_) * A_BYTES + i * 2048);                      \
    _Pragma("unroll") for (int i = 0; i < 4; i++)                                                                    \
        Q_[i] = *reinterpret_cast<const i32x4v *>(lds + st.va1 + (SLOT_) * A_BYTES + i * 2048);
#define MI355_WIDE_READ_B(BF_, VB_, SB_)                                                                             \
    _Pragma("unroll") for (int j = 0; j < WTN; j++)                                                                  \
        BF_[j] = *reinterpret_cast<const i32x4v *>(lds + (VB_) + (SB_) + j * 2048);
    // release of the activation slot just read: the reader publishes, the loader waits for it
#define MI355_WIDE_PUBLISH(VAL_)                                                                                     \
    {                                                                                                                \
        /* the eight activation reads are older than the WTN weight reads; one lane stores the flag */             \
        asm volatile("s_waitcnt lgkmcnt(%2)\n\ts_mov_b64 exec, 1\n\tds_write_b32 %0, %1\n\ts_mov_b64 exec, -1"           \
                     ::"v"(st.flag), "v"((uint32_t)(VAL_)), "n"(WTN) : "memory");                                    \
    }
#define MI355_WIDE_AWAIT(VAL_)                                                                                       \
    {                                                                                                                \
        uint32_t f_;                                                                                                 \
        int spins_ = 0;                                                                                              \
        do {                                                                                                         \
            f_ = __builtin_amdgcn_readfirstlane(*flag);                                                              \
        } while (f_ < (VAL_) && ++spins_ < (1 << 16));                                                               \
    }

    // prologue: stages 0 and 1 are requested, stage 0 has landed behind the barrier
    if constexpr (ROLE == 0) {
        issue_units<NL>(st, lds, st.dst0, k_off(0));
        issue_units<NL>(st, lds, st.dst0 + A_BYTES, k_off(1));
    } else {
        issue_units<NL>(st, lds, B_BASE + st.dst0, k_off(0));
        issue_units<NL>(st, lds, B_BASE + st.dst0 + B_BYTES, k_off(1));
    }
    wait_vmcnt_lgkm0<NL>();                 // (also the caller's LDS stores: the cleared flags)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);

    uint32_t sb_rd = 0;                      // byte offset of the weight slot that is read
    uint32_t sb_wr = 2 * B_BYTES;            // ... of the weight slot refilled next
    // what follows the barrier of "step -1": fragments of stage 0, release and refill of its activation slot
    {
        MI355_WIDE_READ_A(ap, aq0, 0)
        __builtin_amdgcn_sched_barrier(0);   // the order of the reads matters to the publishing wait below
        MI355_WIDE_READ_B(bf0, st.vb0, sb_rd)
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (ROLE == 1) {
            MI355_WIDE_PUBLISH(1u)
            if constexpr (BPOS == 0) {
                issue_units<NL>(st, lds, B_BASE + st.dst0 + sb_wr, k_off(2));
                sb_wr = 0;
            }
        } else {
            MI355_WIDE_AWAIT(1u)
            issue_units<NL>(st, lds, st.dst0, k_off(2));
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    // One K step.  Q_ holds the activation fragments of the second half of this step, QN_ receives those of the next
    // step; ASLOT_ is the activation slot of the next step (compile time: the loop is unrolled by two).
#define MI355_WIDE_STEP(KT_, Q_, QN_, ASLOT_)                                                                        \
    {                                                                                                                \
        /* first half: the weights of the second 64 bytes of K arrive while the first 64 are multiplied */         \
        MI355_WIDE_READ_B(bf1, st.vb1, sb_rd)                                                                        \
        if constexpr (ROLE == 1 && BPOS == 1) issue_units<NL>(st, lds, B_BASE + st.dst0 + sb_wr, k_off((KT_) + 2)); \
        mfma_range<WTN, 0, HALF>(acc, ap, bf0);                                                                      \
        interleave<0x100, WTN, 2>();                                                                                 \
        if constexpr (ROLE == 1 && BPOS == 1) interleave<0x010, NL, 1>();                                            \
        __builtin_amdgcn_sched_group_barrier(0x008, HALF, 0);                                                        \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
        /* stage KT_ + 1 has landed (only this wavefront's newest refill may be in flight) and this wavefront is   \
           done reading the weights of stage KT_ */                                                                 \
        wait_vmcnt_lgkm0<NL>();                                                                                      \
        __builtin_amdgcn_s_barrier();                                                                                \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
        sb_rd = sb_rd == 2 * B_BYTES ? 0u : sb_rd + B_BYTES;                                                         \
        /* second half: all activation fragments of the next step first, then its first weights */                 \
        MI355_WIDE_READ_A(ap, QN_, ASLOT_)                                                                           \
        mfma_range<WTN, 0, 8>(acc, Q_, bf1);                                                                         \
        interleave<0x100, 8, 1>();                                                                                   \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
        MI355_WIDE_READ_B(bf0, st.vb0, sb_rd)                                                                        \
        mfma_range<WTN, 8, 8 + WTN>(acc, Q_, bf1);                                                                   \
        interleave<0x100, WTN, 1>();                                                                                 \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
        if constexpr (ROLE == 1) {                                                                                   \
            MI355_WIDE_PUBLISH((uint32_t)(KT_) + 2u)                                                                 \
            __builtin_amdgcn_sched_barrier(0);                                                                       \
            if constexpr (BPOS == 0) issue_units<NL>(st, lds, B_BASE + st.dst0 + sb_wr, k_off((KT_) + 3));           \
            mfma_range<WTN, 8 + WTN, HALF>(acc, Q_, bf1);                                                            \
            if constexpr (BPOS == 0) interleave<0x010, NL, 1>();                                                     \
            __builtin_amdgcn_sched_group_barrier(0x008, HALF, 0);                                                    \
        } else {                                                                                                     \
            MI355_WIDE_AWAIT((uint32_t)(KT_) + 2u)                                                                   \
            __builtin_amdgcn_sched_barrier(0);                                                                       \
            issue_units<NL>(st, lds, st.dst0 + (ASLOT_) * A_BYTES, k_off((KT_) + 3));                                \
            mfma_range<WTN, 8 + WTN, HALF>(acc, Q_, bf1);                                                            \
            interleave<0x010, NL, 1>();                                                                              \
            __builtin_amdgcn_sched_group_barrier(0x008, HALF, 0);                                                    \
        }                                                                                                            \
        sb_wr = sb_wr == 2 * B_BYTES ? 0u : sb_wr + B_BYTES;                                                         \
        __builtin_amdgcn_sched_barrier(0);                                                                           \
    }

    for (int kt = 0; kt < KT; kt += 2) {
        MI355_WIDE_STEP(kt, aq0, aq1, 1)
        if (kt + 1 >= KT) break;
        MI355_WIDE_STEP(kt + 1, aq1, aq0, 0)
    }
#undef MI355_WIDE_STEP
#undef MI355_WIDE_READ_A
#undef MI355_WIDE_READ_B
#undef MI355_WIDE_PUBLISH
#undef MI355_WIDE_AWAIT
    wait_vmcnt_only<0>();                    // the refills past the end must not land in the epilogue's LDS
}

} // namespace wide
} // namespace mi355
