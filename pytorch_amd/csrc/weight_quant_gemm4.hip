// npu_weight_quant_batchmatmul, int4 weights packed along N (and int8 weights [K, N], see the kernel's template
// parameters), more than 32 activation rows: a tiled GEMM in which the packed weights never exist in expanded form outside
// of registers.  The description is that of the int4 case.
//
// A workgroup owns 64 activation rows x one 128-byte strip of the weight rows (256 columns) and walks its K range in
// stages of 128 rows.  Per stage the activations (64 x 256 B) and the raw strip (128 x 128 B) are copied global -> LDS by
// direct loads into one of four slots.  The strip's 32 dword columns form two spans of 16, a dword's four bytes two
// byte pairs.  A wavefront owns all 64 rows (four MFMA row tiles) x one span x one byte pair: its lane c reads dword
// 16h + c of its eight k rows back from LDS (eight 4-byte reads per 32 k) and expands the four nibbles of its byte pair
// into exact bf16 / fp16 images of the integers, i.e. into the B operands of four MFMA column tiles (tile i = columns
// 128h + 8c + 4jp + i), each of which meets all four row tiles: 16 MFMAs per step for 4 activation fragments and 8
// dwords from LDS and ~40 integer instructions.  No expanded image ever travels through LDS.
// Images (bf16): low nibbles stay where they are, as the low mantissa bits of 128.0 (128 + u, u = w + 8); high nibbles
// move down one bit into the top mantissa bits of 8.0 (8 + u / 2); fp16: both go to the top mantissa bits of 16.0.
// Per scale group  out += scale * (P + offset * X)  as in the other kernels; the row sums X come from one extra MFMA
// per step (wavefront i of a set takes row tile i) and travel through LDS.
//
// A SIMD of this chip does not issue a wavefront's vector-ALU instructions while that wavefront's MFMA executes, but it
// does issue another wavefront's, so the workgroup has eight wavefronts in two sets of four, two per SIMD.  The sets
// share the tile; set 0 computes the even stages of the K range and set 1 the odd ones, side by side from two slots
// while memory is asked for the next two, one barrier per pair.  Both fold their share of a scale group with the
// group's parameters and their own row sums (the fold is linear).  Each wavefront must fit 256 registers, so nothing is
// requested across a stage boundary and a finished group is folded in a block of its own in front of the next stage
// (the other wavefront of the SIMD has matrix work meanwhile).  At the end the sets hand each other half of their totals
// through LDS, and each finishes 32 of the 64 rows.
// K may be split over S workgroups per tile (few tiles): all but the last store their float32 sums in register order
// into the workspace's zero zone, zero mapped to -0.0; the last one (highest index: dispatched after the others) polls
// until no word is zero, adds in chunk order, writes the output and restores the zeros (weight_quant_decode.hip).
// The chunks of a tile sit on one XCD and the collector says on which (a word per tile behind the sums): a producer
// that finds itself there leaves its sums in the shared L2 with ordinary stores, any other writes them through to memory.
#include "weight_quant_common.h"
#include "weight_quant_gemm4.h"

namespace mi355 {
namespace {

struct WqGemm4Args {
    const uint16_t *x, *scale, *offset, *bias;
    const void *w;
    uint16_t *out;
    uint32_t *zone;
    int64_t ldx, ldo;
    uint32_t ldw_bytes, row_bytes;
    int M, N, K;
    int gstages;                    // stages per scale group
    int grouped;
    int tiles_m, strips, S;
    int l2_exchange;                // producers on the collector's XCD leave their sums in the L2
    int max_polls;                  // bound of the collector's wait
    int only_chunk;                 // testing aid: c + 1 = only the workgroups of chunk c run
    uint32_t *status;               // the workspace's sticky status word
};

constexpr int kMaxPolls4 = 1 << 20;

// STAGE_GROUPS: a scale group is one stage, so every stage restarts the group's sums.
// WBITS == 8: the same kernel for int8 weights [K, N].  A weight row of the tile is then 256 bytes (256 columns), a stage
// 64 rows (two steps), and a wavefront owns one 128-byte half of the rows x one span of 16 dwords with all four bytes
// of its dwords: again four column tiles per lane (columns 128 s2 + 64 h + 4 c .. + 3), expanded with a byte-to-float
// conversion and a packing conversion per pair of weights (the weight is its own image, converted with its sign).
template <int ACT, bool STAGE_GROUPS, int WBITS = 4>
__global__ __launch_bounds__(512, 1) void wq_gemm4_kernel(const WqGemm4Args p)
{
    constexpr int SETS = 2, NW = 4 * SETS, BM = 64, BK = WBITS == 4 ? 128 : 64, SLOTS = 4;
    constexpr int STEPS = BK / 32;                             // MFMA steps of a stage
    constexpr int ROW_B = WBITS == 4 ? 128 : 256;              // bytes of a weight row inside the tile
    constexpr int A_BYTES = BM * BK * 2, R_BYTES = BK * ROW_B; // one stage of activations / raw weights
    constexpr int PRM_SLOT = 1024;                             // [256 scales | 256 offsets], 16 bits each
    constexpr int PRM_SLOTS = 8;                               // groups whose parameters are in LDS
    constexpr int SC1 = 16;                                    // cache-policy bit: agent scope
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    char *const raw = lds + SLOTS * A_BYTES;
    char *const prm = raw + SLOTS * R_BYTES;
    float *const xsum = reinterpret_cast<float *>(prm + PRM_SLOTS * PRM_SLOT);   // [SETS][2 slots][BM] row sums

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int set = wave >> 2, ws = wave & 3;
    const int h = ws & 1, jp = ws >> 1;
    // workgroups are dealt round-robin to the 8 XCDs.  The row blocks of a strip and the chunks of a tile sit on one
    // XCD (they share the strip resp. the activations in its L2); the last chunk has the tile's highest index.
    const int xcd_slot = blockIdx.x >> 3;
    const int j = xcd_slot / p.S, chunk = xcd_slot % p.S;
    const int strip = (blockIdx.x & 7) + 8 * (j / p.tiles_m);
    if (strip >= p.strips) return;
    if (p.only_chunk && chunk != (p.only_chunk < 0 ? p.S - 1 : p.only_chunk - 1)) return;      // testing aid (host-driven give-up of the collector)
    const int mb = j % p.tiles_m;
    const int tile = strip * p.tiles_m + mb;
    const int m0 = mb * BM;
    const int n0 = strip * 256;
    const int total_stages = p.K / BK;
    const int units = total_stages / p.gstages;                // K is split in whole scale groups
    const int u0 = (int)((int64_t)units * chunk / p.S), u1 = (int)((int64_t)units * (chunk + 1) / p.S);
    const int s0 = u0 * p.gstages, NSTG = (u1 - u0) * p.gstages;

    // ---- global -> LDS.  Activations: unit = 4 rows x 256 B; LDS slot l of a unit is (row l / 16, chunk l % 16) and
    // holds global chunk (l % 16) ^ (row & 15).  Raw weights: unit = 8 row slots x 128 B; row slot sl holds row
    // sl ^ ((sl >> 3) & 1) and its chunk slot j' holds chunk j' ^ (4 * ((row >> 4) & 1)): with that the four k octets a
    // wavefront reads together fall into four different quarters of the banks.
    // (int8: activation unit = 8 rows x 128 B, chunk slot l % 8 holds chunk (l % 8) ^ (row & 7); weight unit = 4 rows x
    // 256 B, chunk slot j' holds chunk j' ^ (4 * ((row >> 3) & 1)).)
    const int rows_a = min(BM, p.M - m0);
    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(p.x + (int64_t)m0 * p.ldx, (uint32_t)(((int64_t)(rows_a - 1) * p.ldx + p.K) * 2));
    const uint32_t strip_valid = min((uint32_t)ROW_B, p.row_bytes - (uint32_t)strip * (uint32_t)ROW_B);
    const __amdgpu_buffer_rsrc_t rsrc_w =
        make_rsrc(static_cast<const char *>(p.w) + (size_t)strip * ROW_B, (uint32_t)(p.K - 1) * p.ldw_bytes + strip_valid);
    const bool has_offset = p.offset != nullptr;
    const uint32_t param_bytes = (uint32_t)(p.grouped ? units : 1) * (uint32_t)p.N * 2u;
    const __amdgpu_buffer_rsrc_t rsrc_s = make_rsrc(p.scale, param_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_o = make_rsrc(has_offset ? p.offset : p.scale, param_bytes);
    // a stage's 32 load units are dealt to the eight wavefronts; the parameters of a scale group (the strip's 256 scales
    // and offsets) travel with its first stage, issued by the first wavefront of the set that computes that stage.
    // Nothing is issued past the end: the loop waits for vmcnt(0).  Stages are issued in order, so the group of the next
    // stage and its place in the group are counted along.
    int iss_grp = 0, iss_in = 0;
    auto issue_stage = [&](int s) {
        if (s >= NSTG) return;
        char *sa = lds + (s & 3) * A_BYTES, *sr = raw + (s & 3) * R_BYTES;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int u = i * NW + wave;
            if (WBITS == 4 || i == 0) {                        // int8: eight units of activations, one per wavefront
                const int row = WBITS == 4 ? 4 * u + (lane >> 4) : 8 * u + (lane >> 3);
                const uint32_t vo = WBITS == 4 ? (uint32_t)(row * (int)p.ldx * 2 + (((lane & 15) ^ (row & 15)) * 16))
                                               : (uint32_t)(row * (int)p.ldx * 2 + (((lane & 7) ^ (row & 7)) * 16));
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void *)(sa + u * 1024), 16, vo, (uint32_t)(s0 + s) * (uint32_t)(BK * 2), 0, 0);
            }
            if constexpr (WBITS == 4) {
                const int sl = 8 * u + (lane >> 3);
                const int row = sl ^ ((sl >> 3) & 1);
                const uint32_t ch = (uint32_t)((lane & 7) ^ (4 * ((row >> 4) & 1)));
                const uint32_t vo = ch * 16u < strip_valid ? (uint32_t)row * p.ldw_bytes + ch * 16u : kOutOfRange;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_void *)(sr + u * 1024), 16, vo,
                                                         (uint32_t)(s0 + s) * (uint32_t)BK * p.ldw_bytes, 0, kNonTemporal);
            } else {
                const int row = 4 * u + (lane >> 4);
                const uint32_t ch = (uint32_t)((lane & 15) ^ (4 * ((row >> 3) & 1)));
                const uint32_t vo = ch * 16u < strip_valid ? (uint32_t)row * p.ldw_bytes + ch * 16u : kOutOfRange;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_void *)(sr + u * 1024), 16, vo,
                                                         (uint32_t)(s0 + s) * (uint32_t)BK * p.ldw_bytes, 0, kNonTemporal);
            }
        }
        if (wave == 4 * (s & 1) && iss_in == 0) {
            const uint32_t ro = (uint32_t)(p.grouped ? u0 + iss_grp : 0) * (uint32_t)p.N * 2u + (uint32_t)n0 * 2u;
            char *dst = prm + (iss_grp & (PRM_SLOTS - 1)) * PRM_SLOT;
#pragma unroll
            for (int q = 0; q < 2; q++) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_s, (lds_void *)(dst + q * 256), 4, (uint32_t)lane * 4u, ro + q * 256u, 0, 0);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_o, (lds_void *)(dst + 512 + q * 256), 4, (uint32_t)lane * 4u, ro + q * 256u, 0, 0);
            }
        }
        if (++iss_in == p.gstages) {
            iss_in = 0;
            iss_grp++;
        }
    };

    // ---- LDS read addresses
    // raw: dword 16h + c of rows 8g + t; even t and odd t have their own base because odd octets swap row pairs
    // (int8: dword 32 s2 + 16 h + c of rows 8g + t, s2 = jp; rows of one parity of g share their banks: a two-way conflict
    // on reads that are a small part of the step)
    const int jch = WBITS == 4 ? (4 * h + (c >> 2)) ^ (4 * ((g >> 1) & 1)) : (8 * jp + 4 * h + (c >> 2)) ^ (4 * (g & 1));
    const int r_even = WBITS == 4 ? (8 * g + (g & 1)) * 128 + jch * 16 + (c & 3) * 4 : 8 * g * 256 + jch * 16 + (c & 3) * 4;
    const int r_odd = WBITS == 4 ? (8 * g + 1 - (g & 1)) * 128 + jch * 16 + (c & 3) * 4 : r_even + 256;
    // activations: row c of a row tile, chunk 4 ks + g, stored at chunk slot ((ks ^ (c >> 2)) << 2) | (g ^ (c & 3))
    // (int8: rows of 128 bytes, chunk slot (4 ks + g) ^ (c & 7))
    const int a_lane = WBITS == 4 ? c * 256 + ((c >> 2) << 6) + ((g ^ (c & 3)) << 4)
                                  : c * 128 + (((c >> 2) & 1) << 6) + ((g ^ (c & 3)) << 4);   // step ks: a_lane ^ (ks << 6)
    constexpr int A_TILE = 16 * BK * 2;                        // bytes of a row tile in a stage
    // byte offset of this lane's four columns in a parameter slot
    const int prm_col = WBITS == 4 ? (128 * h + 8 * c + 4 * jp) * 2 : (128 * jp + 64 * h + 4 * c) * 2;
    const uint32_t sel0 = 0x0c000c00u | ((4u + 2u * jp) << 16) | (2u * jp);      // byte 2jp of two rows
    const uint32_t sel1 = sel0 + 0x00010001u;                                    // byte 2jp + 1

    f32x4 P[4][4], tot[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int nb = 0; nb < 4; nb++) {
            P[i][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
            tot[i][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    f32x4 Xown = f32x4{0.f, 0.f, 0.f, 0.f};                    // row sums of row tile `ws`
    const u32x4 ones = u32x4{kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>};
    const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
    const BlendRegs br = blend_regs<ACT>();

    // fold of a finished group into the running total: tot += (scale * mul) * (P' + ((offset - bias) / mul) * X)
    float scm[4], ofm[4];
    f32x4 Xg[4];
    auto fetch_fold_operands = [&](int prm_slot, int xsum_slot) {
        const char *pb = prm + prm_slot * PRM_SLOT + prm_col;
        const uint32_t sr0 = *reinterpret_cast<const uint32_t *>(pb), sr1 = *reinterpret_cast<const uint32_t *>(pb + 4);
        const uint32_t or0 = *reinterpret_cast<const uint32_t *>(pb + 512), or1 = *reinterpret_cast<const uint32_t *>(pb + 516);
        const float *xs = xsum + xsum_slot * BM + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) Xg[i] = *reinterpret_cast<const f32x4 *>(xs + 16 * i);
        const float sc[4] = {act_lo<ACT>(sr0), act_hi<ACT>(sr0), act_lo<ACT>(sr1), act_hi<ACT>(sr1)};
        const float of[4] = {has_offset ? act_lo<ACT>(or0) : 0.f, has_offset ? act_hi<ACT>(or0) : 0.f,
                             has_offset ? act_lo<ACT>(or1) : 0.f, has_offset ? act_hi<ACT>(or1) : 0.f};
#pragma unroll
        for (int nb = 0; nb < 4; nb++) {
            const float mul = WBITS == 8 ? 1.0f : (nb & 1) ? kMulHi4<ACT> : kMulLo4<ACT>;
            const float bias = WBITS == 8 ? kImageBias<8> : (nb & 1) ? kBiasHi4<ACT> : kBiasLo4<ACT>;
            scm[nb] = sc[nb] * mul;
            ofm[nb] = (of[nb] - bias) * (1.0f / mul);
        }
    };
    auto fold_tile = [&](int i, int nb) {
#pragma unroll
        for (int q = 0; q < 4; q++) tot[i][nb][q] = __builtin_fmaf(scm[nb], __builtin_fmaf(ofm[nb], Xg[i][q], P[i][nb][q]), tot[i][nb][q]);
    };

    // ---- operands of a step, all from the stage's own slots (a set's next stage is not complete in LDS before the next
    // barrier; the other wavefront of the SIMD covers the latency at the start of a stage): raw dwords are requested two
    // steps ahead (they are expanded one step ahead, between the MFMAs of the step before), activation fragments one
    // step ahead, each into the registers of the fragment that was just used
    uint32_t w[8];
    u32x4 AF[4], AX, b[2][4];
    auto read_w = [&](const char *sr, int ks) {
#pragma unroll
        for (int t = 0; t < 8; t++)
            w[t] = *reinterpret_cast<const uint32_t *>(sr + ks * (32 * ROW_B) + ((t & 1) ? r_odd : r_even) + (t >> 1) * (2 * ROW_B));
    };
    auto read_a = [&](const char *sa, int ks, int i) { return *reinterpret_cast<const u32x4 *>(sa + i * A_TILE + (a_lane ^ (ks << 6))); };
    auto expand = [&](u32x4 (&bn)[4]) {
        if constexpr (WBITS == 8) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const uint32_t wa = w[2 * v], wb = w[2 * v + 1];
#pragma unroll
                for (int nb = 0; nb < 4; nb++)
                    bn[nb][v] = pack_act2<ACT>(sbyte_f32(wa, nb), sbyte_f32(wb, nb));
            }
            return;
        }
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const uint32_t t0 = __builtin_amdgcn_perm(w[2 * v + 1], w[2 * v], sel0);
            const uint32_t t1 = __builtin_amdgcn_perm(w[2 * v + 1], w[2 * v], sel1);
            uint32_t e0, e1, e2, e3;
            expand_byte<ACT>(t0, br.mask_lo, br.c_lo, br.mask_hi, br.c_hi, e0, e1);
            expand_byte<ACT>(t1, br.mask_lo, br.c_lo, br.mask_hi, br.c_hi, e2, e3);
            bn[0][v] = e0;
            bn[1][v] = e1;
            bn[2][v] = e2;
            bn[3][v] = e3;
        }
    };
    // one step of 32 k: the MFMAs of step ks with the expansion of step ks + 1 spread between them
    auto step = [&](const bool restart /* the sums start from the MFMA's zero operand */, const int ks, const char *sa, const char *sr) {
        u32x4(&bc)[4] = b[ks & 1];
        if (ks + 1 < STEPS) expand(b[(ks + 1) & 1]);
        if (ks + 2 < STEPS) read_w(sr, ks + 2);
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int nb = 0; nb < 4; nb++) P[i][nb] = mfma_act<ACT>(AF[i], bc[nb], restart ? zero4 : P[i][nb]);
            if (ks + 1 < STEPS) AF[i] = read_a(sa, ks + 1, i);
        }
        Xown = mfma_act<ACT>(AX, ones, Xown);
        if (ks + 1 < STEPS) AX = read_a(sa, ks + 1, ws);
        // interleave: one MFMA, its share of the integer work, one LDS read
#pragma unroll
        for (int r = 0; r < 17; r++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    };

    // split K: the workgroup that collects a tile's sums says at its start on which XCD it runs (a word behind the
    // exchange area).  A producer on the same XCD shares its L2 and may leave its sums there with ordinary stores, which
    // are acknowledged in a fifth of the time of stores that write through to memory; the collector's polls bypass the
    // vector L1 and see either.
    constexpr uint32_t WAVE_BYTES = 16 * 64 * 16, TILE_BYTES = 4 * WAVE_BYTES;
    const uint32_t tiles = (uint32_t)(p.tiles_m * p.strips);
    const uint32_t flag_base = (uint32_t)(p.S - 1) * tiles * TILE_BYTES;
    const __amdgpu_buffer_rsrc_t rsrc_z = make_rsrc(p.zone, p.S > 1 ? flag_base + tiles * 4u : 0u);
    const uint32_t my_xcd = __builtin_amdgcn_s_getreg(kHwRegXccId) + 1u;
    if (p.S > 1 && chunk == p.S - 1 && threadIdx.x == 0)
        __builtin_amdgcn_raw_buffer_store_b32(my_xcd, rsrc_z, (uint32_t)tile * 4u, flag_base, SC1);

    // ---- main loop: stages 2 it and 2 it + 1 are computed side by side from two slots while memory is asked for the
    // next two; one barrier per pair.  The barrier is issued without the fences of __syncthreads(): the explicit wait
    // above it is what the fence would have to do.
    bool pending = false;
    int pending_prm = 0, pending_x = 0;
    issue_stage(0);
    issue_stage(1);
    int own = 0;
    // group of the set's current stage and the stage's place in it (no divisions in the loop)
    int grp = STAGE_GROUPS ? set : set / p.gstages, in_grp = STAGE_GROUPS ? 0 : set - grp * p.gstages;
    for (int it = 0; 2 * it < NSTG; it++) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();                          // this pair is complete in LDS; everyone is done with the pair before
        asm volatile("" ::: "memory");
        issue_stage(2 * it + 2);
        issue_stage(2 * it + 3);
        const int s = 2 * it + set;
        if (s >= NSTG) continue;
        const char *sa = lds + (s & 3) * A_BYTES, *sr = raw + (s & 3) * R_BYTES;
        read_w(sr, 0);
#pragma unroll
        for (int i = 0; i < 4; i++) AF[i] = read_a(sa, 0, i);
        AX = read_a(sa, 0, ws);
        if (pending) {
            // the other wavefront of the SIMD has matrix work for the time of this fold
            fetch_fold_operands(pending_prm, pending_x);
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int nb = 0; nb < 4; nb++) {
                    fold_tile(i, nb);
                    if (!STAGE_GROUPS) P[i][nb] = zero4;       // otherwise the next step restarts the sums
                }
        }
        expand(b[0]);
        if (STEPS > 1) read_w(sr, 1);
        __builtin_amdgcn_sched_barrier(0);
        // Compile time, not a branch: two copies of the step behind a branch cost a hundred registers, so groups of several
        // stages clear the sums after the fold instead.
        step(STAGE_GROUPS, 0, sa, sr);
#pragma unroll
        for (int ks = 1; ks < STEPS; ks++) {
            __builtin_amdgcn_sched_barrier(0);
            step(false, ks, sa, sr);
        }
        __builtin_amdgcn_sched_barrier(0);
        // the set's share of a group ends with its last stage inside the group
        int next_grp = grp + (STAGE_GROUPS ? 2 : 0), next_in = in_grp + (STAGE_GROUPS ? 0 : 2);
        if (!STAGE_GROUPS)
            for (int r = 0; r < 2; r++)
                if (next_in >= p.gstages) {
                    next_in -= p.gstages;
                    next_grp++;
                }
        const bool last_of_group = s + 2 >= NSTG || next_grp != grp;
        pending = last_of_group;
        pending_prm = grp & (PRM_SLOTS - 1);
        grp = next_grp;
        in_grp = next_in;
        pending_x = 2 * set + (own & 1);
        if (last_of_group) {
            if (c == 0) *reinterpret_cast<f32x4 *>(xsum + pending_x * BM + ws * 16 + 4 * g) = Xown;   // read after the next barrier
            Xown = zero4;
            own++;
        }
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    uint32_t collector_xcd = 0;
    if (p.S > 1 && chunk < p.S - 1) collector_xcd = __builtin_amdgcn_raw_buffer_load_b32(rsrc_z, (uint32_t)tile * 4u, flag_base, SC1);   // used after the fold
    if (pending) {
        fetch_fold_operands(pending_prm, pending_x);
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int nb = 0; nb < 4; nb++) fold_tile(i, nb);
    }

    // each wavefront finishes NE = 8 of its 16 register tiles: the half of the rows that the sets hand each other through
    // LDS (set 1 keeps row tiles 2 and 3 and moves them to the front)
    constexpr int NE = 16 / SETS, NI = NE / 4;
    {
        // the stage slots are free
        f32x4 *red = reinterpret_cast<f32x4 *>(lds) + ws * 16 * 64 + lane;
        if (set == 0) {
#pragma unroll
            for (int e = NE; e < 16; e++) red[e * 64] = tot[e >> 2][e & 3];
        } else {
#pragma unroll
            for (int e = 0; e < NE; e++) red[e * 64] = tot[e >> 2][e & 3];
        }
        __syncthreads();
        if (set == 0) {
#pragma unroll
            for (int e = 0; e < NE; e++) tot[e >> 2][e & 3] += red[e * 64];
        } else {
#pragma unroll
            for (int e = 0; e < NE; e++) tot[e >> 2][e & 3] = red[(e + NE) * 64] + tot[(e + NE) >> 2][e & 3];
        }
    }
    const int e_first = set * NE;                              // register tile e of this wavefront is tile e_first + e of the 16

    // ---- split K: exchange in register order through the zero zone
    if (p.S > 1) {
        const uint32_t lane_off = (uint32_t)tile * TILE_BYTES + (uint32_t)ws * WAVE_BYTES + (uint32_t)e_first * 1024u + (uint32_t)lane * 16u;
        if (chunk < p.S - 1) {
            const bool same_l2 = p.l2_exchange && __builtin_amdgcn_readfirstlane(collector_xcd) == my_xcd;
            u32x4 bits[NE];
#pragma unroll
            for (int e = 0; e < NE; e++) {
                bits[e] = __builtin_bit_cast(u32x4, tot[e >> 2][e & 3]);
#pragma unroll
                for (int q = 0; q < 4; q++) bits[e][q] = bits[e][q] == 0u ? 0x80000000u : bits[e][q];   // no stored word is zero
            }
            // one branch around all stores, not one per store: a 16-byte store that ends a basic block may be followed, in the
            // block the code falls into, by an instruction that overwrites its data registers before the store has read them
            // (the compiler's wait states for that hazard do not reach across the block boundary)
            if (same_l2) {
#pragma unroll
                for (int e = 0; e < NE; e++)
                    buffer_store_b128<0>(bits[e], rsrc_z, lane_off + e * 1024, (uint32_t)chunk * tiles * TILE_BYTES);
            } else {
#pragma unroll
                for (int e = 0; e < NE; e++)
                    buffer_store_b128<SC1>(bits[e], rsrc_z, lane_off + e * 1024, (uint32_t)chunk * tiles * TILE_BYTES);
            }
            return;
        }
        // the sums of up to CB chunks are asked for together and added in chunk order: ((c0 + c1) + ...) + own
        constexpr int CB = 3;
        bool first = true, gave_up = false;
        for (int c0 = 0; c0 < p.S - 1; c0 += CB) {
            u32x4 v[CB][NE];
#pragma unroll
            for (int i = 0; i < CB; i++)
#pragma unroll
                for (int e = 0; e < NE; e++)
                    v[i][e] = c0 + i < p.S - 1 ? __builtin_amdgcn_raw_buffer_load_b128(rsrc_z, lane_off + e * 1024, (uint32_t)(c0 + i) * tiles * TILE_BYTES, SC1)
                                               : u32x4{1u, 1u, 1u, 1u};
            bool missing = true;
            for (int poll = 0; poll < p.max_polls && missing; poll++) {
                missing = false;
                // the polls must be real loads: without a compiler barrier a reload with the operands of the first request is
                // folded into it, and a wavefront that arrived before the data would spin on a stale register until the bound
                asm volatile("" ::: "memory");
#pragma unroll
                for (int i = 0; i < CB; i++)
#pragma unroll
                    for (int e = 0; e < NE; e++)
                        if (v[i][e][0] == 0u || v[i][e][1] == 0u || v[i][e][2] == 0u || v[i][e][3] == 0u) {
                            v[i][e] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_z, lane_off + e * 1024, (uint32_t)(c0 + i) * tiles * TILE_BYTES, SC1);
                            missing = true;
                        }
            }
            gave_up = gave_up || missing;
#pragma unroll
            for (int i = 0; i < CB; i++) {
                if (c0 + i >= p.S - 1) break;
#pragma unroll
                for (int e = 0; e < NE; e++) {
                    if (first) P[e >> 2][e & 3] = __builtin_bit_cast(f32x4, v[i][e]);
                    else P[e >> 2][e & 3] += __builtin_bit_cast(f32x4, v[i][e]);
                }
                first = false;
            }
        }
#pragma unroll
        for (int e = 0; e < NE; e++) tot[e >> 2][e & 3] = P[e >> 2][e & 3] + tot[e >> 2][e & 3];
        if (gave_up) {
            // the wait for the other chunks ran out: the result is marked (NaN), not guessed, and the host is told through
            // the workspace's sticky status word (mi355_workspace_status)
            const float nan = __uint_as_float(0x7fc00000u);
#pragma unroll
            for (int e = 0; e < NE; e++) tot[e >> 2][e & 3] = f32x4{nan, nan, nan, nan};
            *p.status = kStatusExchangeTimeout;
        }
        // the zone goes back to zero for the next launch (no branches around the stores: nothing waits for them).  Ordinary
        // stores: the next launch is what must see them, and a write-through store to a line that a producer left modified
        // in the L2 takes several times as long
        for (int ch = 0; ch < p.S - 1; ch++)
#pragma unroll
            for (int e = 0; e < NE; e++)
                buffer_store_b128<0>(u32x4{0u, 0u, 0u, 0u}, rsrc_z, lane_off + e * 1024, (uint32_t)ch * tiles * TILE_BYTES);
        if (threadIdx.x == 0) __builtin_amdgcn_raw_buffer_store_b32(0u, rsrc_z, (uint32_t)tile * 4u, flag_base, 0);
    }

    // ---- output: lane (c, g) holds rows 16 i + 4 g + q, columns 128 h + 8 c + 4 jp .. + 3: 8 bytes per row
    const int col = WBITS == 4 ? n0 + 128 * h + 8 * c + 4 * jp : n0 + 128 * jp + 64 * h + 4 * c;
    if (col >= p.N) return;                                    // N is a multiple of 8 (int8: of 4): the four columns are inside or outside
    float bv[4];
#pragma unroll
    for (int nb = 0; nb < 4; nb++) bv[nb] = p.bias ? act_1<ACT>(p.bias[col + nb]) : 0.0f;
    const bool out_vec = (p.ldo & 3) == 0 && aligned_dev(p.out, 8);
#pragma unroll
    for (int i = 0; i < NI; i++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int row = m0 + (i + set * NI) * 16 + 4 * g + q;
            if (row >= p.M) continue;
            const uint32_t lo = pack_act2<ACT>(tot[i][0][q] + bv[0], tot[i][1][q] + bv[1]);
            const uint32_t hi = pack_act2<ACT>(tot[i][2][q] + bv[2], tot[i][3][q] + bv[3]);
            uint16_t *o = p.out + (int64_t)row * p.ldo + col;
            if (out_vec) {
                *reinterpret_cast<uint2 *>(o) = uint2{lo, hi};
            } else {
                o[0] = (uint16_t)(lo & 0xffffu);
                o[1] = (uint16_t)(lo >> 16);
                o[2] = (uint16_t)(hi & 0xffffu);
                o[3] = (uint16_t)(hi >> 16);
            }
        }
}

template <int ACT, bool STAGE_GROUPS, int WBITS>
int launch4(const WqGemm4Args &p, unsigned grid, hipStream_t s)
{
    // four slots of activations (64 rows x 128 / 64 k) and raw weights (16 KiB either way), parameters, row sums
    constexpr size_t lds_bytes = (size_t)4 * 64 * (WBITS == 4 ? 256 : 128) + 4 * 16384 + 8 * 1024 + 2 * 2 * 64 * 4;
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");
    auto kern = wq_gemm4_kernel<ACT, STAGE_GROUPS, WBITS>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds_bytes, s, p);
    return check_launch();
}

} // namespace

WqGemm4Plan make_wq_gemm4_plan(int64_t M, int64_t N, int64_t K, int w_bits, int64_t group_size, int64_t ldw_k, int64_t ldx,
                               const void *x, const void *w, const void *scale, const void *offset)
{
    WqGemm4Plan pl{};
    // int4: rows of N / 8 words, 128-row stages, 128-byte strips; int8: rows of N bytes, 64-row stages, 256-byte strips
    const int64_t row_bytes = w_bits == 4 ? N / 2 : N, ldw_bytes = w_bits == 4 ? ldw_k * 4 : ldw_k;
    const int64_t bk = w_bits == 4 ? 128 : 64, strip_bytes = w_bits == 4 ? 128 : 256;
    const int64_t group = group_size > 0 ? group_size : K;
    const bool grouped = group_size > 0 && group != K;
    pl.ok = knob(kKnobWqGemm4Off) != 1 && (w_bits == 4 || w_bits == 8) && M > 32 && K >= 128 && K % 128 == 0 &&
            N % (w_bits == 4 ? 8 : 4) == 0 && (!grouped || group % bk == 0) &&
            ldw_bytes >= row_bytes && ldw_bytes % 16 == 0 && ldx % 8 == 0 && (x == nullptr || aligned(x, 16)) &&
            (w == nullptr || aligned(w, 16)) && (scale == nullptr || aligned(scale, 4)) && (offset == nullptr || aligned(offset, 4)) &&
            (uint64_t)K * (uint64_t)ldw_bytes < (1ull << 31) && (uint64_t)128 * (uint64_t)ldx * 2 + (uint64_t)K * 2 < (1ull << 31) &&
            (uint64_t)(K / group) * (uint64_t)N * 2 < (1ull << 31) && M <= 0x7fffffff;
    if (!pl.ok) return pl;
    pl.strips = (int)((row_bytes + strip_bytes - 1) / strip_bytes);
    const int64_t stages = K / bk;
    const int64_t units = grouped ? K / group : stages;
    // few tiles: split K in whole scale groups (per channel: in equal numbers of stages)
    pl.bm = 64;
    pl.tiles_m = (int)((M + pl.bm - 1) / pl.bm);
    const int64_t tiles = (int64_t)pl.tiles_m * pl.strips;
    int64_t S = tiles < kNumCU ? kNumCU / tiles : 1;
    if (S > units) S = units;
    if (S > 8) S = 8;
    if (const int f = knob(kKnobWqgSplit))
        if (f >= 1 && f <= units) S = f;
    // the sums of S - 1 chunks per tile and one word per tile (the XCD of its collector)
    auto zone = [&](int64_t s) { return (uint64_t)(s - 1) * (uint64_t)tiles * (uint64_t)pl.bm * 256u * 4u + (uint64_t)tiles * 4u; };
    while (S > 1 && (zone(S) > kWorkspaceZoneBytes || (!grouped && stages % S != 0))) S--;
    pl.S = (int)S;
    // per channel: one fold per workgroup, so a "group" is the workgroup's whole range
    pl.gstages = (int)(grouped ? group / bk : stages / S);
    pl.zone_bytes = pl.S > 1 ? (size_t)zone(pl.S) : 0;
    if (tiles * pl.S > 0x7fffffff) pl.ok = false;
    return pl;
}

int launch_wq_gemm4(const WqGemm4Plan &plan, const void *x, int act_f16, const void *w, int w_bits, const void *scale,
                    const void *offset, const void *bias, void *out, int64_t M, int64_t N, int64_t K, int64_t group_size, int64_t ldx,
                    int64_t ldw_k, int64_t ldo, void *workspace, void *stream)
{
    WqGemm4Args p{};
    p.x = static_cast<const uint16_t *>(x);
    p.w = w;
    p.scale = static_cast<const uint16_t *>(scale);
    p.offset = static_cast<const uint16_t *>(offset);
    p.bias = static_cast<const uint16_t *>(bias);
    p.out = static_cast<uint16_t *>(out);
    p.zone = plan.S > 1 ? reinterpret_cast<uint32_t *>(static_cast<char *>(workspace) + kWorkspaceCounterCapacity) : nullptr;
    p.ldx = ldx;
    p.ldo = ldo;
    p.ldw_bytes = (uint32_t)(w_bits == 4 ? ldw_k * 4 : ldw_k);
    p.row_bytes = (uint32_t)(w_bits == 4 ? N / 2 : N);
    p.M = (int)M;
    p.N = (int)N;
    p.K = (int)K;
    p.gstages = plan.gstages;
    p.grouped = group_size > 0 && group_size != K;
    p.tiles_m = plan.tiles_m;
    p.strips = plan.strips;
    p.S = plan.S;
    p.l2_exchange = knob(kKnobWqGemm4Off) != 2;
    p.max_polls = knob(kKnobWqMaxPolls) > 0 ? knob(kKnobWqMaxPolls) : kMaxPolls4;
    p.only_chunk = knob(kKnobWqOnlyChunk);
    p.status = plan.S > 1 ? reinterpret_cast<uint32_t *>(static_cast<char *>(workspace) + kWorkspaceStatusOffset) : nullptr;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t tiles = (int64_t)plan.tiles_m * plan.strips;
    (void)tiles;
    const unsigned grid = (unsigned)((plan.strips + 7) / 8 * 8 * plan.tiles_m * plan.S);
    if (w_bits == 8) return act_f16 ? launch4<1, false, 8>(p, grid, s) : launch4<0, false, 8>(p, grid, s);
    // int4: a variant of its own where a scale group is one stage
    if (p.grouped && plan.gstages == 1) return act_f16 ? launch4<1, true, 4>(p, grid, s) : launch4<0, true, 4>(p, grid, s);
    return act_f16 ? launch4<1, false, 4>(p, grid, s) : launch4<0, false, 4>(p, grid, s);
}

} // namespace mi355
