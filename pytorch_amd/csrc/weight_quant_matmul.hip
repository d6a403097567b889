// npu_weight_quant_batchmatmul for gfx950: bf16 activations x int8 / packed-int4 weights.
//
// The job is weight streaming: every weight byte is read from HBM once, expanded in registers
// and fed to the bf16 MFMA; activations are tiny and stay in cache.
//
// Exact integer weights, float32 scaling.  Rounding (w + offset) * scale to bf16 before the
// MFMA would cost ~2^-9 relative error per product; instead the MFMA multiplies x by an exact
// bf16 image of the integer weight and the antiquant parameters are applied to the float32
// partial sums:
//     out[m,n] = sum_g scale[g,n] * ( P_g[m,n] + offset[g,n] * X_g[m] ),
//     P_g = sum_{k in g} x[m,k] * w[k,n],   X_g = sum_{k in g} x[m,k]
// (X_g comes from one extra MFMA against a vector of ones).
//
// Weight images (chosen so the expansion is a few bit operations per pair of weights):
//   int8 : the weight itself, byte i of a word converted with its sign in one instruction (v_cvt_f32_i32 with a
//          sign-extending byte select) and packed to bf16 (exact: 8 significant bits);  P = P'.
//   int4 : nibble ^ 8 = w + 8 = u in [0,15] is placed in mantissa bits 3..6 of the bf16
//          pattern 0x4100, i.e. the value 8 + u/2 = (w + 24) / 2;  P = 2 P' - 24 X.
//
// Operand mapping.  The weight row is contiguous along N, while an MFMA operand lane wants 8
// consecutive k of ONE column.  A lane therefore takes the same dword column from 8 different
// k rows and one MFMA is issued per byte/nibble position of the dword: MFMA #i covers the
// strided column set { elems_per_dword * dword_column + i }, which only changes the index
// bookkeeping of the epilogue.  The order of k inside a lane's operand is free as long as the
// activation operand uses the same order.
//
// Streaming.  A wavefront owns a 128-byte-wide column strip of the weight (one cache line per row)
// and a contiguous range of K; it loads 32 rows per step straight into registers in the operand
// layout (lane (c, g) takes 8 bytes at column 8c of rows 8g .. 8g+7, so one load instruction covers
// four full cache lines) and keeps PF steps in flight.  The wavefronts of a workgroup cover W
// adjacent strips (W * 128 contiguous bytes of every row: strips streamed side by side keep the
// DRAM pages of a row busy together, which measures close to a linear read) times KS slices of
// the workgroup's K chunk; there is no barrier in the main loop.  Activations and antiquant
// parameters are small, stay in cache and are loaded by every wavefront that needs them.
// Partial sums are reduced over the K slices in LDS; when K is split over several workgroups
// (to occupy all CUs when there are few strips) each workgroup writes its float32 partial to the
// workspace and the workgroup that arrives last at a per-tile counter adds them in chunk order,
// which keeps the result independent of scheduling.
#include "weight_quant_kmajor_decode.h"
#include "weight_quant_common.h"
#include "weight_quant_gemm.h"
#include "weight_quant_kpacked.h"
#include "weight_quant_kpacked_decode.h"
#include "weight_quant_decode.h"
#include "weight_quant_gemm4.h"
#include "weight_quant_repack.h"
#include <type_traits>

namespace mi355 {
namespace {

// One step of a wavefront: 32 weight rows of its strip (8 bytes per lane and row).
// The loads are unconditional so that the main loop stays free of branches around memory instructions (the
// compiler then tracks the outstanding loads exactly); a step past the end of the wavefront's range is given a
// lane offset beyond every buffer size instead, which makes the loads return zero without touching memory.
template <int POLICY>
__device__ __forceinline__ void load_step(u32x2 (&wq)[8], const __amdgpu_buffer_rsrc_t rsrc_w, const uint32_t voff_w,
                                          const uint32_t ldw_bytes, const uint32_t krow, const bool valid)
{
    const uint32_t vw = valid ? voff_w : kOutOfRange;
#pragma unroll
    for (int t = 0; t < 8; t++) wq[t] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, vw, (krow + t) * ldw_bytes, POLICY);
}

// Antiquant parameters of one group for this lane's NPV * 8 consecutive columns.
template <int NPV>
__device__ __forceinline__ void load_params(u32x4 (&sv)[NPV], u32x4 (&ov)[NPV], const __amdgpu_buffer_rsrc_t rsrc_s,
                                            const __amdgpu_buffer_rsrc_t rsrc_o, const bool has_offset,
                                            const uint32_t voff_p, const uint32_t row_off)
{
#pragma unroll
    for (int v = 0; v < NPV; v++) {
        sv[v] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, voff_p + 16u * v, row_off, 0);
        // no offsets: rsrc_o aliases the scales and the loaded values are masked away (no branch around the load)
        ov[v] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_o, voff_p + 16u * v, row_off, 0) & (has_offset ? ~0u : 0u);
    }
}

// Fold one finished group into the running total: tot += (scale * P_MUL) * (P' + ((offset - X_BIAS) / P_MUL) * X);
// both rescalings are exact (powers of two).  Lane (c, g) holds accumulator rows 4g + q; with a single activation
// row only q = 0 of g = 0 is ever stored, so the other components are left alone.
template <int WBITS, int ACT, int MT, int NT, int NPV>
__device__ __forceinline__ void fold_group(f32x4 (&tot)[MT][NT], f32x4 (&P)[MT][NT], f32x4 (&X)[MT], const u32x4 (&sv)[NPV],
                                           const u32x4 (&ov)[NPV], const bool one_row)
{
    constexpr float P_MUL = kImageMul<WBITS, ACT>;
    constexpr float X_BIAS = kImageBias<WBITS>;
#pragma unroll
    for (int i = 0; i < NT; i++) {
        const uint32_t su = sv[i / 8][(i % 8) / 2], ou = ov[i / 8][(i % 8) / 2];
        const float sc = ((i & 1) ? act_hi<ACT>(su) : act_lo<ACT>(su)) * P_MUL;
        const float of = (((i & 1) ? act_hi<ACT>(ou) : act_lo<ACT>(ou)) - X_BIAS) * (1.0f / P_MUL);
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            const float inner0 = __builtin_fmaf(of, X[mt][0], P[mt][i][0]);
            tot[mt][i][0] = __builtin_fmaf(sc, inner0, tot[mt][i][0]);
            if (!one_row) {
#pragma unroll
                for (int q = 1; q < 4; q++) {
                    const float inner = __builtin_fmaf(of, X[mt][q], P[mt][i][q]);
                    tot[mt][i][q] = __builtin_fmaf(sc, inner, tot[mt][i][q]);
                }
            }
        }
    }
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        X[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < NT; i++) P[mt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
}

// BS: steps per loop body (every wavefront's range and every scale group is a whole number of bodies);
// PF: steps kept in flight (PF divides BS or equals it);
// ACCUM: a wavefront may meet more than one scale group, so finished groups are folded into a running total
// inside the loop.  Without it (per channel, or at most one group per wavefront) the single fold happens after
// the loop and the loop carries half as many accumulators.
template <int WBITS, int ACT, int MT, int W, int KS, int BS, int PF, bool ACCUM>
__global__ __launch_bounds__(W * KS * 64) void wq_stream_kernel(const WqArgs p)
{
    static_assert(BS % PF == 0, "the register ring must divide the loop body");
    // with one m tile the weights are read exactly once; with more, other workgroups read the same strip again
    constexpr int POLICY = MT == 1 ? kNonTemporal : 0;
    constexpr int EPD = 32 / WBITS;            // elements per dword
    constexpr int NB = 32 * EPD;               // columns per strip (128 bytes of a weight row)
    constexpr int NT = 2 * EPD;                // MFMA column sets per lane (it holds 2 dword columns)
    constexpr int NPV = NT / 8;                // 16-byte vectors of bf16 parameters per lane
    constexpr int NBW = W * NB;                // columns of the workgroup's tile
    constexpr int THREADS = W * KS * 64;
    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int wstrip = wave % W, kslice = wave / W;
    // workgroups are dealt round-robin to the 8 XCDs: keep the S chunks of a tile on one XCD
    const int xcd_slot = blockIdx.x >> 3;
    const int sgrp = (blockIdx.x & 7) + 8 * (xcd_slot / p.S);
    const int chunk = xcd_slot % p.S;
    if (sgrp >= p.sgroups) return;
    const int strip = sgrp * W + wstrip;
    const int m_base = blockIdx.y * (MT * 16);
    const int rows_valid = min(MT * 16, p.M - m_base);

    // contiguous range of K units for this (chunk, slice); a wavefront whose strip lies past the row has none
    const int R = p.S * KS, r = chunk * KS + kslice;
    const int u0 = (int)((int64_t)p.n_units * r / R), u1 = (int)((int64_t)p.n_units * (r + 1) / R);
    const int step0 = u0 * p.unit_steps;
    const int nsteps = strip < p.strips ? (u1 - u0) * p.unit_steps : 0;
    const int ustep = p.grouped ? p.unit_steps : nsteps;   // steps between folds

    // lanes past the end of the row read (and discard) the first bytes of the row instead
    const bool lane_ok = (uint32_t)strip * 128u + (uint32_t)c * 8u < p.row_bytes;
    const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(p.w, (uint32_t)((uint64_t)(p.K - 1) * p.ldw_bytes + p.row_bytes));
    const uint32_t voff_w = (uint32_t)(8 * g) * p.ldw_bytes + (lane_ok ? (uint32_t)strip * 128u + (uint32_t)c * 8u : 0u);
    // lane (c, g) owns columns strip * NB + (2c) * EPD .. + NT - 1
    const bool has_offset = p.offset != nullptr;
    const uint32_t param_bytes = (uint32_t)(p.grouped ? p.n_units : 1) * (uint32_t)p.N * 2u;
    const __amdgpu_buffer_rsrc_t rsrc_s = make_rsrc(p.scale, param_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_o = make_rsrc(has_offset ? p.offset : p.scale, param_bytes);
    const uint32_t voff_p = lane_ok ? (uint32_t)(strip * NB + 2 * c * EPD) * 2u : 0u;
    const uint32_t param_pitch = (uint32_t)p.N * 2u;

    f32x4 tot[MT][NT], P[MT][NT], X[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        X[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < NT; i++) {
            if constexpr (ACCUM) tot[mt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
            P[mt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    const u32x4 ones = u32x4{kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>};
    uint32_t magic;
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "n"(kInt4Magic<ACT>));   // opaque to the optimiser: stays in a VGPR
    const bool one_row = MT == 1 && rows_valid == 1;

    // register ring: PF steps of weights and activations in flight, the next group's parameters behind them
    u32x2 wq[PF][8];
    u32x4 sv[NPV], ov[NPV], sv_next[NPV], ov_next[NPV];
#pragma unroll
    for (int v = 0; v < NPV; v++) sv[v] = ov[v] = u32x4{0u, 0u, 0u, 0u};
    // scale group of the loop body that follows the current one (parameters are requested a body ahead; per
    // channel, and inside a group, that re-reads the same cached row, which keeps the loop free of branches)
    const int grp_last = p.grouped ? u1 - 1 : 0;
    const int gstep = p.grouped ? p.unit_steps : 0x7fffffff;
    int grp_next = p.grouped ? u0 : 0, next_in_unit = 0;
    load_params<NPV>(sv_next, ov_next, rsrc_s, rsrc_o, has_offset, voff_p, (uint32_t)grp_next * param_pitch);
#pragma unroll
    for (int j = 0; j < PF; j++)
        load_step<POLICY>(wq[j], rsrc_w, voff_w, p.ldw_bytes, (uint32_t)(step0 + j) * 32u, j < nsteps);

    // The activations of the workgroup's K chunk go to LDS once, already in MFMA operand order: the fragment of
    // (step, m tile) is 1 KiB, lane (c, g) finds x[m tile * 16 + c][32 * step + 8g .. + 7] at lane * 16.  The global
    // side reads whole rows (consecutive threads take consecutive 16-byte pieces of one row).  Rows past the last
    // valid one stay unwritten: they only feed accumulator rows that are never stored.
    const int cu0 = (int)((int64_t)p.n_units * (chunk * KS) / R), cu1 = (int)((int64_t)p.n_units * (chunk * KS + KS) / R);
    const int cstep0 = cu0 * p.unit_steps;
    const int pieces = (cu1 - cu0) * p.unit_steps * 4;      // 16-byte pieces per activation row
    char *xs = lds + 16;
    {
        // rows are dealt to the wavefronts, the lanes walk along a row; the loads of a lane are independent of
        // its LDS stores, so they all go out before the first one is needed
        const uint16_t *xsrc = p.x + (int64_t)m_base * p.ldx + (int64_t)cstep0 * 32;
        for (int r = wave; r < rows_valid; r += W * KS) {
            const uint16_t *xrow = xsrc + (int64_t)r * p.ldx;
            char *dst = xs + (((r >> 4) * 64 + (r & 15)) << 4);
#pragma unroll 4
            for (int q = lane; q < pieces; q += 64) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(xrow + q * 8);
                *reinterpret_cast<u32x4 *>(dst + ((((q >> 2) * MT) * 64 + (q & 3) * 16) << 4)) = v;
            }
        }
    }
    __syncthreads();
    const char *xw = xs + ((size_t)(step0 - cstep0) * MT * 64 + lane) * 16;   // this wavefront's first fragment

    int in_unit = 0;
#pragma unroll 1
    for (int s = 0; s < nsteps; s += BS) {
#pragma unroll
        for (int v = 0; v < NPV; v++) sv[v] = sv_next[v], ov[v] = ov_next[v];
        next_in_unit += BS;
        if (next_in_unit == gstep) next_in_unit = 0, grp_next = min(grp_next + 1, grp_last);
        load_params<NPV>(sv_next, ov_next, rsrc_s, rsrc_o, has_offset, voff_p, (uint32_t)grp_next * param_pitch);
#pragma unroll
        for (int j = 0; j < BS; j++) {
            const int slot = j % PF;
            uint32_t w0[8], w1[8];
#pragma unroll
            for (int t = 0; t < 8; t++) {
                w0[t] = wq[slot][t].x ^ (WBITS == 4 ? 0x88888888u : 0u);      // int4: nibbles u = w + 8; int8 converts signed
                w1[t] = wq[slot][t].y ^ (WBITS == 4 ? 0x88888888u : 0u);
            }
            u32x4 xa[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) xa[mt] = *reinterpret_cast<const u32x4 *>(xw + ((s + j) * MT + mt) * 1024);
            // keep the order: wait for this slot, refill it, then compute
            __builtin_amdgcn_sched_barrier(0);
            load_step<POLICY>(wq[slot], rsrc_w, voff_w, p.ldw_bytes, (uint32_t)(step0 + s + j + PF) * 32u, s + j + PF < nsteps);
            __builtin_amdgcn_sched_barrier(0);

#pragma unroll
            for (int h = 0; h < 2; h++) {
#pragma unroll
                for (int jb = 0; jb < EPD / 2; jb++) {
                    u32x4 b0, b1;
                    expand_pair<WBITS, ACT>(h ? w1 : w0, jb, magic, b0, b1);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        P[mt][h * EPD + 2 * jb] = mfma_act<ACT>(xa[mt], b0, P[mt][h * EPD + 2 * jb]);
                        P[mt][h * EPD + 2 * jb + 1] = mfma_act<ACT>(xa[mt], b1, P[mt][h * EPD + 2 * jb + 1]);
                    }
                }
            }
#pragma unroll
            for (int mt = 0; mt < MT; mt++) X[mt] = mfma_act<ACT>(xa[mt], ones, X[mt]);
        }
        if constexpr (ACCUM) {
            in_unit += BS;
            if (in_unit == ustep) {
                fold_group<WBITS, ACT, MT, NT, NPV>(tot, P, X, sv, ov, one_row);
                in_unit = 0;
            }
        }
    }
    if constexpr (!ACCUM) {
        // the wavefront met a single parameter row: one fold, and the running total only starts to exist here
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int i = 0; i < NT; i++) tot[mt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        fold_group<WBITS, ACT, MT, NT, NPV>(tot, P, X, sv, ov, one_row);
    }

    // ---- reduce over the K slices, one m tile at a time: red[slice][row of the m tile][column of the tile]
    float *red = reinterpret_cast<float *>(lds + 16);
    TileOut<NBW, KS, THREADS, ACT> outp(p, lds, m_base, sgrp * NBW, chunk);
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        const int rows_mt = min(16, rows_valid - mt * 16);
        __syncthreads();                      // the activation fragments / the previous m tile's sums are dead
        if (lane_ok) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int row = 4 * g + q;
                if (row >= rows_mt) continue;
                float *dst = red + ((size_t)kslice * 16 + row) * NBW + wstrip * NB + (2 * c) * EPD;
#pragma unroll
                for (int i = 0; i < NT; i += 4)
                    *reinterpret_cast<f32x4 *>(dst + i) = f32x4{tot[mt][i][q], tot[mt][i + 1][q], tot[mt][i + 2][q], tot[mt][i + 3][q]};
            }
        }
        __syncthreads();
        outp.emit_mtile(red, mt * 16, rows_mt);
    }
    outp.finish(rows_valid, sgrp);
}

// int8 weights stored K-major ([N, K] row-major: the transposed view that torch_npu's LinearWeightQuant passes,
// torch_npu/contrib/module/linear_weight_quant.py:106).  Here a weight row already holds consecutive k of one output
// column, which is what an MFMA operand lane wants, so a wavefront simply owns 16 columns (16 weight rows) for the whole
// K range of its workgroup and keeps one accumulator tile per m tile; the eight wavefronts of a workgroup cover 128
// columns, i.e. one contiguous block of 128 weight rows in memory.  Nothing is reduced across wavefronts.
// K advances in steps of 128: lane (c, g) loads bytes [16g, 16g+16) and [64+16g, 64+16g+16) of the step from row c
// (two 16-byte loads) and feeds four MFMAs with the 8-byte halves; the activation fragments are laid out to match.
// Activations are staged through LDS in chunks of 8 steps, already in fragment order, double buffered: the loads of
// the next chunk are issued at the top of a chunk, written to LDS at its end, one barrier per chunk.
// Per group:  out = sum_g scale_g * (P_g + offset_g * X_g)  with the weight as its own image (see the top of the file).
template <int MT, bool GROUPED, int ACT>
__global__ __launch_bounds__(512) void wq_kmajor_kernel(const WqArgs p)
{
    constexpr int NBW = 128, THREADS = 512;
    constexpr int CH = 8 / MT;                          // steps per chunk of activations (32 KiB of LDS per buffer)
    constexpr int BODY = CH / 2;                        // steps per batch of weight loads: two batches per chunk, so
                                                        // that the register slot of a step is known at compile time
    constexpr int POLICY = MT == 1 ? kNonTemporal : 0;
    constexpr int XBUF = CH * MT * 4096;       // bytes of one activation chunk in LDS
    constexpr int TBUF = 2048;                 // one step of one wavefront's weights (16 rows x 128 bytes)
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int xcd_slot = blockIdx.x >> 3;
    const int tile = (blockIdx.x & 7) + 8 * (xcd_slot / p.S);
    const int chunk = xcd_slot % p.S;
    if (tile >= p.sgroups) return;
    const int m_base = blockIdx.y * (MT * 16);
    const int rows_valid = min(MT * 16, p.M - m_base);
    const int n0 = tile * NBW;

    // K range of this workgroup in steps of 128 (whole units: scale groups, or single steps per channel)
    const int u0 = (int)((int64_t)p.n_units * chunk / p.S), u1 = (int)((int64_t)p.n_units * (chunk + 1) / p.S);
    const int step0 = u0 * p.unit_steps, nsteps = (u1 - u0) * p.unit_steps;
    const int nchunks = (nsteps + CH - 1) / CH;

    // Weights: this wavefront's 16 rows (rows past N repeat the last valid row; N is a multiple of 4, so quads of columns past N are skipped whole).
    // A load instruction fetches whole cache lines - lane l takes 16 bytes of row l/8 (+8 for the second load) - which
    // reads HBM a quarter faster than fetching the MFMA operand layout directly (16 rows x 64 bytes per
    // instruction); the wavefront then turns the step around through a private 2 KiB LDS tile.  The 16-byte chunk a
    // lane fetches is XOR-swizzled with the row pair so that the operand reads (16 rows x 16 bytes) are free of bank
    // conflicts; LDS slot s of row r holds chunk s ^ ((r >> 1) & 7).
    const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(p.w, (uint32_t)((uint64_t)(p.N - 1) * p.ldw_bytes + (uint32_t)p.K));
    uint32_t voff_w[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int rl = 8 * h + (lane >> 3);
        voff_w[h] = (uint32_t)min(n0 + wave * 16 + rl, p.N - 1) * p.ldw_bytes + (uint32_t)(((lane & 7) ^ ((rl >> 1) & 7)) * 16);
    }
    char *tbuf = lds + 16 + 2 * XBUF + wave * (2 * TBUF);
    const int t_rd = c * 128 + ((g ^ ((c >> 1) & 7)) * 16);   // chunk g of row c; chunk g + 4 is at slot ^ 4, i.e. +-64 bytes
    // activations: staging reads whole rows, rows are dealt to the wavefronts; what lies past the last row or the
    // last step is given an out-of-range offset (zeros, no memory traffic, no branch around the load)
    const __amdgpu_buffer_rsrc_t rsrc_x =
        make_rsrc(p.x + (int64_t)m_base * p.ldx, (uint32_t)(((int64_t)(rows_valid - 1) * p.ldx + p.K) * 2));
    // antiquant parameters of this lane's column (accumulator column = c)
    const int pcol = min(n0 + wave * 16 + c, p.N - 1);
    const bool has_offset = p.offset != nullptr;

    // Weight loads are issued in batches of BODY steps (512 consecutive bytes of each of the 16 rows go out back to
    // back, so the memory controller sees them together), two batches in registers: one being consumed, one in flight.
    u32x4 wq[2][BODY][2];
    auto load_body = [&](int slot, int st) {    // st: first step of the batch, relative to step0
#pragma unroll
        for (int j = 0; j < BODY; j++) {
            const bool ok = st + j < nsteps;
            const uint32_t kb = (uint32_t)(step0 + st + j) * 128u;
            wq[slot][j][0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, ok ? voff_w[0] : kOutOfRange, kb, POLICY);
            wq[slot][j][1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, ok ? voff_w[1] : kOutOfRange, kb, POLICY);
        }
    };
    // staging: 16-byte piece q of a row's chunk (8 consecutive k) belongs to step q/16, sub-step t and lane group g with
    // q % 16 = 8 * (t / 2) + 2 * g + (t % 2); it goes to fragment (step, m tile, t) at lane (g, row % 16)
    constexpr int XR = (MT * 16 + 7) / 8;          // rows per wavefront
    constexpr int XH = CH * 16 / 64;               // a row's chunk is CH * 16 pieces, 64 per load instruction
    u32x4 xst[XR][XH];
    auto stage_load = [&](int ch) {
#pragma unroll
        for (int i = 0; i < XR; i++) {
            const int r = wave + 8 * i;
#pragma unroll
            for (int h = 0; h < XH; h++) {
                const int q = lane + 64 * h;
                const int st = ch * CH + (q >> 4);
                const bool ok = r < rows_valid && st < nsteps;
                // lane-dependent part in the vector offset, the chunk's position in the scalar offset
                xst[i][h] = __builtin_amdgcn_raw_buffer_load_b128(
                    rsrc_x, ok ? (uint32_t)((r * (int)p.ldx + q * 8) * 2) : kOutOfRange, (uint32_t)(step0 + ch * CH) * 256u, 0);
            }
        }
    };
    auto stage_store = [&](int ch) {
        char *buf = lds + 16 + (ch & 1) * XBUF;
#pragma unroll
        for (int i = 0; i < XR; i++) {
            const int r = wave + 8 * i;
            if (r >= MT * 16) continue;
#pragma unroll
            for (int h = 0; h < XH; h++) {
                const int q = lane + 64 * h;
                const int sl = q >> 4, rr = q & 15;
                const int t = 2 * (rr >> 3) + (rr & 1), gg = (rr & 7) >> 1;
                *reinterpret_cast<u32x4 *>(buf + (((sl * MT + (r >> 4)) * 4 + t) * 64 + gg * 16 + (r & 15)) * 16) = xst[i][h];
            }
        }
    };

    f32x4 P[MT], X[MT], tot[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) P[mt] = X[mt] = tot[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    const u32x4 ones = u32x4{kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>};
    auto fold = [&](int grp) {
        const float sc = act_1<ACT>(p.scale[(int64_t)grp * p.N + pcol]);
        const float of = has_offset ? act_1<ACT>(p.offset[(int64_t)grp * p.N + pcol]) : 0.0f;
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
#pragma unroll
            for (int q = 0; q < 4; q++) tot[mt][q] = __builtin_fmaf(sc, __builtin_fmaf(of, X[mt][q], P[mt][q]), tot[mt][q]);
            P[mt] = X[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    };

    // prologue: first weight steps in flight, first activation chunk in LDS
    stage_load(0);                              // before the weights: loads retire in order, and these come from cache
    load_body(0, 0);
    load_body(1, BODY);
    stage_store(0);
    __syncthreads();
    // step 0 of the weights goes into the wavefront's turn-around tile
    *reinterpret_cast<u32x4 *>(tbuf + lane * 16) = wq[0][0][0];
    *reinterpret_cast<u32x4 *>(tbuf + 1024 + lane * 16) = wq[0][0][1];

    int in_unit = 0, grp = GROUPED ? u0 : 0;
    for (int ch = 0; ch < nchunks; ch++) {
        stage_load(ch + 1);                     // past the end: zeros, no memory traffic
        const char *xb = lds + 16 + (ch & 1) * XBUF + lane * 16;
#pragma unroll
        for (int j = 0; j < CH; j++) {
            const int st = ch * CH + j;
            const int slot = j / BODY, js = j % BODY;
            u32x4 xa[4][MT];                    // this step's activation fragments, all requested up front
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int mt = 0; mt < MT; mt++) xa[t][mt] = *reinterpret_cast<const u32x4 *>(xb + ((j * MT + mt) * 4 + t) * 1024);
            // this step's weights in operand order (written during the previous step), then the next step's
            // registers take their place in the other half of the tile
            const char *tr = tbuf + (j & 1) * TBUF + t_rd;
            u32x4 w0 = *reinterpret_cast<const u32x4 *>(tr);
            u32x4 w1 = *reinterpret_cast<const u32x4 *>(tbuf + (j & 1) * TBUF + (t_rd ^ 64));
            {
                const int sn = ((j + 1) / BODY) & 1, jsn = (j + 1) % BODY;
                char *tw = tbuf + ((j + 1) & 1) * TBUF + lane * 16;
                *reinterpret_cast<u32x4 *>(tw) = wq[sn][jsn][0];
                *reinterpret_cast<u32x4 *>(tw + 1024) = wq[sn][jsn][1];
            }
            if (js == BODY - 1) {               // the batch has left the registers: refill its slot two batches ahead
                __builtin_amdgcn_sched_barrier(0);
                load_body(slot, st + 1 + BODY);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const uint32_t lo = t < 2 ? w0[2 * (t & 1)] : w1[2 * (t & 1)], hi = t < 2 ? w0[2 * (t & 1) + 1] : w1[2 * (t & 1) + 1];
                u32x4 b;
                b[0] = pack_act2<ACT>(sbyte_f32(lo, 0), sbyte_f32(lo, 1));
                b[1] = pack_act2<ACT>(sbyte_f32(lo, 2), sbyte_f32(lo, 3));
                b[2] = pack_act2<ACT>(sbyte_f32(hi, 0), sbyte_f32(hi, 1));
                b[3] = pack_act2<ACT>(sbyte_f32(hi, 2), sbyte_f32(hi, 3));
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    P[mt] = mfma_act<ACT>(xa[t][mt], b, P[mt]);
                    X[mt] = mfma_act<ACT>(xa[t][mt], ones, X[mt]);
                }
            }
            if constexpr (GROUPED) {
                if (st < nsteps && ++in_unit == p.unit_steps) {
                    fold(grp);
                    in_unit = 0;
                    grp++;
                }
            }
        }
        stage_store(ch + 1);
        __syncthreads();
    }
    if constexpr (!GROUPED) fold(0);

    // ---- output: the wavefront's [rows x 16 columns] tile goes through LDS to the shared output / exchange code
    float *red = reinterpret_cast<float *>(lds + 16);
    TileOut<NBW, 1, THREADS, ACT> outp(p, lds, m_base, n0, chunk);
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        const int rows_mt = min(16, rows_valid - mt * 16);
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int row = 4 * g + q;
            if (row < rows_mt) red[row * NBW + wave * 16 + c] = tot[mt][q];
        }
        __syncthreads();
        outp.emit_mtile(red, mt * 16, rows_mt);
    }
    outp.finish(rows_valid, tile);
}

// Any layout (including K-major int8 weights, i.e. the transposed view of an [N,K] tensor, int4 words along either
// dimension and strided parameters), any alignment: one thread per output element, golden operation order.
__global__ __launch_bounds__(256) void wq_generic_kernel(const uint16_t *__restrict__ x, const void *__restrict__ w,
                                                         int w_bits, const uint16_t *__restrict__ scale,
                                                         const uint16_t *__restrict__ offset,
                                                         const uint16_t *__restrict__ bias,
                                                         uint16_t *__restrict__ out, int M, int N, int K, int group,
                                                         int64_t ldx, int64_t ldw_k, int64_t ldw_n, int64_t ldo,
                                                         int64_t ld_param_g, int64_t ld_param_n, int kpacked, int act)
{
    const int n = blockIdx.x * 64 + (threadIdx.x & 63);
    const int m = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (m >= M || n >= N) return;
    float acc = 0.0f;
    for (int k = 0; k < K; k++) {
        const int gidx = k / group;
        float wv;
        if (w_bits == 8) {
            wv = (float)static_cast<const int8_t *>(w)[(int64_t)k * ldw_k + (int64_t)n * ldw_n];
        } else {
            // words along N (element n & 7 of word n / 8 of row k) or along K (element k & 7 of word k / 8 of column n)
            const uint32_t word = kpacked ? static_cast<const uint32_t *>(w)[(int64_t)n * ldw_n + (k >> 3)]
                                          : static_cast<const uint32_t *>(w)[(int64_t)k * ldw_k + (n >> 3)];
            const int v = (int)((word >> (4 * ((kpacked ? k : n) & 7))) & 0xfu);
            wv = (float)((v ^ 8) - 8);
        }
        auto cvt = [&](uint16_t h) { return act ? act_1<1>(h) : act_1<0>(h); };
        if (offset) wv = wv + cvt(offset[(int64_t)gidx * ld_param_g + (int64_t)n * ld_param_n]);
        wv = wv * cvt(scale[(int64_t)gidx * ld_param_g + (int64_t)n * ld_param_n]);
        acc = acc + cvt(x[(int64_t)m * ldx + k]) * wv;
    }
    if (bias) acc = acc + (act ? act_1<1>(bias[n]) : act_1<0>(bias[n]));
    out[(int64_t)m * ldo + n] = (uint16_t)(act ? pack_act2<1>(acc, 0.0f) : pack_act2<0>(acc, 0.0f));
}

struct WqPlan {
    bool fast;
    int mt;             // m tiles (16 rows) per workgroup
    int w, ks;          // adjacent strips per workgroup, K slices per workgroup: w * ks wavefronts
    bool accum;         // a wavefront may meet more than one scale group
    int strips, sgroups, mchunks, S;
    int unit_steps, n_units;
    int bs;             // steps per loop body of the kernel
    size_t partial_bytes, counter_bytes;
    size_t slab_bytes;  // activations of one K chunk in LDS
};

WqPlan make_plan(int64_t M, int64_t N, int64_t K, int w_bits, int64_t group_size, bool n_major, int64_t ldw_k,
                 int64_t ldx, const void *x, const void *w, const void *scale, const void *offset)
{
    WqPlan pl{};
    const int64_t row_bytes = w_bits == 4 ? N / 2 : N;
    const int64_t ldw_bytes = w_bits == 4 ? ldw_k * 4 : ldw_k;
    const int64_t group = group_size > 0 ? group_size : K;
    pl.fast = K > 0 && K % 32 == 0 && group % 32 == 0 && n_major && row_bytes % 16 == 0 && ldw_bytes % 16 == 0 &&
              ldx % 8 == 0 && (x == nullptr || aligned(x, 16)) && (w == nullptr || aligned(w, 16)) &&
              (scale == nullptr || aligned(scale, 16)) && (offset == nullptr || aligned(offset, 16)) &&
              (uint64_t)K * (uint64_t)ldw_bytes < (1ull << 32) && (uint64_t)M * (uint64_t)ldx * 2 < (1ull << 32) &&
              (uint64_t)(K / group) * (uint64_t)N * 2 < (1ull << 32);
    if (!pl.fast) return pl;
    pl.mt = M <= 16 ? 1 : 2;
    pl.strips = (int)((row_bytes + 127) / 128);
    pl.mchunks = (int)((M + pl.mt * 16 - 1) / (pl.mt * 16));
    const bool grouped = group_size > 0 && group != K;
    // loop body of 4 steps when a scale group (per channel: the whole of K) is a whole number of them, else 1 step
    const int64_t span = (grouped ? group : K) / 32;
    pl.bs = span % 4 == 0 ? 4 : 1;
    pl.unit_steps = grouped ? (int)(group / 32) : pl.bs;
    pl.n_units = (int)(K / (32 * pl.unit_steps));
    // W adjacent strips per workgroup; the remaining wavefronts slice K.  Pairs of strips read DRAM markedly
    // better, but halve the number of tiles: with few strips that means a deeper split of K and a longer exchange.
    pl.w = pl.strips >= 112 ? 2 : 1;
    if (const int f = knob(kKnobWqW))      // tuning aid
        if (f == 1 || f == 2) pl.w = f;
    pl.sgroups = (pl.strips + pl.w - 1) / pl.w;
    constexpr int kMaxSlabSteps = (160 * 1024 - 16) / 1024;
    // Eight wavefronts per workgroup, except where the accumulators of two m tiles plus a running total need the
    // whole register file of a SIMD (int4, several groups per wavefront): then four.
    for (int nwv = 8; nwv >= 4; nwv -= 4) {
        pl.ks = nwv / pl.w;
        // split K over S workgroups until all CUs have work; every wavefront keeps at least one unit
        int S = kNumCU / (pl.sgroups * pl.mchunks);
        const int s_max = pl.n_units / pl.ks > 0 ? pl.n_units / pl.ks : 1;
        if (S > s_max) S = s_max;
        if (S > 16) S = 16;
        if (S < 1) S = 1;
        // the activations of a workgroup's K chunk must fit in LDS (1 KiB per step and m tile)
        auto slab_steps = [&](int chunks) { return (pl.n_units + chunks - 1) / chunks * pl.unit_steps * pl.mt; };
        while (slab_steps(S) > kMaxSlabSteps && S < s_max) S++;
        if (const int f = knob(kKnobWqSplit))  // tuning aid: force the number of K chunks
            if (f >= 1 && f <= s_max) S = f;
        if (w_bits == 4 && pl.mt == 2 && grouped && nwv == 8 && pl.bs == 4) {
            // two m tiles of int4 run much better without the running total (eight wavefronts, no spills): split K
            // further, down to one scale group per wavefront, when that stays within 16 chunks (measured at
            // M = 128, K = 4096: 73 us against 92 us)
            const int s_one = (pl.n_units + pl.ks - 1) / pl.ks;
            if (s_one > S && s_one <= 16 && s_one <= s_max && !knob(kKnobWqSplit)) S = s_one;
        }
        if ((uint64_t)S * (uint64_t)M * (uint64_t)N * 4 >= (1ull << 32)) S = 1; // exchange offsets are 32-bit
        pl.S = S;
        pl.slab_bytes = (size_t)slab_steps(S) * 1024;
        pl.accum = grouped && (pl.n_units + S * pl.ks - 1) / (S * pl.ks) > 1;
        if (pl.bs == 1) pl.accum = true;              // only instantiated with the running total
        if (slab_steps(S) > kMaxSlabSteps) {
            pl.fast = false;
            return pl;
        }
        if (!(w_bits == 4 && pl.mt == 2 && pl.accum)) break;
    }
    // the four-wavefront int4 kernel for two m tiles exists only with the running total (which also serves a
    // wavefront that meets a single group)
    if (w_bits == 4 && pl.mt == 2 && pl.w * pl.ks == 4) pl.accum = true;
    pl.partial_bytes = pl.S > 1 ? (size_t)pl.S * M * N * sizeof(float) : 0;
    if (pl.S > 1 && (size_t)pl.sgroups * pl.mchunks * sizeof(uint32_t) > kWorkspaceCounterBytes) {
        pl.fast = false;                              // more tiles than arrival counters
        return pl;
    }
    pl.counter_bytes = pl.S > 1 ? kWorkspaceZeroBytes : 0;
    return pl;
}

template <int WBITS, int ACT, int MT, int W, int KS, int BS, bool ACCUM>
int launch_stream(const WqArgs &p, const WqPlan &pl, hipStream_t s)
{
    constexpr int EPD = 32 / WBITS, NB = 32 * EPD;
    // Steps in flight per wavefront.  Measured: deeper register rings only lengthen the queues in front of HBM
    // (int4, K = 4096: 11.8 / 12.7 / 13.6 us with 1 / 2 / 4 steps; int8, K = 8192: 46.5 / 46.1 / 47.9 us).
    // Four-wavefront workgroups (int4, two m tiles, running total) have half the loads in flight: two steps.
    constexpr int PF = BS > 1 && (WBITS == 8 || W * KS == 4) ? 2 : 1;
    constexpr size_t red_bytes = (size_t)KS * 16 * W * NB * sizeof(float);
    static_assert(16 + red_bytes <= 160 * 1024, "LDS budget");
    const size_t lds_bytes = 16 + (red_bytes > pl.slab_bytes ? red_bytes : pl.slab_bytes);
    auto kern = wq_stream_kernel<WBITS, ACT, MT, W, KS, BS, PF, ACCUM>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)((pl.sgroups + 7) / 8 * 8 * pl.S), (unsigned)pl.mchunks), dim3(W * KS * 64),
                       lds_bytes, s, p);
    return check_launch();
}

// ACC_MODES: 0 = both accumulation modes are instantiated, 1 = only the running total, 2 = only the single fold
template <int WBITS, int ACT, int MT, int W, int KS, int ACC_MODES>
int launch_body(const WqArgs &p, const WqPlan &pl, hipStream_t s)
{
    if constexpr (ACC_MODES != 2) {
        if (pl.bs == 1) return launch_stream<WBITS, ACT, MT, W, KS, 1, true>(p, pl, s);
        if (pl.accum) return launch_stream<WBITS, ACT, MT, W, KS, 4, true>(p, pl, s);
    }
    if constexpr (ACC_MODES != 1) {
        if (pl.bs == 4 && !pl.accum) return launch_stream<WBITS, ACT, MT, W, KS, 4, false>(p, pl, s);
    }
    return MI355_ERR_UNSUPPORTED;
}

// K-major int8 weights ([N, K] storage).
struct WqKmPlan {
    bool fast;
    int mt, mchunks, tiles, S, unit_steps, n_units;
    bool grouped;
    size_t partial_bytes, counter_bytes, lds_bytes;
};

WqKmPlan make_kmajor_plan(int64_t M, int64_t N, int64_t K, int64_t group_size, int64_t ldw_n, int64_t ldx, const void *x,
                          const void *w)
{
    WqKmPlan pl{};
    const int64_t group = group_size > 0 ? group_size : K;
    // N % 4: the output side stores quads of four columns (other N take the generic kernel)
    pl.fast = K > 0 && K % 128 == 0 && group % 128 == 0 && N % 4 == 0 && ldw_n >= K && ldw_n % 16 == 0 && ldx % 8 == 0 &&
              (x == nullptr || aligned(x, 16)) && (w == nullptr || aligned(w, 16)) &&
              (uint64_t)N * (uint64_t)ldw_n < (1ull << 32) && (uint64_t)M * (uint64_t)ldx * 2 < (1ull << 32);
    if (!pl.fast) return pl;
    pl.mt = M <= 16 ? 1 : 2;
    pl.mchunks = (int)((M + pl.mt * 16 - 1) / (pl.mt * 16));
    pl.tiles = (int)((N + 127) / 128);
    pl.grouped = group_size > 0 && group != K;
    pl.unit_steps = pl.grouped ? (int)(group / 128) : 1;
    pl.n_units = (int)(K / (128 * pl.unit_steps));
    int S = kNumCU / (pl.tiles * pl.mchunks);
    if (S > pl.n_units) S = pl.n_units;
    if (S > 16) S = 16;
    if (S < 1) S = 1;
    if (const int f = knob(kKnobWqSplit))
        if (f >= 1 && f <= pl.n_units) S = f;
    if ((uint64_t)S * (uint64_t)M * (uint64_t)N * 4 >= (1ull << 32)) S = 1;
    if (S > 1 && (size_t)pl.tiles * pl.mchunks * sizeof(uint32_t) > kWorkspaceCounterBytes) S = 1;
    if (wq_kmajor_decode_shape(M, N, K, group_size)) S = 1;   // the decode kernel splits K inside its workgroups
    pl.S = S;
    pl.partial_bytes = S > 1 ? (size_t)S * M * N * sizeof(float) : 0;
    pl.counter_bytes = S > 1 ? kWorkspaceZeroBytes : 0;
    pl.lds_bytes = 16 + (size_t)2 * 32768 + 8 * 2 * 2048;   // two activation chunks + the turn-around tiles
    return pl;
}

template <int MT, bool GROUPED, int ACT>
int launch_kmajor(const WqArgs &p, const WqKmPlan &pl, hipStream_t s)
{
    auto kern = wq_kmajor_kernel<MT, GROUPED, ACT>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)((pl.tiles + 7) / 8 * 8 * pl.S), (unsigned)pl.mchunks), dim3(512), pl.lds_bytes, s, p);
    return check_launch();
}

template <int WBITS, int ACT>
int launch_bits(const WqArgs &p, const WqPlan &pl, hipStream_t s)
{
    if (pl.mt == 1)
        return pl.w == 1 ? launch_body<WBITS, ACT, 1, 1, 8, 0>(p, pl, s) : launch_body<WBITS, ACT, 1, 2, 4, 0>(p, pl, s);
    if constexpr (WBITS == 8) {
        return pl.w == 1 ? launch_body<8, ACT, 2, 1, 8, 0>(p, pl, s) : launch_body<8, ACT, 2, 2, 4, 0>(p, pl, s);
    } else {
        // two m tiles of int4: eight wavefronts only without the running total (see make_plan)
        if (pl.w * pl.ks == 8)
            return pl.w == 1 ? launch_body<4, ACT, 2, 1, 8, 2>(p, pl, s) : launch_body<4, ACT, 2, 2, 4, 2>(p, pl, s);
        return pl.w == 1 ? launch_body<4, ACT, 2, 1, 4, 1>(p, pl, s) : launch_body<4, ACT, 2, 2, 2, 1>(p, pl, s);
    }
}

template <int ACT>
int launch_kmajor_any(const WqArgs &p, const WqKmPlan &km, hipStream_t s)
{
    if (km.mt == 1) return km.grouped ? launch_kmajor<1, true, ACT>(p, km, s) : launch_kmajor<1, false, ACT>(p, km, s);
    return km.grouped ? launch_kmajor<2, true, ACT>(p, km, s) : launch_kmajor<2, false, ACT>(p, km, s);
}

} // namespace
} // namespace mi355

namespace mi355 {
namespace {
// Which kernel a launch with rows along N takes when every pointer is aligned, in the order of the launch: the int4 decode
// kernel, the int4 register-expanding GEMM, the tiled GEMM through LDS images, the streaming kernel.
enum { kPreferDecode, kPreferGemm4, kPreferGemm, kPreferStream };

// int4 words along K, many rows: the weight is rewritten into the workspace with its words along N (and the parameters
// gathered into row-major [G, N]) for the register-expanding GEMM.  Layout of the workspace: the zero area, the weight
// ([K, repack_pitch_words(N)] words), scales, offsets.
constexpr int64_t kRepackRows = 256;
int64_t repack_pitch_words(int64_t N) { return (N / 8 + 3) / 4 * 4; }
size_t align256(size_t v) { return (v + 255) / 256 * 256; }
size_t repack_weight_bytes(int64_t N, int64_t K) { return align256((size_t)K * (size_t)repack_pitch_words(N) * 4); }
size_t repack_param_bytes(int64_t N, int64_t K, int64_t group_size)
{
    return align256((size_t)(group_size > 0 ? K / group_size : 1) * (size_t)N * 2);
}
size_t repack_workspace_bytes(int64_t N, int64_t K, int64_t group_size)
{
    return kWorkspaceZeroBytes + repack_weight_bytes(N, K) + 2 * repack_param_bytes(N, K, group_size);
}
bool repack_applies(int64_t M, int64_t N, int64_t K, int64_t group_size, int64_t ldx, const void *x)
{
    return M >= kRepackRows && N % 8 == 0 && K % 128 == 0 &&
           make_wq_gemm4_plan(M, N, K, 4, group_size, repack_pitch_words(N), ldx, x, nullptr, nullptr, nullptr).ok;
}
int preferred_n_major_kernel(int64_t M, int64_t N, int64_t K, int w_bits, int64_t group_size, int64_t ldw_k, int64_t ldx)
{
    if (w_bits == 4 && make_wq_decode_plan(M, N, K, 4, group_size, ldw_k, ldx, nullptr, nullptr, nullptr, nullptr).ok) return kPreferDecode;
    if (make_wq_gemm4_plan(M, N, K, w_bits, group_size, ldw_k, ldx, nullptr, nullptr, nullptr, nullptr).ok) return kPreferGemm4;
    if (make_wq_gemm_plan(M, N, K, w_bits, group_size, 1, ldw_k, ldx, nullptr, nullptr, nullptr, nullptr).ok) return kPreferGemm;
    return kPreferStream;
}
} // namespace
} // namespace mi355

extern "C" size_t mi355_weight_quant_matmul_workspace(int64_t M, int64_t N, int64_t K, int w_bits, int64_t group_size)
{
    using namespace mi355;
    if (M <= 0 || N <= 0 || K <= 0 || (w_bits != 4 && w_bits != 8) || group_size < 0) return 0;
    // The query knows neither strides nor alignments, the launch plans with the real ones: the answer is the largest
    // request over every layout the kernels accept, once with dense rows (pitch = row length) and once with rows padded
    // to 128 bytes, which is what lets a shape with a ragged row length onto a fast kernel that the dense pitch rules out.
    // Per layout it asks for the kernel the launch prefers (preferred_n_major_kernel); a kernel further down the order, which
    // only runs when a pointer is misaligned, falls through to the generic kernel if its own request is not met (the
    // streaming kernel would ask for S x M x N x 4 bytes at large M: hundreds of MiB that no launch of a sane caller uses).
    auto pad = [](int64_t v, int64_t to) { return (v + to - 1) / to * to; };
    size_t need = 0;
    for (int padded = 0; padded < 2; padded++) {
        const int64_t ldx = padded ? pad(K, 64) : K;                                  // activation pitch, elements
        const int64_t ldw_n_major = padded ? pad(w_bits == 4 ? N / 8 : N, w_bits == 4 ? 32 : 128) : (w_bits == 4 ? N / 8 : N);
        const int64_t ldw_k_major = padded ? pad(w_bits == 4 ? K / 8 : K, w_bits == 4 ? 32 : 128) : (w_bits == 4 ? K / 8 : K);
        const int preferred = preferred_n_major_kernel(M, N, K, w_bits, group_size, ldw_n_major, ldx);
        if (preferred == kPreferStream) {
            const WqPlan pl = make_plan(M, N, K, w_bits, group_size, true, ldw_n_major, ldx, nullptr, nullptr, nullptr, nullptr);
            if (pl.fast && pl.partial_bytes + pl.counter_bytes > need) need = pl.partial_bytes + pl.counter_bytes;
        }
        for (int layout = 1; layout <= (w_bits == 8 ? 2 : 1); layout++) {
            if (layout == 1 && preferred != kPreferGemm) continue;
            const WqGemmPlan gp = make_wq_gemm_plan(M, N, K, w_bits, group_size, layout, layout == 2 ? ldw_k_major : ldw_n_major, ldx,
                                                    nullptr, nullptr, nullptr, nullptr);
            const size_t gneed = gp.counter_bytes + gp.partial_bytes;
            if (gp.ok && gneed > need) need = gneed;
        }
        if (w_bits == 4) {                  // words along N: the decode and register-expanding kernels exchange in the zero area
            const WqDecodePlan dp = make_wq_decode_plan(M, N, K, 4, group_size, ldw_n_major, ldx, nullptr, nullptr, nullptr, nullptr);
            if (dp.ok && dp.S > 1 && kWorkspaceZeroBytes > need) need = kWorkspaceZeroBytes;
            const WqGemm4Plan g4 = make_wq_gemm4_plan(M, N, K, 4, group_size, ldw_n_major, ldx, nullptr, nullptr, nullptr, nullptr);
            if (g4.ok && g4.S > 1 && kWorkspaceZeroBytes > need) need = kWorkspaceZeroBytes;
            // words along K: rewritten per call from kRepackRows rows up, a kernel of their own below
            if (repack_applies(M, N, K, group_size, ldx, nullptr)) {
                if (repack_workspace_bytes(N, K, group_size) > need) need = repack_workspace_bytes(N, K, group_size);
            } else {
                const WqKpackedPlan kp = make_wq_kpacked_plan(M, N, K, group_size, ldw_k_major, ldx, nullptr, nullptr);
                if (kp.ok && kp.partial_bytes + kp.counter_bytes > need) need = kp.partial_bytes + kp.counter_bytes;
            }
        } else {                            // the K-major layout may split differently
            const WqGemm4Plan g8 = make_wq_gemm4_plan(M, N, K, 8, group_size, ldw_n_major, ldx, nullptr, nullptr, nullptr, nullptr);
            if (g8.ok && g8.S > 1 && kWorkspaceZeroBytes > need) need = kWorkspaceZeroBytes;
            const WqKmPlan km = make_kmajor_plan(M, N, K, group_size, ldw_k_major, ldx, nullptr, nullptr);
            if (km.fast && km.partial_bytes + km.counter_bytes > need) need = km.partial_bytes + km.counter_bytes;
        }
    }
    return need;
}

extern "C" int mi355_weight_quant_matmul(const void *x_bf16, int act_dtype, const void *w, int w_bits, const void *scale_bf16,
                                         const void *offset_bf16, const void *bias, void *out_bf16, int64_t M, int64_t N, int64_t K,
                                         int64_t group_size, int64_t ld_param_g, int64_t ld_param_n, int64_t ldx,
                                         int64_t ldw_k, int64_t ldw_n, int64_t ldo, void *workspace, size_t workspace_bytes,
                                         void *stream)
{
    using namespace mi355;
    if (M < 0 || N < 0 || K < 0 || group_size < 0) return MI355_ERR_BAD_ARGUMENT;
    if (w_bits != 8 && w_bits != 4) return MI355_ERR_BAD_ARGUMENT;
    if (act_dtype != MI355_DTYPE_BF16 && act_dtype != MI355_DTYPE_FP16) return MI355_ERR_BAD_ARGUMENT;
    const bool f16 = act_dtype == MI355_DTYPE_FP16;
    if (M == 0 || N == 0) return MI355_OK;
    if (!out_bf16 || ldo < N) return MI355_ERR_BAD_ARGUMENT;
    if (K > 0 && (!x_bf16 || !w || !scale_bf16 || ldx < K)) return MI355_ERR_BAD_ARGUMENT;
    // int4 words run along N (ldw_n == 1: rows of N/8 words, ldw_k words apart) or along K (ldw_k == 1: columns of K/8
    // words, ldw_n words apart)
    const bool kpacked = w_bits == 4 && ldw_n != 1 && ldw_k == 1;
    if (w_bits == 4 && !kpacked && (ldw_n != 1 || N % 8 != 0 || ldw_k < N / 8)) return MI355_ERR_BAD_ARGUMENT;
    if (kpacked && (K % 8 != 0 || ldw_n < K / 8)) return MI355_ERR_BAD_ARGUMENT;
    if (w_bits == 8 && ldw_k != 1 && ldw_n != 1) return MI355_ERR_UNSUPPORTED;
    if (group_size > 0 && (K % group_size != 0)) return MI355_ERR_BAD_ARGUMENT;
    const int64_t n_groups = group_size > 0 && K > 0 ? K / group_size : 1;
    if (ld_param_g < 0 || ld_param_n < 1) return MI355_ERR_BAD_ARGUMENT;
    // every kernel but the one for K-packed int4 (and the generic one) reads [G, N] row-major parameters
    const bool params_rowmajor = ld_param_n == 1 && (n_groups == 1 || ld_param_g == N);
    if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return MI355_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int group = (int)(group_size > 0 ? group_size : (K > 0 ? K : 1));

    const auto generic = [&]() {
        hipLaunchKernelGGL(wq_generic_kernel, dim3((unsigned)((N + 63) / 64), (unsigned)((M + 3) / 4)), dim3(256), 0, s,
                           static_cast<const uint16_t *>(x_bf16), w, w_bits, static_cast<const uint16_t *>(scale_bf16),
                           static_cast<const uint16_t *>(offset_bf16), static_cast<const uint16_t *>(bias),
                           static_cast<uint16_t *>(out_bf16), (int)M, (int)N, (int)K, group, ldx, ldw_k, ldw_n, ldo, ld_param_g,
                           ld_param_n, kpacked ? 1 : 0, f16 ? 1 : 0);
        return check_launch();
    };
    if (kpacked) {
        if (repack_applies(M, N, K, group_size, ldx, x_bf16) && ldw_n % 4 == 0 && aligned(w, 16) && aligned(scale_bf16, 2) &&
            (!offset_bf16 || aligned(offset_bf16, 2)) && aligned(out_bf16, 2) && (!bias || aligned(bias, 2)) && workspace &&
            aligned(workspace, 256) && workspace_bytes >= repack_workspace_bytes(N, K, group_size)) {
            char *ws = static_cast<char *>(workspace);
            void *w_kn = ws + kWorkspaceZeroBytes;
            void *scale_gn = ws + kWorkspaceZeroBytes + repack_weight_bytes(N, K);
            void *offset_gn = offset_bf16 ? static_cast<char *>(scale_gn) + repack_param_bytes(N, K, group_size) : nullptr;
            const int64_t pitch = repack_pitch_words(N);
            int st = launch_repack_int4_k_to_n(w, ldw_n, w_kn, pitch, N, K, stream);
            if (st == MI355_OK) st = launch_gather_params_u16(scale_bf16, ld_param_g, ld_param_n, scale_gn, n_groups, N, stream);
            if (st == MI355_OK && offset_bf16)
                st = launch_gather_params_u16(offset_bf16, ld_param_g, ld_param_n, offset_gn, n_groups, N, stream);
            if (st != MI355_OK) return st;
            const WqGemm4Plan g4 = make_wq_gemm4_plan(M, N, K, 4, group_size, pitch, ldx, x_bf16, w_kn, scale_gn, offset_gn);
            if (!g4.ok) return MI355_ERR_LAUNCH;       // planned with these strides a few lines up
            return launch_wq_gemm4(g4, x_bf16, f16 ? 1 : 0, w_kn, 4, scale_gn, offset_gn, bias, out_bf16, M, N, K, group_size, ldx, pitch,
                                   ldo, workspace, stream);
        }
        if (wq_kpacked_decode_shape(M, N, K, group_size) && ldw_n < (1ll << 29)) {
            // at most 32 rows, groups of 128: the barrier-free kernel that splits K inside the workgroup
            WqKpDecodeArgs d;
            d.x = static_cast<const uint16_t *>(x_bf16);
            d.w = w;
            d.scale = static_cast<const uint16_t *>(scale_bf16);
            d.offset = static_cast<const uint16_t *>(offset_bf16);
            d.bias = static_cast<const uint16_t *>(bias);
            d.out = static_cast<uint16_t *>(out_bf16);
            d.ldx = ldx;
            d.ldo = ldo;
            d.ld_param_g = ld_param_g;
            d.ld_param_n = ld_param_n;
            d.ldw_bytes = (uint32_t)(ldw_n * 4);
            d.M = (int)M;
            d.N = (int)N;
            d.K = (int)K;
            const int st = launch_wq_kpacked_decode(d, f16 ? 1 : 0, static_cast<hipStream_t>(stream));
            if (st != MI355_ERR_UNSUPPORTED) return st;
        }
        const WqKpackedPlan kp = make_wq_kpacked_plan(M, N, K, group_size, ldw_n, ldx, x_bf16, w);
        const bool ptrs_ok = aligned(scale_bf16, 2) && (!offset_bf16 || aligned(offset_bf16, 2)) && aligned(out_bf16, 2) &&
                             (!bias || aligned(bias, 2));
        if (!kp.ok || !ptrs_ok) return generic();
        if (kp.S > 1) {
            if (!workspace || workspace_bytes < kp.counter_bytes + kp.partial_bytes) return MI355_ERR_WORKSPACE;
            if (!aligned(workspace, 16)) return MI355_ERR_ALIGNMENT;
        }
        return launch_wq_kpacked(kp, x_bf16, f16 ? 1 : 0, w, scale_bf16, offset_bf16, bias, out_bf16, M, N, K, ldx, ldw_n, ldo,
                                 ld_param_g, ld_param_n, workspace, stream);
    }
    if (!params_rowmajor) return generic();
    if (w_bits == 8 && ldw_k == 1 && ldw_n != 1) {
        // K-major: the transposed view of an [N, K] weight
        const WqGemmPlan gk = make_wq_gemm_plan(M, N, K, 8, group_size, 2, ldw_n, ldx, x_bf16, w, scale_bf16, offset_bf16);
        if (gk.ok && aligned(out_bf16, 2) && (!bias || aligned(bias, 2))) {
            if (gk.S > 1) {
                if (!workspace || workspace_bytes < gk.counter_bytes + gk.partial_bytes) return MI355_ERR_WORKSPACE;
                if (!aligned(workspace, 16)) return MI355_ERR_ALIGNMENT;
            }
            return launch_wq_gemm(gk, x_bf16, f16 ? 1 : 0, w, 8, scale_bf16, offset_bf16, bias, out_bf16, M, N, K, ldx, ldw_n, ldo,
                                  workspace, stream);
        }
        const WqKmPlan km = make_kmajor_plan(M, N, K, group_size, ldw_n, ldx, x_bf16, w);
        const bool params_ok = aligned(scale_bf16, 2) && (!offset_bf16 || aligned(offset_bf16, 2));
        if (km.fast && params_ok) {
            if (wq_kmajor_decode_shape(M, N, K, group_size)) {
                // at most 32 rows, one scale per column: the barrier-free kernel that splits K inside the workgroup
                WqKmDecodeArgs d;
                d.x = static_cast<const uint16_t *>(x_bf16);
                d.w = static_cast<const int8_t *>(w);
                d.scale = static_cast<const uint16_t *>(scale_bf16);
                d.offset = static_cast<const uint16_t *>(offset_bf16);
                d.bias = static_cast<const uint16_t *>(bias);
                d.out = static_cast<uint16_t *>(out_bf16);
                d.ldx = ldx;
                d.ldw = ldw_n;
                d.ldo = ldo;
                d.M = (int)M;
                d.N = (int)N;
                d.K = (int)K;
                const int st = launch_wq_kmajor_decode(d, f16 ? 1 : 0, s);
                if (st != MI355_ERR_UNSUPPORTED) return st;
            }
            if (km.S > 1) {
                if (!workspace || workspace_bytes < km.partial_bytes + km.counter_bytes) return MI355_ERR_WORKSPACE;
                if (!aligned(workspace, 16)) return MI355_ERR_ALIGNMENT;
            }
            WqArgs p{};
            p.x = static_cast<const uint16_t *>(x_bf16);
            p.w = w;
            p.scale = static_cast<const uint16_t *>(scale_bf16);
            p.offset = static_cast<const uint16_t *>(offset_bf16);
            p.bias = static_cast<const uint16_t *>(bias);
            p.out = static_cast<uint16_t *>(out_bf16);
            p.counter = km.S > 1 ? static_cast<uint32_t *>(workspace) : nullptr;
            p.partial = km.S > 1 ? reinterpret_cast<float *>(static_cast<char *>(workspace) + km.counter_bytes) : nullptr;
            p.ldx = ldx;
            p.ldo = ldo;
            p.ldw_bytes = (uint32_t)ldw_n;
            p.row_bytes = (uint32_t)K;
            p.M = (int)M;
            p.N = (int)N;
            p.K = (int)K;
            p.unit_steps = km.unit_steps;
            p.n_units = km.n_units;
            p.grouped = km.grouped;
            p.strips = km.tiles;
            p.sgroups = km.tiles;
            p.S = km.S;
            return f16 ? launch_kmajor_any<1>(p, km, s) : launch_kmajor_any<0>(p, km, s);
        }
    }
    const bool n_major = w_bits == 4 || (ldw_n == 1 && ldw_k >= N);
    if (w_bits == 4) {
        // at most 32 rows, words along N: the barrier-free decode kernel
        const WqDecodePlan dp = make_wq_decode_plan(M, N, K, 4, group_size, ldw_k, ldx, x_bf16, w, scale_bf16, offset_bf16);
        if (dp.ok && aligned(out_bf16, 2) && (!bias || aligned(bias, 2))) {
            if (dp.S > 1) {
                if (!workspace || workspace_bytes < kWorkspaceZeroBytes) return MI355_ERR_WORKSPACE;
                if (!aligned(workspace, 16)) return MI355_ERR_ALIGNMENT;
            }
            return launch_wq_decode(dp, x_bf16, f16 ? 1 : 0, w, scale_bf16, offset_bf16, bias, out_bf16, M, N, K, group_size, ldx,
                                    ldw_k, ldo, workspace, stream);
        }
        // more than 32 rows: the tiled kernel that expands the nibbles in registers
        const WqGemm4Plan g4 = make_wq_gemm4_plan(M, N, K, 4, group_size, ldw_k, ldx, x_bf16, w, scale_bf16, offset_bf16);
        if (g4.ok && aligned(out_bf16, 2) && (!bias || aligned(bias, 2))) {
            if (g4.S > 1) {
                if (!workspace || workspace_bytes < kWorkspaceZeroBytes) return MI355_ERR_WORKSPACE;
                if (!aligned(workspace, 16)) return MI355_ERR_ALIGNMENT;
            }
            return launch_wq_gemm4(g4, x_bf16, f16 ? 1 : 0, w, 4, scale_bf16, offset_bf16, bias, out_bf16, M, N, K, group_size, ldx, ldw_k,
                                   ldo, workspace, stream);
        }
    }
    if (w_bits == 8 && n_major) {
        // int8 [K, N], more than 32 rows: the same register-expanding kernel
        const WqGemm4Plan g8 = make_wq_gemm4_plan(M, N, K, 8, group_size, ldw_k, ldx, x_bf16, w, scale_bf16, offset_bf16);
        if (g8.ok && aligned(out_bf16, 2) && (!bias || aligned(bias, 2))) {
            if (g8.S > 1) {
                if (!workspace || workspace_bytes < kWorkspaceZeroBytes) return MI355_ERR_WORKSPACE;
                if (!aligned(workspace, 16)) return MI355_ERR_ALIGNMENT;
            }
            return launch_wq_gemm4(g8, x_bf16, f16 ? 1 : 0, w, 8, scale_bf16, offset_bf16, bias, out_bf16, M, N, K, group_size, ldx, ldw_k,
                                   ldo, workspace, stream);
        }
    }
    // more than 32 rows: the tiled kernel decodes every weight once per 64 or 128 rows
    // A kernel that the workspace query did not plan for (it only runs because a pointer kept the preferred one away) goes
    // on to the next one when its own request is not met; the preferred one reports the missing workspace.
    const int preferred = n_major ? preferred_n_major_kernel(M, N, K, w_bits, group_size, ldw_k, ldx) : kPreferStream;
    const auto workspace_holds = [&](size_t bytes) { return workspace && workspace_bytes >= bytes && aligned(workspace, 16); };
    const WqGemmPlan gp = make_wq_gemm_plan(M, N, K, w_bits, group_size, n_major ? 1 : 0, ldw_k, ldx, x_bf16, w, scale_bf16, offset_bf16);
    if (gp.ok && aligned(out_bf16, 2) && (!bias || aligned(bias, 2)) &&
        (gp.S == 1 || preferred >= kPreferGemm || workspace_holds(gp.counter_bytes + gp.partial_bytes))) {
        if (gp.S > 1) {
            if (!workspace || workspace_bytes < gp.counter_bytes + gp.partial_bytes) return MI355_ERR_WORKSPACE;
            if (!aligned(workspace, 16)) return MI355_ERR_ALIGNMENT;
        }
        return launch_wq_gemm(gp, x_bf16, f16 ? 1 : 0, w, w_bits, scale_bf16, offset_bf16, bias, out_bf16, M, N, K, ldx, ldw_k,
                              ldo, workspace, stream);
    }
    const WqPlan pl = make_plan(M, N, K, w_bits, group_size, n_major, ldw_k, ldx, x_bf16, w, scale_bf16, offset_bf16);
    if (!pl.fast) return generic();
    if (pl.S > 1) {
        if (preferred != kPreferStream && !workspace_holds(pl.partial_bytes + pl.counter_bytes)) return generic();
        if (!workspace || workspace_bytes < pl.partial_bytes + pl.counter_bytes) return MI355_ERR_WORKSPACE;
        if (!aligned(workspace, 16)) return MI355_ERR_ALIGNMENT;
    }

    WqArgs p;
    p.x = static_cast<const uint16_t *>(x_bf16);
    p.w = w;
    p.scale = static_cast<const uint16_t *>(scale_bf16);
    p.offset = static_cast<const uint16_t *>(offset_bf16);
    p.bias = static_cast<const uint16_t *>(bias);
    p.out = static_cast<uint16_t *>(out_bf16);
    // counters first (they must start at zero and are left at zero), partial sums after them
    p.counter = pl.S > 1 ? static_cast<uint32_t *>(workspace) : nullptr;
    p.partial = pl.S > 1 ? reinterpret_cast<float *>(static_cast<char *>(workspace) + pl.counter_bytes) : nullptr;
    p.ldx = ldx;
    p.ldo = ldo;
    p.ldw_bytes = (uint32_t)(w_bits == 4 ? ldw_k * 4 : ldw_k);
    p.row_bytes = (uint32_t)(w_bits == 4 ? N / 2 : N);
    p.M = (int)M;
    p.N = (int)N;
    p.K = (int)K;
    p.unit_steps = pl.unit_steps;
    p.n_units = pl.n_units;
    p.grouped = group_size > 0 && group != K;
    p.strips = pl.strips;
    p.sgroups = pl.sgroups;
    p.S = pl.S;
    if (f16) return w_bits == 4 ? launch_bits<4, 1>(p, pl, s) : launch_bits<8, 1>(p, pl, s);
    return w_bits == 4 ? launch_bits<4, 0>(p, pl, s) : launch_bits<8, 0>(p, pl, s);
}
