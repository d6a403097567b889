// npu_weight_quant_batchmatmul with int4 weights packed along K: the int32 words of a column hold consecutive k
// (storage [N, K/8]), which is what the contrib module passes - it keeps the weight [out_features, in_features/8] and
// hands over the transposed view (torch_npu/contrib/module/linear_weight_quant.py:71,106).
//
// In this layout a weight row already holds consecutive k of ONE output column, the order an MFMA operand lane
// wants: a wavefront owns 16 columns (16 weight rows) for the whole K range of its workgroup, loads them straight
// into registers and keeps one accumulator tile per m tile.  Nothing is reduced across wavefronts, and with 16
// columns per wavefront there are enough tiles to fill the chip without splitting K (the N-packed layout needs a
// 32-way split of K at the same shape, and an exchange of partial sums after it).
//
// K advances in steps of 128 bytes per row = 256 k = two sub-steps of 128 k.  Lane (c, g) gets bytes [16g, 16g+16) of
// both 64-byte halves of row c: 32 nibbles each, four MFMAs per half, one per dword.  The eight nibbles of a dword
// are expanded to the exact integer image of weight_quant_common.h with two mask operations and four byte permutes,
// which leaves them in the order 0,2,4,6,1,3,5,7; the activation fragments are staged in the same order.
// Per scale group (a whole number of sub-steps):  out += scale_g * (P_g + offset_g * X_g), see weight_quant_matmul.hip.
#include "weight_quant_common.h"
#include "weight_quant_kpacked.h"

namespace mi355 {
namespace {

// eight nibbles (already XORed with 8: u = w + 8) -> eight 16-bit images in the order 0,2,4,6,1,3,5,7
template <int ACT>
__device__ __forceinline__ u32x4 expand_word(uint32_t v)
{
    u32x4 b;
    if constexpr (ACT == 0) {
        // bf16 image 0x4100 | u << 3: the shifted nibble fills the low byte, 0x41 is the high byte
        const uint32_t e = (v << 3) & 0x78787878u, o = (v >> 1) & 0x78787878u;
        b[0] = __builtin_amdgcn_perm(0x41414141u, e, 0x04010400u);
        b[1] = __builtin_amdgcn_perm(0x41414141u, e, 0x04030402u);
        b[2] = __builtin_amdgcn_perm(0x41414141u, o, 0x04010400u);
        b[3] = __builtin_amdgcn_perm(0x41414141u, o, 0x04030402u);
    } else {
        // fp16 image 0x4c00 | u << 6
        const uint32_t e = v & 0x0f0f0f0fu, o = (v >> 4) & 0x0f0f0f0fu;
        b[0] = (__builtin_amdgcn_perm(0u, e, 0x0c010c00u) << 6) | 0x4c004c00u;
        b[1] = (__builtin_amdgcn_perm(0u, e, 0x0c030c02u) << 6) | 0x4c004c00u;
        b[2] = (__builtin_amdgcn_perm(0u, o, 0x0c010c00u) << 6) | 0x4c004c00u;
        b[3] = (__builtin_amdgcn_perm(0u, o, 0x0c030c02u) << 6) | 0x4c004c00u;
    }
    return b;
}

// 16-bit elements 0..7 of a 16-byte piece -> order 0,2,4,6,1,3,5,7
__device__ __forceinline__ u32x4 even_odd(u32x4 v)
{
    u32x4 r;
    r[0] = __builtin_amdgcn_perm(v[1], v[0], 0x05040100u);
    r[1] = __builtin_amdgcn_perm(v[3], v[2], 0x05040100u);
    r[2] = __builtin_amdgcn_perm(v[1], v[0], 0x07060302u);
    r[3] = __builtin_amdgcn_perm(v[3], v[2], 0x07060302u);
    return r;
}

// MT: m tiles (16 rows) per workgroup; NW x NTW: 16-column tiles per workgroup, NTW of them per wavefront (with four
// m tiles a wavefront takes two: an activation fragment read from LDS then feeds two weight tiles, and the row sums
// are formed once per wavefront instead of once per column tile); KS: slices of the workgroup's K range -
// NW * KS wavefronts, the slices are added in LDS at the end (two wavefronts per SIMD where the column tiles alone
// would leave one: a single wavefront cannot hide its own MFMA and LDS latencies); G128: a scale group is one
// sub-step (group_size 128), so every half step starts its sums from zero and ends with a fold - no counters, and
// the first MFMA of a half takes a zero accumulator instead of a cleared register
template <int MT, int NW, int KS, int NTW, int ACT, bool G128>
__global__ __launch_bounds__(NW * KS * 64) void wq_kpacked_kernel(const WqArgs p)
{
    static_assert(MT * KS <= 4, "a chunk holds at least one step of every slice");
    constexpr int WAVES = NW * KS, NBW = NW * NTW * 16, THREADS = WAVES * 64;
    constexpr int DA = MT * NTW >= 8 ? 1 : 2;           // accumulators per sum, used alternately (short dependent chains)
    constexpr int CH = 4 / (MT * KS);                   // steps per slice and chunk of activations (32 KiB of LDS per buffer)
    constexpr int RS = MT == 4 ? (NW == 8 ? 2 : 4) : 8;                 // steps per round of the main loop: two batches of weight loads in
    constexpr int BODY = RS / 2;                        // registers (one consumed, one in flight; 2 KiB per step and
                                                        // wavefront), the slot of a step known at compile time
    constexpr int POLICY = MT == 1 ? kNonTemporal : 0;
    constexpr int FP = 1024 + 16;                       // pitch of a 1 KiB activation fragment in LDS: the staging writes
                                                        // of a wavefront go to sixteen fragments at the same lane
                                                        // position, which an unpadded pitch puts into the same banks
    constexpr int XBUF = 32 * FP;                       // bytes of one activation chunk in LDS
    constexpr int TBUF = 2048;                          // one step of one wavefront's weights (16 rows x 128 bytes)
    constexpr int PPR = CH * 32;                        // 16-byte pieces of an activation row per slice and chunk
    constexpr int PPT = 2048 / THREADS;                 // pieces per thread and chunk
    constexpr float P_MUL = kImageMul<4, ACT>, X_BIAS = kImageBias<4>;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int ct = wave % NW, ks = wave / NW;           // column tile and K slice of this wavefront
    const int xcd_slot = blockIdx.x >> 3;
    const int tile = (blockIdx.x & 7) + 8 * (xcd_slot / p.S);
    const int chunk = xcd_slot % p.S;
    if (tile >= p.sgroups) return;
    const int m_base = blockIdx.y * (MT * 16);
    const int rows_valid = min(MT * 16, p.M - m_base);
    const int n0 = tile * NBW;

    // K range of this workgroup in steps of 256 (whole units: a unit is a whole number of steps and of scale groups)
    const int u0 = (int)((int64_t)p.n_units * chunk / p.S), u1 = (int)((int64_t)p.n_units * (chunk + 1) / p.S);
    const int wg_step0 = u0 * p.unit_steps, wg_nsteps = (u1 - u0) * p.unit_steps;
    // ... and of slice s of the workgroup (whole units again); every wavefront runs the rounds of the longest slice
    auto slice_u0 = [&](int s) { return (int)((int64_t)(u1 - u0) * s / KS); };
    const int step0 = wg_step0 + slice_u0(ks) * p.unit_steps, nsteps = (slice_u0(ks + 1) - slice_u0(ks)) * p.unit_steps;
    const int nrounds = ((u1 - u0 + KS - 1) / KS * p.unit_steps + RS - 1) / RS;
    // scale groups in sub-steps of 128 k (per channel: one group that ends with the wavefront's range)
    const int gsub = p.grouped ? p.unit_sub : 2 * nsteps;
    const int grp0 = p.grouped ? (2 * wg_step0) / p.unit_sub : 0;                       // first group of the workgroup
    const int ngroups = p.grouped ? (2 * wg_nsteps) / p.unit_sub : 1;                   // groups of the workgroup
    const int gl0 = p.grouped ? (2 * (step0 - wg_step0)) / p.unit_sub : 0;              // first group of this wavefront

    // Weights: a load instruction fetches whole cache lines - lane l takes 16 bytes of row l/8 (+8 for the second
    // load) - and the wavefront turns the step around through a private 2 KiB LDS tile into operand order.  The
    // 16-byte chunk a lane fetches is XOR-swizzled with the row pair so that the operand reads (16 rows x 16 bytes)
    // are free of bank conflicts; LDS slot s of row r holds chunk s ^ ((r >> 1) & 7).
    const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(p.w, (uint32_t)((uint64_t)(p.N - 1) * p.ldw_bytes + p.row_bytes));
    uint32_t voff_w[NTW][2];
#pragma unroll
    for (int tt = 0; tt < NTW; tt++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int rl = 8 * h + (lane >> 3);
            voff_w[tt][h] = (uint32_t)min(n0 + (ct * NTW + tt) * 16 + rl, p.N - 1) * p.ldw_bytes +
                            (uint32_t)(((lane & 7) ^ ((rl >> 1) & 7)) * 16);
        }
    char *tbuf = lds + 16 + 2 * XBUF + wave * (NTW * 2 * TBUF);                               // [step parity][tile][2 KiB]
    uint32_t *prm = reinterpret_cast<uint32_t *>(lds + 16 + 2 * XBUF + WAVES * NTW * 2 * TBUF);   // [group][column]: scale | offset << 16
    const int t_rd = c * 128 + ((g ^ ((c >> 1) & 7)) * 16);   // chunk g of row c; chunk g + 4 is at slot ^ 4, i.e. +-64 bytes
    const __amdgpu_buffer_rsrc_t rsrc_x =
        make_rsrc(p.x + (int64_t)m_base * p.ldx, (uint32_t)(((int64_t)(rows_valid - 1) * p.ldx + p.K) * 2));

    u32x4 wq[2][BODY][NTW][2];
    auto load_body = [&](int slot, int st) {    // st: first step of the batch, relative to step0
#pragma unroll
        for (int j = 0; j < BODY; j++) {
            const bool ok = st + j < nsteps;
            const uint32_t kb = (uint32_t)(step0 + st + j) * 128u;
#pragma unroll
            for (int tt = 0; tt < NTW; tt++) {
                wq[slot][j][tt][0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, ok ? voff_w[tt][0] : kOutOfRange, kb, POLICY);
                wq[slot][j][tt][1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, ok ? voff_w[tt][1] : kOutOfRange, kb, POLICY);
            }
        }
    };
    // Activation staging: piece q of a row's chunk of one slice (8 consecutive k) belongs to step q / 32, half
    // (q % 32) / 16, lane group (q % 16) / 4 and dword q % 4 of that lane's 16 bytes; it goes to fragment
    // (slice, step, m tile, 4 * half + dword) at lane (group, row % 16).  Consecutive threads read consecutive pieces
    // of a row.
    u32x4 xst[PPT];
    auto stage_load = [&](int ch) {
#pragma unroll
        for (int i = 0; i < PPT; i++) {
            const int pid = i * THREADS + threadIdx.x;
            const int r = pid / (KS * PPR), sl = (pid / PPR) % KS, q = pid % PPR;
            const int s0 = slice_u0(sl) * p.unit_steps, sn = (slice_u0(sl + 1) - slice_u0(sl)) * p.unit_steps;
            const bool ok = r < rows_valid && ch * CH + (q >> 5) < sn;
            xst[i] = __builtin_amdgcn_raw_buffer_load_b128(
                rsrc_x, ok ? (uint32_t)((r * (int)p.ldx + (wg_step0 + s0 + ch * CH) * 256 + q * 8) * 2) : kOutOfRange, 0u, 0);
        }
    };
    // rows past the last valid one are never written: they only feed accumulator rows that are never stored
    const int valid_pieces = rows_valid * KS * PPR;
    auto stage_store = [&](int ch) {
        char *buf = lds + 16 + (ch & 1) * XBUF;
#pragma unroll
        for (int i = 0; i < PPT; i++) {
            if (i * THREADS >= valid_pieces) break;         // uniform over the workgroup
            const int pid = i * THREADS + threadIdx.x;
            const int r = pid / (KS * PPR), sl = (pid / PPR) % KS, q = pid % PPR;
            const int st = q >> 5, f = 4 * ((q >> 4) & 1) + (q & 3), gg = (q >> 2) & 3;
            *reinterpret_cast<u32x4 *>(buf + (((sl * CH + st) * MT + (r >> 4)) * 8 + f) * FP + (gg * 16 + (r & 15)) * 16) =
                even_odd(xst[i]);
        }
    };

    f32x4 P[MT][NTW][DA], X[MT][DA], tot[MT][NTW];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int a = 0; a < DA; a++) {
            X[mt][a] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int tt = 0; tt < NTW; tt++) P[mt][tt][a] = tot[mt][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    const u32x4 ones = u32x4{kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>};
    auto fold = [&](int gl) {
        f32x4 xs[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) xs[mt] = DA == 2 ? X[mt][0] + X[mt][DA - 1] : X[mt][0];
#pragma unroll
        for (int tt = 0; tt < NTW; tt++) {
            const uint32_t pr = prm[gl * NBW + (ct * NTW + tt) * 16 + c];
            const float sc = act_lo<ACT>(pr) * P_MUL;
            const float of = (act_hi<ACT>(pr) - X_BIAS) * (1.0f / P_MUL);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const f32x4 ps = DA == 2 ? P[mt][tt][0] + P[mt][tt][DA - 1] : P[mt][tt][0];
#pragma unroll
                for (int q = 0; q < 4; q++)
                    tot[mt][tt][q] = __builtin_fmaf(sc, __builtin_fmaf(of, xs[mt][q], ps[q]), tot[mt][tt][q]);
            }
        }
        if constexpr (!G128) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int a = 0; a < DA; a++) {
                    X[mt][a] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int tt = 0; tt < NTW; tt++) P[mt][tt][a] = f32x4{0.f, 0.f, 0.f, 0.f};
                }
        }
    };

    // prologue: the antiquant parameters are requested first (they come from HBM, and the first barrier waits for
    // them), then the activations of chunk 0 (from cache) and the first batch of weights
    {
        // parameters of the workgroup's columns and groups, any strides: walk along whichever dimension is
        // contiguous in memory; eight loads in flight per thread, no branches around them (indices past the end
        // repeat the last entry; without offsets the scale is loaded twice and masked).  `inner` is a power of two in
        // all usual cases, which spares the integer divisions.
        const bool n_inner = p.ld_param_n == 1;
        const int inner = n_inner ? NBW : ngroups, total = ngroups * NBW;
        const int shift = (inner & (inner - 1)) == 0 ? 31 - __builtin_clz(inner) : -1;
        const uint16_t *offp = p.offset ? p.offset : p.scale;
        const uint32_t omask = p.offset ? 0xffffu : 0u;
        auto batch = [&](int base, bool first) {
            uint32_t sv[8], ov[8];
            int at_lds[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int idx = min(base + i * THREADS + (int)threadIdx.x, total - 1);
                int a, b;
                if (shift >= 0) a = idx & (inner - 1), b = idx >> shift;
                else a = idx % inner, b = idx / inner;
                const int col = n_inner ? a : b, gl = n_inner ? b : a;
                const int64_t at = (int64_t)(grp0 + gl) * p.ld_param_g + (int64_t)min(n0 + col, p.N - 1) * p.ld_param_n;
                sv[i] = p.scale[at];
                ov[i] = offp[at];
                at_lds[i] = gl * NBW + col;
            }
            if (first) {
                __builtin_amdgcn_sched_barrier(0);
                stage_load(0);
                load_body(0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) prm[at_lds[i]] = sv[i] | ((ov[i] & omask) << 16);
        };
        for (int base = 8 * THREADS; base < total; base += 8 * THREADS) batch(base, false);
        batch(0, true);
    }
    stage_store(0);
    __syncthreads();
    // the second batch of weights goes out behind the barrier: ahead of it, it would sit in the memory queues in
    // front of the activation and parameter loads of the wavefronts that arrive later
    load_body(1, BODY);
    __builtin_amdgcn_sched_barrier(0);
    // step 0 of the weights goes through the wavefront's turn-around tile into operand order
    u32x4 w[NTW][2];
#pragma unroll
    for (int tt = 0; tt < NTW; tt++) {
        *reinterpret_cast<u32x4 *>(tbuf + tt * TBUF + lane * 16) = wq[0][0][tt][0];
        *reinterpret_cast<u32x4 *>(tbuf + tt * TBUF + 1024 + lane * 16) = wq[0][0][tt][1];
        w[tt][0] = *reinterpret_cast<const u32x4 *>(tbuf + tt * TBUF + t_rd);
        w[tt][1] = *reinterpret_cast<const u32x4 *>(tbuf + tt * TBUF + (t_rd ^ 64));
    }

    // activation fragments of one half step (four MFMA k blocks per m tile); with one or two m tiles the next half
    // of the same chunk is requested while the current one is multiplied
    // (with four m tiles: one buffer, filled two k blocks at a time)
    constexpr int XA = MT <= 2 ? 2 : 1;
    constexpr int DG = MT <= 2 ? 4 : 2;                 // k blocks per request
    u32x4 xa[XA][DG][MT];
    auto read_xa = [&](int buf, const char *xb, int jc, int h, int d0) {
#pragma unroll
        for (int d = 0; d < DG; d++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
                xa[buf][d][mt] = *reinterpret_cast<const u32x4 *>(xb + (((ks * CH + jc) * MT + mt) * 8 + 4 * h + d0 + d) * FP);
    };

    int in_group = 0, gl = gl0, ch = 0;
    for (int rd = 0; rd < nrounds; rd++) {
#pragma unroll
        for (int j = 0; j < RS; j++) {
            const int st = rd * RS + j;
            const int jc = j % CH;                          // step inside the activation chunk
            const int slot = j / BODY, js = j % BODY;
            if (jc == 0) stage_load(ch + 1);                // past the end: zeros, no memory traffic
            const char *xb = lds + 16 + (ch & 1) * XBUF + lane * 16;
            // this step's weights are in w (operand order); the next step's registers go through the other half of
            // the turn-around tile and are read back at once, so that their latency hides behind this step
            u32x4 wc[NTW][2];
#pragma unroll
            for (int tt = 0; tt < NTW; tt++) {
                wc[tt][0] = w[tt][0] ^ 0x88888888u;
                wc[tt][1] = w[tt][1] ^ 0x88888888u;
                const int sn = ((j + 1) / BODY) & 1, jsn = (j + 1) % BODY;
                char *tn = tbuf + (((j + 1) & 1) * NTW + tt) * TBUF;
                *reinterpret_cast<u32x4 *>(tn + lane * 16) = wq[sn][jsn][tt][0];
                *reinterpret_cast<u32x4 *>(tn + 1024 + lane * 16) = wq[sn][jsn][tt][1];
                w[tt][0] = *reinterpret_cast<const u32x4 *>(tn + t_rd);
                w[tt][1] = *reinterpret_cast<const u32x4 *>(tn + (t_rd ^ 64));
            }
            if (js == BODY - 1) {               // the batch has left the registers: refill its slot two batches ahead
                __builtin_amdgcn_sched_barrier(0);
                load_body(slot, st + 1 + BODY);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int cur = XA == 2 ? (2 * j + h) & 1 : 0;
                if constexpr (XA == 2) {
                    if (jc == 0 && h == 0) read_xa(cur, xb, jc, h, 0);
                    if (!(jc == CH - 1 && h == 1)) read_xa(cur ^ 1, xb, h ? jc + 1 : jc, h ^ 1, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    if constexpr (XA == 1) {
                        if (d % DG == 0) read_xa(0, xb, jc, h, d);
                    }
                    u32x4 b[NTW];
#pragma unroll
                    for (int tt = 0; tt < NTW; tt++) b[tt] = expand_word<ACT>(wc[tt][h][d]);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        const f32x4 zero = f32x4{0.f, 0.f, 0.f, 0.f};
                        const bool first = G128 && d < DA;          // a group starts with this half step
#pragma unroll
                        for (int tt = 0; tt < NTW; tt++)
                            P[mt][tt][d % DA] = mfma_act<ACT>(xa[cur][d % DG][mt], b[tt], first ? zero : P[mt][tt][d % DA]);
                        X[mt][d % DA] = mfma_act<ACT>(xa[cur][d % DG][mt], ones, first ? zero : X[mt][d % DA]);
                    }
                }
                if constexpr (G128) {
                    if (st < nsteps) fold(gl++);
                } else if (st < nsteps && ++in_group == gsub) {
                    fold(gl);
                    in_group = 0;
                    gl++;
                }
            }
            if (jc == CH - 1) {
                stage_store(ch + 1);
                __syncthreads();
                ch++;
            }
        }
    }

    // ---- output: the wavefront's [rows x 16 columns] tile goes through LDS to the shared output / exchange code
    float *red = reinterpret_cast<float *>(lds + 16);
    TileOut<NBW, KS, THREADS, ACT> outp(p, lds, m_base, n0, chunk);
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        const int rows_mt = min(16, rows_valid - mt * 16);
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int row = 4 * g + q;
#pragma unroll
            for (int tt = 0; tt < NTW; tt++)
                if (row < rows_mt) red[(ks * 16 + row) * NBW + (ct * NTW + tt) * 16 + c] = tot[mt][tt][q];
        }
        __syncthreads();
        outp.emit_mtile(red, mt * 16, rows_mt);
    }
    outp.finish(rows_valid, tile);
}

template <int MT, int NW, int KS, int NTW, int ACT, bool G128>
int launch_one(const WqArgs &p, const WqKpackedPlan &pl, hipStream_t s)
{
    auto kern = wq_kpacked_kernel<MT, NW, KS, NTW, ACT, G128>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)((pl.tiles + 7) / 8 * 8 * pl.S), (unsigned)pl.mchunks), dim3(NW * KS * 64),
                       pl.lds_bytes, s, p);
    return check_launch();
}

template <int ACT, bool G128>
int launch_shape(const WqArgs &p, const WqKpackedPlan &pl, hipStream_t s)
{
    if (pl.mt == 4)     // two column tiles per wavefront
        return pl.nw == 4 ? launch_one<4, 4, 1, 2, ACT, G128>(p, pl, s) : launch_one<4, 8, 1, 2, ACT, G128>(p, pl, s);
    if (pl.nw == 4 && pl.ks == 2)
        return pl.mt == 1 ? launch_one<1, 4, 2, 1, ACT, G128>(p, pl, s) : launch_one<2, 4, 2, 1, ACT, G128>(p, pl, s);
    if (pl.nw == 4) return pl.mt == 1 ? launch_one<1, 4, 1, 1, ACT, G128>(p, pl, s) : launch_one<2, 4, 1, 1, ACT, G128>(p, pl, s);
    return pl.mt == 1 ? launch_one<1, 8, 1, 1, ACT, G128>(p, pl, s) : launch_one<2, 8, 1, 1, ACT, G128>(p, pl, s);
}

template <int ACT>
int launch_act(const WqArgs &p, const WqKpackedPlan &pl, hipStream_t s)
{
    const bool g128 = pl.grouped && pl.unit_sub == 1;
    return g128 ? launch_shape<ACT, true>(p, pl, s) : launch_shape<ACT, false>(p, pl, s);
}

int64_t gcd64(int64_t a, int64_t b)
{
    while (b) {
        const int64_t t = a % b;
        a = b;
        b = t;
    }
    return a;
}

} // namespace

WqKpackedPlan make_wq_kpacked_plan(int64_t M, int64_t N, int64_t K, int64_t group_size, int64_t ldw_n, int64_t ldx, const void *x,
                                   const void *w)
{
    WqKpackedPlan pl{};
    const int64_t group = group_size > 0 ? group_size : K;
    pl.ok = M > 0 && K > 0 && K % 256 == 0 && group % 128 == 0 && N % 8 == 0 && ldw_n >= K / 8 && ldw_n % 4 == 0 && ldx % 8 == 0 &&
            (x == nullptr || aligned(x, 16)) && (w == nullptr || aligned(w, 16)) &&
            (uint64_t)N * (uint64_t)ldw_n * 4 < (1ull << 32) && (uint64_t)M * (uint64_t)ldx * 2 < (1ull << 32);
    if (!pl.ok) return pl;
    pl.mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
    if (const int f = knob(kKnobWqkMt))      // tuning aid
        if (f == 1 || f == 2 || f == 4) pl.mt = f;
    pl.mchunks = (int)((M + pl.mt * 16 - 1) / (pl.mt * 16));
    pl.grouped = group_size > 0 && group != K;
    pl.unit_sub = pl.grouped ? (int)(group / 128) : 0;
    // K may be split between workgroups at multiples of a step (256) that are also multiples of a scale group
    const int64_t unit = pl.grouped ? group / gcd64(group, 256) * 256 : 256;
    pl.unit_steps = (int)(unit / 256);
    pl.n_units = (int)(K / unit);
    if (K % unit != 0) {                  // one unit: no split
        pl.unit_steps = (int)(K / 256);
        pl.n_units = 1;
    }
    // eight wavefronts per workgroup when that still gives (nearly) every CU a workgroup, else four; with four m tiles a
    // wavefront owns two column tiles
    pl.ntw = pl.mt == 4 ? 2 : 1;
    const int tiles8 = (int)((N + 8 * pl.ntw * 16 - 1) / (8 * pl.ntw * 16));
    const int64_t wgs8 = (int64_t)tiles8 * pl.mchunks;
    bool eight = wgs8 >= 200;
    if (pl.mt == 4 && !eight) {
        // ... or, with four m tiles, when a split of K of at most eight fills the CUs with them (measured on layer
        // projections at 48-192 rows: 14336x4096 at 128 rows 47.4 -> 40.4 us, 8192x8192 47.6 -> 38.3, 4096x14336 at 48
        // rows 27.5 -> 24.2; a sixteen-way split of eight-wavefront workgroups loses to an eight-way one of four)
        const int64_t s8 = kNumCU / wgs8;
        eight = wgs8 >= 160 || (s8 <= 8 && s8 <= pl.n_units && wgs8 * s8 >= 224);
    }
    pl.nw = eight ? 8 : 4;
    if (const int f = knob(kKnobWqkNw))      // tuning aid
        if (f == 4 || f == 8) pl.nw = f;
    const int wg_cols = pl.nw * pl.ntw * 16;
    pl.tiles = (int)((N + wg_cols - 1) / wg_cols);
    pl.ks = 1;
    int S = kNumCU / (pl.tiles * pl.mchunks);
    if (S > pl.n_units) S = pl.n_units;
    if (S > 16) S = 16;
    if (S < 1) S = 1;
    if (const int f = knob(kKnobWqSplit))
        if (f >= 1 && f <= pl.n_units) S = f;
    if ((uint64_t)S * (uint64_t)M * (uint64_t)N * 4 >= (1ull << 32)) S = 1;
    if (S > 1 && (size_t)pl.tiles * pl.mchunks * sizeof(uint32_t) > kWorkspaceCounterBytes) S = 1;
    // the parameter table of a workgroup's K range must fit in LDS beside the activation chunks and turn-around tiles
    auto lds_need = [&](int s) {
        const int64_t units = (pl.n_units + s - 1) / s;
        const int64_t groups = pl.grouped ? units * pl.unit_steps * 2 / pl.unit_sub : 1;
        const int waves = pl.nw * (pl.nw == 4 && pl.mt <= 2 ? 2 : 1);                    // two K slices at most
        return (size_t)16 + 2 * 32 * (1024 + 16) + (size_t)waves * pl.ntw * 4096 + (size_t)groups * wg_cols * 4;
    };
    while (lds_need(S) > 160 * 1024 && S < pl.n_units && S < 16) S++;
    if (lds_need(S) > 160 * 1024) {
        pl.ok = false;
        return pl;
    }
    pl.S = S;
    // with four column tiles and at most two m tiles the workgroup's K range is cut into two slices (eight wavefronts,
    // two per SIMD) when it holds at least two units
    if (pl.nw == 4 && pl.mt <= 2 && (pl.n_units + S - 1) / S >= 2 && knob(kKnobWqkKs) != 1) pl.ks = 2;
    pl.lds_bytes = lds_need(S);
    pl.partial_bytes = S > 1 ? (size_t)S * M * N * sizeof(float) : 0;
    pl.counter_bytes = S > 1 ? kWorkspaceZeroBytes : 0;
    return pl;
}

int launch_wq_kpacked(const WqKpackedPlan &pl, const void *x, int act_f16, const void *w, const void *scale, const void *offset,
                      const void *bias, void *out, int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw_n, int64_t ldo,
                      int64_t ld_param_g, int64_t ld_param_n, void *workspace, void *stream)
{
    WqArgs p{};
    p.x = static_cast<const uint16_t *>(x);
    p.w = w;
    p.scale = static_cast<const uint16_t *>(scale);
    p.offset = static_cast<const uint16_t *>(offset);
    p.bias = static_cast<const uint16_t *>(bias);
    p.out = static_cast<uint16_t *>(out);
    p.counter = pl.S > 1 ? static_cast<uint32_t *>(workspace) : nullptr;
    p.partial = pl.S > 1 ? reinterpret_cast<float *>(static_cast<char *>(workspace) + pl.counter_bytes) : nullptr;
    p.ldx = ldx;
    p.ldo = ldo;
    p.ldw_bytes = (uint32_t)(ldw_n * 4);
    p.row_bytes = (uint32_t)(K / 2);
    p.M = (int)M;
    p.N = (int)N;
    p.K = (int)K;
    p.unit_steps = pl.unit_steps;
    p.n_units = pl.n_units;
    p.grouped = pl.grouped;
    p.unit_sub = pl.unit_sub;
    p.ld_param_g = ld_param_g;
    p.ld_param_n = ld_param_n;
    p.strips = pl.tiles;
    p.sgroups = pl.tiles;
    p.S = pl.S;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return act_f16 ? launch_act<1>(p, pl, s) : launch_act<0>(p, pl, s);
}

} // namespace mi355
