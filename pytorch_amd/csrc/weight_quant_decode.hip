// npu_weight_quant_batchmatmul, decode shapes (at most 32 activation rows) with int4 weights packed along N: the job
// is one pass over the packed weights, and at these sizes (tens of megabytes) the launch is as much a latency
// problem as a bandwidth problem.  The kernel is therefore built around three rules:
//   * every byte a wavefront will ever need is requested in its first instructions (its activations, its antiquant
//     parameters, its whole weight tile) and consumed in arrival order: there is no barrier, no LDS staging and no
//     dependent load in front of the arithmetic;
//   * a wavefront's tile is 128 weight rows x one 128-byte strip (256 columns): the rows of one scale group, so the
//     per-group fold  out += scale * (P + offset * X)  (see weight_quant_matmul.hip) happens once, after the loop;
//   * the partial sums of the workgroups that share a strip meet without counters or fences: every workgroup but
//     the one with the highest index stores its partial with agent-scope write-through stores into a region of the
//     workspace that is zero between launches, mapping a zero sum to -0.0 so that every stored word is non-zero; the
//     workgroup with the highest index of the strip (dispatched after the others, so those are running or done)
//     reads the words back with agent-scope loads until none is zero, adds them in chunk order to its own sum,
//     writes the output and stores the zeros back.  The critical path after the last weight byte is one store, one
//     load and the output store; the relaxed agent-scope counter it replaces cost an acknowledged store, an atomic
//     round trip and a load.  The wait is bounded: after max_polls unanswered polls a thread gives up, stores NaN where
//     its sums should be and sets the workspace's sticky status word, which mi355_workspace_status() reports to the host
//     (the launch still ends).  The order of dispatch that the scheme leans on - a strip's highest workgroup index
//     starts last - is what the hardware does today, not a guarantee; the bound and the status word are the net.
#include "weight_quant_common.h"
#include "weight_quant_decode.h"

namespace mi355 {
namespace {

struct WqDecArgs {
    const uint16_t *x, *scale, *offset, *bias;
    const void *w;
    uint16_t *out;
    uint32_t *zone;                 // [S-1][M][N] float32 bit patterns, zero between launches
    int64_t ldx, ldo;
    uint32_t ldw_bytes, row_bytes;
    int M, N, K;
    int group_rows;                 // rows of a scale group (K when per channel)
    int strips, S;
    int l2_exchange;                // producers on the collector's XCD leave their sums in the L2
    int max_polls;                  // bound of the collector's wait
    int only_chunk;                 // testing aid: c + 1 = only the workgroups of chunk c run
    uint32_t *status;               // the workspace's sticky status word
};

constexpr int kMaxPolls = 1 << 20;
constexpr int SC1 = 16;             // cache-policy bit: agent scope

// MT: m tiles of 16 activation rows (1 or 2); QPT: output quads per thread and m tile (rows x 64 quads over 512 threads):
// 1 up to 8 rows, 2 up to 16.  With two m tiles the accumulators take half of the register file, so the weight tile is
// requested two steps at a time instead of all at once.
template <int ACT, int MT, int QPT>
__global__ __launch_bounds__(512) void wq_decode4_kernel(const WqDecArgs p)
{
    constexpr int STEPS = 4;                    // 32-row steps of a wavefront's tile
    constexpr int PFS = MT == 1 ? 4 : 2;        // steps in flight
    constexpr int NT = 16;                      // MFMA column sets per lane = its 16 consecutive columns
    constexpr int NBW = 256;                    // columns of a strip
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    // Workgroups are dealt round-robin to the 8 XCDs; the last chunk of a strip has the highest index of the strip.
    const int xcd_slot = blockIdx.x >> 3;
    const int strip = (blockIdx.x & 7) + 8 * (xcd_slot / p.S), chunk = xcd_slot % p.S;
    if (strip >= p.strips) return;
    if (p.only_chunk && chunk != (p.only_chunk < 0 ? p.S - 1 : p.only_chunk - 1)) return;      // testing aid (host-driven give-up of the collector)
    // The chunks of a strip sit on one XCD.  The collector says on which it runs (a word per strip behind the sums); a
    // producer that finds itself there leaves its sums in the shared L2 with ordinary stores, which the collector's polls
    // (they bypass the vector L1) see a microsecond before stores that write through to memory.
    const uint32_t zone_chunk_bytes = (uint32_t)p.M * (uint32_t)p.N * 4u;
    const uint32_t flag_base = zone_chunk_bytes * (uint32_t)(p.S - 1);
    const __amdgpu_buffer_rsrc_t rsrc_z = make_rsrc(p.zone, p.S > 1 ? flag_base + (uint32_t)p.strips * 4u : 0u);
    const bool collector = p.S > 1 && chunk == p.S - 1;
    const uint32_t my_xcd = __builtin_amdgcn_s_getreg(kHwRegXccId) + 1u;
    if (collector && threadIdx.x == 0) __builtin_amdgcn_raw_buffer_store_b32(my_xcd, rsrc_z, (uint32_t)strip * 4u, flag_base, SC1);
    const int row0 = (chunk * 8 + wave) * (32 * STEPS);
    const bool wave_live = row0 < p.K;          // K is a multiple of 128: a wavefront's tile is inside K or wholly outside
    const int n0 = strip * NBW;

    const bool lane_ok = (uint32_t)strip * 128u + (uint32_t)c * 8u < p.row_bytes;
    f32x4 tot[MT][NT];
    if (wave_live) {
        // ---- requests: activations, parameters, the weight tile
        const __amdgpu_buffer_rsrc_t rsrc_x = make_rsrc(p.x, (uint32_t)(((int64_t)(p.M - 1) * p.ldx + p.K) * 2));
        u32x4 xa[PFS][MT];
        auto load_x = [&](int slot, int s) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const int m = mt * 16 + c;
                xa[slot][mt] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, m < p.M ? (uint32_t)((m * (int)p.ldx + 8 * g) * 2) : kOutOfRange,
                                                                     (uint32_t)(row0 + 32 * s) * 2u, 0);
            }
        };
#pragma unroll
        for (int s = 0; s < PFS; s++) load_x(s, s);
        const bool has_offset = p.offset != nullptr;
        const int grp = row0 / p.group_rows;
        const uint32_t param_bytes = (uint32_t)(p.K / p.group_rows) * (uint32_t)p.N * 2u;
        const __amdgpu_buffer_rsrc_t rsrc_s = make_rsrc(p.scale, param_bytes);
        const __amdgpu_buffer_rsrc_t rsrc_o = make_rsrc(has_offset ? p.offset : p.scale, param_bytes);
        const uint32_t voff_p = lane_ok ? (uint32_t)(n0 + 16 * c) * 2u : kOutOfRange;
        // A lane needs 64 bytes of parameters (16 scales, 16 offsets).  Lane (c, g) fetches the g-th 16-byte quarter
        // (g = 0, 1: scales, g = 2, 3: offsets; without offsets rsrc_o aliases the scales and the values are dropped at
        // the fold) so that the instruction carries no duplicate bytes; the four lanes of a column group exchange the
        // quarters through the LDS crossbar before the fold.
        const u32x4 pq = __builtin_amdgcn_raw_buffer_load_b128(g < 2 ? rsrc_s : rsrc_o, voff_p + 16u * (g & 1),
                                                               (uint32_t)grp * (uint32_t)p.N * 2u, 0);
        const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(p.w, (uint32_t)((uint64_t)(p.K - 1) * p.ldw_bytes + p.row_bytes));
        const uint32_t voff_w = lane_ok ? (uint32_t)(8 * g) * p.ldw_bytes + (uint32_t)strip * 128u + (uint32_t)c * 8u : kOutOfRange;
        u32x2 wq[PFS][8];
        auto load_step = [&](int slot, int s) {
#pragma unroll
            for (int t = 0; t < 8; t++)
                wq[slot][t] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, voff_w, (uint32_t)(row0 + 32 * s + t) * p.ldw_bytes,
                                                                   kNonTemporal);
        };
#pragma unroll
        for (int s = 0; s < PFS; s++) load_step(s, s);

        f32x4 P[MT][NT], X[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            X[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < NT; i++) P[mt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        const u32x4 ones = u32x4{kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>};
        const BlendRegs br = blend_regs<ACT>();

#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            // a step's arithmetic stays behind the previous step's: otherwise the compiler gathers the unpacking of
            // all steps in front of the first MFMA, which then waits for the last load
            __builtin_amdgcn_sched_barrier(0);
            const int slot = s % PFS;
            uint32_t w0[8], w1[8];
#pragma unroll
            for (int t = 0; t < 8; t++) {
                w0[t] = wq[slot][t].x;
                w1[t] = wq[slot][t].y;
            }
            u32x4 xs[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) xs[mt] = xa[slot][mt];
            if (s + PFS < STEPS) {
                __builtin_amdgcn_sched_barrier(0);
                load_x(slot, s + PFS);
                load_step(slot, s + PFS);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int h = 0; h < 2; h++) {
#pragma unroll
                for (int jb = 0; jb < 4; jb++) {
                    u32x4 b0, b1;
                    expand_pair_blend<ACT>(h ? w1 : w0, jb, br, b0, b1);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        P[mt][h * 8 + 2 * jb] = mfma_act<ACT>(xs[mt], b0, P[mt][h * 8 + 2 * jb]);
                        P[mt][h * 8 + 2 * jb + 1] = mfma_act<ACT>(xs[mt], b1, P[mt][h * 8 + 2 * jb + 1]);
                    }
                }
            }
#pragma unroll
            for (int mt = 0; mt < MT; mt++) X[mt] = mfma_act<ACT>(xs[mt], ones, X[mt]);
        }
        __builtin_amdgcn_sched_barrier(0);
        u32x4 sv[2], ov[2];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            sv[0][i] = (uint32_t)__builtin_amdgcn_ds_bpermute(c * 4, (int)pq[i]);
            sv[1][i] = (uint32_t)__builtin_amdgcn_ds_bpermute((16 + c) * 4, (int)pq[i]);
            ov[0][i] = (uint32_t)__builtin_amdgcn_ds_bpermute((32 + c) * 4, (int)pq[i]);
            ov[1][i] = (uint32_t)__builtin_amdgcn_ds_bpermute((48 + c) * 4, (int)pq[i]);
        }
        // ---- the single fold: tot = (scale * mul) * (P' + ((offset - bias) / mul) * X), both rescalings exact
#pragma unroll
        for (int i = 0; i < NT; i++) {
            const float P_MUL = (i & 1) ? kMulHi4<ACT> : kMulLo4<ACT>, X_BIAS = (i & 1) ? kBiasHi4<ACT> : kBiasLo4<ACT>;
            const uint32_t su = sv[i / 8][(i % 8) / 2], ou = ov[i / 8][(i % 8) / 2];
            const float sc = ((i & 1) ? act_hi<ACT>(su) : act_lo<ACT>(su)) * P_MUL;
            const float of = ((has_offset ? ((i & 1) ? act_hi<ACT>(ou) : act_lo<ACT>(ou)) : 0.0f) - X_BIAS) * (1.0f / P_MUL);
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int q = 0; q < 4; q++) tot[mt][i][q] = sc * __builtin_fmaf(of, X[mt][q], P[mt][i][q]);
        }
    } else {
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int i = 0; i < NT; i++) tot[mt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // ---- the eight wavefronts' sums meet in LDS, one m tile at a time: red[wave][row][column]
    float *red = reinterpret_cast<float *>(lds);
    constexpr int NQ = MT * QPT;                 // output quads per thread
    constexpr int CB = NQ <= 2 ? 4 : 3;          // chunks collected per batch
    f32x4 acc[NQ];
    uint32_t zoff[NQ];
    bool live[NQ];
#pragma unroll
    for (int e = 0; e < NQ; e++) {
        const int qd = (int)threadIdx.x + 512 * (e % QPT);
        const int row = qd / (NBW / 4), nl = (qd % (NBW / 4)) * 4, mt = e / QPT;
        live[e] = row < min(16, p.M - mt * 16) && n0 + nl < p.N;  // N is a multiple of 8: a quad is inside or outside
        zoff[e] = live[e] ? (uint32_t)(((mt * 16 + row) * p.N + n0 + nl) * 4) : kOutOfRange;
    }
    uint32_t collector_xcd = 0;
    if (p.S > 1 && !collector) collector_xcd = __builtin_amdgcn_raw_buffer_load_b32(rsrc_z, (uint32_t)strip * 4u, flag_base, SC1);   // used after the reduction
    // The strip's last workgroup asks for the other chunks' sums before it reduces its own: it was dispatched last, so
    // the others have usually stored theirs by now and the answers arrive while the LDS reduction runs.
    u32x4 v[NQ][CB];
#pragma unroll
    for (int e = 0; e < NQ; e++)
#pragma unroll
        for (int i = 0; i < CB; i++)
            v[e][i] = collector && live[e] && i < p.S - 1
                          ? __builtin_amdgcn_raw_buffer_load_b128(rsrc_z, zoff[e], (uint32_t)i * zone_chunk_bytes, SC1)
                          : u32x4{1u, 1u, 1u, 1u};
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        const int rows_mt = min(16, p.M - mt * 16);
        if (mt > 0) __syncthreads();             // the previous m tile's sums have been read
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int row = 4 * g + q;
            if (row < rows_mt) {
                // a lane's four 16-byte pieces are rotated by its column group: with the pieces of neighbouring lanes 64 bytes
                // apart, unrotated stores would meet in two groups of banks
                float *dst = red + ((size_t)wave * rows_mt + row) * NBW + 16 * c;
#pragma unroll
                for (int i = 0; i < NT; i += 4)
                    *reinterpret_cast<f32x4 *>(dst + 4 * ((i / 4 + c) & 3)) =
                        f32x4{tot[mt][i][q], tot[mt][i + 1][q], tot[mt][i + 2][q], tot[mt][i + 3][q]};
            }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < QPT; j++) {
            const int qd = (int)threadIdx.x + 512 * j;
            const int row = qd / (NBW / 4), nl = (qd % (NBW / 4)) * 4;
            const int e = mt * QPT + j;
            acc[e] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (live[e]) {
                const int piece = nl >> 2, nl_rot = (piece & ~3) * 4 + 4 * ((piece + (piece >> 2)) & 3);   // where the stores put it
#pragma unroll
                for (int wv = 0; wv < 8; wv++) acc[e] += *reinterpret_cast<const f32x4 *>(red + ((size_t)wv * rows_mt + row) * NBW + nl_rot);
            }
        }
    }
    if (p.S > 1) {
        if (chunk < p.S - 1) {
            u32x4 bits[NQ];
#pragma unroll
            for (int e = 0; e < NQ; e++) {
                bits[e] = __builtin_bit_cast(u32x4, acc[e]);
#pragma unroll
                for (int i = 0; i < 4; i++) bits[e][i] = bits[e][i] == 0u ? 0x80000000u : bits[e][i];   // +0 travels as -0: no stored word is zero
            }
            if (p.l2_exchange && __builtin_amdgcn_readfirstlane(collector_xcd) == my_xcd) {
#pragma unroll
                for (int e = 0; e < NQ; e++) buffer_store_b128<0>(bits[e], rsrc_z, zoff[e], (uint32_t)chunk * zone_chunk_bytes);   // dead quads: out of range
            } else {
#pragma unroll
                for (int e = 0; e < NQ; e++) buffer_store_b128<SC1>(bits[e], rsrc_z, zoff[e], (uint32_t)chunk * zone_chunk_bytes);
            }
            return;
        }
        // the strip's last workgroup collects the other chunks in chunk order; all of a thread's requests go out
        // before the first answer is looked at
        f32x4 sum[NQ];
        bool gave_up = false;
#pragma unroll
        for (int e = 0; e < NQ; e++) sum[e] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int c0 = 0; c0 < p.S - 1; c0 += CB) {
            if (c0 > 0) {                        // the first batch is already on its way
#pragma unroll
                for (int e = 0; e < NQ; e++)
#pragma unroll
                    for (int i = 0; i < CB; i++)
                        v[e][i] = live[e] && c0 + i < p.S - 1
                                      ? __builtin_amdgcn_raw_buffer_load_b128(rsrc_z, zoff[e], (uint32_t)(c0 + i) * zone_chunk_bytes, SC1)
                                      : u32x4{1u, 1u, 1u, 1u};
            }
            bool missing = true;
            for (int poll = 0; poll < p.max_polls && missing; poll++) {
                missing = false;
                // the polls must be real loads: without a compiler barrier a reload with the operands of the first request is
                // folded into it, and a wavefront that arrived before the data would spin on a stale register until the bound
                asm volatile("" ::: "memory");
#pragma unroll
                for (int e = 0; e < NQ; e++)
#pragma unroll
                    for (int i = 0; i < CB; i++)
                        if (v[e][i][0] == 0u || v[e][i][1] == 0u || v[e][i][2] == 0u || v[e][i][3] == 0u) {
                            v[e][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_z, zoff[e], (uint32_t)(c0 + i) * zone_chunk_bytes, SC1);
                            missing = true;
                        }
            }
            gave_up = gave_up || missing;
#pragma unroll
            for (int i = 0; i < CB; i++)
#pragma unroll
                for (int e = 0; e < NQ; e++) {
                    const f32x4 f = __builtin_bit_cast(f32x4, v[e][i]);
                    sum[e] += live[e] && c0 + i < p.S - 1 ? f : f32x4{0.f, 0.f, 0.f, 0.f};
                }
        }
#pragma unroll
        for (int e = 0; e < NQ; e++) acc[e] = sum[e] + acc[e];
        if (gave_up) {
            // some partial sums never came: the result is marked (NaN), not guessed, and the host is told
            const float nan = __uint_as_float(0x7fc00000u);
#pragma unroll
            for (int e = 0; e < NQ; e++) acc[e] = f32x4{nan, nan, nan, nan};
            *p.status = kStatusExchangeTimeout;
        }
    }
    const bool out_vec = (p.ldo & 3) == 0 && aligned_dev(p.out, 8);
#pragma unroll
    for (int e = 0; e < NQ; e++) {
        if (!live[e]) continue;
        const int qd = (int)threadIdx.x + 512 * (e % QPT);
        const int row = (e / QPT) * 16 + qd / (NBW / 4), nl = (qd % (NBW / 4)) * 4;
        f32x4 a = acc[e];
        if (p.bias) {
#pragma unroll
            for (int i = 0; i < 4; i++) a[i] = a[i] + act_1<ACT>(p.bias[n0 + nl + i]);
        }
        uint16_t *o = p.out + (int64_t)row * p.ldo + n0 + nl;
        if (out_vec) {
            u32x2 pk;
            pk.x = pack_act2<ACT>(a[0], a[1]);
            pk.y = pack_act2<ACT>(a[2], a[3]);
            *reinterpret_cast<u32x2 *>(o) = pk;
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = (uint16_t)pack_act2<ACT>(a[i], 0.0f);
        }
    }
    if (p.S > 1) {
        // the zone goes back to zero for the next launch; no branch around the stores (a dead quad or chunk gets an
        // out-of-range offset), so nothing waits for their acknowledgements.  Ordinary stores: the next launch is what must
        // see them, and a write-through store to a line that a producer left modified in the L2 takes several times as long
        for (int c0 = 0; c0 < p.S - 1; c0 += 4) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < NQ; e++)
                    buffer_store_b128<0>(u32x4{0u, 0u, 0u, 0u}, rsrc_z, c0 + i < p.S - 1 ? zoff[e] : kOutOfRange,
                                         (uint32_t)(c0 + i) * zone_chunk_bytes);
        }
        if (threadIdx.x == 0) __builtin_amdgcn_raw_buffer_store_b32(0u, rsrc_z, (uint32_t)strip * 4u, flag_base, 0);
    }
}

} // namespace

WqDecodePlan make_wq_decode_plan(int64_t M, int64_t N, int64_t K, int w_bits, int64_t group_size, int64_t ldw_k, int64_t ldx,
                                 const void *x, const void *w, const void *scale, const void *offset)
{
    WqDecodePlan pl{};
    const int64_t row_bytes = N / 2, ldw_bytes = ldw_k * 4;
    const int64_t group = group_size > 0 ? group_size : K;
    pl.grouped = group_size > 0 && group != K;
    // a wavefront's 128 rows lie inside one scale group; every offset the kernel forms fits in 32 bits
    pl.ok = knob(kKnobWqDecodeOff) != 1 && w_bits == 4 && M >= 1 && M <= 32 && K >= 128 && K % 128 == 0 && N % 8 == 0 &&
            (pl.grouped ? group % 128 == 0 : true) && ldw_bytes >= row_bytes && ldw_bytes % 8 == 0 && ldx % 8 == 0 &&
            (x == nullptr || aligned(x, 16)) && (w == nullptr || aligned(w, 8)) && (scale == nullptr || aligned(scale, 16)) &&
            (offset == nullptr || aligned(offset, 16)) && (uint64_t)K * (uint64_t)ldw_bytes < (1ull << 31) &&
            (uint64_t)M * (uint64_t)ldx * 2 < (1ull << 31) && (uint64_t)(K / group) * (uint64_t)N * 2 < (1ull << 31);
    if (!pl.ok) return pl;
    pl.mt = M <= 16 ? 1 : 2;
    pl.strips = (int)((row_bytes + 127) / 128);
    pl.S = (int)((K + 1023) / 1024);
    pl.zone_bytes = pl.S > 1 ? (size_t)(pl.S - 1) * (size_t)M * (size_t)N * 4 + (size_t)pl.strips * 4 : 0;   // sums, and a word per strip
    if (pl.zone_bytes > kWorkspaceZoneBytes || (uint64_t)pl.strips * pl.S > 0x7fffffffu) pl.ok = false;
    return pl;
}

int launch_wq_decode(const WqDecodePlan &plan, const void *x, int act_f16, const void *w, const void *scale, const void *offset,
                     const void *bias, void *out, int64_t M, int64_t N, int64_t K, int64_t group_size, int64_t ldx, int64_t ldw_k,
                     int64_t ldo, void *workspace, void *stream)
{
    WqDecArgs p{};
    p.x = static_cast<const uint16_t *>(x);
    p.w = w;
    p.scale = static_cast<const uint16_t *>(scale);
    p.offset = static_cast<const uint16_t *>(offset);
    p.bias = static_cast<const uint16_t *>(bias);
    p.out = static_cast<uint16_t *>(out);
    p.zone = plan.S > 1 ? reinterpret_cast<uint32_t *>(static_cast<char *>(workspace) + kWorkspaceCounterCapacity) : nullptr;
    p.ldx = ldx;
    p.ldo = ldo;
    p.ldw_bytes = (uint32_t)(ldw_k * 4);
    p.row_bytes = (uint32_t)(N / 2);
    p.M = (int)M;
    p.N = (int)N;
    p.K = (int)K;
    p.group_rows = (int)(plan.grouped ? group_size : K);
    p.strips = plan.strips;
    p.S = plan.S;
    p.l2_exchange = knob(kKnobWqDecodeOff) != 2;
    p.max_polls = knob(kKnobWqMaxPolls) > 0 ? knob(kKnobWqMaxPolls) : kMaxPolls;
    p.only_chunk = knob(kKnobWqOnlyChunk);
    p.status = plan.S > 1 ? reinterpret_cast<uint32_t *>(static_cast<char *>(workspace) + kWorkspaceStatusOffset) : nullptr;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int rows = (int)(M < 16 ? M : 16);
    const size_t lds_bytes = (size_t)8 * rows * 256 * sizeof(float);
    auto go = [&](auto kern) {
        static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (attr_status != hipSuccess) return (int)MI355_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, dim3((unsigned)((plan.strips + 7) / 8 * 8 * plan.S)), dim3(512), lds_bytes, s, p);
        return check_launch();
    };
    if (M <= 8) return act_f16 ? go(wq_decode4_kernel<1, 1, 1>) : go(wq_decode4_kernel<0, 1, 1>);
    if (M <= 16) return act_f16 ? go(wq_decode4_kernel<1, 1, 2>) : go(wq_decode4_kernel<0, 1, 2>);
    return act_f16 ? go(wq_decode4_kernel<1, 2, 2>) : go(wq_decode4_kernel<0, 2, 2>);
}

} // namespace mi355

