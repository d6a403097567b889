// npu_weight_quant_batchmatmul for more than 32 activation rows: a tiled GEMM that decodes every weight once
// per workgroup tile instead of streaming the weight once per 32 rows.
//
// A workgroup of eight wavefronts owns BM activation rows x one 128-byte strip of the weight rows (128 int8 or
// 256 int4 columns) and walks its K range in stages of 64 rows:
//   * weights: wavefront w copies rows 8w .. 8w+7 of the stage global -> LDS with one 1 KiB load instruction, three
//     stages ahead (vector-memory instructions cost the CU ~16 clocks each however few bytes they move, so the raw
//     bytes travel 16 per lane); it then reads its two bytes of each of the eight rows back, expands them to the
//     exact 16-bit images of the integers (the same images as the streaming kernel) and writes them to LDS as
//     [column][8 k] 16-byte chunks;
//   * activations: copied global -> LDS without passing registers, two stages ahead (three slots);
//   * both LDS tiles have a 128-byte row pitch (64 k x 2 bytes) with the 16-byte chunks XOR-swizzled by the row
//     pair, so the fragment reads of the 16x16x32 MFMA are conflict free; two image slots, one barrier per stage;
//   * the VALU work (folding a finished scale group into the running total, expanding the next stage's weights)
//     is placed between the MFMAs of a stage, so that it runs in their shadow.
// The antiquant parameters are applied to the float32 sums per scale group exactly as in the streaming kernel:
//     out[m,n] = sum_g scale[g,n] * ( P_g[m,n] + offset[g,n] * X_g[m] ),
// where the row sums X_g[m] of the activations come from MFMAs against a vector of ones.  Every column tile needs the
// same sums, so the wavefronts of a workgroup share the work: each accumulates the sums of ONE 16-row tile (one or two
// extra MFMAs per stage and four registers instead of eight MFMAs and sixteen registers) and publishes them through
// LDS when a group ends.
// The weight fragment is the first MFMA operand, so a lane owns four consecutive output columns of one row.
// K may be split over S workgroups per tile: each publishes its float32 sums in register order and the last
// arrival adds all of them in chunk order (the result does not depend on the order of arrival).
#include "weight_quant_common.h"
#include "weight_quant_gemm.h"

namespace mi355 {
namespace {

struct WqGemmArgs {
    const uint16_t *x;
    const void *w;
    const uint16_t *scale, *offset, *bias;
    uint16_t *out;
    float *partial;                 // workspace [tile][chunk][wavefront][accumulator quad][lane] float32x4 (S > 1)
    uint32_t *counter;              // workspace [tile], zero on entry, left zero (S > 1)
    int64_t ldx, ldo;
    uint32_t ldw_bytes, row_bytes;
    int M, N, K;
    int unit_stages, n_units, grouped;
    int tiles_m, tiles_n, tiles_per_xcd, S;
};

// KM: int8 weights stored [N, K] (K-major, the transposed view the LinearWeightQuant module passes); otherwise the
// weight rows are contiguous along N.
template <int WBITS, int ACT, int BM, bool ACCUM, bool KM>
__global__ __launch_bounds__(512, 1) void wq_gemm_kernel(const WqGemmArgs p)
{
    static_assert(!KM || WBITS == 8, "K-major weights are int8");
    constexpr int NW = 8;
    constexpr int BN = WBITS == 4 ? 256 : 128;
    constexpr int WGM = BM / 64, WGN = NW / WGM;
    constexpr int WTM = 4, WTN = BN / (16 * WGN);
    constexpr int PITCH = 128;                                 // bytes per LDS tile row: 64 k of 16 bits
    constexpr int A_BYTES = BM * PITCH, B_BYTES = BN * PITCH;
    constexpr int A_RING = 3 * A_BYTES;                        // LDS: three activation slots, two image slots, raw weight ring
    constexpr int LA = BM / 8 / NW;                            // activation loads of a wavefront per stage
    constexpr int CPL = WBITS == 4 ? 4 : 2;                    // weight columns per lane of the loader
    constexpr int NPIECE = KM ? 2 : CPL / 2;                   // expansion steps of a lane per stage (row-major: two columns each; K-major: one 16-byte chunk each)
    constexpr int PPJ = (NPIECE + WTN - 1) / WTN;              // of which this many follow each tile column of the second half
    constexpr float P_MUL = kImageMul<WBITS, ACT>;
    constexpr float X_BIAS = kImageBias<WBITS>;
    static_assert(BM == 64 || BM == 128, "tile rows");
    static_assert(WTN >= 1, "tile columns");
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    // workgroup -> (tile, K chunk): every XCD gets a contiguous run of tiles, rows fastest, so the row tiles
    // of one weight strip share an L2
    const int xcd = blockIdx.x & 7;
    const int slot_id = blockIdx.x >> 3;
    const int tile = xcd * p.tiles_per_xcd + slot_id % p.tiles_per_xcd;
    const int chunk = slot_id / p.tiles_per_xcd;
    if (tile >= p.tiles_m * p.tiles_n) return;
    const int m0 = (tile % p.tiles_m) * BM;
    const int tn = tile / p.tiles_m;
    const int n0 = tn * BN;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int u0 = (int)((int64_t)p.n_units * chunk / p.S), u1 = (int)((int64_t)p.n_units * (chunk + 1) / p.S);
    const int s0 = u0 * p.unit_stages;                         // first stage of this workgroup
    const int NSTG = (u1 - u0) * p.unit_stages;                // its number of stages (even)

    // ---- activations: global -> LDS.  Lane l of a unit (8 rows x 128 B) fills LDS slot l: row l/8, chunk slot
    // l%8, which must hold global chunk (l%8) ^ ((row >> 1) & 7).  unit = i * 8 + wave, so (row >> 1) & 7 =
    // 4 * (wave & 1) + (l/8) / 2.
    const int rows_a = min(BM, p.M - m0);
    const __amdgpu_buffer_rsrc_t rsrc_a =
        make_rsrc(p.x + (int64_t)m0 * p.ldx, (uint32_t)(((int64_t)(rows_a - 1) * p.ldx + p.K) * 2));
    const int rr = lane >> 3;
    const uint32_t voff_a = (uint32_t)(rr * (int)p.ldx * 2 + (((lane & 7) ^ (((wave & 1) << 2) | (rr >> 1))) * 16));
    const uint32_t unit_stride_a = 16u * (uint32_t)p.ldx;
    auto issue_a = [&](int s) {
        char *slot = lds + (s % 3) * A_BYTES;
        const uint32_t vo = s < NSTG ? voff_a : kOutOfRange;
#pragma unroll
        for (int i = 0; i < LA; i++) {
            const int u = i * NW + wave;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void *)(slot + u * 1024), 16, vo,
                                                     (uint32_t)u * unit_stride_a + (uint32_t)(s0 + s) * PITCH, 0, 0);
        }
    };

    // ---- weights: global -> LDS raw ring (three slots of 8 KiB = one stage of the strip), 1 KiB per wavefront and load.
    // Row-major along N: wavefront w copies k rows 8w .. 8w+7 (128 B each).  K-major: it copies columns 16w .. 16w+15
    // (64 B = the stage's 64 k each).
    constexpr int RAW_BYTES = 64 * 128;
    char *const raw = lds + A_RING + 2 * B_BYTES;
    const uint32_t strip_valid = KM ? 0u : min(128u, p.row_bytes - (uint32_t)tn * 128u);
    const int cols_valid = min(BN, p.N - n0);
    const __amdgpu_buffer_rsrc_t rsrc_w =
        KM ? make_rsrc(static_cast<const char *>(p.w) + (size_t)n0 * p.ldw_bytes, (uint32_t)(cols_valid - 1) * p.ldw_bytes + (uint32_t)p.K)
           : make_rsrc(static_cast<const char *>(p.w) + (size_t)tn * 128, (uint32_t)(p.K - 1) * p.ldw_bytes + strip_valid);
    const uint32_t voff_w = KM ? (uint32_t)(lane >> 2) * p.ldw_bytes + (uint32_t)(lane & 3) * 16u
                               : ((uint32_t)(lane & 7) * 16u < strip_valid
                                      ? (uint32_t)(lane >> 3) * p.ldw_bytes + (uint32_t)(lane & 7) * 16u
                                      : kOutOfRange);
    auto issue_w = [&](int s) {
        const uint32_t vo = s < NSTG ? voff_w : kOutOfRange;
        const uint32_t so = KM ? (uint32_t)wave * 16u * p.ldw_bytes + (uint32_t)(s0 + s) * 64u
                               : ((uint32_t)(s0 + s) * 64u + (uint32_t)wave * 8u) * p.ldw_bytes;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_void *)(raw + (s % 3) * RAW_BYTES + wave * 1024), 16, vo, so, 0, 0);
    };
    // Row-major: this lane's two bytes (2 int8 / 4 int4 columns) of the wavefront's eight rows.  K-major: two runs of
    // eight consecutive k of one column each (chunk c = t * 512 + wave * 64 + lane: column c / 8, k octet c % 8).
    auto read_raw = [&](uint32_t (&wr)[8], int s) {
        if constexpr (KM) {
            const char *src = raw + (s % 3) * RAW_BYTES + (wave * 64 + lane) * 8;
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const u32x2 v = *reinterpret_cast<const u32x2 *>(src + t * 4096);
                wr[2 * t] = v.x;
                wr[2 * t + 1] = v.y;
            }
        } else {
            const char *src = raw + (s % 3) * RAW_BYTES + wave * 1024 + lane * 2;
#pragma unroll
            for (int t = 0; t < 8; t++) wr[t] = *reinterpret_cast<const uint16_t *>(src + t * 128);
        }
    };
    uint32_t magic;
    asm volatile("v_mov_b32 %0, %1" : "=v"(magic) : "n"(kInt4Magic<ACT>));   // opaque to the optimiser: stays in a VGPR
    // int4: two's complement -> offset binary (nibble + 8); then the 16-bit images -> LDS
    auto flip_w = [&](uint32_t (&wx)[8], const uint32_t (&wr)[8]) {
#pragma unroll
        for (int t = 0; t < (KM ? 4 : 8); t++) wx[t] = wr[t] ^ (WBITS == 4 ? 0x8888u : 0u);   // int8 converts signed
    };
    // registers -> LDS, one piece: column n, k octet o -> chunk slot o ^ ((n >> 1) & 7) of row n
    auto expand_piece = [&](const uint32_t (&wx)[8], int piece, int s) {
        char *bs = lds + A_RING + (s & 1) * B_BYTES;
        if constexpr (KM) {
            const int c = piece * 512 + wave * 64 + lane;
            const int n = c >> 3, o = c & 7;
            const uint32_t lo = wx[2 * piece], hi = wx[2 * piece + 1];
            u32x4 b;
            b[0] = pack_act2<ACT>(sbyte_f32(lo, 0), sbyte_f32(lo, 1));
            b[1] = pack_act2<ACT>(sbyte_f32(lo, 2), sbyte_f32(lo, 3));
            b[2] = pack_act2<ACT>(sbyte_f32(hi, 0), sbyte_f32(hi, 1));
            b[3] = pack_act2<ACT>(sbyte_f32(hi, 2), sbyte_f32(hi, 3));
            *reinterpret_cast<u32x4 *>(bs + n * PITCH + ((o ^ ((n >> 1) & 7)) * 16)) = b;
        } else {
            u32x4 b0, b1;
            expand_pair<WBITS, ACT>(wx, piece, magic, b0, b1);
            const int n = lane * CPL + 2 * piece;              // even: n and n + 1 share the swizzle
            const int sw = (wave ^ ((n >> 1) & 7)) * 16;
            *reinterpret_cast<u32x4 *>(bs + n * PITCH + sw) = b0;
            *reinterpret_cast<u32x4 *>(bs + (n + 1) * PITCH + sw) = b1;
        }
    };
    auto expand_w = [&](const uint32_t (&wx)[8], int s) {
#pragma unroll
        for (int piece = 0; piece < NPIECE; piece++) expand_piece(wx, piece, s);
    };

    // ---- antiquant parameters of this lane's columns: tile j covers n0 + (wn * WTN + j) * 16 + 4 * (lane / 16) + r
    const int ncol0 = n0 + wn * WTN * 16 + (lane >> 4) * 4;
    const uint32_t param_bytes = (uint32_t)(p.grouped ? p.K / (64 * p.unit_stages) : 1) * (uint32_t)p.N * 2u;
    const __amdgpu_buffer_rsrc_t rsrc_s = make_rsrc(p.scale, param_bytes);
    const bool has_offset = p.offset != nullptr;
    const __amdgpu_buffer_rsrc_t rsrc_o = make_rsrc(has_offset ? p.offset : p.scale, param_bytes);
    const uint32_t omask = has_offset ? ~0u : 0u;
    const uint32_t voff_p = (uint32_t)ncol0 * 2u;
    // Inside the loop the parameters of a finished group travel through LDS: wavefront 0 copies the tile's BN scales and
    // offsets global -> LDS (a few load instructions for the whole workgroup instead of 2 * WTN per wavefront, and no
    // registers held across the stage); two slots, by group parity.  After the loop they are loaded into registers.
    constexpr int PRM_SLOT = 2048;                             // [BN scales | +512: BN offsets] 16-bit each, [+1024 | +1536: BM row sums] float32
    char *const prm = lds + A_RING + 2 * B_BYTES + 3 * RAW_BYTES;
    auto issue_params = [&](int group_row) {
        const uint32_t ro = (uint32_t)group_row * (uint32_t)p.N * 2u + (uint32_t)n0 * 2u;
        char *dst = prm + (group_row & 1) * PRM_SLOT;
#pragma unroll
        for (int h = 0; h < BN / 128; h++) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_s, (lds_void *)(dst + h * 256), 4, (uint32_t)lane * 4u, ro + h * 256u, 0, 0);
            if (has_offset)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_o, (lds_void *)(dst + 512 + h * 256), 4, (uint32_t)lane * 4u,
                                                         ro + h * 256u, 0, 0);
        }
    };
    const int prm_col = (wn * WTN * 16 + (lane >> 4) * 4) * 2;  // byte offset of this lane's first column in a slot
    u32x2 sv[WTN], ov[WTN];
    auto load_params = [&](int group_row) {
        const uint32_t ro = (uint32_t)group_row * (uint32_t)p.N * 2u;
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            sv[j] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_s, voff_p + 32u * j, ro, 0);
            ov[j] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_o, voff_p + 32u * j, ro, 0);   // masked where it is used
        }
    };

    f32x4 P[WTM][WTN], tot[WTM][WTN];
    float X[WTM];                                              // row sums of the group being folded
#pragma unroll
    for (int i = 0; i < WTM; i++) {
        X[i] = 0.0f;
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            P[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
            tot[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    // Folding a finished group: tot += scale * (P' + ((offset - X_BIAS) / P_MUL) * X), with the common factor P_MUL
    // applied once at the output (both rescalings are powers of two, hence exact).
    float sc[4], of[4];
    auto fold_params = [&](const u32x2 s2, const u32x2 o2) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint32_t su = s2[r >> 1], ou = o2[r >> 1] & omask;
            sc[r] = (r & 1) ? act_hi<ACT>(su) : act_lo<ACT>(su);
            of[r] = __builtin_fmaf((r & 1) ? act_hi<ACT>(ou) : act_lo<ACT>(ou), 1.0f / P_MUL, -X_BIAS / P_MUL);
        }
    };
    auto fold_tile = [&](int i, int j) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float inner = __builtin_fmaf(of[r], X[i], P[i][j][r]);
            tot[i][j][r] = __builtin_fmaf(sc[r], inner, tot[i][j][r]);
        }
    };

    // ---- row sums: wavefront (wm, wn) owns 16-row tile wn % 4 of its 64 rows; with eight wavefronts across (64-row
    // workgroup tiles) two wavefronts share a tile and take one half stage each.  acc[r] of the ones-MFMA is the sum
    // of row lane % 16 for every r, so lanes 0..15 publish component 0.
    constexpr int XSPLIT = WGN / 4;
    const int xi = wn & 3, xk = wn >> 2;
    f32x4 Xown = f32x4{0.f, 0.f, 0.f, 0.f};
    const u32x4 ones = u32x4{kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>};
    auto publish_x = [&](int slot) {
        float *dst = reinterpret_cast<float *>(prm + slot * PRM_SLOT + 1024 + xk * 512) + wm * 64 + xi * 16 + (lane & 15);
        if (lane < 16) *dst = Xown[0];
        Xown = f32x4{0.f, 0.f, 0.f, 0.f};
    };
    auto read_x = [&](int slot) {
        const float *src = reinterpret_cast<const float *>(prm + slot * PRM_SLOT + 1024) + wm * 64 + (lane & 15);
#pragma unroll
        for (int i = 0; i < WTM; i++) {
            X[i] = src[i * 16];
            if constexpr (XSPLIT == 2) X[i] = X[i] + src[128 + i * 16];
        }
    };

    // ---- fragment reads: lane reads row (lane % 16) of a 16-row tile, chunk (ks * 4 + lane / 16), stored at slot
    // chunk ^ ((row >> 1) & 7); for ks = 1 the slot is the ks = 0 slot with bit 2 flipped
    const int frow = lane & 15;
    const int sw0 = ((lane >> 4) ^ ((frow >> 1) & 7)) * 16;
    const int a_off = (wm * 64 + frow) * PITCH;
    const int b_off = A_RING + (wn * WTN * 16 + frow) * PITCH;
    const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
    // activation fragments of a half stage are read together; weight fragments are streamed one tile column ahead
    // (two live instead of WTN: the 64 x 64 tile with a running total has no registers to spare)
    u32x4 AF[WTM], BF[2];
    const char *sb_cur = nullptr;
    auto read_frags = [&](int s, int ks) {
        const char *sa = lds + (s % 3) * A_BYTES + a_off;
        const int sw = sw0 ^ (ks * 64);
        sb_cur = lds + (s & 1) * B_BYTES + b_off + sw;
#pragma unroll
        for (int i = 0; i < WTM; i++) AF[i] = *reinterpret_cast<const u32x4 *>(sa + i * 16 * PITCH + sw);
        BF[0] = *reinterpret_cast<const u32x4 *>(sb_cur);
    };
    auto read_b = [&](int j) { BF[j & 1] = *reinterpret_cast<const u32x4 *>(sb_cur + j * 16 * PITCH); };
    // this wavefront's share of the row sums for half stage ks (uniform branches: one MFMA is executed)
    auto rowsum_mfma = [&](int ks) {
        if (XSPLIT == 2 && xk != ks) return;
        if (xi == 0) Xown = mfma_act<ACT>(ones, AF[0], Xown);
        else if (xi == 1) Xown = mfma_act<ACT>(ones, AF[1], Xown);
        else if (xi == 2) Xown = mfma_act<ACT>(ones, AF[2], Xown);
        else Xown = mfma_act<ACT>(ones, AF[3], Xown);
    };

    // ---- main loop.  Stage s is computed from activation slot s % 3 and image slot s & 1.  Meanwhile image slot
    // (s + 1) & 1 receives the images of stage s + 1, expanded from the raw ring, and memory is asked for the
    // activations of stage s + 2 and the raw weights of stage s + 3.  Loads are never skipped (a stage past the end
    // gets an out-of-range lane offset and moves no bytes), so the number of loads in flight is the same in every
    // iteration: at the top, "at most LA + 1 outstanding" means everything but the newest refills has landed.
    //
    // The VALU work rides in the shadow of the MFMAs of the same wavefront: a finished scale group is folded tile by
    // tile in the first half of the next stage (fold tile t, then restart its accumulator with an MFMA whose C
    // operand is zero, while the VALU goes on to tile t + 1), and the images of stage s + 1 are expanded between the
    // MFMAs of the second half.  sched_barrier pins that order.
    uint32_t wx[8];
    issue_w(0);
    issue_a(0);
    issue_w(1);
    issue_a(1);
    issue_w(2);
    wait_vmcnt<2 * LA + 2>();
    __syncthreads();
    read_raw(wx, 0);
    flip_w(wx, wx);
    expand_w(wx, 0);
    bool pending = false;                                      // a finished group awaits its fold
    int pending_row = 0;
    for (int s = 0; s < NSTG; s++) {
        wait_vmcnt<LA + 1>();
        wait_lgkmcnt0();
        __syncthreads();                                       // stage s is complete in LDS; everyone is done with stage s - 1
        read_frags(s, 0);
        // the parameters of a group are fetched in its last stage, ahead of the refills (the wait at the next top
        // then covers them)
        const bool last_of_group = ACCUM && (s0 + s + 1) % p.unit_stages == 0;
        const int group_row = (s0 + s) / p.unit_stages;
        if (last_of_group && wave == 0) issue_params(group_row);
        issue_a(s + 2);
        issue_w(s + 3);
        __builtin_amdgcn_sched_barrier(0);
        if (ACCUM && pending) {
            const char *pb = prm + (pending_row & 1) * PRM_SLOT + prm_col;
            read_x(pending_row & 1);
#pragma unroll
            for (int j = 0; j < WTN; j++) {
                if (j + 1 < WTN) read_b(j + 1);
                fold_params(*reinterpret_cast<const u32x2 *>(pb + j * 32), *reinterpret_cast<const u32x2 *>(pb + 512 + j * 32));
#pragma unroll
                for (int i = 0; i < WTM; i++) {
                    fold_tile(i, j);
                    P[i][j] = mfma_act<ACT>(BF[j & 1], AF[i], zero4);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < WTN; j++) {
                if (j + 1 < WTN) read_b(j + 1);
#pragma unroll
                for (int i = 0; i < WTM; i++) P[i][j] = mfma_act<ACT>(BF[j & 1], AF[i], P[i][j]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        rowsum_mfma(0);
        __builtin_amdgcn_sched_barrier(0);
        pending = last_of_group;
        pending_row = group_row;
        read_raw(wx, s + 1);
        read_frags(s, 1);
        flip_w(wx, wx);
        __builtin_amdgcn_sched_barrier(0);
        // second half: MFMAs with the expansion of stage s + 1 in between
        {
#pragma unroll
            for (int j = 0; j < WTN; j++) {
                if (j + 1 < WTN) read_b(j + 1);
#pragma unroll
                for (int i = 0; i < WTM; i++) P[i][j] = mfma_act<ACT>(BF[j & 1], AF[i], P[i][j]);
#pragma unroll
                for (int piece = j * PPJ; piece < (j + 1) * PPJ && piece < NPIECE; piece++) expand_piece(wx, piece, s + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        rowsum_mfma(1);
        if (last_of_group) publish_x(group_row & 1);           // read by everyone after the next barrier
    }
    if constexpr (!ACCUM) publish_x(0);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // the refills past the end (zeros) have landed
    __syncthreads();
    // the last group (without the running total: the only one)
    load_params(p.grouped ? u1 - 1 : 0);
    read_x(ACCUM ? (u1 - 1) & 1 : 0);
#pragma unroll
    for (int j = 0; j < WTN; j++) {
        fold_params(sv[j], ov[j]);
#pragma unroll
        for (int i = 0; i < WTM; i++) {
            fold_tile(i, j);
            tot[i][j] = tot[i][j] * P_MUL;
        }
    }

    // ---- split K: publish, count, last arrival sums in chunk order
    if (p.S > 1) {
        constexpr int SC1 = 16;                                // cache-policy bit: agent scope
        constexpr uint32_t WAVE_BYTES = WTM * WTN * 64 * 16;
        constexpr uint32_t CHUNK_BYTES = NW * WAVE_BYTES;
        const __amdgpu_buffer_rsrc_t rsrc_p =
            make_rsrc(p.partial + (size_t)tile * p.S * (CHUNK_BYTES / 4), (uint32_t)p.S * CHUNK_BYTES);
        const uint32_t lane_off = (uint32_t)wave * WAVE_BYTES + (uint32_t)lane * 16u;
#pragma unroll
        for (int i = 0; i < WTM; i++)
#pragma unroll
            for (int j = 0; j < WTN; j++)
                buffer_store_b128<SC1>(__builtin_bit_cast(u32x4, tot[i][j]), rsrc_p,
                                                       lane_off + (i * WTN + j) * 1024, (uint32_t)chunk * CHUNK_BYTES);
        wait_vmcnt<0>();                                       // this wavefront's sums have reached the coherence point
        __syncthreads();
        int &is_last = *reinterpret_cast<int *>(lds);
        if (threadIdx.x == 0) {
            const uint32_t old = __hip_atomic_fetch_add(p.counter + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = old == (uint32_t)(p.S - 1);
        }
        __syncthreads();
        if (!is_last) return;
#pragma unroll
        for (int i = 0; i < WTM; i++)
#pragma unroll
            for (int j = 0; j < WTN; j++) tot[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        // two chunks per round: all their loads are in flight together; the sums stay in chunk order
        for (int ch = 0; ch < p.S; ch += 2) {
            f32x4 v0[WTM][WTN], v1[WTM][WTN];
            const uint32_t second = ch + 1 < p.S ? 0u : kOutOfRange;   // an odd tail reads zeros
#pragma unroll
            for (int i = 0; i < WTM; i++)
#pragma unroll
                for (int j = 0; j < WTN; j++) {
                    v0[i][j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                        rsrc_p, lane_off + (i * WTN + j) * 1024, (uint32_t)ch * CHUNK_BYTES, SC1));
                    v1[i][j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                        rsrc_p, (lane_off + (i * WTN + j) * 1024) | second, (uint32_t)(ch + 1) * CHUNK_BYTES, SC1));
                }
#pragma unroll
            for (int i = 0; i < WTM; i++)
#pragma unroll
                for (int j = 0; j < WTN; j++) tot[i][j] = (tot[i][j] + v0[i][j]) + v1[i][j];
        }
        if (threadIdx.x == 0) __hip_atomic_store(p.counter + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- output: lane holds row m = ... + lane % 16, columns ncol0 + 16 j + r
    const bool out_vec = (p.ldo & 3) == 0 && aligned_dev(p.out, 8);
#pragma unroll
    for (int j = 0; j < WTN; j++) {
        const int n = ncol0 + j * 16;
        if (n >= p.N) continue;                                // N is a multiple of 8: a quad is valid as a whole
        f32x4 bv = f32x4{0.f, 0.f, 0.f, 0.f};
        if (p.bias) {
#pragma unroll
            for (int r = 0; r < 4; r++) bv[r] = act_1<ACT>(p.bias[n + r]);
        }
#pragma unroll
        for (int i = 0; i < WTM; i++) {
            const int m = m0 + wm * 64 + i * 16 + frow;
            if (m >= p.M) continue;
            const f32x4 v = tot[i][j] + bv;
            uint16_t *o = p.out + (int64_t)m * p.ldo + n;
            if (out_vec) {
                u32x2 pk;
                pk.x = pack_act2<ACT>(v[0], v[1]);
                pk.y = pack_act2<ACT>(v[2], v[3]);
                *reinterpret_cast<u32x2 *>(o) = pk;
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++) o[r] = (uint16_t)pack_act2<ACT>(v[r], 0.0f);
            }
        }
    }
}

template <int WBITS, int ACT, int BM, bool ACCUM, bool KM>
int launch_tile(WqGemmArgs &p, hipStream_t s)
{
    constexpr int BN = WBITS == 4 ? 256 : 128;
    constexpr size_t lds_bytes = (size_t)(3 * BM + 2 * BN) * 128 + 3 * 64 * 128 + 2 * 2048;   // activation ring, image slots, raw ring, parameters
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");
    auto kern = wq_gemm_kernel<WBITS, ACT, BM, ACCUM, KM>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)(8 * p.tiles_per_xcd * p.S)), dim3(512), lds_bytes, s, p);
    return check_launch();
}

template <int WBITS, int ACT, bool KM>
int launch_any(WqGemmArgs &p, const WqGemmPlan &pl, hipStream_t s)
{
    if (pl.bm == 64)
        return pl.accum ? launch_tile<WBITS, ACT, 64, true, KM>(p, s) : launch_tile<WBITS, ACT, 64, false, KM>(p, s);
    return pl.accum ? launch_tile<WBITS, ACT, 128, true, KM>(p, s) : launch_tile<WBITS, ACT, 128, false, KM>(p, s);
}

} // namespace

WqGemmPlan make_wq_gemm_plan(int64_t M, int64_t N, int64_t K, int w_bits, int64_t group_size, int layout, int64_t ldw,
                             int64_t ldx, const void *x, const void *w, const void *scale, const void *offset)
{
    WqGemmPlan pl{};
    pl.k_major = layout == 2;
    const int64_t row_bytes = w_bits == 4 ? N / 2 : N;
    const int64_t ldw_bytes = w_bits == 4 ? ldw * 4 : ldw;     // bytes between k rows, or (K-major) between columns
    const int64_t group = group_size > 0 ? group_size : K;
    pl.grouped = group_size > 0 && group != K;
    const bool layout_ok = layout == 1 ? ldw_bytes >= row_bytes && (uint64_t)K * (uint64_t)ldw_bytes < (1ull << 32)
                                       : layout == 2 && w_bits == 8 && ldw >= K && (uint64_t)N * (uint64_t)ldw < (1ull << 32);
    pl.ok = M > 32 && layout_ok && K >= 128 && K % 128 == 0 && group % 128 == 0 && N % 8 == 0 && ldw_bytes % 4 == 0 &&
            ldx % 8 == 0 && (x == nullptr || aligned(x, 16)) && (w == nullptr || aligned(w, 4)) &&
            (scale == nullptr || aligned(scale, 4)) && (offset == nullptr || aligned(offset, 4)) &&
            (uint64_t)128 * (uint64_t)ldx * 2 < (1ull << 31) &&
            (uint64_t)(K / group) * (uint64_t)N * 2 < (1ull << 31) && !knob(kKnobWqGemmOff) /* tuning aid: keeps every shape on the streaming kernels */;
    if (!pl.ok) return pl;
    const int bn = w_bits == 4 ? 256 : 128;
    pl.bm = M <= 64 ? 64 : 128;
    if (const int f = knob(kKnobWqgBm))                 // tuning aid
        if (f == 64 || f == 128) pl.bm = f;
    pl.tiles_m = (int)((M + pl.bm - 1) / pl.bm);
    pl.tiles_n = pl.k_major ? (int)((N + 127) / 128) : (int)((row_bytes + 127) / 128);
    pl.unit_stages = pl.grouped ? (int)(group / 64) : 2;
    pl.n_units = (int)(K / (64 * pl.unit_stages));
    const int64_t tiles = (int64_t)pl.tiles_m * pl.tiles_n;
    int64_t S = tiles < kNumCU ? kNumCU / tiles : 1;
    if (S > pl.n_units) S = pl.n_units;
    if (S > 8) S = 8;
    if (const int f = knob(kKnobWqgSplit))              // tuning aid
        if (f >= 1 && f <= pl.n_units) S = f;
    if (S > 1 && ((uint64_t)S * pl.bm * bn * 4 >= (1ull << 32) || (size_t)tiles * 4 > kWorkspaceCounterBytes)) S = 1;
    pl.S = (int)S;
    pl.accum = pl.grouped && (pl.n_units + pl.S - 1) / pl.S > 1;
    pl.partial_bytes = pl.S > 1 ? (size_t)tiles * pl.S * pl.bm * bn * 4 : 0;
    pl.counter_bytes = pl.S > 1 ? kWorkspaceZeroBytes : 0;
    (void)bn;
    return pl;
}

int launch_wq_gemm(const WqGemmPlan &pl, const void *x, int act_f16, const void *w, int w_bits, const void *scale,
                   const void *offset, const void *bias, void *out, int64_t M, int64_t N, int64_t K, int64_t ldx,
                   int64_t ldw, int64_t ldo, void *workspace, void *stream)
{
    WqGemmArgs p{};
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
    p.ldw_bytes = (uint32_t)(w_bits == 4 ? ldw * 4 : ldw);
    p.row_bytes = (uint32_t)(w_bits == 4 ? N / 2 : N);
    p.M = (int)M;
    p.N = (int)N;
    p.K = (int)K;
    p.unit_stages = pl.unit_stages;
    p.n_units = pl.n_units;
    p.grouped = pl.grouped;
    p.tiles_m = pl.tiles_m;
    p.tiles_n = pl.tiles_n;
    p.tiles_per_xcd = (pl.tiles_m * pl.tiles_n + 7) / 8;
    p.S = pl.S;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (pl.k_major) return act_f16 ? launch_any<8, 1, true>(p, pl, s) : launch_any<8, 0, true>(p, pl, s);
    if (act_f16) return w_bits == 4 ? launch_any<4, 1, false>(p, pl, s) : launch_any<8, 1, false>(p, pl, s);
    return w_bits == 4 ? launch_any<4, 0, false>(p, pl, s) : launch_any<8, 0, false>(p, pl, s);
}

} // namespace mi355
