// npu_quant_matmul for gfx950: int8 x int8 -> int32 on the MFMA units with the dequantising
// epilogue fused (per-token scale, per-channel scale, bias, bf16 rounding).
//
// Data layout.  A is [M,K] row-major int8.  The B operand is consumed K-major ("[N,K]", the
// storage of an nn.Linear-style weight whose transposed view the callers pass); a contiguous
// [K,N] weight is first transposed into the caller's workspace.
//
// Kernel.  A workgroup of 8 wavefronts (two per SIMD, arranged WGM x WGN) owns a BM x BN tile of
// the output.  K is walked in steps of BK = 128 bytes.  Global memory -> LDS goes through
// the direct-to-LDS load (16 bytes per lane, no register staging); the 16-byte chunks of a row
// are XOR-swizzled with the row number (applied on the global-address side, because the LDS
// side of a direct load is fixed at lane * 16) so that the 16 rows x 16 bytes a wavefront
// reads per MFMA operand spread over all banks.  Every wavefront keeps WTM x WTN
// accumulator tiles of v_mfma_i32_16x16x64_i8 in registers.
//
// The MFMA is issued with the weight fragment as the first operand, so each lane ends up with
// four consecutive output columns of one row: the epilogue then needs one per-token scale and
// four consecutive per-channel scales per accumulator quad and stores 8 bytes per lane.
//
// Exactness.  Accumulation is integer and therefore independent of the tiling.  The epilogue
// evaluates ((float(acc) * pertoken[m]) * scale[n]) + bias[n] with separately rounded binary32
// operations (contraction is disabled for this library) and rounds once to bf16.
#include "common.h"
#include "quant_matmul_decode.h"
#include "quant_matmul_wide.h"
#include <stdio.h>
#include <type_traits>
#include <stdlib.h>
#include <mutex>

namespace mi355 {
namespace {

constexpr int BK = 128;          // bytes (= int8 elements) of K per LDS stage

typedef int32_t i32x4v __attribute__((ext_vector_type(4)));

typedef __attribute__((address_space(3))) void lds_void;

template <int VM>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(VM >= 0 && VM < 64, "vmcnt range");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(VM) : "memory");
}

template <int VM>
__device__ __forceinline__ void wait_vmcnt_lgkm0()
{
    static_assert(VM >= 0 && VM < 64, "vmcnt range");
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(VM) : "memory");
}

// Raw buffer descriptor (stride 0, 32-bit data format): loads beyond `bytes` return zero.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

struct QmmArgs {
    const int8_t *a;
    const int8_t *bt;          // [N, K] K-major
    const float *pertoken;     // [M] or null
    const float *scale;        // [scale_len]
    const void *bias;          // [N] of bias_kind, or null
    int bias_kind;             // MI355_BIAS_*
    int out_f16;               // round to fp16 instead of bf16
    void *out;
    int64_t lda, ldbt, ldc;
    int M, N, K;
    int scale_len;
    int out_i32;
    const uint64_t *qparam;    // packed quantisation parameters [scale_len] (replace `scale`), or null
    int out_i8;                // re-quantised int8 output (needs qparam)
    int stream_out;            // 16-bit and int8 outputs with aligned rows: non-temporal row stores (chosen by the launcher)
    int tiles_m, tiles_n, tiles_per_xcd;
    int S;                     // workgroups that share the K range of a tile
    int32_t *partial;          // workspace [tile][chunk][wavefront][accumulator quad][lane] int32x4 (S > 1)
    uint32_t *counter;         // workspace [tile], zero on entry, left zero (S > 1)
#ifdef MI355_QMM_TS
    unsigned long long *ts;    // debugging aid: [workgroup][wavefront][64] cycle counter stamps
#endif
};

#ifdef MI355_QMM_TS
#define MI355_TS(IDX) if (p.ts && lane == 0) p.ts[((size_t)blockIdx.x * 8 + wave) * 128 + (IDX)] = __builtin_readcyclecounter();
#else
#define MI355_TS(IDX)
#endif

// Packed quantisation parameter (the 64-bit words npu_trans_quant_param produces): bits 0-31 the float32 scale,
// bits 37-45 the offset as a 9-bit two's-complement integer, bit 46 set.
__device__ __forceinline__ float qparam_scale(uint64_t q) { return __uint_as_float((uint32_t)q); }
__device__ __forceinline__ float qparam_offset(uint64_t q) { return (float)(((int32_t)((uint32_t)(q >> 37) << 23)) >> 23); }

// out = clamp(rint((acc + int32 bias) * scale + offset)) as int8; each operation rounded to float32
__device__ __forceinline__ int32_t requant1(int32_t a, int32_t bi, float sc, float off)
{
    float v = (float)(int32_t)((uint32_t)a + (uint32_t)bi);
    v = v * sc;
    v = v + off;
    v = rintf(v);
    v = fminf(fmaxf(v, -128.0f), 127.0f);
    return (int32_t)v;
}

// WGM x WGN wavefronts per workgroup, each owning (16*WTM) x (16*WTN) of the output tile.
// LOOP 0: the generic K loop below; 3: the same with as many activation slots as weight slots (whole stages requested
// NS steps ahead); 1, 2: the loop of quant_matmul_wide.h (4 x 2 wavefronts of 64 rows) with its
// instruction order 0 (refills in a block) or 1 (refills spread over the step)
// EPI (the widest wavefront tile only, see LEAN below): which variants of the LDS-parameter epilogue this instantiation holds
template <int WGM, int WGN, int WTM, int WTN, int NS, int LOOP = 0, int EPI = 0>
__global__ __launch_bounds__(WGM *WGN * 64, 1) void qmm_kernel(const QmmArgs p)
{
    constexpr int NW = WGM * WGN;
    constexpr int BM = 16 * WTM * WGM, BN = 16 * WTN * WGN;
    constexpr int UNITS_A = BM / 8, UNITS_B = BN / 8;        // unit = 8 rows x 128 B = one wavefront-wide load
    constexpr int UNITS_BP = (UNITS_B + NW - 1) / NW * NW;
    constexpr int LA = UNITS_A / NW, LB = UNITS_BP / NW;     // loads of a wavefront per activation / weight stage
    constexpr int A_BYTES = UNITS_A * 1024, B_BYTES = UNITS_BP * 1024;
    constexpr bool WIDE = LOOP == 1 || LOOP == 2;
    constexpr bool WHOLE = NS >= 4 || LOOP == 3;             // whole stages: activations get NS slots as well
    // the epilogues that take their parameters from LDS (quant_matmul_wide.h: wavefronts of 64 rows): the wide loop's tiles
    // and the whole-stage 128-row tiles, which keep the vectors behind their ring
    constexpr bool LDSP = WIDE || (LOOP == 3 && WTM == 4);
    constexpr int NSA = WHOLE ? NS : 2;                      // activation slots; NS weight slots follow them in LDS
    constexpr uint32_t kOutOfRange = 0x80000000u;            // lane offset beyond every buffer: the load writes zeros
    static_assert(UNITS_A % NW == 0, "A units must divide evenly over the wavefronts");
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    // XCD-aware rasterisation: workgroups are dealt round-robin to the 8 XCDs, each of which has
    // a private L2; give every XCD a contiguous run of tiles, M fastest, so its workgroups
    // share weight columns.
    const int xcd = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    const int tile = xcd * p.tiles_per_xcd + slot % p.tiles_per_xcd;
    const int chunk = slot / p.tiles_per_xcd;                // K chunk of this workgroup (split K)
    if (tile >= p.tiles_m * p.tiles_n) return;
    const int m0 = (tile % p.tiles_m) * BM;
    const int n0 = (tile / p.tiles_m) * BN;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    MI355_TS(0)
    // Wavefronts w and w + 4 of a workgroup share a SIMD.  In the wide loop the two wavefronts of a SIMD take different
    // roles (one refills activations, one weights): wn = 0, 1, 0, 1, 1, 0, 1, 0 for wavefronts 0 .. 7.
    const int wm = LOOP == 1 || LOOP == 2 ? ((wave & 3) >> 1) + 2 * (wave >> 2) : wave / WGN;
    const int wn = LOOP == 1 || LOOP == 2 ? ((wave >> 2) ^ wave) & 1 : wave % WGN;
    const int kt0 = (int)((int64_t)(p.K / BK) * chunk / p.S);            // first K step of this workgroup
    const int KT = (int)((int64_t)(p.K / BK) * (chunk + 1) / p.S) - kt0;  // its number of K steps

    // Global -> LDS addressing.  Lane l of a unit fills LDS slot l (16 B): row l/8, chunk slot l%8,
    // which must hold global chunk (l%8) ^ (l/8) of that row (XOR swizzle).
    const int rows_a = min(BM, p.M - m0), rows_b = min(BN, p.N - n0);
    // (timing ablations 32 / 64: every tile reads the activation rows / weight columns of the first tile)
    const __amdgpu_buffer_rsrc_t rsrc_a =
        make_rsrc(p.a + (int64_t)((MI355_WIDE_ABL & 32) ? 0 : m0) * p.lda, (uint32_t)((int64_t)(rows_a - 1) * p.lda + p.K));
    const __amdgpu_buffer_rsrc_t rsrc_b =
        make_rsrc(p.bt + (int64_t)((MI355_WIDE_ABL & 64) ? 0 : n0) * p.ldbt, (uint32_t)((int64_t)(rows_b - 1) * p.ldbt + p.K));
    const int rr = lane >> 3;
    // row of the tile = 8 * unit + rr and unit = i * NW + wave with NW even: (row >> 1) & 7 = 4 * (wave & 1) + rr / 2
    const int gchunk = ((lane & 7) ^ (((wave & 1) << 2) | (rr >> 1))) * 16;
    const uint32_t voff_a = (uint32_t)(rr * (int)p.lda + gchunk);
    const uint32_t voff_b = (uint32_t)(rr * (int)p.ldbt + gchunk);
    const uint32_t unit_stride_a = 8u * (uint32_t)p.lda, unit_stride_b = 8u * (uint32_t)p.ldbt;

    // Loads are never skipped, so that the number of outstanding loads at every point of the loop is a
    // compile-time constant; a K step past the end gets an out-of-range lane offset instead (no memory traffic).
    auto issue_a = [&](int kt, int KT) {
        char *slot = lds + (kt % NSA) * A_BYTES;
        const uint32_t vo = kt < KT ? voff_a : kOutOfRange;
#pragma unroll
        for (int i = 0; i < LA; i++) {
            const int u = i * NW + wave;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void *)(slot + u * 1024), 16, vo,
                                                     (uint32_t)u * unit_stride_a + (uint32_t)(kt0 + kt) * BK, 0, 0);
        }
    };
    // B units are padded to a multiple of the wavefront count (rows past the tile read as zero), so every
    // wavefront issues the same number of loads per stage
    auto issue_b = [&](int kt, int KT) {
        char *slot = lds + NSA * A_BYTES + (kt % (NS > 0 ? NS : 1)) * B_BYTES;
        const uint32_t vo = kt < KT ? voff_b : kOutOfRange;
#pragma unroll
        for (int i = 0; i < LB; i++) {
            const int u = i * NW + wave;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void *)(slot + u * 1024), 16, vo,
                                                     (uint32_t)u * unit_stride_b + (uint32_t)(kt0 + kt) * BK, 0, 0);
        }
    };

    i32x4v acc[WTM][WTN];
#pragma unroll
    for (int i = 0; i < WTM; i++)
#pragma unroll
        for (int j = 0; j < WTN; j++) acc[i][j] = i32x4v{0, 0, 0, 0};

    // the wide loop's epilogue for the common case takes its parameters from LDS (quant_matmul_wide.h)
    // (the widest wavefront tile holds few variants of it at a time: every further one costs the K loop registers it does not
    // have - 2048x4096x28672 went from 203 to 219 us with all of them in one kernel.  EPI 0: no bias or a bf16 one; 1: an
    // int32 or float32 bias; 2: packed parameter words with no bias or an int32 one.)
    constexpr bool LEAN = WTN >= 7;
    const bool lean_bias = EPI == 0 ? p.bias_kind == MI355_BIAS_NONE || p.bias_kind == MI355_BIAS_BF16
                                    : EPI == 1 && (p.bias_kind == MI355_BIAS_INT32 || p.bias_kind == MI355_BIAS_FP32);
    const bool lean_qp = EPI == 2 && (p.bias_kind == MI355_BIAS_NONE || p.bias_kind == MI355_BIAS_INT32);
    const bool fast_epilogue = LDSP && !p.out_i32 && !p.out_i8 && !p.qparam && (p.scale_len == p.N || p.scale_len == 1) &&
                               (!LEAN || lean_bias) && (p.ldc & 7) == 0 &&
                               aligned_dev(p.out, 16) && (!p.pertoken || aligned_dev(p.pertoken, 16)) &&
                               (p.scale_len == 1 || aligned_dev(p.scale, 16)) && (!p.bias || aligned_dev(p.bias, 16));
    // ... the same with the column scales taken from packed 64-bit parameter words (no per-token scales then)
    const bool fast_epilogue_qp = LDSP && (!LEAN || lean_qp) && !p.out_i32 && !p.out_i8 && p.qparam && !p.pertoken && p.scale_len == p.N && (p.ldc & 7) == 0 &&
                                  aligned_dev(p.out, 16) && aligned_dev(p.qparam, 16) && (!p.bias || aligned_dev(p.bias, 16));
    // ... and so does the one for the re-quantised int8 output with per-channel parameter words
    const bool fast_epilogue_i8 = LDSP && p.out_i8 && p.qparam && p.scale_len == p.N &&
                                  (p.bias_kind == MI355_BIAS_NONE || p.bias_kind == MI355_BIAS_INT32) && (p.ldc & 15) == 0 &&
                                  aligned_dev(p.out, 16) && aligned_dev(p.qparam, 16) && (!p.bias || aligned_dev(p.bias, 16));

    // requested by one wavefront in front of its first stage (loads retire in order: they have landed when stage 0 has)
    constexpr int PARAM_BASE = WIDE ? wide::Geometry<WTN>::PARAM_BASE : NSA * A_BYTES + (NS > 0 ? NS : 1) * B_BYTES;
    if constexpr (LDSP) {
        if (fast_epilogue && wave == 0)
            wide::request_params(lds, PARAM_BASE, p.pertoken, p.scale, p.scale_len == 1, p.bias, p.bias_kind == MI355_BIAS_BF16 ? 2 : 4,
                                 m0, n0, rows_a, rows_b, lane);
        if (fast_epilogue_qp && wave == 0)
            wide::request_params_i8(lds, PARAM_BASE, p.qparam, p.bias, n0, rows_b, lane, p.bias_kind == MI355_BIAS_BF16 ? 2 : 4);
        if (fast_epilogue_i8 && wave == 0)
            wide::request_params_i8(lds, PARAM_BASE, p.qparam, p.bias_kind == MI355_BIAS_INT32 ? p.bias : nullptr, n0, rows_b, lane);
    }
    if constexpr (WIDE) {
        static_assert(WGM == 4 && WGN == 2 && WTM == 4 && NS == 3, "wide loop: 4 x 2 wavefronts of 64 rows");
        using G = wide::Geometry<WTN>;
        if (threadIdx.x < 16) reinterpret_cast<uint32_t *>(lds + G::FLAG_BASE)[threadIdx.x] = 0u;
        const int frow = lane & 15;
        const uint32_t sw0 = (uint32_t)(((lane >> 4) ^ ((frow >> 1) & 7)) * 16);
        wide::LoopState st;
        st.va0 = (uint32_t)((wm * 64 + frow) * BK) + sw0;
        st.va1 = (uint32_t)((wm * 64 + frow) * BK) + (sw0 ^ 64u);
        st.vb0 = (uint32_t)(G::B_BASE + (wn * WTN * 16 + frow) * BK) + sw0;
        st.vb1 = (uint32_t)(G::B_BASE + (wn * WTN * 16 + frow) * BK) + (sw0 ^ 64u);
        st.flag = (uint32_t)(G::FLAG_BASE + wm * 4);
        st.KT = KT;
#ifdef MI355_QMM_TS
        st.ts = p.ts ? p.ts + ((size_t)blockIdx.x * 8 + wave) * 128 : nullptr;
#endif
        // unit u of a stage holds rows 8u .. 8u+7; lane l fills row l / 8, 16-byte slot l % 8 with the row's chunk
        // (l % 8) ^ ((row >> 1) & 7), and (row >> 1) & 7 = 4 * (u & 1) + (l / 8) / 2
        auto lane_off = [&](int par, int64_t ld) { return (uint32_t)(rr * (int)ld + (((lane & 7) ^ ((par << 2) | (rr >> 1))) * 16)); };
        if (wn == 0) {
            const int u0 = wm * wide::LAW;                                // its own 64 activation rows
            st.rsrc = rsrc_a;
            st.voff0 = lane_off(0, p.lda);
            st.voff1 = lane_off(1, p.lda);
            st.unit_stride = unit_stride_a;
            st.sbase = (uint32_t)u0 * unit_stride_a + (uint32_t)kt0 * BK;
            st.dst0 = (uint32_t)u0 * 1024u;
            wide::k_loop<WTN, 0, LOOP - 1>(acc, lds, st);
        } else {
            const int u0 = wm * G::LBW;                                   // a quarter of the weight rows
            st.rsrc = rsrc_b;
            st.voff0 = lane_off(u0 & 1, p.ldbt);
            st.voff1 = lane_off((u0 & 1) ^ 1, p.ldbt);
            st.unit_stride = unit_stride_b;
            st.sbase = (uint32_t)u0 * unit_stride_b + (uint32_t)kt0 * BK;
            st.dst0 = (uint32_t)u0 * 1024u;
            wide::k_loop<WTN, 1, LOOP - 1>(acc, lds, st);
        }
        MI355_TS(2)
        __syncthreads();
        MI355_TS(3)
    } else if constexpr (NS == 0) {
        // ---- streaming K loop (at most 64 rows, few workgroups per CU: the weights are a pure HBM stream).  No workgroup
        // ring and no barrier per K step: a wavefront owns its 16 weight rows (= 16 output columns) for the whole K range
        // of the workgroup and loads 128 bytes of each row per step by direct-to-LDS loads into a private ring of five
        // XOR-swizzled 2 KiB tiles, four steps in flight - whole cache lines per instruction (lane l: 16 bytes of row l / 8,
        // and of row 8 + l / 8) -, from which it reads the step in operand order (its own loads and reads: no barrier, only
        // the wait for the step's two loads).  Activations are staged in fragment order, four steps at a time, double
        // buffered, by direct-to-LDS loads as well: the loads of the next chunk are issued at the top of a chunk, one
        // barrier per chunk.  No register holds an operand before its fragment read.
        static_assert(WGM == 1 && WGN == 8 && WTM == 4 && WTN == 1, "streaming loop: eight wavefronts of 64 rows x 16 columns");
        constexpr int CH = 4;                                   // steps per chunk of activations
        constexpr int XBUF = CH * WTM * 2048;                   // bytes of one activation chunk: [step][m tile][half][lane] x 16
        constexpr int TBUF = 2048;
        constexpr int R = 4;                                    // weight steps in flight per wavefront
        constexpr int RING = R + 1;                             // ... and the one being read
        char *const tbuf = lds + 2 * XBUF + wave * (RING * TBUF);
        const int c16 = lane & 15, g4 = lane >> 4;
        uint32_t voff_w[2];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int rl = 8 * h + (lane >> 3);
            voff_w[h] = (uint32_t)((wn * 16 + rl) * (int)p.ldbt + (((lane & 7) ^ ((rl >> 1) & 7)) * 16));
        }
        const int t_rd = c16 * 128 + ((g4 ^ ((c16 >> 1) & 7)) * 16);   // chunk g of row c; chunk g + 4 is at slot ^ 4
        // a step's 16 rows x 128 bytes go straight into a slot of the wavefront's ring (lane l at l * 16, i.e. row l / 8 and
        // row 8 + l / 8 in the swizzled piece order the reads expect)
        auto load_w = [&](int slot, int st) {
            const bool ok = st < KT;
            const uint32_t kb = (uint32_t)(kt0 + st) * BK;
            char *dst = tbuf + slot * TBUF;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void *)dst, 16, ok ? voff_w[0] : kOutOfRange, kb, 0, 2);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_void *)(dst + 1024), 16, ok ? voff_w[1] : kOutOfRange, kb, 0, 2);
        };
        // staging: the chunk is 64 rows x 512 bytes = 2048 pieces of 16 bytes, four per thread, by direct-to-LDS loads.  A
        // wavefront's instruction takes 16 rows x 4 consecutive pieces (64 bytes of a row): in fragment order those are one
        // contiguous KiB of LDS (piece g of row r at g * 256 + r * 16), which is what a direct load writes (lane l at
        // l * 16 behind the instruction's base).
        const int st_row = lane & 15, st_g = lane >> 4;
        auto stage = [&](int ch) {
            char *buf = lds + (ch & 1) * XBUF;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int combo = wave * 4 + j;                              // (group of 16 rows, group of 4 pieces)
                const int mt = combo % WTM, qg = combo / WTM;                // pieces 4 qg .. 4 qg + 3: step qg / 2, half qg % 2
                const int row = mt * 16 + st_row, q = qg * 4 + st_g;
                const bool ok = ch * CH + (q >> 3) < KT;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void *)(buf + (((qg >> 1) * WTM + mt) * 2 + (qg & 1)) * 1024), 16,
                                                         ok ? (uint32_t)(row * (int)p.lda + q * 16) : kOutOfRange,
                                                         (uint32_t)(kt0 + ch * CH) * BK, 0, 0);
            }
        };
        // a chunk has landed: at most the `younger` loads issued behind its four are outstanding; and every wavefront is
        // done with the other buffer
        auto chunk_barrier = [&](auto younger) {
            wait_vmcnt_lgkm0<decltype(younger)::value>();
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };
        stage(0);                                   // before the weights: loads retire in order, and these come from cache
#pragma unroll
        for (int r = 0; r < R; r++) load_w(r, r);
        chunk_barrier(std::integral_constant<int, 2 * R>{});
        const int nchunks = (KT + CH - 1) / CH;
        int slot0 = 0;                              // ring slot of the chunk's first step: (ch * CH) % RING
        for (int ch = 0; ch < nchunks; ch++) {
            stage(ch + 1);                          // into the other buffer; past the end: zeros, no memory traffic
            const char *xb = lds + (ch & 1) * XBUF + lane * 16;
#pragma unroll
            for (int j = 0; j < CH; j++) {
                const int st = ch * CH + j;
                const int slot = slot0 + j >= RING ? slot0 + j - RING : slot0 + j;
                i32x4v xa[2][WTM];
#pragma unroll
                for (int t = 0; t < 2; t++)
#pragma unroll
                    for (int mt = 0; mt < WTM; mt++) xa[t][mt] = *reinterpret_cast<const i32x4v *>(xb + ((j * WTM + mt) * 2 + t) * 1024);
                // this step's weights have landed: behind them are the loads of the R - 1 steps after it and the one chunk of
                // activations requested within the last R steps (R = CH: always exactly one)
                static_assert(R == CH, "the count below");
                wait_vmcnt<2 * (R - 1) + 4>();
                asm volatile("" ::: "memory");
                const char *tr = tbuf + slot * TBUF;
                const i32x4v w0 = *reinterpret_cast<const i32x4v *>(tr + t_rd);
                const i32x4v w1 = *reinterpret_cast<const i32x4v *>(tr + (t_rd ^ 64));
                __builtin_amdgcn_sched_barrier(0);
                load_w(slot == 0 ? RING - 1 : slot - 1, st + R);             // the slot read one step ago
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int mt = 0; mt < WTM; mt++) acc[mt][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, xa[0][mt], acc[mt][0], 0, 0, 0);
#pragma unroll
                for (int mt = 0; mt < WTM; mt++) acc[mt][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, xa[1][mt], acc[mt][0], 0, 0, 0);
            }
            chunk_barrier(std::integral_constant<int, 2 * CH>{});       // the chunk's weight loads were issued behind its activations
            slot0 = slot0 + CH >= RING ? slot0 + CH - RING : slot0 + CH;
        }
        wait_vmcnt<0>();                            // nothing is on its way into LDS when the epilogue takes it over
        __syncthreads();
    } else {
    // LDS read addressing: lane reads row (lane % 16) of a 16-row tile, 16-byte chunk (ks*4 + lane/16),
    // stored at slot chunk ^ (row % 8).  For ks = 1 the slot is the ks = 0 slot with bit 2 flipped.
    const int frow = lane & 15;
    const int sw0 = ((lane >> 4) ^ ((frow >> 1) & 7)) * 16;
    const int a_off = (wm * WTM * 16 + frow) * BK;
    const int b_off = NSA * A_BYTES + (wn * WTN * 16 + frow) * BK;

    // Fragments are double buffered in registers: the LDS reads of the next 64-wide K step are issued before
    // the MFMAs of the current one, so LDS latency hides behind the matrix pipe instead of in front of it.
    i32x4v af0[WTM], bf0[WTN], af1[WTM], bf1[WTN];
#define MI355_READ_FRAGS(AF, BF, KT_, KS)                                                                        \
    {                                                                                                            \
        const char *sa_ = lds + ((KT_) % NSA) * A_BYTES + a_off, *sb_ = lds + ((KT_) % (NS > 0 ? NS : 1)) * B_BYTES + b_off; \
        const int sw_ = sw0 ^ ((KS) * 64);                                                                       \
        _Pragma("unroll") for (int i = 0; i < WTM; i++)                                                          \
            AF[i] = *reinterpret_cast<const i32x4v *>(sa_ + i * 16 * BK + sw_);                                  \
        _Pragma("unroll") for (int j = 0; j < WTN; j++)                                                          \
            BF[j] = *reinterpret_cast<const i32x4v *>(sb_ + j * 16 * BK + sw_);                                  \
    }
#define MI355_MFMA_BLOCK(AF, BF)                                                                                 \
    {                                                                                                            \
        _Pragma("unroll") for (int i = 0; i < WTM; i++)                                                          \
            _Pragma("unroll") for (int j = 0; j < WTN; j++)                                                      \
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(BF[j], AF[i], acc[i][j], 0, 0, 0);             \
    }

    // Instruction order of half a K step: the fragment reads of the next half, each followed by PER MFMAs, then the
    // refills, each followed by two MFMAs, then the remaining MFMAs.  A wavefront that issues its memory
    // instructions in a burst waits while their queues drain and issues no MFMA meanwhile.  (The refills follow
    // the reads in program order because the compiler orders a direct-to-LDS load against later LDS reads.)
#define MI355_INTERLEAVE(NDMA, PER)                                                                              \
    {                                                                                                            \
        _Pragma("unroll") for (int q = 0; q < WTM + WTN; q++) {                                                  \
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                                   \
            __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);                                                 \
        }                                                                                                        \
        _Pragma("unroll") for (int q = 0; q < (NDMA); q++) {                                                     \
            __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);                                                   \
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);                                                   \
        }                                                                                                        \
        __builtin_amdgcn_sched_group_barrier(0x008, WTM * WTN, 0);                                               \
    }

    // Two activation slots and NS weight slots (NS = 3 described).  In the middle of K step kt, once every wavefront is done
    // with stage kt, its slots are refilled with the activations of step kt+2 and the weights of step kt+3:
    // activations come from cache and get one step to land, weights come from HBM and get two.  Loads retire in
    // order and every refill issues the activation loads first, so "at most LB outstanding" means that
    // everything up to the activations of step kt+1 has landed and only the newest weight refill may be in flight.
    // (With NS = 2 the weights of step kt+2 are requested instead and nothing may stay in flight; small tiles
    // use that to keep two workgroups resident per CU.)
    // (With NS >= 4, for launches of at most one small tile per CU, activations get NS slots as well and whole stages
    // are requested NS steps ahead: NS-1 stages in flight per CU instead of one is what a weight stream from HBM
    // needs when no second workgroup shares the CU.)
    static_assert(NS >= 2 && NS <= 4 && (NS < 4 || WTM * WTN <= 16), "weight slots");
    issue_a(0, KT);
    issue_b(0, KT);
    issue_a(1, KT);
    issue_b(1, KT);
    if constexpr (NS == 3 && !WHOLE) issue_b(2, KT);
    if constexpr (WHOLE) {
#pragma unroll
        for (int st = 2; st < NS; st++) {
            issue_a(st, KT);
            issue_b(st, KT);
        }
        wait_vmcnt<(NS - 1) * (LA + LB)>();                            // stage 0 has landed
    } else {
        wait_vmcnt<LA + (NS - 1) * LB>();                              // stage 0 has landed
    }
    __syncthreads();
    MI355_READ_FRAGS(af0, bf0, 0, 0)

    for (int kt = 0; kt < KT; kt++) {
        if constexpr (NS == 3 && WTM * WTN > 16 && !WHOLE) {
            MI355_READ_FRAGS(af1, bf1, kt, 1)
            MI355_MFMA_BLOCK(af0, bf0)
            MI355_INTERLEAVE(0, 2)
            __builtin_amdgcn_sched_barrier(0);
            wait_vmcnt_lgkm0<LB>();            // stage kt+1 has landed and this wavefront is done reading stage kt
            __syncthreads();
            MI355_READ_FRAGS(af0, bf0, kt + 1, 0)
            issue_a(kt + 2, KT);
            issue_b(kt + NS, KT);
            MI355_MFMA_BLOCK(af1, bf1)
            MI355_INTERLEAVE(LA + LB, 1)
            __builtin_amdgcn_sched_barrier(0);
        } else {
            // small wavefront tiles (and two resident workgroups per CU, which overlap each other's bursts) gain
            // nothing from spreading the instructions
            MI355_READ_FRAGS(af1, bf1, kt, 1)
            __builtin_amdgcn_sched_barrier(0);
            MI355_MFMA_BLOCK(af0, bf0)
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (WHOLE) wait_vmcnt_lgkm0<(NS - 2) * (LA + LB)>();     // stage kt+1 has landed, NS-2 more may be in flight
            else wait_vmcnt_lgkm0<(NS - 2) * LB>();
            __syncthreads();
            issue_a(kt + NSA, KT);
            issue_b(kt + NS, KT);
            MI355_READ_FRAGS(af0, bf0, kt + 1, 0)
            __builtin_amdgcn_sched_barrier(0);
            MI355_MFMA_BLOCK(af1, bf1)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    wait_vmcnt<0>();                       // the refills past the end (zeros) must not land in the epilogue's LDS
    __syncthreads();
#undef MI355_READ_FRAGS
#undef MI355_MFMA_BLOCK
#undef MI355_INTERLEAVE
    }

    if (p.S > 1) {
        // Split K: every workgroup of the tile publishes its int32 partial sums in register order (16 bytes per
        // lane, fully coalesced); the one that arrives last at the tile's counter adds the others to its own and
        // runs the epilogue.  Integer addition is exact, so the result does not depend on the order of arrival.
        // Publication uses agent-scope (sc1) write-through stores and cache-bypassing loads, ordered by the
        // wavefronts' own store counters, the workgroup barrier and a relaxed agent-scope counter (a full
        // release/acquire fence would write back and invalidate the whole L2 of the XCD).
        constexpr int SC1 = 16;
        constexpr uint32_t WAVE_BYTES = WTM * WTN * 64 * 16;
        constexpr uint32_t CHUNK_BYTES = NW * WAVE_BYTES;
        const __amdgpu_buffer_rsrc_t rsrc_p = make_rsrc(p.partial + (size_t)tile * p.S * (CHUNK_BYTES / 4), (uint32_t)p.S * CHUNK_BYTES);
        const uint32_t lane_off = (uint32_t)wave * WAVE_BYTES + (uint32_t)lane * 16u;
#pragma unroll
        for (int i = 0; i < WTM; i++)
#pragma unroll
            for (int j = 0; j < WTN; j++)
                buffer_store_b128<SC1>(__builtin_bit_cast(u32x4, acc[i][j]), rsrc_p, lane_off + (i * WTN + j) * 1024,
                                                       (uint32_t)chunk * CHUNK_BYTES);
        wait_vmcnt<0>();                                          // this wavefront's partial sums have reached the coherence point
        __syncthreads();                                          // (also: every wavefront is done with the LDS stages)
        int &is_last = *reinterpret_cast<int *>(lds);
        if (threadIdx.x == 0) {
            const uint32_t old = __hip_atomic_fetch_add(p.counter + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = old == (uint32_t)(p.S - 1);
        }
        __syncthreads();
        const bool last = is_last != 0;
        __syncthreads();                                          // the flag's LDS word is reused by the epilogue
        if (!last) return;
        // the other chunks' sums are asked for CB chunks at a time (as many as the registers hold): one round trip to the
        // coherence point per batch instead of one per chunk.  The own chunk and chunks past the end get an out-of-range
        // lane offset, i.e. zeros.
        constexpr int TL = WTM * WTN;
        constexpr int CB = TL <= 4 ? 8 : TL <= 8 ? 4 : TL <= 16 ? 2 : 1;
        for (int c0 = 0; c0 < p.S; c0 += CB) {
            u32x4 v[CB][TL];
#pragma unroll
            for (int b = 0; b < CB; b++) {
                const int ch = c0 + b;
                const uint32_t lo = ch < p.S && ch != chunk ? lane_off : kOutOfRange;
#pragma unroll
                for (int t = 0; t < TL; t++)
                    v[b][t] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_p, lo + t * 1024, (uint32_t)min(ch, p.S - 1) * CHUNK_BYTES, SC1);
            }
#pragma unroll
            for (int b = 0; b < CB; b++)
#pragma unroll
                for (int t = 0; t < TL; t++) acc[t / WTN][t % WTN] += __builtin_bit_cast(i32x4v, v[b][t]);
        }
        if (threadIdx.x == 0) __hip_atomic_store(p.counter + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    if constexpr (LDSP) {
        if (fast_epilogue_i8) {
            wide::EpilogueArgs e;
            e.param_base = PARAM_BASE;
            e.out = p.out;
            e.ldc = p.ldc;
            e.M = p.M;
            e.N = p.N;
            e.m0 = m0;
            e.n0 = n0;
            e.has_bias = p.bias_kind == MI355_BIAS_INT32;
            e.out_f16 = 0;
            e.stream_out = p.stream_out;
            e.wm = wm;
            e.wn = wn;
            wide::epilogue_fast_i8<WTN>(acc, lds, e, wave, lane);
            return;
        }
        if (fast_epilogue || fast_epilogue_qp) {
            wide::EpilogueArgs e;
            e.param_base = PARAM_BASE;
            e.packed_scale = fast_epilogue_qp;
            e.out = p.out;
            e.ldc = p.ldc;
            e.M = p.M;
            e.N = p.N;
            e.m0 = m0;
            e.n0 = n0;
            e.has_bias = p.bias ? p.bias_kind : MI355_BIAS_NONE;
            e.out_f16 = p.out_f16;
            e.stream_out = p.stream_out;
            e.wm = wm;
            e.wn = wn;
            wide::epilogue_fast<WTN, EPI>(acc, lds, e, wave, lane);
            MI355_TS(4)
            return;
        }
    }
    // Epilogue.  The weight fragment was the first MFMA operand, so
    // acc[i][j][r] = C[m = tile row (lane % 16)][n = 4 * (lane / 16) + r].
    const int mrow = lane & 15;
    const int nquad = (lane >> 4) * 4;
    if (p.out_i32) {
        if (p.bias_kind == MI355_BIAS_INT32) {
            const int32_t *bb = static_cast<const int32_t *>(p.bias);
#pragma unroll
            for (int j = 0; j < WTN; j++) {
                const int n = n0 + (wn * WTN + j) * 16 + nquad;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int32_t bi = bb[min(n + r, p.N - 1)];
#pragma unroll
                    for (int i = 0; i < WTM; i++) acc[i][j][r] = (int32_t)((uint32_t)acc[i][j][r] + (uint32_t)bi);
                }
            }
        }
        const bool vec = (p.ldc & 3) == 0 && aligned_dev(p.out, 16);
#pragma unroll
        for (int i = 0; i < WTM; i++) {
            const int m = m0 + (wm * WTM + i) * 16 + mrow;
#pragma unroll
            for (int j = 0; j < WTN; j++) {
                const int n = n0 + (wn * WTN + j) * 16 + nquad;
                if (m >= p.M || n >= p.N) continue;
                int32_t *o = static_cast<int32_t *>(p.out) + (int64_t)m * p.ldc + n;
                if (vec && n + 3 < p.N) {
                    *reinterpret_cast<i32x4v *>(o) = acc[i][j];
                } else {
                    for (int r = 0; r < 4; r++)
                        if (n + r < p.N) o[r] = acc[i][j][r];
                }
            }
        }
        return;
    }
    if (p.out_i8) {
        // Re-quantised output: a lane owns four consecutive columns of a row in every 16x16 tile, i.e. one 32-bit word
        // of int8 results.  With aligned output rows the words of the wavefront's tile go through its own LDS region
        // (the stage buffers are idle after the last barrier) and leave as 16-byte stores over whole tile rows.
        constexpr int ROWQ = WTN * 16 + 16;                   // padded row pitch in bytes
        constexpr int CHQ = WTN;                              // 16-byte chunks per row
        char *stq = lds + wave * (WTM * 16 * ROWQ);
        const bool wide8 = (p.ldc & 15) == 0 && aligned_dev(p.out, 16);
        const bool words = (p.ldc & 3) == 0 && aligned_dev(p.out, 4);
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            const int n = n0 + (wn * WTN + j) * 16 + nquad;
            float sc[4], of[4];
            int32_t bi[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int nn = min(n + r, p.N - 1);
                const uint64_t q = p.qparam[p.scale_len == 1 ? 0 : nn];
                sc[r] = qparam_scale(q);
                of[r] = qparam_offset(q);
                bi[r] = p.bias_kind == MI355_BIAS_INT32 ? static_cast<const int32_t *>(p.bias)[nn] : 0;
            }
#pragma unroll
            for (int i = 0; i < WTM; i++) {
                const int m = m0 + (wm * WTM + i) * 16 + mrow;
                uint32_t w = 0;
#pragma unroll
                for (int r = 0; r < 4; r++) w |= ((uint32_t)requant1(acc[i][j][r], bi[r], sc[r], of[r]) & 0xffu) << (8 * r);
                if (wide8) {
                    *reinterpret_cast<uint32_t *>(stq + (i * 16 + mrow) * ROWQ + j * 16 + nquad) = w;
                    continue;
                }
                if (m >= p.M || n >= p.N) continue;
                int8_t *o = static_cast<int8_t *>(p.out) + (int64_t)m * p.ldc + n;
                if (words && n + 3 < p.N) {
                    *reinterpret_cast<uint32_t *>(o) = w;
                } else {
                    for (int r = 0; r < 4; r++)
                        if (n + r < p.N) o[r] = (int8_t)(w >> (8 * r));
                }
            }
        }
        if (wide8) {
            const int mw = m0 + wm * WTM * 16, nw = n0 + wn * WTN * 16;
#pragma unroll
            for (int q0 = 0; q0 < WTM * 16 * CHQ; q0 += 64) {
                const int q = q0 + lane;
                const int row = q / CHQ, ch = q % CHQ;
                if ((WTM * 16 * CHQ) % 64 != 0 && row >= WTM * 16) continue;
                const int m = mw + row, n = nw + ch * 16;
                if (m >= p.M || n >= p.N) continue;
                const u32x4 v = *reinterpret_cast<const u32x4 *>(stq + row * ROWQ + ch * 16);
                int8_t *o = static_cast<int8_t *>(p.out) + (int64_t)m * p.ldc + n;
                if (n + 15 < p.N) {
                    *reinterpret_cast<u32x4 *>(o) = v;
                } else {
                    for (int r = 0; r < 16; r++)
                        if (n + r < p.N) o[r] = (int8_t)(v[r >> 2] >> ((r & 3) * 8));
                }
            }
        }
        return;
    }
    // All dequantisation parameters of this wavefront are fetched in one batch (indices clamped so that every
    // load is in bounds), then every accumulator quad is scaled and rounded.
    float psv[WTM];
#pragma unroll
    for (int i = 0; i < WTM; i++) {
        const int m = min(m0 + (wm * WTM + i) * 16 + mrow, p.M - 1);
        psv[i] = p.pertoken ? p.pertoken[m] : 1.0f;
    }
    f32x4 scv[WTN], bsv[WTN];
    i32x4v biv[WTN];                                          // int32 bias: added to the accumulator before dequantisation
    const bool quads = (p.N & 3) == 0 && (p.qparam || aligned_dev(p.scale, 16)) && (!p.bias || aligned_dev(p.bias, 16));
#pragma unroll
    for (int j = 0; j < WTN; j++) {
        const int n = n0 + (wn * WTN + j) * 16 + nquad;
        if (p.qparam) {
#pragma unroll
            for (int r = 0; r < 4; r++) scv[j][r] = qparam_scale(p.qparam[p.scale_len == 1 ? 0 : min(n + r, p.N - 1)]);
        } else if (p.scale_len == 1) {
            const float s1 = p.scale[0];
            scv[j] = f32x4{s1, s1, s1, s1};
        } else if (quads) {
            scv[j] = *reinterpret_cast<const f32x4 *>(p.scale + min(n, p.N - 4));
        } else {
#pragma unroll
            for (int r = 0; r < 4; r++) scv[j][r] = p.scale[min(n + r, p.N - 1)];
        }
        bsv[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        biv[j] = i32x4v{0, 0, 0, 0};
        if (p.bias_kind == MI355_BIAS_BF16) {
            const uint16_t *bb = static_cast<const uint16_t *>(p.bias);
            if (quads) {
                const u32x2 b2 = *reinterpret_cast<const u32x2 *>(bb + min(n, p.N - 4));
                bsv[j] = f32x4{bf16_lo(b2.x), bf16_hi(b2.x), bf16_lo(b2.y), bf16_hi(b2.y)};
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++) bsv[j][r] = bf16_1(bb[min(n + r, p.N - 1)]);
            }
        } else if (p.bias_kind == MI355_BIAS_FP32) {
            const float *bb = static_cast<const float *>(p.bias);
#pragma unroll
            for (int r = 0; r < 4; r++) bsv[j][r] = bb[min(n + r, p.N - 1)];
        } else if (p.bias_kind == MI355_BIAS_INT32) {
            const int32_t *bb = static_cast<const int32_t *>(p.bias);
#pragma unroll
            for (int r = 0; r < 4; r++) biv[j][r] = bb[min(n + r, p.N - 1)];
        }
    }
    const bool has_ps = p.pertoken != nullptr;
    const bool has_bias = p.bias_kind == MI355_BIAS_BF16 || p.bias_kind == MI355_BIAS_FP32;
    const bool f16 = p.out_f16 != 0;
    // (acc + int32 bias) wraps like the hardware accumulator; float bias is added after both scales
    auto dequant = [&](int32_t a, int32_t bi, float ps, float sc, float bf) {
        float v = (float)(int32_t)((uint32_t)a + (uint32_t)bi);
        if (has_ps) v = v * ps;
        v = v * sc;
        if (has_bias) v = v + bf;
        return v;
    };
    auto pack2 = [&](float lo, float hi) { return f16 ? pack_f16x2(lo, hi) : pack_bf16x2(lo, hi); };

    // The rounded bf16 tile of a wavefront goes through its own LDS region (the stage buffers are idle after the
    // last barrier) so that global stores are 16 bytes per lane and cover whole rows of the wavefront tile.
    constexpr int ROWB = WTN * 32 + 16;                       // padded row pitch: spreads rows over the banks
    constexpr int CHUNKS = WTN * 2;                           // 16-byte chunks per row
    static_assert(NW * WTM * 16 * ROWB <= 160 * 1024, "epilogue staging must fit in LDS");
    char *stg = lds + wave * (WTM * 16 * ROWB);
    const bool wide = (p.ldc & 7) == 0 && aligned_dev(p.out, 16);
    if (wide) {
        // The output type, and the common case of a per-token scale with a float bias, are chosen once per
        // wavefront here and not once per element: a scalar branch per converted pair costs more than the
        // arithmetic between two of them.
        auto stage_tile = [&](auto f16_c, auto fast_c) {
            constexpr bool F16 = decltype(f16_c)::value, FAST = decltype(fast_c)::value;
#pragma unroll
            for (int i = 0; i < WTM; i++)
#pragma unroll
                for (int j = 0; j < WTN; j++) {
                    float f[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        if constexpr (FAST) {
                            float v = (float)acc[i][j][r];
                            v = v * psv[i];
                            v = v * scv[j][r];
                            f[r] = v + bsv[j][r];
                        } else {
                            f[r] = dequant(acc[i][j][r], biv[j][r], psv[i], scv[j][r], bsv[j][r]);
                        }
                    }
                    u32x2 pk;
                    pk.x = F16 ? pack_f16x2(f[0], f[1]) : pack_bf16x2(f[0], f[1]);
                    pk.y = F16 ? pack_f16x2(f[2], f[3]) : pack_bf16x2(f[2], f[3]);
                    *reinterpret_cast<u32x2 *>(stg + (i * 16 + mrow) * ROWB + (j * 16 + nquad) * 2) = pk;
                }
        };
        const bool fast = has_ps && has_bias;                 // a float bias excludes the int32 one
        using T = std::true_type;
        using F = std::false_type;
        if (f16) {
            if (fast) stage_tile(T{}, T{}); else stage_tile(T{}, F{});
        } else {
            if (fast) stage_tile(F{}, T{}); else stage_tile(F{}, F{});
        }
        const int mw = m0 + wm * WTM * 16, nw = n0 + wn * WTN * 16;
        // the kind of store is a compile-time choice (a run-time choice between the two is merged into ordinary stores)
        auto store_rows = [&](auto nt_c) {
#pragma unroll
            for (int q0 = 0; q0 < WTM * 16 * CHUNKS; q0 += 64) {
                const int q = q0 + lane;
                const int row = q / CHUNKS, ch = q % CHUNKS;
                if ((WTM * 16 * CHUNKS) % 64 != 0 && row >= WTM * 16) continue;
                const int m = mw + row, n = nw + ch * 8;
                if (m >= p.M || n >= p.N) continue;
                const u32x4 v = *reinterpret_cast<const u32x4 *>(stg + row * ROWB + ch * 16);
                uint16_t *o = static_cast<uint16_t *>(p.out) + (int64_t)m * p.ldc + n;
                if (n + 7 < p.N) {
                    if constexpr (decltype(nt_c)::value) __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(o));
                    else *reinterpret_cast<u32x4 *>(o) = v;
                } else {
                    for (int r = 0; r < 8; r++)
                        if (n + r < p.N) o[r] = (uint16_t)(v[r >> 1] >> ((r & 1) * 16));
                }
            }
        };
        if (p.stream_out) store_rows(T{}); else store_rows(F{});
        return;
    }
    const bool vec = (p.ldc & 3) == 0 && aligned_dev(p.out, 8);
#pragma unroll
    for (int i = 0; i < WTM; i++) {
        const int m = m0 + (wm * WTM + i) * 16 + mrow;
#pragma unroll
        for (int j = 0; j < WTN; j++) {
            const int n = n0 + (wn * WTN + j) * 16 + nquad;
            float f[4];
#pragma unroll
            for (int r = 0; r < 4; r++) f[r] = dequant(acc[i][j][r], biv[j][r], psv[i], scv[j][r], bsv[j][r]);
            if (m >= p.M || n >= p.N) continue;
            uint16_t *o = static_cast<uint16_t *>(p.out) + (int64_t)m * p.ldc + n;
            if (vec && n + 3 < p.N) {
                u32x2 pk;
                pk.x = pack2(f[0], f[1]);
                pk.y = pack2(f[2], f[3]);
                *reinterpret_cast<u32x2 *>(o) = pk;
            } else {
                for (int r = 0; r < 4; r++)
                    if (n + r < p.N) o[r] = (uint16_t)pack2(f[r], 0.0f);
            }
        }
    }
}

// Correct for every shape, stride and alignment; used when the tiled kernel's preconditions
// (K multiple of 128, 16-byte aligned rows) do not hold.  One thread per output element.
__global__ __launch_bounds__(256) void qmm_generic_kernel(const int8_t *__restrict__ a, const int8_t *__restrict__ b,
                                                          const float *__restrict__ pertoken,
                                                          const float *__restrict__ scale, int scale_len,
                                                          const void *__restrict__ bias, int bias_kind, int out_f16, void *out,
                                                          int out_i32, const uint64_t *__restrict__ qparam, int out_i8,
                                                          int M, int N, int K, int64_t lda, int64_t ldb_k,
                                                          int64_t ldb_n, int64_t ldc)
{
    const int n = blockIdx.x * 16 + (threadIdx.x & 15);
    const int m = blockIdx.y * 16 + (threadIdx.x >> 4);
    if (m >= M || n >= N) return;
    int32_t s = 0;
    for (int k = 0; k < K; k++) s += (int32_t)a[(int64_t)m * lda + k] * (int32_t)b[(int64_t)k * ldb_k + (int64_t)n * ldb_n];
    if (out_i8) {
        const uint64_t q = qparam[scale_len == 1 ? 0 : n];
        const int32_t bi = bias_kind == MI355_BIAS_INT32 ? static_cast<const int32_t *>(bias)[n] : 0;
        static_cast<int8_t *>(out)[(int64_t)m * ldc + n] = (int8_t)requant1(s, bi, qparam_scale(q), qparam_offset(q));
        return;
    }
    if (bias_kind == MI355_BIAS_INT32) s = (int32_t)((uint32_t)s + (uint32_t)static_cast<const int32_t *>(bias)[n]);
    if (out_i32) {
        static_cast<int32_t *>(out)[(int64_t)m * ldc + n] = s;
        return;
    }
    float v = (float)s;
    if (pertoken) v = v * pertoken[m];
    v = v * (qparam ? qparam_scale(qparam[scale_len == 1 ? 0 : n]) : scale[scale_len == 1 ? 0 : n]);
    if (bias_kind == MI355_BIAS_BF16) v = v + bf16_1(static_cast<const uint16_t *>(bias)[n]);
    if (bias_kind == MI355_BIAS_FP32) v = v + static_cast<const float *>(bias)[n];
    static_cast<uint16_t *>(out)[(int64_t)m * ldc + n] = (uint16_t)(out_f16 ? pack_f16x2(v, 0.0f) : pack_bf16x2(v, 0.0f));
}

// [K,N] contiguous -> [N,K] contiguous, 64x64 byte tiles through LDS.
__global__ __launch_bounds__(256) void transpose_i8_kernel(const int8_t *__restrict__ src, int8_t *__restrict__ dst,
                                                           int K, int N, int64_t ld_src)
{
    __shared__ int8_t tile[64][64 + 4];
    const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < 64; r += 4) {
        const int k = k0 + r, n = n0 + tx;
        tile[r][tx] = (k < K && n < N) ? src[(int64_t)k * ld_src + n] : (int8_t)0;
    }
    __syncthreads();
    for (int r = ty; r < 64; r += 4) {
        const int n = n0 + r, k = k0 + tx;
        if (n < N && k < K) dst[(int64_t)n * K + k] = tile[tx][r];
    }
}

// The same for 16-byte aligned rows on both sides: 128x128 byte tiles, 16-byte loads along N and 16-byte stores along K
// (whole 128-byte lines either way); the transposition itself is done by byte reads from LDS.
__global__ __launch_bounds__(256) void transpose_i8_wide_kernel(const int8_t *__restrict__ src, int8_t *__restrict__ dst,
                                                                int K, int N, int64_t ld_src)
{
    constexpr int T = 128, PITCH = T + 4;                     // pitch 33 dwords: a column walk changes bank every row
    __shared__ __attribute__((aligned(16))) int8_t tile[T * PITCH];
    const int k0 = blockIdx.y * T, n0 = blockIdx.x * T;
    const int t = threadIdx.x;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int r = (t >> 3) + 32 * i, c = (t & 7) * 16;    // row k0 + r, bytes n0 + c .. + 15
        u32x4 v{0u, 0u, 0u, 0u};
        if (k0 + r < K && n0 + c < N) {                       // N % 16 == 0: a chunk is inside or outside as a whole
            v = *reinterpret_cast<const u32x4 *>(src + (int64_t)(k0 + r) * ld_src + n0 + c);
        }
        uint32_t *d = reinterpret_cast<uint32_t *>(tile + r * PITCH + c);
        d[0] = v.x, d[1] = v.y, d[2] = v.z, d[3] = v.w;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int n = (t >> 3) + 32 * i, kc = (t & 7) * 16;   // output row n0 + n, bytes k0 + kc .. + 15
        if (n0 + n >= N || k0 + kc >= K) continue;            // K % 16 == 0
        u32x4 v;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            uint32_t x = 0;
#pragma unroll
            for (int b = 0; b < 4; b++) x |= (uint32_t)(uint8_t)tile[(kc + 4 * w + b) * PITCH + n] << (8 * b);
            v[w] = x;
        }
        *reinterpret_cast<u32x4 *>(dst + (int64_t)(n0 + n) * K + k0 + kc) = v;
    }
}

template <int WGM, int WGN, int WTM, int WTN, int DEEP = 0, int LOOP = 0, int EPI = 0>
int launch_qmm(QmmArgs p, hipStream_t s)
{
    constexpr int BM = 16 * WTM * WGM, BN = 16 * WTN * WGN;
    constexpr int NWL = WGM * WGN;
    // Two activation slots and three weight slots (weights come from HBM and need the longer lead), unless two
    // weight slots let two workgroups share a CU (80 KiB each): sixteen resident wavefronts hide barriers and
    // epilogues better than the deeper ring does.
    constexpr size_t a_bytes = (size_t)(BM / 8) * 1024, b_bytes = (size_t)((BN / 8 + NWL - 1) / NWL * NWL) * 1024;
    constexpr size_t staging_bytes = (size_t)BM * WGN * ((BN / WGN) * 2 + 16);   // epilogue: padded bf16 tile rows
    // DEEP: that many whole stages, one workgroup per CU (for launches that put at most one of these small tiles on a CU)
    constexpr int NS = DEEP < 0 ? 0 : DEEP ? DEEP : 2 * a_bytes + 2 * b_bytes <= 80 * 1024 && staging_bytes <= 80 * 1024 ? 2 : 3;
    // DEEP < 0: the streaming K loop (two activation chunks of 32 KiB and a ring of five 2 KiB weight steps per wavefront)
    constexpr size_t stage_bytes = DEEP < 0 ? (size_t)2 * 32768 + 8 * 5 * 2048 : (DEEP ? DEEP : 2) * a_bytes + NS * b_bytes;
    constexpr size_t ring_bytes = LOOP == 1 || LOOP == 2 ? (size_t)wide::Geometry<WTN>::LDS_BYTES : stage_bytes + (LOOP == 3 ? 3072 : 0);
    constexpr size_t lds_bytes = ring_bytes > staging_bytes ? ring_bytes : staging_bytes;
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    const int tiles = p.tiles_m * p.tiles_n;
    p.tiles_per_xcd = (tiles + 7) / 8;
    if (p.S > 1 && (uint64_t)p.S * BM * BN * 4 >= (1ull << 32)) return MI355_ERR_UNSUPPORTED;
    auto kern = qmm_kernel<WGM, WGN, WTM, WTN, NS, LOOP, EPI>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(8 * p.tiles_per_xcd * p.S), dim3(WGM * WGN * 64), lds_bytes, s, p);
    return check_launch();
}

// Tile shapes (rows x columns of the workgroup tile) the library instantiates, with measured times at K = 4096
// on operands that are not cache resident: `slots` workgroups are resident at once (256 CUs x 1 or 2), a launch
// that fits in one round of them takes `single_us` in all, longer launches take `round_us` per round.
// `whole`: the variant of a 128-row tile that keeps three whole stages (as many activation slots as weight slots) and
// has a CU to itself: its activation refills get two K steps to land instead of one, which is what a tile needs when no
// second workgroup on the CU covers the wait (128x192 at K = 4096: 37.2 -> 31.6 us per round, 128x128: 33.0 -> 24.7).
struct TileChoice {
    int bm, bn, slots;
    double single_us, round_us;
    int whole;
};
constexpr TileChoice kTiles[] = {{256, 256, 256, 58.0, 59.0, 0}, {256, 224, 256, 52.5, 52.0, 0}, {256, 192, 256, 44.5, 45.5, 0},
                                 {128, 320, 256, 48.0, 43.0, 0}, {128, 256, 256, 40.0, 45.6, 0}, {128, 192, 512, 55.8, 58.8, 0},
                                 {128, 128, 512, 40.0, 43.3, 0}, {64, 256, 512, 40.0, 52.6, 0},  {64, 128, 512, 24.0, 30.0, 0},
                                 {128, 192, 256, 32.0, 32.0, 1}, {128, 128, 256, 24.0, 24.8, 1}};

// Workspace layout: [arrival counters | split-K partial sums | transposed weight].
struct QmmPlan {
    TileChoice tile;
    int S;                       // K chunks per tile
    size_t counter_bytes, partial_bytes, transpose_bytes;
};

// Pick the tile shape and the split of K with the smallest estimated time.  The table above gives a launch at K = 4096
// without a split; other depths scale the part of it that is the K loop (`kBaseUs` is what a launch costs around the
// loop).  Two terms that the table does not hold are added: every tile reads (bm + bn) x K bytes through the L2, which
// bounds small tiles on a long K (64x128 tiles on 1024x14336x4096: 1.4 GB, 107 us), and a split of K moves
// wgs x bm x bn x 4 bytes of partial sums out and in again, the S - 1 foreign chunks of a tile through the one workgroup
// that collects them (128x256 tiles split twelve ways: 39 us where a four-way split of 64x128 tiles takes 25).
// Constants fitted to sweeps over tile x split on M = 128 .. 2048, K = 8192 .. 28672 and on M = 80 .. 512 over the
// projections of transformer layers with K = 4096 .. 14336 (46 shapes: the estimate's choice is 0.7 % slower than the
// measured best on average and 8 % at worst; at K = 4096 without a split the estimate is the table itself).
constexpr size_t kMaxPartialBytes = (size_t)128 << 20;
constexpr uint64_t kStreamOutMaxBytes = (uint64_t)32 << 20;     // the L2s of the eight XCDs together
constexpr double kBaseUs = 6.0, kL2BytesPerUs = 12e6, kExchangeUs = 1.0, kExchangeBytesPerUs = 10e6, kCollectorBytesPerUs = 100e3;
constexpr double kAloneOnCu = 0.85;
// a split of a whole-stage tile measured 2-4 us above what the terms below give (its partial sums are 64-96 KiB per
// workgroup); and of two plans with the same estimate the one that leaves fewer CUs idle is the faster one
constexpr double kWholeSplitUs = 3.0, kIdleCuUs = 2.0;

void choose_tile_and_split(int64_t M, int64_t N, int64_t K, bool may_split, size_t partial_cap, TileChoice *tile, int *split)
{
    const int forced_tile = knob(kKnobQmmTile);             // debugging aids: bm * 1000 + bn, and the split
    const int forced_split = knob(kKnobQmmSplit);
    const int64_t kt = K / BK;
    double best_cost = 1e300;
    *tile = kTiles[0];
    *split = 1;
    for (const TileChoice &c : kTiles) {
        if (forced_tile && (c.bm != forced_tile / 1000 || c.bn != forced_tile % 1000)) continue;
        if (c.whole && knob(kKnobQmmLoop) == 1) continue;   // MI355_QMM_LOOP = 1: only the generic loop with its usual rings
        if (!c.whole && knob(kKnobQmmLoop) == 4 && c.bm == 128 && (c.bn == 128 || c.bn == 192)) continue;   // 4: only their whole-stage variants
        const int64_t tiles = ((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn);
        for (const int S : {1, 2, 3, 4, 6, 8, 12, 16}) {
            if (forced_split >= 1 && forced_split <= kt && may_split) {
                if (S != 1) continue;                       // one candidate per tile: the forced split
            } else if (S > 1 && (!may_split || tiles > 128 || kt / S < 4)) {
                continue;                                   // few tiles and at least four K steps per workgroup
            }
            const int s_eff = forced_split >= 1 && forced_split <= kt && may_split ? forced_split : S;
            const int64_t wgs = tiles * s_eff;
            // a caller with a fixed scratch area (mi355_quant_matmul_noalloc) only gets splits whose partial sums fit it
            // ... and nobody gets more than 128 MiB of them
            // (a split forced through the knob is bound by a fixed scratch area too, and no split may need more arrival
            // counters than the workspace holds)
            if (s_eff > 1 && (s_eff == S || partial_cap < kMaxPartialBytes) &&
                (uint64_t)wgs * c.bm * c.bn * 4 > (partial_cap < kMaxPartialBytes ? partial_cap : kMaxPartialBytes))
                continue;
            if (s_eff > 1 && (uint64_t)tiles * 4 > kWorkspaceCounterBytes) continue;
            const int64_t rounds = (wgs + c.slots - 1) / c.slots;
            const double at_4096 = rounds == 1 ? c.single_us : (double)rounds * c.round_us;
            double loop_us = (at_4096 - kBaseUs) * ((double)kt / s_eff) / 32.0;
            // tiles that run two to a CU: with more than 256 and fewer than 512 workgroups the CUs that hold two set the
            // time, as if all did (128x128 split six ways, 384 workgroups: 42 us where eight ways, 512, take 38)
            if (c.slots == 512 && rounds == 1 && wgs > 256) loop_us *= 512.0 / (double)wgs;
            // ... and with at most 256 every workgroup has a CU to itself
            if (c.slots == 512 && wgs <= 256) loop_us *= kAloneOnCu;
            double cost = kBaseUs + loop_us;
            const double l2 = kBaseUs + (double)tiles * (c.bm + c.bn) * (double)K / kL2BytesPerUs;
            if (l2 > cost) cost = l2;
            if (s_eff > 1)
                cost += kExchangeUs + (double)wgs * c.bm * c.bn * 8.0 / kExchangeBytesPerUs +
                        (double)(s_eff - 1) * c.bm * c.bn * 4.0 / kCollectorBytesPerUs + (c.whole ? kWholeSplitUs : 0.0);
            if (wgs < 256) cost += kIdleCuUs * (1.0 - (double)wgs / 256.0);
            if (cost < best_cost) {
                best_cost = cost;
                *tile = c;
                *split = s_eff;
            }
        }
    }
}

// `zero_area`: bytes in front of the scratch part of the workspace (the shared zero area, or just the counters when the
// workspace is private to this operator)
QmmPlan make_qmm_plan(int64_t M, int64_t N, int64_t K, int64_t ldb_k, int64_t ldb_n, size_t zero_area = kWorkspaceZeroBytes,
                      size_t scratch_cap = ~(size_t)0)
{
    QmmPlan pl{};
    const bool tiled_shape = K >= BK && K % BK == 0;
    // the decode kernel splits K inside its workgroups (it is not used while a tile or a split is forced)
    const bool decode = qmm_decode_shape(M, N, K) && knob(kKnobQmmSplit) == 0 && knob(kKnobQmmTile) == 0;
    // a contiguous [K,N] weight is transposed into the workspace
    pl.transpose_bytes = tiled_shape && ldb_k != 1 && ldb_n == 1 ? (size_t)N * (size_t)K : 0;
    const size_t fixed = zero_area + pl.transpose_bytes;
    choose_tile_and_split(M, N, K, tiled_shape && !decode, scratch_cap > fixed ? scratch_cap - fixed : 0, &pl.tile, &pl.S);
    if (tiled_shape && pl.S > 1) {
        const int64_t tiles = ((M + pl.tile.bm - 1) / pl.tile.bm) * ((N + pl.tile.bn - 1) / pl.tile.bn);
        pl.partial_bytes = (size_t)tiles * pl.S * pl.tile.bm * pl.tile.bn * 4;   // tiles <= 128 counters
    }
    pl.counter_bytes = pl.partial_bytes + pl.transpose_bytes > 0 ? zero_area : 0;
    return pl;
}

} // namespace
} // namespace mi355

extern "C" size_t mi355_quant_matmul_workspace(int64_t M, int64_t N, int64_t K, int64_t ldb_k, int64_t ldb_n)
{
    using namespace mi355;
    if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffffff || N > 0x7fffffff) return 0;
    const QmmPlan pl = make_qmm_plan(M, N, K, ldb_k, ldb_n);
    return pl.counter_bytes + pl.partial_bytes + pl.transpose_bytes;
}

namespace mi355 {
namespace {

__global__ __launch_bounds__(256) void trans_quant_param_kernel(const float *__restrict__ scale, int scale_one,
                                                                const float *__restrict__ offset, int offset_one,
                                                                uint64_t *__restrict__ out, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    uint64_t q = (uint64_t)__float_as_uint(scale[scale_one ? 0 : i]) | (1ull << 46);
    if (offset) {
        float o = rintf(offset[offset_one ? 0 : i]);
        o = fminf(fmaxf(o, -256.0f), 255.0f);
        q |= (uint64_t)((uint32_t)(int32_t)o & 0x1ffu) << 37;
    }
    out[i] = q;
}

#ifdef MI355_QMM_TS
unsigned long long *g_dbg_ts = nullptr;
#endif

// One implementation behind both entry points: `scale` (float32) or `qparam` (packed) carries the per-channel factors.
int run_quant_matmul(const int8_t *a, const int8_t *b, const float *pertoken_scale, const float *scale, const uint64_t *qparam,
                     int64_t scale_len, const void *bias, int bias_dtype, void *out, int out_dtype, int64_t M,
                     int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                     void *workspace, size_t workspace_bytes, void *stream, size_t zero_area = kWorkspaceZeroBytes,
                     size_t scratch_cap = ~(size_t)0)
{
    if (M < 0 || N < 0 || K < 0) return MI355_ERR_BAD_ARGUMENT;
    if (out_dtype != MI355_OUT_BF16 && out_dtype != MI355_OUT_INT32 && out_dtype != MI355_OUT_FP16 && out_dtype != MI355_OUT_INT8)
        return MI355_ERR_BAD_ARGUMENT;
    const int out_i8 = out_dtype == MI355_OUT_INT8;
    if (out_i8 && (!qparam || pertoken_scale)) return MI355_ERR_BAD_ARGUMENT;
    if (out_i8 && bias_dtype != MI355_BIAS_NONE && bias_dtype != MI355_BIAS_INT32) return MI355_ERR_UNSUPPORTED;
    if (qparam && !aligned(qparam, 8)) return MI355_ERR_ALIGNMENT;
    if (bias_dtype < MI355_BIAS_NONE || bias_dtype > MI355_BIAS_FP32) return MI355_ERR_BAD_ARGUMENT;
    if ((bias != nullptr) != (bias_dtype != MI355_BIAS_NONE)) return MI355_ERR_BAD_ARGUMENT;
    if (M == 0 || N == 0) return MI355_OK;
    if (!out || ldc < N) return MI355_ERR_BAD_ARGUMENT;
    if (K > 0 && (!a || !b || lda < K)) return MI355_ERR_BAD_ARGUMENT;
    if (ldb_k != 1 && ldb_n != 1) return MI355_ERR_UNSUPPORTED;
    if (out_dtype != MI355_OUT_INT32 && ((!scale && !qparam) || (scale_len != 1 && scale_len != N))) return MI355_ERR_BAD_ARGUMENT;
    if (out_dtype == MI355_OUT_INT32 && bias_dtype != MI355_BIAS_NONE && bias_dtype != MI355_BIAS_INT32) return MI355_ERR_UNSUPPORTED;
    if (bias && !aligned(bias, bias_dtype == MI355_BIAS_BF16 ? 2 : 4)) return MI355_ERR_ALIGNMENT;
    if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return MI355_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int out_i32 = out_dtype == MI355_OUT_INT32;

    const int8_t *bt = b;
    int64_t ldbt = ldb_n;
    // the tiled kernel addresses a tile's rows with 32-bit buffer offsets: 256 rows of either operand must stay below 2^31
    const bool offsets_fit = (uint64_t)256 * (uint64_t)lda + (uint64_t)K < (1ull << 31) &&
                             (uint64_t)256 * (uint64_t)(ldb_k != 1 ? K : ldb_n) + (uint64_t)K < (1ull << 31);
    bool tiled = K >= BK && K % BK == 0 && (lda & 15) == 0 && aligned(a, 16) && offsets_fit;
    const QmmPlan pl = make_qmm_plan(M, N, K, ldb_k, ldb_n, zero_area, scratch_cap);
    char *ws = static_cast<char *>(workspace);
    if (tiled && pl.counter_bytes + pl.partial_bytes + pl.transpose_bytes > 0) {
        if (!ws || workspace_bytes < pl.counter_bytes + pl.partial_bytes + pl.transpose_bytes) return MI355_ERR_WORKSPACE;
        if (!aligned(ws, 16)) return MI355_ERR_ALIGNMENT;
    }
    if (tiled && ldb_k != 1) {
        // contiguous [K,N]: transpose once into the workspace
        int8_t *dst = reinterpret_cast<int8_t *>(ws + pl.counter_bytes + pl.partial_bytes);
        if ((N & 15) == 0 && (K & 15) == 0 && (ldb_k & 15) == 0 && aligned(b, 16) && aligned(dst, 16))
            hipLaunchKernelGGL(transpose_i8_wide_kernel, dim3((unsigned)((N + 127) / 128), (unsigned)((K + 127) / 128)),
                               dim3(256), 0, s, b, dst, (int)K, (int)N, ldb_k);
        else
            hipLaunchKernelGGL(transpose_i8_kernel, dim3((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64)), dim3(256), 0,
                               s, b, dst, (int)K, (int)N, ldb_k);
        bt = dst;
        ldbt = K;
    }
    tiled = tiled && (ldbt & 15) == 0 && aligned(bt, 16);
    if (tiled && knob(kKnobQmmSplit) == 0 && knob(kKnobQmmTile) == 0) {
        // at most 64 rows: the barrier-free kernel that splits K inside the workgroup (quant_matmul_decode.hip)
        QmmDecodeArgs d;
        d.a = a;
        d.bt = bt;
        d.pertoken = out_i32 ? nullptr : pertoken_scale;
        d.scale = out_i32 ? nullptr : scale;             // an int32 output takes no scales: empty descriptors
        d.qparam = out_i32 ? nullptr : qparam;
        d.bias = bias;
        d.bias_kind = bias_dtype;
        d.out_f16 = out_dtype == MI355_OUT_FP16;
        d.out_i8 = out_i8;
        d.out_i32 = out_i32;
        d.out = out;
        d.lda = lda;
        d.ldbt = ldbt;
        d.ldc = ldc;
        d.M = (int)M;
        d.N = (int)N;
        d.K = (int)K;
        d.scale_len = out_i32 ? 0 : (int)scale_len;
        const int st = launch_qmm_decode(d, s);
        if (st != MI355_ERR_UNSUPPORTED) return st;
    }
    if (!tiled) {
        hipLaunchKernelGGL(qmm_generic_kernel, dim3((unsigned)((N + 15) / 16), (unsigned)((M + 15) / 16)), dim3(256), 0, s,
                           a, b, pertoken_scale, scale, (int)scale_len, bias, bias_dtype, out_dtype == MI355_OUT_FP16 ? 1 : 0, out,
                           out_i32, qparam, out_i8, (int)M, (int)N, (int)K, lda, ldb_k, ldb_n, ldc);
        return check_launch();
    }

    QmmArgs p;
    p.a = a;
    p.bt = bt;
    p.pertoken = out_i32 ? nullptr : pertoken_scale;
    p.scale = scale;
    p.bias = bias;
    p.bias_kind = bias_dtype;
    p.out_f16 = out_dtype == MI355_OUT_FP16;
    p.out = out;
    p.lda = lda;
    p.ldbt = ldbt;
    p.ldc = ldc;
    p.M = (int)M;
    p.N = (int)N;
    p.K = (int)K;
    p.scale_len = (int)scale_len;
    p.out_i32 = out_i32;
    p.qparam = qparam;
    p.out_i8 = out_i8;
    // An output that the L2s could hold (8 x 4 MiB) would leave them only in the write-back at the end of the kernel, a
    // burst that nothing overlaps; streaming the rows out while other tiles still compute makes the launch 2.5 us
    // (1024x4096x11008) shorter and costs the next reader nothing (product + dynamic_quant of it: 60.1 -> 58.5 us).  A
    // larger output spills into the Infinity Cache during the kernel anyway, and a reader finds it there: non-temporal
    // stores would take that away (2048x4096x28672 followed by the fused SwiGLU + quantisation: +11 us), so it keeps
    // ordinary stores.  MI355_QMM_STREAM_OUT: 1 never, 2 always.
    {
        const int so = knob(kKnobQmmStreamOut);
        const uint64_t out_bytes = (uint64_t)M * (uint64_t)N * (out_i8 ? 1u : 2u);
        p.stream_out = so == 2 || (so != 1 && out_bytes <= kStreamOutMaxBytes);
    }
    const TileChoice c = pl.tile;
    p.S = pl.S;
    p.counter = pl.S > 1 ? reinterpret_cast<uint32_t *>(ws) : nullptr;
    p.partial = pl.S > 1 ? reinterpret_cast<int32_t *>(ws + pl.counter_bytes) : nullptr;
#ifdef MI355_QMM_TS
    p.ts = g_dbg_ts;
#endif
#define MI355_QMM_CASE(bm_, bn_, wgm_, wgn_)  \
    if (c.bm == bm_ && c.bn == bn_) return launch_qmm<wgm_, wgn_, bm_ / (16 * wgm_), bn_ / (16 * wgn_)>(p, s);
    MI355_QMM_CASE(256, 256, 2, 4)
    {
        const int lk = knob(kKnobQmmLoop);                 // 0: automatic; 1: the generic loop; 2, 3: the wide loop with refills in a block / spread; 4: see the planner
        if (lk != 1) {
            if (c.bm == 256 && c.bn == 224) {
                if (lk == 2) return launch_qmm<4, 2, 4, 7, 0, 1>(p, s);
                // the instantiation whose LDS-parameter epilogue serves this call's kind of bias and scale
                const bool to16 = !p.out_i32 && !p.out_i8;
                if (to16 && !p.qparam && (p.bias_kind == MI355_BIAS_INT32 || p.bias_kind == MI355_BIAS_FP32)) return launch_qmm<4, 2, 4, 7, 0, 2, 1>(p, s);
                if (to16 && p.qparam && !p.pertoken && (p.bias_kind == MI355_BIAS_NONE || p.bias_kind == MI355_BIAS_INT32)) return launch_qmm<4, 2, 4, 7, 0, 2, 2>(p, s);
                return launch_qmm<4, 2, 4, 7, 0, 2>(p, s);
            }
            if (c.bm == 256 && c.bn == 192) return lk == 2 ? launch_qmm<4, 2, 4, 6, 0, 1>(p, s) : launch_qmm<4, 2, 4, 6, 0, 2>(p, s);
        }
    }
    MI355_QMM_CASE(256, 224, 4, 2)
    MI355_QMM_CASE(256, 192, 4, 2)
    if (c.whole) {
        if (c.bm == 128 && c.bn == 192) return launch_qmm<2, 4, 4, 3, 3, 3>(p, s);
        if (c.bm == 128 && c.bn == 128) return launch_qmm<2, 4, 4, 2, 3, 3>(p, s);
        return MI355_ERR_UNSUPPORTED;
    }
    MI355_QMM_CASE(128, 320, 2, 4)
    MI355_QMM_CASE(128, 256, 2, 4)
    MI355_QMM_CASE(128, 192, 2, 4)
    MI355_QMM_CASE(128, 128, 2, 4)
    {
        // the 64-row tiles normally rely on two resident workgroups per CU to keep loads in flight; when the launch has
        // no second workgroup for a CU, one workgroup with a four-stage ring streams the weights instead
        const int64_t wgs = (int64_t)((p.M + c.bm - 1) / c.bm) * ((p.N + c.bn - 1) / c.bn) * p.S;
        const int dk = knob(kKnobQmmDeepOff);              // 1: neither; 2: the ring instead of the streaming loop
        const bool deep = wgs <= 256 && dk != 1;
        if (deep && c.bm == 64 && c.bn == 256) return launch_qmm<1, 8, 4, 2, 3>(p, s);
        if (deep && c.bm == 64 && c.bn == 128) return dk == 2 ? launch_qmm<1, 8, 4, 1, 4>(p, s) : launch_qmm<1, 8, 4, 1, -1>(p, s);
    }
    MI355_QMM_CASE(64, 256, 1, 8)
    MI355_QMM_CASE(64, 128, 1, 8)
#undef MI355_QMM_CASE
    return MI355_ERR_UNSUPPORTED;
}

} // namespace
} // namespace mi355

#ifdef MI355_QMM_TS
extern "C" void mi355_dbg_set_ts(unsigned long long *p) { mi355::g_dbg_ts = p; }
#endif

extern "C" int mi355_quant_matmul(const int8_t *a, const int8_t *b, const float *pertoken_scale, const float *scale,
                                  int64_t scale_len, const void *bias, int bias_dtype, void *out, int out_dtype, int64_t M,
                                  int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                                  void *workspace, size_t workspace_bytes, void *stream)
{
    if (out_dtype == MI355_OUT_INT8) return MI355_ERR_BAD_ARGUMENT;          // needs packed parameters
    return mi355::run_quant_matmul(a, b, pertoken_scale, scale, nullptr, scale_len, bias, bias_dtype, out, out_dtype, M, N, K,
                                   lda, ldb_k, ldb_n, ldc, workspace, workspace_bytes, stream);
}

extern "C" int mi355_quant_matmul_qparam(const int8_t *a, const int8_t *b, const uint64_t *qparam, int64_t qparam_len,
                                         const void *bias, int bias_dtype, void *out, int out_dtype, int64_t M, int64_t N,
                                         int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc, void *workspace,
                                         size_t workspace_bytes, void *stream)
{
    if (out_dtype == MI355_OUT_INT32) return MI355_ERR_BAD_ARGUMENT;         // an int32 result has no scale
    if (!qparam && M > 0 && N > 0) return MI355_ERR_BAD_ARGUMENT;
    return mi355::run_quant_matmul(a, b, nullptr, nullptr, qparam, qparam_len, bias, bias_dtype, out, out_dtype, M, N, K, lda,
                                   ldb_k, ldb_n, ldc, workspace, workspace_bytes, stream);
}

extern "C" int mi355_trans_quant_param(const float *scale, int64_t scale_len, const float *offset, int64_t offset_len,
                                       uint64_t *out, int64_t n, void *stream)
{
    using namespace mi355;
    if (n < 0 || scale_len < 0 || offset_len < 0) return MI355_ERR_BAD_ARGUMENT;
    if (n == 0) return MI355_OK;
    if (!scale || !out || (scale_len != 1 && scale_len != n)) return MI355_ERR_BAD_ARGUMENT;
    if (offset && offset_len != 1 && offset_len != n) return MI355_ERR_BAD_ARGUMENT;
    if (!aligned(scale, 4) || !aligned(out, 8) || (offset && !aligned(offset, 4))) return MI355_ERR_ALIGNMENT;
    hipLaunchKernelGGL(trans_quant_param_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), scale, scale_len == 1, offset, offset_len == 1, out, n);
    return check_launch();
}

// ---------------------------------------------------------------------------------------------------------------
// mi355_quant_matmul_noalloc: the same product for callers that cannot provide or allocate a workspace (code under
// HIP graph capture, serving loops and harnesses that forbid hipMalloc).  The workspace the kernels need (arrival
// counters, split-K partial sums, the transposed copy of a [K,N] weight) lives in a file-scope device array of
// fixed size; every GPU the library runs on holds its own copy until the process ends.
namespace mi355 {
namespace {

constexpr size_t kStaticScratchBytes = MI355_NOALLOC_SCRATCH_BYTES;
__device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

__global__ __launch_bounds__(256) void scratch_clear_kernel(uint32_t *p, int words)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < words) p[i] = 0u;
}

constexpr int kMaxDevices = 64;
struct DeviceScratch {
    void *ptr = nullptr;        // device address of this GPU's copy of `scratch`
    bool ready = false;
};
DeviceScratch g_scratch[kMaxDevices];
std::mutex g_scratch_mu;

// Device address of the current device's scratch array; on first use per device the address is resolved and the
// arrival counters are cleared by a small kernel on the caller's stream (a fill kernel, not a memset node, so that
// a caller who captures this first call records something that replays correctly).
int scratch_of_current_device(void **out, hipStream_t s)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MI355_ERR_LAUNCH;
    // the array's address is resolved for the current device: a stream of another device cannot use it
    if (s) {
        int sdev = -1;
        if (hipStreamGetDevice(s, &sdev) != hipSuccess) return MI355_ERR_LAUNCH;
        if (sdev != dev) return MI355_ERR_BAD_ARGUMENT;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    DeviceScratch &d = g_scratch[dev];
    if (!d.ptr) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return MI355_ERR_LAUNCH;
        d.ptr = ptr;
    }
    if (!d.ready) {
        // A __device__ array starts out zeroed and every launch leaves the counters zero, so this clear only guards
        // against a process that wrote to the array by other means.  While the stream is capturing the kernel is merely
        // recorded, so the array does not count as cleared until a call outside a capture has enqueued the clear.
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &capturing) != hipSuccess) return MI355_ERR_LAUNCH;
        hipLaunchKernelGGL(scratch_clear_kernel, dim3((unsigned)(kWorkspaceCounterCapacity / 4 / 256)), dim3(256), 0, s,
                           static_cast<uint32_t *>(d.ptr), (int)(kWorkspaceCounterCapacity / 4));
        if (check_launch() != MI355_OK) return MI355_ERR_LAUNCH;
        if (capturing == hipStreamCaptureStatusNone) d.ready = true;
    }
    *out = d.ptr;
    return MI355_OK;
}

} // namespace
} // namespace mi355

extern "C" int mi355_quant_matmul_noalloc(const int8_t *a, const int8_t *b, const float *pertoken_scale, const float *scale,
                                          int64_t scale_len, const void *bias, int bias_dtype, void *out, int out_dtype,
                                          int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n,
                                          int64_t ldc, void *stream)
{
    using namespace mi355;
    if (out_dtype == MI355_OUT_INT8) return MI355_ERR_BAD_ARGUMENT;
    if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffffff || N > 0x7fffffff)
        return run_quant_matmul(a, b, pertoken_scale, scale, nullptr, scale_len, bias, bias_dtype, out, out_dtype, M, N, K, lda,
                                ldb_k, ldb_n, ldc, nullptr, 0, stream);
    // the scratch array is private to this operator: the arrival counters are followed directly by the partial sums
    const QmmPlan pl = make_qmm_plan(M, N, K, ldb_k, ldb_n, kWorkspaceCounterCapacity, kStaticScratchBytes);
    const size_t need = pl.counter_bytes + pl.partial_bytes + pl.transpose_bytes;
    if (need > kStaticScratchBytes) return MI355_ERR_WORKSPACE;      // beyond the fixed scratch: use mi355_quant_matmul
    void *ws = nullptr;
    if (need > 0) {
        const int st = scratch_of_current_device(&ws, static_cast<hipStream_t>(stream));
        if (st != MI355_OK) return st;
    }
    return run_quant_matmul(a, b, pertoken_scale, scale, nullptr, scale_len, bias, bias_dtype, out, out_dtype, M, N, K, lda,
                            ldb_k, ldb_n, ldc, ws, need > 0 ? kStaticScratchBytes : 0, stream, kWorkspaceCounterCapacity, kStaticScratchBytes);
}

// One-time weight pre-layout for npu_quant_matmul: a contiguous [K,N] int8 weight is rewritten K-major ([N,K] storage),
// the layout the GEMM consumes without its per-call transposing pre-pass.
extern "C" int mi355_transpose_int8(const int8_t *src, int8_t *dst, int64_t K, int64_t N, int64_t ld_src, void *stream)
{
    using namespace mi355;
    if (K < 0 || N < 0 || ld_src < N) return MI355_ERR_BAD_ARGUMENT;
    if (K == 0 || N == 0) return MI355_OK;
    if (!src || !dst) return MI355_ERR_BAD_ARGUMENT;
    if (K > 0x7fffffff || N > 0x7fffffff) return MI355_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if ((N & 15) == 0 && (K & 15) == 0 && (ld_src & 15) == 0 && aligned(src, 16) && aligned(dst, 16))
        hipLaunchKernelGGL(transpose_i8_wide_kernel, dim3((unsigned)((N + 127) / 128), (unsigned)((K + 127) / 128)), dim3(256), 0, s,
                           src, dst, (int)K, (int)N, ld_src);
    else
        hipLaunchKernelGGL(transpose_i8_kernel, dim3((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64)), dim3(256), 0, s, src, dst,
                           (int)K, (int)N, ld_src);
    return check_launch();
}
