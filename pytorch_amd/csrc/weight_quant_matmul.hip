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
//   int8 : u = w ^ 0x80 = w + 128 in [0,255], converted with v_cvt_f32_ubyteN and packed to
//          bf16 (exact: 8 significant bits);  P = P' - 128 X.
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
// Streaming.  A workgroup owns a 128-byte-wide column strip of the weight (one cache line per
// row) and one chunk of K; its wavefronts split that chunk.  Each wavefront streams its own rows
// through a private LDS ring with direct-to-LDS buffer loads (16 bytes per lane, no register
// staging, up to D steps of 32 rows in flight) and synchronises with nothing but its own
// s_waitcnt counters, so the main loop has no barrier.  The activations of a step travel through
// the same ring.  Partial sums are reduced over the wavefronts in LDS; when K is split over
// several workgroups (to occupy all CUs when there are few strips) each workgroup writes its
// float32 partial to the workspace and the workgroup that arrives last at a per-strip counter
// adds them in chunk order, which keeps the result independent of scheduling.
#include "common.h"
#include <stdlib.h>
#include <type_traits>

namespace mi355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) void lds_void;

constexpr int kNumCU = 256;

struct WqArgs {
    const uint16_t *x;              // bf16 [M, K]
    const void *w;                  // weight rows, contiguous along N
    const uint16_t *scale;          // bf16 [G, N]
    const uint16_t *offset;         // bf16 [G, N] or null
    uint16_t *out;                  // bf16 [M, N]
    float *partial;                 // workspace [S][M][N] float32 (S > 1)
    uint32_t *counter;              // workspace [mchunks][strips], zero on entry, left zero
    int64_t ldx, ldo;
    uint32_t ldw_bytes;             // bytes between weight rows
    uint32_t row_bytes;             // valid bytes of a weight row
    int M, N, K;
    int unit_steps;                 // 32-row steps per scale group (per channel: 1)
    int n_units;                    // K / (32 * unit_steps)
    int grouped;                    // 0: one scale row for all K
    int strips, S;
};

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
template <int WBITS>
__device__ __forceinline__ void expand_pair(const uint32_t (&w)[8], int jb, uint32_t magic, u32x4 &b0, u32x4 &b1)
{
    if constexpr (WBITS == 4) {
        // `magic` (0x41004100) lives in a VGPR so that (x & mask) | magic is one v_and_or_b32 (mask from an SGPR)
        const uint32_t sel = 0x0c000c00u | ((4u + jb) << 16) | (uint32_t)jb;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const uint32_t t = __builtin_amdgcn_perm(w[2 * v + 1], w[2 * v], sel); // [byte jb of row 2v, 0, byte jb of row 2v+1, 0]
            b0[v] = ((t << 3) & 0x00780078u) | magic;                              // low nibble  -> element 2*jb
            b1[v] = ((t >> 1) & 0x00780078u) | magic;                              // high nibble -> element 2*jb+1
        }
    } else {
        (void)magic;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            b0[v] = pack_bf16x2((float)((w[2 * v] >> (16 * jb)) & 0xffu), (float)((w[2 * v + 1] >> (16 * jb)) & 0xffu));
            b1[v] = pack_bf16x2((float)((w[2 * v] >> (16 * jb + 8)) & 0xffu),
                                (float)((w[2 * v + 1] >> (16 * jb + 8)) & 0xffu));
        }
    }
}

template <int WBITS, int MT, int NWV, int D>
__global__ __launch_bounds__(NWV * 64) void wq_stream_kernel(const WqArgs p)
{
    constexpr int EPD = 32 / WBITS;            // elements per dword
    constexpr int NB = 32 * EPD;               // columns per strip (128 bytes of a weight row)
    constexpr int NT = 2 * EPD;                // MFMA column sets per lane (it holds 2 dword columns)
    constexpr int PB = NB * 4;                 // antiquant parameters of a group: NB scales + NB offsets, bf16
    constexpr int SLOT = 4096 + MT * 1024 + PB; // ring slot: 32 weight rows x 128 B, MT activation fragments, parameters
    constexpr int LOADS = 4 + MT;              // direct-to-LDS loads per step (one more on the first step of a group)
    constexpr float P_MUL = WBITS == 4 ? 2.0f : 1.0f;
    constexpr float X_BIAS = WBITS == 4 ? 24.0f : 128.0f;
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    // workgroups are dealt round-robin to the 8 XCDs: keep the S chunks of a strip on one XCD
    const int xcd_slot = blockIdx.x >> 3;
    const int strip = (blockIdx.x & 7) + 8 * (xcd_slot / p.S);
    const int chunk = xcd_slot % p.S;
    if (strip >= p.strips) return;
    const int m_base = blockIdx.y * (MT * 16);
    const int rows_valid = min(MT * 16, p.M - m_base);

    // contiguous range of K units for this (chunk, wavefront)
    const int R = p.S * NWV, r = chunk * NWV + wave;
    const int u0 = (int)((int64_t)p.n_units * r / R), u1 = (int)((int64_t)p.n_units * (r + 1) / R);
    const int step0 = u0 * p.unit_steps;
    const int nsteps = (u1 - u0) * p.unit_steps;

    const __amdgpu_buffer_rsrc_t rsrc_w =
        make_rsrc(static_cast<const char *>(p.w) + (size_t)strip * 128,
                  (uint32_t)((uint64_t)(p.K - 1) * p.ldw_bytes + p.row_bytes - (uint32_t)strip * 128u));
    const __amdgpu_buffer_rsrc_t rsrc_x =
        make_rsrc(p.x + (int64_t)m_base * p.ldx, (uint32_t)(((int64_t)(rows_valid - 1) * p.ldx + p.K) * 2));
    const uint32_t voff_w = (uint32_t)(lane >> 3) * p.ldw_bytes + (uint32_t)(lane & 7) * 16u;
    const uint32_t voff_x = (uint32_t)((c * (int)p.ldx + 8 * g) * 2);
    const uint32_t mt_stride_x = 16u * (uint32_t)p.ldx * 2u;

    // parameter load of a group: lanes [0, NB/8) fetch 16 bytes of the scale row each, the next NB/8 lanes the offset row
    constexpr int PL = NB / 8;
    const int pcol = strip * NB + (lane % PL) * 8;              // first of this lane's 8 parameter columns
    const bool p_lane = lane < 2 * PL && pcol < p.N && (lane < PL || p.offset != nullptr);
    const uint16_t *p_base = (lane < PL ? p.scale : p.offset) + pcol;

    // per channel there is a single parameter row: it travels with step 0 only
    auto group_first = [&](int s) { return p.grouped ? s % p.unit_steps == 0 : s == 0; };
    char *ring = lds + wave * (D * SLOT);
    auto issue = [&](int s) {
        char *slot = ring + (s % D) * SLOT;
        const uint32_t krow = (uint32_t)(step0 + s) * 32u;
        if (group_first(s) && p_lane) {
            const int grp = p.grouped ? u0 + s / p.unit_steps : 0;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(p_base + (int64_t)grp * p.N),
                                             (lds_void *)(slot + 4096 + MT * 1024), 16, 0, 0);
        }
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_void *)(slot + 4096 + mt * 1024), 16, voff_x,
                                                     krow * 2u + (uint32_t)mt * mt_stride_x, 0, 0);
#pragma unroll
        for (int u = 0; u < 4; u++)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_void *)(slot + u * 1024), 16, voff_w,
                                                     (krow + 8u * u) * p.ldw_bytes, 0, 0);
    };

    f32x4 tot[MT][NT], P[MT][NT], X[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        X[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < NT; i++) {
            tot[mt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
            P[mt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    const u32x4 ones = u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x41004100" : "=v"(magic));   // opaque to the optimiser: stays in a VGPR
    const int dwcol = strip * 32 + 2 * c;                      // first of this lane's two dword columns
    const int ncols_dw = (int)(p.row_bytes >> 2);
    const bool dw_ok[2] = {dwcol < ncols_dw, dwcol + 1 < ncols_dw};

    // Antiquant parameters of the current group: they arrive in the ring slot of the group's first step and are
    // copied to registers when that step is consumed.  Lane (c, g) owns columns (2c)*EPD .. (2c+2)*EPD-1.
    typedef typename std::conditional<EPD == 8, u32x4, u32x2>::type PV;
    PV sv[2], ov[2];
#pragma unroll
    for (int h = 0; h < 2; h++) sv[h] = PV{}, ov[h] = PV{};
    const bool has_offset = p.offset != nullptr;

    // fold one finished group: tot += (scale * P_MUL) * (P' + ((offset - X_BIAS) / P_MUL) * X); both rescalings are
    // exact (powers of two).  Only accumulator rows that exist are touched: lane (c, g) holds rows 4g + q.
    const bool one_row = MT == 1 && rows_valid == 1;
    auto fold = [&]() {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            if (!dw_ok[h]) continue;
#pragma unroll
            for (int i = 0; i < EPD; i++) {
                const float sc = ((i & 1) ? bf16_hi(sv[h][i / 2]) : bf16_lo(sv[h][i / 2])) * P_MUL;
                const float of = ((has_offset ? ((i & 1) ? bf16_hi(ov[h][i / 2]) : bf16_lo(ov[h][i / 2])) : 0.0f) - X_BIAS) *
                                 (1.0f / P_MUL);
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    const float inner0 = __builtin_fmaf(of, X[mt][0], P[mt][h * EPD + i][0]);
                    tot[mt][h * EPD + i][0] = __builtin_fmaf(sc, inner0, tot[mt][h * EPD + i][0]);
                    if (!one_row) {
#pragma unroll
                        for (int q = 1; q < 4; q++) {
                            const float inner = __builtin_fmaf(of, X[mt][q], P[mt][h * EPD + i][q]);
                            tot[mt][h * EPD + i][q] = __builtin_fmaf(sc, inner, tot[mt][h * EPD + i][q]);
                        }
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
    };

    const int pro = nsteps < D ? nsteps : D;
    for (int s = 0; s < pro; s++) issue(s);

    for (int s = 0; s < nsteps; s++) {
        // steps s+1 .. min(s+D-1, nsteps-1) may stay in flight; each has at least LOADS loads, so allowing
        // ahead * LOADS outstanding loads guarantees that everything of step s has landed
        const int ahead = min(D - 1, nsteps - 1 - s);
        if (ahead >= 3) wait_vmcnt<3 * LOADS>();
        else if (ahead == 2) wait_vmcnt<2 * LOADS>();
        else if (ahead == 1) wait_vmcnt<1 * LOADS>();
        else wait_vmcnt<0>();
        const char *slot = ring + (s % D) * SLOT;
        if (group_first(s)) {                 // first step of a group: take its parameters out of the slot
            const char *pp = slot + 4096 + MT * 1024 + (2 * c) * EPD * 2;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                sv[h] = *reinterpret_cast<const PV *>(pp + h * EPD * 2);
                ov[h] = *reinterpret_cast<const PV *>(pp + NB * 2 + h * EPD * 2);
            }
        }
        uint32_t w0[8], w1[8];
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const u32x2 v = *reinterpret_cast<const u32x2 *>(slot + (8 * g + t) * 128 + c * 8);
            w0[t] = v.x ^ (WBITS == 4 ? 0x88888888u : 0x80808080u);
            w1[t] = v.y ^ (WBITS == 4 ? 0x88888888u : 0x80808080u);
        }
        u32x4 xa[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) xa[mt] = *reinterpret_cast<const u32x4 *>(slot + 4096 + mt * 1024 + lane * 16);
        wait_lgkmcnt0();                      // the slot is in registers: it can be refilled
        if (s + D < nsteps) issue(s + D);

#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int jb = 0; jb < EPD / 2; jb++) {
                u32x4 b0, b1;
                expand_pair<WBITS>(h ? w1 : w0, jb, magic, b0, b1);
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    const bf16x8 a = __builtin_bit_cast(bf16x8, xa[mt]);
                    P[mt][h * EPD + 2 * jb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, b0),
                                                                                   P[mt][h * EPD + 2 * jb], 0, 0, 0);
                    P[mt][h * EPD + 2 * jb + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        a, __builtin_bit_cast(bf16x8, b1), P[mt][h * EPD + 2 * jb + 1], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
            X[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[mt]),
                                                            __builtin_bit_cast(bf16x8, ones), X[mt], 0, 0, 0);
        if (p.grouped && (s + 1) % p.unit_steps == 0) fold();
    }
    if (!p.grouped && nsteps > 0) fold();

    // ---- reduce over the wavefronts: red[wave][row][col], rows_valid rows of NB columns
    __syncthreads();                          // every ring is drained: LDS can be reused
    float *red = reinterpret_cast<float *>(lds);
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int row = mt * 16 + 4 * g + q;
            if (row >= rows_valid) continue;
            float *dst = red + ((size_t)wave * rows_valid + row) * NB + (2 * c) * EPD;
#pragma unroll
            for (int i = 0; i < NT; i++) dst[i] = tot[mt][i][q];
        }
    __syncthreads();
    // every thread owns quads of 4 consecutive columns of the [rows_valid x NB] tile
    constexpr int QPR = NB / 4;
    constexpr int THREADS = NWV * 64;
    const int n0 = strip * NB;
    const int nquads = rows_valid * QPR;
    constexpr size_t RED_BYTES = (size_t)NWV * MT * 16 * NB * sizeof(float);
    int &is_last = *reinterpret_cast<int *>(lds + RED_BYTES);   // just past the reduction buffer
    auto sum_waves = [&](int qd) {
        const int row = qd / QPR, nl = (qd % QPR) * 4;
        f32x4 acc = *reinterpret_cast<const f32x4 *>(red + ((size_t)0 * rows_valid + row) * NB + nl);
#pragma unroll
        for (int wv = 1; wv < NWV; wv++) acc += *reinterpret_cast<const f32x4 *>(red + ((size_t)wv * rows_valid + row) * NB + nl);
        return acc;
    };
    const bool out_vec = (p.ldo & 3) == 0 && aligned_dev(p.out, 8);
    auto store_out = [&](int qd, f32x4 v) {
        const int row = qd / QPR, nl = (qd % QPR) * 4;
        uint16_t *o = p.out + (int64_t)(m_base + row) * p.ldo + n0 + nl;
        if (out_vec) {
            u32x2 pk;
            pk.x = pack_bf16x2(v[0], v[1]);
            pk.y = pack_bf16x2(v[2], v[3]);
            *reinterpret_cast<u32x2 *>(o) = pk;
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = f32_to_bf16(v[i]);
        }
    };
    if (p.S == 1) {
        for (int qd = threadIdx.x; qd < nquads; qd += THREADS)
            if (n0 + (qd % QPR) * 4 < p.N) store_out(qd, sum_waves(qd));
        return;
    }
    // K split over S workgroups: publish this chunk's partial, the last arrival adds them in chunk order.
    // The exchange uses agent-scope (sc1) write-through stores and cache-bypassing loads, ordered by the
    // wavefronts' own store counters, the workgroup barrier and a relaxed agent-scope counter; a full
    // release/acquire fence would write back and invalidate the whole L2 of the XCD, which costs far
    // more than the kernel itself.
    constexpr int SC1 = 16;                   // cache-policy bit: agent scope
    const uint32_t chunk_bytes = (uint32_t)p.M * (uint32_t)p.N * 4u;
    const __amdgpu_buffer_rsrc_t rsrc_p = make_rsrc(p.partial, chunk_bytes * (uint32_t)p.S);
    auto quad_off = [&](int qd) {
        const int row = qd / QPR, nl = (qd % QPR) * 4;
        return (uint32_t)(((m_base + row) * p.N + n0 + nl) * 4);
    };
    for (int qd = threadIdx.x; qd < nquads; qd += THREADS) {
        if (n0 + (qd % QPR) * 4 >= p.N) continue;
        const f32x4 v = sum_waves(qd);
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rsrc_p, quad_off(qd), (uint32_t)chunk * chunk_bytes, SC1);
    }
    wait_vmcnt<0>();                          // this wavefront's partial sums have reached the coherence point
    __syncthreads();
    uint32_t *cnt = p.counter + (size_t)blockIdx.y * p.strips + strip;
    if (threadIdx.x == 0) {
        const uint32_t old = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = old == (uint32_t)(p.S - 1);
    }
    __syncthreads();
    if (!is_last) return;
    for (int qd = threadIdx.x; qd < nquads; qd += THREADS) {
        if (n0 + (qd % QPR) * 4 >= p.N) continue;
        const uint32_t off = quad_off(qd);
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int ch = 0; ch < p.S; ch += 4) {
            // four loads in flight; chunks past S fall outside the buffer and read as zero
            f32x4 v[4];
#pragma unroll
            for (int i = 0; i < 4; i++)
                v[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_p, off, (uint32_t)(ch + i) * chunk_bytes, SC1));
#pragma unroll
            for (int i = 0; i < 4; i++) acc += v[i];
        }
        store_out(qd, acc);
    }
    if (threadIdx.x == 0) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // ready for the next launch
}

// Any layout (including K-major int8 weights, i.e. the transposed view of an [N,K] tensor),
// any alignment: one thread per output element, golden operation order.
__global__ __launch_bounds__(256) void wq_generic_kernel(const uint16_t *__restrict__ x, const void *__restrict__ w,
                                                         int w_bits, const uint16_t *__restrict__ scale,
                                                         const uint16_t *__restrict__ offset,
                                                         uint16_t *__restrict__ out, int M, int N, int K, int group,
                                                         int64_t ldx, int64_t ldw_k, int64_t ldw_n, int64_t ldo)
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
            const uint32_t word = static_cast<const uint32_t *>(w)[(int64_t)k * ldw_k + (n >> 3)];
            const int v = (int)((word >> (4 * (n & 7))) & 0xfu);
            wv = (float)((v ^ 8) - 8);
        }
        if (offset) wv = wv + bf16_1(offset[(int64_t)gidx * N + n]);
        wv = wv * bf16_1(scale[(int64_t)gidx * N + n]);
        acc = acc + bf16_1(x[(int64_t)m * ldx + k]) * wv;
    }
    out[(int64_t)m * ldo + n] = f32_to_bf16(acc);
}

struct WqPlan {
    bool fast;
    int mt, nwv;        // m tiles per workgroup, wavefronts per workgroup
    int strips, mchunks, S;
    int unit_steps, n_units;
    size_t partial_bytes, counter_bytes;
};

WqPlan make_plan(int64_t M, int64_t N, int64_t K, int w_bits, int64_t group_size, bool n_major, int64_t ldw_k,
                 int64_t ldx, const void *x, const void *w)
{
    WqPlan pl{};
    const int64_t row_bytes = w_bits == 4 ? N / 2 : N;
    const int64_t ldw_bytes = w_bits == 4 ? ldw_k * 4 : ldw_k;
    const int64_t group = group_size > 0 ? group_size : K;
    pl.fast = K > 0 && K % 32 == 0 && group % 32 == 0 && n_major && row_bytes % 16 == 0 && ldw_bytes % 16 == 0 &&
              ldx % 8 == 0 && (x == nullptr || aligned(x, 16)) && (w == nullptr || aligned(w, 16)) &&
              (uint64_t)K * (uint64_t)ldw_bytes < (1ull << 32) && (uint64_t)M * (uint64_t)ldx * 2 < (1ull << 32);
    if (!pl.fast) return pl;
    pl.mt = M <= 16 ? 1 : 2;
    pl.nwv = pl.mt == 1 ? 8 : 4;
    pl.strips = (int)((row_bytes + 127) / 128);
    pl.mchunks = (int)((M + pl.mt * 16 - 1) / (pl.mt * 16));
    const bool grouped = group_size > 0 && group != K;
    pl.unit_steps = grouped ? (int)(group / 32) : 1;
    pl.n_units = (int)(K / (32 * pl.unit_steps));
    // split K over S workgroups until all CUs have work; every wavefront keeps at least one unit
    int S = kNumCU / (pl.strips * pl.mchunks);
    const int s_max = pl.n_units / pl.nwv;
    if (S > s_max) S = s_max;
    if (S > 16) S = 16;
    if (S < 1) S = 1;
    if (const char *e = getenv("MI355_WQ_SPLIT")) { // debugging aid: force the number of K chunks
        const int f = atoi(e);
        if (f >= 1 && f <= s_max) S = f;
    }
    if ((uint64_t)S * (uint64_t)M * (uint64_t)N * 4 >= (1ull << 32)) S = 1; // exchange offsets are 32-bit
    pl.S = S;
    pl.partial_bytes = S > 1 ? (size_t)S * M * N * sizeof(float) : 0;
    pl.counter_bytes = S > 1 ? (((size_t)pl.strips * pl.mchunks * sizeof(uint32_t)) + 255) / 256 * 256 : 0;
    return pl;
}

template <int WBITS, int MT, int NWV>
int launch_stream(const WqArgs &p, const WqPlan &pl, hipStream_t s)
{
    constexpr int EPD = 32 / WBITS, NB = 32 * EPD, SLOT = 4096 + MT * 1024 + NB * 4;
    constexpr int D = (160 * 1024) / (NWV * SLOT) >= 4 ? 4 : (160 * 1024) / (NWV * SLOT);   // ring depth that fits LDS
    static_assert(D >= 2, "ring depth");
    constexpr size_t ring_bytes = (size_t)NWV * D * SLOT;
    constexpr size_t red_bytes = (size_t)NWV * MT * 16 * NB * sizeof(float);
    constexpr size_t lds_bytes = ring_bytes > red_bytes + 16 ? ring_bytes : red_bytes + 16;
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");
    auto kern = wq_stream_kernel<WBITS, MT, NWV, D>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)((pl.strips + 7) / 8 * 8 * pl.S), (unsigned)pl.mchunks), dim3(NWV * 64), lds_bytes, s,
                       p);
    return check_launch();
}

} // namespace
} // namespace mi355

extern "C" size_t mi355_weight_quant_matmul_workspace(int64_t M, int64_t N, int64_t K, int w_bits, int64_t group_size)
{
    using namespace mi355;
    if (M <= 0 || N <= 0 || K <= 0 || (w_bits != 4 && w_bits != 8) || group_size < 0) return 0;
    // the largest request over the layouts the streaming kernel accepts (row pitch = row length)
    const WqPlan pl = make_plan(M, N, K, w_bits, group_size, true, w_bits == 4 ? N / 8 : N, K, nullptr, nullptr);
    return pl.fast ? pl.partial_bytes + pl.counter_bytes : 0;
}

extern "C" int mi355_weight_quant_matmul(const void *x_bf16, const void *w, int w_bits, const void *scale_bf16,
                                         const void *offset_bf16, void *out_bf16, int64_t M, int64_t N, int64_t K,
                                         int64_t group_size, int64_t ldx, int64_t ldw_k, int64_t ldw_n, int64_t ldo,
                                         void *workspace, size_t workspace_bytes, void *stream)
{
    using namespace mi355;
    if (M < 0 || N < 0 || K < 0 || group_size < 0) return MI355_ERR_BAD_ARGUMENT;
    if (w_bits != 8 && w_bits != 4) return MI355_ERR_BAD_ARGUMENT;
    if (M == 0 || N == 0) return MI355_OK;
    if (!out_bf16 || ldo < N) return MI355_ERR_BAD_ARGUMENT;
    if (K > 0 && (!x_bf16 || !w || !scale_bf16 || ldx < K)) return MI355_ERR_BAD_ARGUMENT;
    if (w_bits == 4 && (N % 8 != 0 || ldw_k < N / 8)) return MI355_ERR_BAD_ARGUMENT;
    if (w_bits == 8 && ldw_k != 1 && ldw_n != 1) return MI355_ERR_UNSUPPORTED;
    if (group_size > 0 && (K % group_size != 0)) return MI355_ERR_BAD_ARGUMENT;
    if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return MI355_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int group = (int)(group_size > 0 ? group_size : (K > 0 ? K : 1));

    const bool n_major = w_bits == 4 || (ldw_n == 1 && ldw_k >= N);
    const WqPlan pl = make_plan(M, N, K, w_bits, group_size, n_major, ldw_k, ldx, x_bf16, w);
    if (!pl.fast) {
        hipLaunchKernelGGL(wq_generic_kernel, dim3((unsigned)((N + 63) / 64), (unsigned)((M + 3) / 4)), dim3(256), 0, s,
                           static_cast<const uint16_t *>(x_bf16), w, w_bits, static_cast<const uint16_t *>(scale_bf16),
                           static_cast<const uint16_t *>(offset_bf16), static_cast<uint16_t *>(out_bf16), (int)M, (int)N,
                           (int)K, group, ldx, ldw_k, ldw_n, ldo);
        return check_launch();
    }
    if (pl.S > 1) {
        if (!workspace || workspace_bytes < pl.partial_bytes + pl.counter_bytes) return MI355_ERR_WORKSPACE;
        if (!aligned(workspace, 16)) return MI355_ERR_ALIGNMENT;
    }

    WqArgs p;
    p.x = static_cast<const uint16_t *>(x_bf16);
    p.w = w;
    p.scale = static_cast<const uint16_t *>(scale_bf16);
    p.offset = static_cast<const uint16_t *>(offset_bf16);
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
    p.S = pl.S;
    if (w_bits == 4) return pl.mt == 1 ? launch_stream<4, 1, 8>(p, pl, s) : launch_stream<4, 2, 4>(p, pl, s);
    return pl.mt == 1 ? launch_stream<8, 1, 8>(p, pl, s) : launch_stream<8, 2, 4>(p, pl, s);
}
