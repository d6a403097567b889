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
// Weight images (chosen so the expansion is a couple of bit operations per pair of weights):
//   int8 : u = w ^ 0x80 = w + 128 in [0,255], converted with v_cvt_f32_ubyteN and packed to
//          bf16 (exact: 8 significant bits);  P = P' - 128 X.
//   int4 : nibble ^ 8 = w + 8 = u in [0,15] is placed in mantissa bits 3..6 of the bf16
//          pattern 0x4100, i.e. the value 8 + u/2 = (w + 24) / 2;  P = 2 P' - 24 X.
//
// Mapping.  The packed weight row is contiguous along N, while an MFMA operand lane wants 8
// consecutive k of ONE column.  A lane therefore loads the same dword column from 8 different
// k rows and one MFMA is issued per byte/nibble position: MFMA #i covers the columns
// { elems_per_dword * (j0 + c) + i : c = 0..15 }, a strided set, which only changes the index
// bookkeeping of the epilogue.  The order of k inside a lane's operand is free as long as the
// activation operand uses the same order.
//
// A workgroup owns a strip of 16 dword columns; its wavefronts split K and reduce through
// LDS in a fixed order (deterministic).
#include "common.h"

namespace mi355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int NWV = 8;              // wavefronts per workgroup (K split)

struct WqArgs {
    const uint16_t *x;              // bf16 [M, K]
    const uint32_t *w;              // dwords: int4 -> [K, N/8], int8 -> [K, N/4]
    const uint16_t *scale;          // bf16 [G, N]
    const uint16_t *offset;         // bf16 [G, N] or null
    uint16_t *out;                  // bf16 [M, N]
    int64_t ldx, ldw, ldo;          // ldw in dwords
    int M, N, K;
    int group;                      // K for per-channel
    int ncols_dw;                   // dword columns per row (N/8 or N/4)
};

template <int WBITS>
__device__ __forceinline__ void expand(const uint32_t (&w)[8], int i, u32x4 &b)
{
    // B fragment of MFMA #i: VGPR v holds (k slot 2v, k slot 2v+1) = rows (2v, 2v+1) of this lane's 8 rows
    if constexpr (WBITS == 4) {
        const int jb = i >> 1;
        const uint32_t sel = 0x0c000c00u | ((4u + jb) << 16) | (uint32_t)jb;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const uint32_t t = __builtin_amdgcn_perm(w[2 * v + 1], w[2 * v], sel);
            const uint32_t sh = (i & 1) ? (t >> 1) : (t << 3);
            b[v] = (sh & 0x00780078u) | 0x41004100u;
        }
    } else {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const float lo = (float)((w[2 * v] >> (8 * i)) & 0xffu);
            const float hi = (float)((w[2 * v + 1] >> (8 * i)) & 0xffu);
            b[v] = pack_bf16x2(lo, hi);
        }
    }
}

template <int WBITS, int MT>
__global__ __launch_bounds__(NWV * 64) void wq_strip_kernel(const WqArgs p)
{
    constexpr int EPD = 32 / WBITS;          // elements per dword = MFMAs per k-step
    constexpr int NS = 16 * EPD;             // columns per strip
    constexpr float P_MUL = WBITS == 4 ? 2.0f : 1.0f;
    constexpr float X_BIAS = WBITS == 4 ? 24.0f : 128.0f;
    extern __shared__ float red[];           // [NWV][MT*16][NS]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int j = blockIdx.x * 16 + c;       // this lane's dword column
    const bool col_ok = j < p.ncols_dw;
    const int m_base = blockIdx.y * (MT * 16);

    // K units (groups) dealt contiguously to the wavefronts
    const int n_groups = p.K / p.group;
    const int gpw = (n_groups + NWV - 1) / NWV;
    // per-channel: the "group" is the whole K; split it in k-steps of 32 instead
    const bool per_channel = n_groups == 1;
    const int steps_total = p.K / 32;
    const int spw = (steps_total + NWV - 1) / NWV;

    int grp_begin, grp_end;
    if (per_channel) {
        grp_begin = 0;
        grp_end = 1;
    } else {
        grp_begin = min(wave * gpw, n_groups);
        grp_end = min(grp_begin + gpw, n_groups);
    }

    f32x4 tot[MT][EPD];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int i = 0; i < EPD; i++) tot[mt][i] = f32x4{0.f, 0.f, 0.f, 0.f};

    const u32x4 ones = u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};

    for (int grp = grp_begin; grp < grp_end; grp++) {
        int ks_begin, ks_end;
        if (per_channel) {
            ks_begin = min(wave * spw, steps_total);
            ks_end = min(ks_begin + spw, steps_total);
        } else {
            ks_begin = grp * (p.group / 32);
            ks_end = ks_begin + p.group / 32;
        }
        f32x4 P[MT][EPD], X[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            X[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < EPD; i++) P[mt][i] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll 2
        for (int ks = ks_begin; ks < ks_end; ks++) {
            const int kb = ks * 32 + 8 * g;
            uint32_t w[8];
#pragma unroll
            for (int t = 0; t < 8; t++) {
                uint32_t v = col_ok ? __builtin_nontemporal_load(p.w + (int64_t)(kb + t) * p.ldw + j) : 0u;
                w[t] = v ^ (WBITS == 4 ? 0x88888888u : 0x80808080u);
            }
            u32x4 xa[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const int m = m_base + mt * 16 + c;
                xa[mt] = m < p.M ? *reinterpret_cast<const u32x4 *>(p.x + (int64_t)m * p.ldx + kb) : u32x4{0, 0, 0, 0};
            }
#pragma unroll
            for (int i = 0; i < EPD; i++) {
                u32x4 b;
                expand<WBITS>(w, i, b);
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
                    P[mt][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[mt]),
                                                                       __builtin_bit_cast(bf16x8, b), P[mt][i], 0, 0, 0);
            }
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
                X[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[mt]),
                                                                __builtin_bit_cast(bf16x8, ones), X[mt], 0, 0, 0);
        }
        // fold the group: tot += scale * (P_MUL * P' + (offset - X_BIAS) * X)
        if (col_ok && ks_end > ks_begin) {
            const int64_t pbase = (int64_t)grp * p.N + (int64_t)j * EPD;
#pragma unroll
            for (int i = 0; i < EPD; i++) {
                const float sc = bf16_1(p.scale[pbase + i]);
                // a wavefront that holds only part of a per-channel K range must not add the offset twice:
                // the offset term is linear in X, so each wavefront adds it for its own X.
                const float of = (p.offset ? bf16_1(p.offset[pbase + i]) : 0.0f) - X_BIAS;
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const float inner = __builtin_fmaf(of, X[mt][r], P_MUL * P[mt][i][r]);
                        tot[mt][i][r] = __builtin_fmaf(sc, inner, tot[mt][i][r]);
                    }
            }
        }
    }

    // reduce over the wavefronts through LDS: red[wave][m][n_local], n_local = c * EPD + i
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int i = 0; i < EPD; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int ml = mt * 16 + 4 * g + r;
                red[(wave * (MT * 16) + ml) * NS + c * EPD + i] = tot[mt][i][r];
            }
    __syncthreads();
    const int n0 = blockIdx.x * NS;
    for (int e = threadIdx.x; e < MT * 16 * NS; e += NWV * 64) {
        const int ml = e / NS, nl = e % NS;
        const int m = m_base + ml, n = n0 + nl;
        if (m >= p.M || n >= p.N) continue;
        float s = 0.0f;
#pragma unroll
        for (int wv = 0; wv < NWV; wv++) s += red[(wv * (MT * 16) + ml) * NS + nl];
        p.out[(int64_t)m * p.ldo + n] = f32_to_bf16(s);
    }
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

template <int WBITS, int MT>
int launch_strip(const WqArgs &p, hipStream_t s)
{
    constexpr int EPD = 32 / WBITS, NS = 16 * EPD;
    constexpr size_t lds_bytes = (size_t)NWV * MT * 16 * NS * sizeof(float);
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");
    auto kern = wq_strip_kernel<WBITS, MT>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    const unsigned strips = (unsigned)((p.ncols_dw + 15) / 16);
    const unsigned mchunks = (unsigned)((p.M + MT * 16 - 1) / (MT * 16));
    hipLaunchKernelGGL(kern, dim3(strips, mchunks), dim3(NWV * 64), lds_bytes, s, p);
    return check_launch();
}

} // namespace
} // namespace mi355

extern "C" size_t mi355_weight_quant_matmul_workspace(int64_t M, int64_t N, int64_t K, int w_bits, int64_t group_size)
{
    (void)M;
    (void)N;
    (void)K;
    (void)w_bits;
    (void)group_size;
    return 0;
}

extern "C" int mi355_weight_quant_matmul(const void *x_bf16, const void *w, int w_bits, const void *scale_bf16,
                                         const void *offset_bf16, void *out_bf16, int64_t M, int64_t N, int64_t K,
                                         int64_t group_size, int64_t ldx, int64_t ldw_k, int64_t ldw_n, int64_t ldo,
                                         void *workspace, size_t workspace_bytes, void *stream)
{
    using namespace mi355;
    (void)workspace;
    (void)workspace_bytes;
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

    const bool n_major = w_bits == 4 || (ldw_n == 1 && N % 4 == 0 && ldw_k % 4 == 0);
    const bool fast = K > 0 && K % 32 == 0 && group % 32 == 0 && n_major && aligned(w, 4) && aligned(x_bf16, 16) &&
                      ldx % 8 == 0;
    if (!fast) {
        hipLaunchKernelGGL(wq_generic_kernel, dim3((unsigned)((N + 63) / 64), (unsigned)((M + 3) / 4)), dim3(256), 0, s,
                           static_cast<const uint16_t *>(x_bf16), w, w_bits, static_cast<const uint16_t *>(scale_bf16),
                           static_cast<const uint16_t *>(offset_bf16), static_cast<uint16_t *>(out_bf16), (int)M, (int)N,
                           (int)K, group, ldx, ldw_k, ldw_n, ldo);
        return check_launch();
    }

    WqArgs p;
    p.x = static_cast<const uint16_t *>(x_bf16);
    p.w = static_cast<const uint32_t *>(w);
    p.scale = static_cast<const uint16_t *>(scale_bf16);
    p.offset = static_cast<const uint16_t *>(offset_bf16);
    p.out = static_cast<uint16_t *>(out_bf16);
    p.ldx = ldx;
    p.ldw = w_bits == 4 ? ldw_k : ldw_k / 4;
    p.ldo = ldo;
    p.M = (int)M;
    p.N = (int)N;
    p.K = (int)K;
    p.group = group;
    p.ncols_dw = (int)(w_bits == 4 ? N / 8 : N / 4);
    if (w_bits == 4) return M <= 16 ? launch_strip<4, 1>(p, s) : launch_strip<4, 2>(p, s);
    return M <= 16 ? launch_strip<8, 1>(p, s) : launch_strip<8, 2>(p, s);
}
