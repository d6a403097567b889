// npu_weight_quant_batchmatmul for decode-sized batches of int4 weights packed along K (storage [N, K/8] int32, the
// layout torch_npu's LinearWeightQuant passes as a transposed view, torch_npu/contrib/module/linear_weight_quant.py:71,106)
// with scale groups of 128, at most 32 activation rows.
//
// The structure is that of the other decode kernels (quant_matmul_decode.hip, weight_quant_kmajor_decode.hip): a
// workgroup of eight wavefronts owns strips of weight rows (= output columns) over the whole of K, wavefront w the w-th
// eighth of K; at most one workgroup per CU walks over strips b, b + 256, ... with its ring of weight loads running
// across strip boundaries; weights arrive as whole cache lines and are turned into MFMA operand order through a private
// swizzled LDS tile; the wavefront's slice of the activations is loaded once and kept in registers, and so are its row
// sums per scale group; the partial sums of a strip meet in LDS (two areas in turn, one barrier per strip) and the first
// wavefronts write it out while the others go on.  No split of K over workgroups, no workspace.
//
// A step is 128 bytes of a weight row = 256 k = two scale groups.  Lane (c, g) gets bytes [16 g, 16 g + 16) of both
// 64-byte halves of row c: four words of eight nibbles each, one MFMA per word, so MFMA d of half h multiplies the k
// at 128 h + 32 g + 8 d .. + 7.  The nibbles of a word are expanded to the exact images of weight_quant_common.h in the
// order 0,2,4,6,1,3,5,7 and the activation fragments are kept in the same order.  Per group:
// out += scale_g * (2 P_g + (offset_g - 24) * X_g)  (bf16; fp16: P_g + (offset_g - 24) X_g), as in weight_quant_kpacked.hip.
#include "weight_quant_common.h"
#include "weight_quant_kpacked_decode.h"

namespace mi355 {
namespace {

constexpr int kStep = 128;                      // weight bytes per row and step: 256 k
constexpr int kMaxWorkgroups = 256;

// eight nibbles (already XORed with 8: u = w + 8) -> eight 16-bit images in the order 0,2,4,6,1,3,5,7
template <int ACT>
__device__ __forceinline__ u32x4 expand_word(uint32_t v)
{
    u32x4 b;
    if constexpr (ACT == 0) {
        const uint32_t e = (v << 3) & 0x78787878u, o = (v >> 1) & 0x78787878u;
        b[0] = __builtin_amdgcn_perm(0x41414141u, e, 0x04010400u);
        b[1] = __builtin_amdgcn_perm(0x41414141u, e, 0x04030402u);
        b[2] = __builtin_amdgcn_perm(0x41414141u, o, 0x04010400u);
        b[3] = __builtin_amdgcn_perm(0x41414141u, o, 0x04030402u);
    } else {
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

// MT tiles of 16 activation rows; NS steps per wavefront and column tile, NT column tiles of 16 per strip (NS * NT steps
// per strip), PF steps in flight; ACT 0 bf16, 1 fp16.
template <int MT, int NS, int NT, int PF, int ACT>
__global__ __launch_bounds__(512) void wq_kpacked_decode_kernel(const WqKpDecodeArgs p)
{
    constexpr int FS = NS * NT;                                           // flat steps per strip
    static_assert(FS % PF == 0 && PF % 2 == 0, "static ring slots and LDS buffer parities");
    constexpr int NG = 2 * NS;                                            // scale groups of a wavefront
    static_assert(NG == 4 || NG == 8, "parameters travel in lane groups of four");
    constexpr float P_MUL = kImageMul<4, ACT>, X_BIAS = kImageBias<4>;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int KT = p.K / (2 * kStep);
    const int s0 = KT * wave / 8, ns = KT * (wave + 1) / 8 - s0;          // this wavefront's steps (at most NS)
    const int strips = (p.N + 16 * NT - 1) / (16 * NT);
    const int my_strips = (strips - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;

    const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(p.w, (uint32_t)((int64_t)(p.N - 1) * p.ldw_bytes + p.K / 2));
    const __amdgpu_buffer_rsrc_t rsrc_x = make_rsrc(p.x, (uint32_t)(((int64_t)(p.M - 1) * p.ldx + p.K) * 2));
    const int n_groups = p.K / 128;
    const uint32_t prm_bytes = (uint32_t)(((int64_t)(n_groups - 1) * p.ld_param_g + (int64_t)(p.N - 1) * p.ld_param_n + 1) * 2);
    const __amdgpu_buffer_rsrc_t rsrc_sc = make_rsrc(p.scale, prm_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_of = make_rsrc(p.offset, p.offset ? prm_bytes : 0u);
    const __amdgpu_buffer_rsrc_t rsrc_bias = make_rsrc(p.bias, p.bias ? (uint32_t)p.N * 2u : 0u);
    uint32_t voff_w[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int rl = 8 * h + (lane >> 3);
        voff_w[h] = (uint32_t)rl * p.ldw_bytes + (uint32_t)(((lane & 7) ^ ((rl >> 1) & 7)) * 16);
    }
    const int t_rd = c * 128 + ((g ^ ((c >> 1) & 7)) * 16);               // piece g of row c; piece g + 4 is at slot ^ 4
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    char *const tb = lds + wave * 4096;                                   // two weight buffers of 2 KiB
    char *const shared = lds + 8 * 4096;                                  // activation turn-around first, then the sums
    float *const red = reinterpret_cast<float *>(shared);                 // [parity][wavefront][column tile][lane][4]

    // The wavefront's slice of the activations, once: a step is 16 rows x 512 bytes; an instruction loads two whole rows
    // (lane l: 16 bytes of row 2 i + l / 32), the step goes through LDS, and lane (c, g) reads for MFMA d of half h the
    // 8 k at 128 h + 32 g + 8 d of row c, even elements first.  All of the loads are requested before the first weights,
    // so one memory round trip covers both (the counter of outstanding loads runs in order).
    u32x4 xl[NS][MT][8];
#pragma unroll
    for (int j = 0; j < NS; j++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int row = mt * 16 + 2 * i + (lane >> 5);
                xl[j][mt][i] = __builtin_amdgcn_raw_buffer_load_b128(
                    rsrc_x, j < ns && row < p.M ? (uint32_t)((row * (int)p.ldx) * 2 + (lane & 31) * 16) : kOutOfRange,
                    (uint32_t)(s0 + j) * (4 * kStep), 0);
            }

    // weights: flat step f = strip index * FS + column tile * NS + step; ring slot f % PF, LDS buffer f % 2
    u32x4 wr[PF][2];
    auto load_w = [&](int slot, int t, int f) {
        const int nt = f / NS, st = f % NS;
        const bool ok = t < my_strips && st < ns;
        const uint32_t so = (uint32_t)((((int)blockIdx.x + t * (int)gridDim.x) * NT + nt) * 16) * p.ldw_bytes + (uint32_t)(s0 + st) * kStep;
#pragma unroll
        for (int h = 0; h < 2; h++) wr[slot][h] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, ok ? voff_w[h] : kOutOfRange, so, kNonTemporal);
    };
    auto to_lds_w = [&](int slot, int buf) {
        char *dst = tb + buf * 2048 + lane * 16;
#pragma unroll
        for (int h = 0; h < 2; h++) *reinterpret_cast<u32x4 *>(dst + h * 1024) = wr[slot][h];
    };
    // antiquantisation parameters of a strip: lane (c, g) holds (scale, offset) of column c and of this wavefront's
    // groups g (and g + 4); at the fold of group j every lane fetches its column's pair from lane (c, j % 4)
    auto load_params = [&](int t, uint32_t (&prm)[NT][NG / 4]) {
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
#pragma unroll
            for (int r = 0; r < NG / 4; r++) {
                const int col = min((((int)blockIdx.x + t * (int)gridDim.x) * NT + nt) * 16 + c, p.N - 1);
                const int grp = 2 * s0 + 4 * r + g;
                const bool ok = t < my_strips && grp < n_groups;
                const uint32_t off = ok ? (uint32_t)(((int64_t)grp * p.ld_param_g + (int64_t)col * p.ld_param_n) * 2) : kOutOfRange;
                const uint32_t s16 = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc_sc, off, 0, 0);
                const uint32_t o16 = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc_of, off, 0, 0);
                prm[nt][r] = s16 | (o16 << 16);
            }
    };
#pragma unroll
    for (int r = 0; r < PF; r++) load_w(r, r / FS, r % FS);
    uint32_t prm_next[NT][NG / 4];
    load_params(0, prm_next);

    // turn the activations around while the first weights are on their way
    u32x4 xf[NS][MT][2][4];
    f32x4 Xg[NS][MT][2];
    const u32x4 ones = u32x4{kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>};
    {
        char *xb = shared + wave * 8192;
#pragma unroll
        for (int j = 0; j < NS; j++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
#pragma unroll
            for (int i = 0; i < 8; i++) *reinterpret_cast<u32x4 *>(xb + i * 1024 + lane * 16) = xl[j][mt][i];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                Xg[j][mt][h] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    xf[j][mt][h][d] = even_odd(*reinterpret_cast<const u32x4 *>(xb + c * 512 + (16 * h + 4 * g + d) * 16));
                    Xg[j][mt][h] = mfma_act<ACT>(xf[j][mt][h][d], ones, Xg[j][mt][h]);
                }
            }
        }
    }


    // wavefront f < NT * MT finishes tile (column tile f / MT, row tile f % MT) of every strip: lane l writes row l / 4,
    // columns 4 (l % 4) .. + 3
    const bool finisher = wave < NT * MT;
    const int fnt = wave / MT, fmt = wave % MT;
    const int er = lane >> 2, ec = (lane & 3) * 4;
    const int em = fmt * 16 + er;
    const int e_idx = (16 * (er >> 2)) * 4 + (er & 3);                    // accumulator element (row, column 0) of a tile

    __syncthreads();                                                      // every wavefront is done with its activation tile
    to_lds_w(0, 0);
    for (int t = 0; t < my_strips; t++) {
        uint32_t prm[NT][NG / 4];
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
#pragma unroll
            for (int r = 0; r < NG / 4; r++) prm[nt][r] = prm_next[nt][r];
        load_params(t + 1, prm_next);
        const int en = (((int)blockIdx.x + t * (int)gridDim.x) * NT + fnt) * 16 + ec;
        const u32x2 bq = __builtin_amdgcn_raw_buffer_load_b64(rsrc_bias, finisher && en < p.N ? (uint32_t)en * 2u : kOutOfRange, 0, 0);

        f32x4 tot[NT][MT];
#pragma unroll
        for (int f = 0; f < FS; f++) {
            const int nt = f / NS, j = f % NS;
            if (j == 0) {
#pragma unroll
                for (int mt = 0; mt < MT; mt++) tot[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            const char *src = tb + (f & 1) * 2048;
            const u32x4 w0 = *reinterpret_cast<const u32x4 *>(src + t_rd) ^ 0x88888888u;          // nibbles u = w + 8
            const u32x4 w1 = *reinterpret_cast<const u32x4 *>(src + (t_rd ^ 64)) ^ 0x88888888u;
            to_lds_w((f + 1) % PF, (f + 1) & 1);                          // the next step's registers take the other buffer
            __builtin_amdgcn_sched_barrier(0);
            load_w(f % PF, t + (f + PF) / FS, (f + PF) % FS);             // this step's registers are free again
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int h = 0; h < 2; h++) {
                f32x4 P[MT];
#pragma unroll
                for (int mt = 0; mt < MT; mt++) P[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    const u32x4 b = expand_word<ACT>(h ? w1[d] : w0[d]);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) P[mt] = mfma_act<ACT>(xf[j][mt][h][d], b, P[mt]);
                }
                const int gl = 2 * j + h;                                 // group of this half among the wavefront's
                const uint32_t pr = (uint32_t)__builtin_amdgcn_ds_bpermute((c + 16 * (gl & 3)) * 4, (int)prm[nt][gl >> 2]);
                const float sc = act_lo<ACT>(pr) * P_MUL;
                const float of = ((p.offset ? act_hi<ACT>(pr) : 0.0f) - X_BIAS) * (1.0f / P_MUL);
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int q = 0; q < 4; q++) tot[nt][mt][q] = __builtin_fmaf(sc, __builtin_fmaf(of, Xg[j][mt][h][q], P[mt][q]), tot[nt][mt][q]);
            }
        }

        float *const rd = red + (t & 1) * (8 * NT * MT * 256);
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) *reinterpret_cast<f32x4 *>(rd + (((wave * NT + nt) * MT + mt) * 64 + lane) * 4) = tot[nt][mt];
        __syncthreads();
        if (finisher) {
            float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < 8; w++)
#pragma unroll
                for (int i = 0; i < 4; i++) sum[i] += rd[(w * NT * MT + wave) * 256 + e_idx + 4 * (ec + i)];
            if (em < p.M && en < p.N) {
                if (p.bias) {
#pragma unroll
                    for (int i = 0; i < 4; i++) sum[i] = sum[i] + ((i & 1) ? act_hi<ACT>(bq[i >> 1]) : act_lo<ACT>(bq[i >> 1]));
                }
                u32x2 pk;
                pk.x = pack_act2<ACT>(sum[0], sum[1]);
                pk.y = pack_act2<ACT>(sum[2], sum[3]);
                *reinterpret_cast<u32x2 *>(p.out + (int64_t)em * p.ldo + en) = pk;
            }
        }
    }
}

template <int MT, int NS, int NT, int PF, int ACT>
int launch(const WqKpDecodeArgs &p, hipStream_t s)
{
    constexpr int lds_bytes = 8 * 4096 + 8 * 8192;                        // weight tiles, activation tiles (later: the sums)
    static_assert(2 * 8 * NT * MT * 1024 <= 8 * 8192, "the sums fit where the activation tiles were");
    auto kern = wq_kpacked_decode_kernel<MT, NS, NT, PF, ACT>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    const int strips = (p.N + 16 * NT - 1) / (16 * NT);
    hipLaunchKernelGGL(kern, dim3((unsigned)(strips < kMaxWorkgroups ? strips : kMaxWorkgroups)), dim3(512), lds_bytes, s, p);
    return check_launch();
}

template <int ACT>
int launch_act(const WqKpDecodeArgs &p, hipStream_t s)
{
    const int ns = (p.K / (2 * kStep) + 7) / 8;
    if (p.M > 16) return launch<2, 2, 1, 2, ACT>(p, s);
    if (ns > 2) return launch<1, 4, 1, 4, ACT>(p, s);
    // strips of 32 columns keep four steps in flight across strips; when strips of 16 give every workgroup at most one,
    // they fill twice as many CUs (4096 x 4096 at one row: 7.5 -> 6.4 us; with several strips per workgroup the deeper
    // ring wins: 4096 x 28672 16.1 against 18.9 us)
    return p.N <= 16 * kMaxWorkgroups ? launch<1, 2, 1, 2, ACT>(p, s) : launch<1, 2, 2, 4, ACT>(p, s);
}

} // namespace

bool wq_kpacked_decode_shape(int64_t M, int64_t N, int64_t K, int64_t group_size)
{
    if (knob(kKnobWqDecodeOff) == 1 || knob(kKnobWqSplit) != 0) return false;
    if (group_size != 128) return false;
    if (M < 1 || M > 32 || K % (2 * kStep) != 0 || K < 8 * 2 * kStep || N < 2048 || N % 4 != 0) return false;
    // the activations of a wavefront's eighth of K stay in registers: at most four steps of 256 k with one tile of 16
    // rows, two with two
    return (K / (2 * kStep) + 7) / 8 <= (M <= 16 ? 4 : 2);
}

int launch_wq_kpacked_decode(const WqKpDecodeArgs &p, int act_f16, hipStream_t s)
{
    if (!wq_kpacked_decode_shape(p.M, p.N, p.K, 128)) return MI355_ERR_UNSUPPORTED;
    if ((p.ldw_bytes & 15) != 0 || (int64_t)p.ldw_bytes < p.K / 2 || !aligned(p.w, 16) || (p.ldx & 7) != 0 || !aligned(p.x, 16))
        return MI355_ERR_UNSUPPORTED;
    if ((p.ldo & 3) != 0 || !aligned(p.out, 8) || !aligned(p.scale, 2) || (p.offset && !aligned(p.offset, 2)) || (p.bias && !aligned(p.bias, 8)))
        return MI355_ERR_UNSUPPORTED;
    if (p.ld_param_g < 0 || p.ld_param_n < 0) return MI355_ERR_UNSUPPORTED;
    const uint64_t prm_span = ((uint64_t)(p.K / 128 - 1) * (uint64_t)p.ld_param_g + (uint64_t)(p.N - 1) * (uint64_t)p.ld_param_n + 1) * 2;
    if ((uint64_t)(p.N + 32) * (uint64_t)p.ldw_bytes + (uint64_t)p.K / 2 >= (1ull << 31) ||
        ((uint64_t)p.M * (uint64_t)p.ldx + (uint64_t)p.K) * 2 >= (1ull << 31) || prm_span >= (1ull << 31))
        return MI355_ERR_UNSUPPORTED;
    return act_f16 ? launch_act<1>(p, s) : launch_act<0>(p, s);
}

} // namespace mi355
