// npu_weight_quant_batchmatmul for decode-sized batches of int8 weights stored [N, K] (the transposed view that
// torch_npu's LinearWeightQuant passes, torch_npu/contrib/module/linear_weight_quant.py:106), one scale / offset per
// output column, at most 32 activation rows.
//
// The structure is that of the decode kernel of npu_quant_matmul (quant_matmul_decode.hip): a workgroup of eight
// wavefronts owns strips of 16 weight rows (= 16 output columns) over the whole of K, wavefront w the w-th eighth of K; at
// most one workgroup per CU, workgroup b walks over strips b, b + 256, ... with its ring of weight loads running across
// strip boundaries; weights arrive as whole cache lines (lane l: 16 bytes of row l / 8 and of row 8 + l / 8 of a 128-byte
// step) and are turned into MFMA operand order through a private swizzled LDS tile; the wavefront's slice of the
// activations is loaded once, turned around the same way and kept in registers for all strips; the eight partial sums of
// a strip meet in LDS (two areas in turn, one barrier per strip) and the first wavefronts write it out while the others go
// on.  No split of K over workgroups, no workspace, no barrier in front of the data.
//
// Arithmetic as in the other weight-only kernels: the MFMA multiplies the activations by the integer weight, which is an
// exact bf16 / fp16 number, and  out = scale * (P + offset * X) + bias  in float32 with P the sum of products and X the
// sum of the row's activations (formed once per launch: it does not depend on the strip), then one rounding.
#include "weight_quant_common.h"
#include "weight_quant_kmajor_decode.h"

namespace mi355 {
namespace {

constexpr int kStep = 128;                      // weight bytes (= k) per step: four MFMAs of 32
constexpr int kMaxWorkgroups = 256;

// MT tiles of 16 activation rows; NS (even) steps per wavefront and strip, PF of them in flight; ACT 0 bf16, 1 fp16.
template <int MT, int NS, int PF, int ACT>
__global__ __launch_bounds__(512) void wq_kmajor_decode_kernel(const WqKmDecodeArgs p)
{
    static_assert(NS % 2 == 0 && NS % PF == 0 && PF % 2 == 0, "static ring slots and LDS buffer parities");
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int KT = p.K / kStep;
    const int s0 = KT * wave / 8, ns = KT * (wave + 1) / 8 - s0;          // this wavefront's steps (at most NS)
    const int strips = (p.N + 15) / 16;
    const int my_strips = (strips - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;

    const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(p.w, (uint32_t)((int64_t)(p.N - 1) * p.ldw + p.K));
    const __amdgpu_buffer_rsrc_t rsrc_x = make_rsrc(p.x, (uint32_t)(((int64_t)(p.M - 1) * p.ldx + p.K) * 2));
    const __amdgpu_buffer_rsrc_t rsrc_sc = make_rsrc(p.scale, (uint32_t)p.N * 2u);
    const __amdgpu_buffer_rsrc_t rsrc_of = make_rsrc(p.offset, p.offset ? (uint32_t)p.N * 2u : 0u);
    const __amdgpu_buffer_rsrc_t rsrc_bias = make_rsrc(p.bias, p.bias ? (uint32_t)p.N * 2u : 0u);
    uint32_t voff_w[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int rl = 8 * h + (lane >> 3);
        voff_w[h] = (uint32_t)(rl * (int)p.ldw + (((lane & 7) ^ ((rl >> 1) & 7)) * 16));
    }
    const int t_rd = c * 128 + ((g ^ ((c >> 1) & 7)) * 16);               // piece g of row c; piece g + 4 is at slot ^ 4
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    constexpr int kWaveBytes = 4096 + 4096;                               // two weight buffers, one activation step
    char *const tb = lds + wave * kWaveBytes;
    float *const red = reinterpret_cast<float *>(lds + 8 * kWaveBytes);   // [parity][wavefront][tile][lane][4]
    float *const xsum = red + 2 * 8 * MT * 256;                           // [wavefront][tile][lane][4]

    // The wavefront's slice of the activations, once: a step is 16 rows x 256 bytes; an instruction loads four whole
    // rows (lane l: 16 bytes of row 4 i + l / 16), the step goes through LDS, and lane (c, g) reads for MFMA t the
    // 8 k at 64 (t / 2) + 16 g + 8 (t % 2) of row c.
    u32x4 xf[NS][MT][4];
#pragma unroll
    for (int j = 0; j < NS; j++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = mt * 16 + 4 * i + (lane >> 4);
                xf[j][mt][i] = __builtin_amdgcn_raw_buffer_load_b128(
                    rsrc_x, j < ns && row < p.M ? (uint32_t)((row * (int)p.ldx) * 2 + (lane & 15) * 16) : kOutOfRange,
                    (uint32_t)(s0 + j) * (kStep * 2), 0);
            }

    // weights: flat step f = strip index * NS + step; ring slot f % PF, LDS buffer f % 2
    u32x4 wr[PF][2];
    auto load_w = [&](int slot, int t, int st) {
        const bool ok = t < my_strips && st < ns;
        const uint32_t so = (uint32_t)(((int)blockIdx.x + t * (int)gridDim.x) * 16) * (uint32_t)p.ldw + (uint32_t)(s0 + st) * kStep;
#pragma unroll
        for (int h = 0; h < 2; h++) wr[slot][h] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, ok ? voff_w[h] : kOutOfRange, so, kNonTemporal);
    };
    auto to_lds_w = [&](int slot, int buf) {
        char *dst = tb + buf * 2048 + lane * 16;
#pragma unroll
        for (int h = 0; h < 2; h++) *reinterpret_cast<u32x4 *>(dst + h * 1024) = wr[slot][h];
    };
#pragma unroll
    for (int r = 0; r < PF; r++) load_w(r, r / NS, r % NS);

    // turn the activation steps around (a wavefront's LDS operations complete in order) and add up the rows
    const u32x4 ones = u32x4{kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>, kOnes2<ACT>};
    f32x4 X[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) X[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < NS; j++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            char *xb = tb + 4096;
#pragma unroll
            for (int i = 0; i < 4; i++) *reinterpret_cast<u32x4 *>(xb + i * 1024 + lane * 16) = xf[j][mt][i];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                xf[j][mt][t] = *reinterpret_cast<const u32x4 *>(xb + c * 256 + ((t >> 1) * 8 + 2 * g + (t & 1)) * 16);
                X[mt] = mfma_act<ACT>(xf[j][mt][t], ones, X[mt]);
            }
        }
    // every wavefront's row sums meet once: lane (c, g) of the accumulator holds rows 4 g + q (the same for every column)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) *reinterpret_cast<f32x4 *>(xsum + ((wave * MT + mt) * 64 + lane) * 4) = X[mt];

    // wavefront t < MT finishes tile t of every strip: lane l writes row l / 4, columns 4 (l % 4) .. + 3
    const bool finisher = wave < MT;
    const int er = lane >> 2, ec = (lane & 3) * 4;
    const int em = wave * 16 + er;
    // accumulator element (row 4 g + q, column c) lies at float index (c + 16 g) * 4 + q of a wavefront's tile
    const int e_idx = (16 * (er >> 2)) * 4 + (er & 3);                    // + 4 * column
    float xtot = 0.0f;
    bool xtot_ready = false;

    to_lds_w(0, 0);
    for (int t = 0; t < my_strips; t++) {
        const int n0 = ((int)blockIdx.x + t * (int)gridDim.x) * 16;
        const int en = n0 + ec;
        // antiquantisation parameters of this strip (wavefronts that finish no tile get an out-of-range offset: no branch
        // around loads)
        const uint32_t po = finisher && en < p.N ? (uint32_t)en * 2u : kOutOfRange;
        const u32x2 scq = __builtin_amdgcn_raw_buffer_load_b64(rsrc_sc, po, 0, 0);
        const u32x2 ofq = __builtin_amdgcn_raw_buffer_load_b64(rsrc_of, po, 0, 0);
        const u32x2 bq = __builtin_amdgcn_raw_buffer_load_b64(rsrc_bias, po, 0, 0);

        f32x4 P[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) P[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < NS; j++) {
            const char *src = tb + (j & 1) * 2048;
            const u32x4 w0 = *reinterpret_cast<const u32x4 *>(src + t_rd);
            const u32x4 w1 = *reinterpret_cast<const u32x4 *>(src + (t_rd ^ 64));
            to_lds_w((j + 1) % PF, (j + 1) & 1);                          // the next step's registers take the other buffer
            __builtin_amdgcn_sched_barrier(0);
            load_w(j % PF, t + (j + PF) / NS, (j + PF) % NS);             // this step's registers are free again
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t lo = q < 2 ? w0[2 * (q & 1)] : w1[2 * (q & 1)], hi = q < 2 ? w0[2 * (q & 1) + 1] : w1[2 * (q & 1) + 1];
                u32x4 b;
                b[0] = pack_act2<ACT>(sbyte_f32(lo, 0), sbyte_f32(lo, 1));
                b[1] = pack_act2<ACT>(sbyte_f32(lo, 2), sbyte_f32(lo, 3));
                b[2] = pack_act2<ACT>(sbyte_f32(hi, 0), sbyte_f32(hi, 1));
                b[3] = pack_act2<ACT>(sbyte_f32(hi, 2), sbyte_f32(hi, 3));
#pragma unroll
                for (int mt = 0; mt < MT; mt++) P[mt] = mfma_act<ACT>(xf[j][mt][q], b, P[mt]);
            }
        }

        float *const rd = red + (t & 1) * (8 * MT * 256);
#pragma unroll
        for (int mt = 0; mt < MT; mt++) *reinterpret_cast<f32x4 *>(rd + ((wave * MT + mt) * 64 + lane) * 4) = P[mt];
        __syncthreads();
        if (finisher) {
            if (!xtot_ready) {                                            // behind the first barrier every row sum is there
#pragma unroll
                for (int w = 0; w < 8; w++) xtot += xsum[(w * MT + wave) * 256 + e_idx];
                xtot_ready = true;
            }
            float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < 8; w++)
#pragma unroll
                for (int i = 0; i < 4; i++) sum[i] += rd[(w * MT + wave) * 256 + e_idx + 4 * (ec + i)];
            if (em < p.M && en < p.N) {
                float f[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float sc = (i & 1) ? act_hi<ACT>(scq[i >> 1]) : act_lo<ACT>(scq[i >> 1]);
                    const float of = p.offset ? ((i & 1) ? act_hi<ACT>(ofq[i >> 1]) : act_lo<ACT>(ofq[i >> 1])) : 0.0f;
                    float v = sc * __builtin_fmaf(of, xtot, sum[i]);
                    if (p.bias) v = v + ((i & 1) ? act_hi<ACT>(bq[i >> 1]) : act_lo<ACT>(bq[i >> 1]));
                    f[i] = v;
                }
                u32x2 pk;
                pk.x = pack_act2<ACT>(f[0], f[1]);
                pk.y = pack_act2<ACT>(f[2], f[3]);
                *reinterpret_cast<u32x2 *>(p.out + (int64_t)em * p.ldo + en) = pk;
            }
        }
    }
}

template <int MT, int NS, int ACT>
int launch(const WqKmDecodeArgs &p, hipStream_t s)
{
    constexpr int lds_bytes = 8 * 8192 + 2 * 8 * MT * 1024 + 8 * MT * 1024;
    auto kern = wq_kmajor_decode_kernel<MT, NS, 4, ACT>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    const int strips = (p.N + 15) / 16;
    hipLaunchKernelGGL(kern, dim3((unsigned)(strips < kMaxWorkgroups ? strips : kMaxWorkgroups)), dim3(512), lds_bytes, s, p);
    return check_launch();
}

template <int ACT>
int launch_act(const WqKmDecodeArgs &p, hipStream_t s)
{
    const int ns = (p.K / kStep + 7) / 8;
    if (p.M <= 16) return ns <= 4 ? launch<1, 4, ACT>(p, s) : launch<1, 8, ACT>(p, s);
    return launch<2, 4, ACT>(p, s);
}

} // namespace

bool wq_kmajor_decode_shape(int64_t M, int64_t N, int64_t K, int64_t group_size)
{
    if (knob(kKnobWqDecodeOff) == 1 || knob(kKnobWqSplit) != 0) return false;
    if (group_size > 0 && group_size != K) return false;                  // one scale per column
    if (M < 1 || M > 32 || K % kStep != 0 || K < 8 * kStep || N < 2048 || N % 4 != 0) return false;
    // the activations of a wavefront's eighth of K stay in registers: 8 steps with one tile of 16 rows, 4 with two
    const int64_t steps = (K / kStep + 7) / 8;
    return M <= 16 ? steps <= 8 : steps <= 4;
}

int launch_wq_kmajor_decode(const WqKmDecodeArgs &p, int act_f16, hipStream_t s)
{
    if (!wq_kmajor_decode_shape(p.M, p.N, p.K, 0)) return MI355_ERR_UNSUPPORTED;
    if ((p.ldw & 15) != 0 || p.ldw < p.K || !aligned(p.w, 16) || (p.ldx & 7) != 0 || !aligned(p.x, 16)) return MI355_ERR_UNSUPPORTED;
    if ((p.ldo & 3) != 0 || !aligned(p.out, 8) || !aligned(p.scale, 8) || (p.offset && !aligned(p.offset, 8)) ||
        (p.bias && !aligned(p.bias, 8)))
        return MI355_ERR_UNSUPPORTED;
    if ((uint64_t)(p.N + 16) * (uint64_t)p.ldw + (uint64_t)p.K >= (1ull << 31) ||
        ((uint64_t)p.M * (uint64_t)p.ldx + (uint64_t)p.K) * 2 >= (1ull << 31))
        return MI355_ERR_UNSUPPORTED;
    return act_f16 ? launch_act<1>(p, s) : launch_act<0>(p, s);
}

} // namespace mi355
