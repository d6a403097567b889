// npu_quant_matmul for decode-sized batches on gfx950: int8 [M,K] x int8 weight stored [N,K], few rows; bf16, fp16, re-quantised int8 or int32 output.
//
// With so few rows the operator is a stream of the weight from HBM, and what the tiled kernel spends around that stream
// (an activation staging barrier before the first weight byte is used, a split of K over workgroups with partial sums and
// arrival counters in memory, a second round of loads in the workgroup that arrives last) is as long as the stream itself
// for the projection sizes of a transformer layer.  Here nothing stands between the launch and the data:
//   * a workgroup of eight wavefronts owns 16 weight rows (= 16 output columns) over the whole of K; wavefront w owns the
//     w-th eighth of K, so K is split inside the workgroup and the only exchange is one pass through LDS;
//   * a wavefront loads whole cache lines - lane l takes 16 bytes of row l / 8 (and of row 8 + l / 8) of a 128-byte step,
//     of the weight and of each tile of 16 activation rows alike (the latter come from the L2) - and turns each step
//     around through a private, XOR-swizzled LDS tile into MFMA operand order (lane (c, g): bytes 16 g.. and 64 + 16 g..
//     of row c).  Loading in operand order directly needs no LDS but puts four different rows in front of the address
//     coalescer every cycle: 3.3 TB/s instead of 6;
//   * a wavefront's LDS operations complete in order, so the turn-around needs no barrier; PF steps are in flight per
//     wavefront from the first instructions on, and a step past the end of the wavefront's range gets an out-of-range
//     lane offset (zeros, no memory traffic), so the loop has no branch around its loads;
//   * dequantisation parameters are requested before the weights and wait in registers.
// Integer accumulation makes the result independent of the split; the epilogue is the tiled kernel's, operation for
// operation: ((float(acc + int32 bias) * pertoken[m]) * scale[n]) + bias[n], each operation rounded to float32, then one
// rounding to the output type; or clamp(rint((acc + int32 bias) * scale[n] + offset[n])) for an int8 output, acc + int32 bias for an int32 one.
#include "common.h"
#include "quant_matmul_decode.h"

namespace mi355 {
namespace {

typedef int32_t i32x4v __attribute__((ext_vector_type(4)));
constexpr uint32_t kOutOfRange = 0x80000000u;   // lane offset beyond every buffer size: the load returns zero, no traffic
constexpr int kStep = 128;                      // bytes of K per step: two MFMAs of 64
constexpr int kMaxWorkgroups = 256;             // one per CU; a workgroup walks over strips b, b + 256, ...

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

// The offset of a packed quantisation parameter, from its high word: bits 37-45 of the 64, a 9-bit two's-complement integer.
__device__ __forceinline__ float qparam_hi_offset(uint32_t hi) { return (float)(((int32_t)((hi >> 5) << 23)) >> 23); }

// MT tiles of 16 activation rows; NS (even) steps of 128 bytes of K per wavefront and strip, PF of them in flight.
template <int MT, int NS, int PF>
__global__ __launch_bounds__(512) void qmm_decode_kernel(const QmmDecodeArgs p)
{
    static_assert(NS % 2 == 0 && NS % PF == 0 && PF % 2 == 0, "static ring slots and LDS buffer parities");
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int KT = p.K / kStep;
    const int s0 = KT * wave / 8, ns = KT * (wave + 1) / 8 - s0;          // this wavefront's steps (at most NS)
    const int strips = (p.N + 15) / 16;
    const int my_strips = (strips - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;   // strips b, b + grid, ...

    const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(p.bt, (uint32_t)((int64_t)(p.N - 1) * p.ldbt + p.K));
    const __amdgpu_buffer_rsrc_t rsrc_x = make_rsrc(p.a, (uint32_t)((int64_t)(p.M - 1) * p.lda + p.K));
    // per-channel factors: float32 words, or the low halves of 64-bit packed parameters
    const uint32_t sc_elem = p.qparam ? 8u : 4u;
    const __amdgpu_buffer_rsrc_t rsrc_sc = make_rsrc(p.qparam ? static_cast<const void *>(p.qparam) : static_cast<const void *>(p.scale), (uint32_t)p.scale_len * sc_elem);
    const uint32_t bias_elem = p.bias_kind == MI355_BIAS_BF16 ? 2u : 4u;
    const __amdgpu_buffer_rsrc_t rsrc_bias = make_rsrc(p.bias, p.bias ? (uint32_t)p.N * bias_elem : 0u);
    // lane l of half h loads row 8 h + l / 8, and the 16-byte piece that belongs in slot l % 8 of that row's swizzled
    // LDS image: piece (l % 8) ^ ((row / 2) % 8).  Weight rows past N lie beyond the descriptor's range.
    uint32_t voff_w[2], voff_x[MT][2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int rl = 8 * h + (lane >> 3);
        const int piece = ((lane & 7) ^ ((rl >> 1) & 7)) * 16;
        voff_w[h] = (uint32_t)(rl * (int)p.ldbt + piece);
#pragma unroll
        for (int mt = 0; mt < MT; mt++) voff_x[mt][h] = mt * 16 + rl < p.M ? (uint32_t)((mt * 16 + rl) * (int)p.lda + piece) : kOutOfRange;
    }
    const int t_rd = c * 128 + ((g ^ ((c >> 1) & 7)) * 16);               // piece g of row c; piece g + 4 is at slot ^ 4
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    constexpr int kWaveBytes = 4096 + MT * 2048;                          // two weight buffers, one activation buffer per tile
    char *const tb = lds + wave * kWaveBytes;
    i32x4v *const red = reinterpret_cast<i32x4v *>(lds + 8 * kWaveBytes); // [parity][wavefront][tile][lane]

    // The wavefront's slice of the activations, once, in operand order: every strip multiplies the same fragments.
    i32x4v xf[NS][MT][2];
#pragma unroll
    for (int j = 0; j < NS; j++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int h = 0; h < 2; h++)
                xf[j][mt][h] = __builtin_bit_cast(i32x4v, __builtin_amdgcn_raw_buffer_load_b128(
                    rsrc_x, j < ns ? voff_x[mt][h] : kOutOfRange, (uint32_t)(s0 + j) * kStep, 0));

    // weights: flat step f = strip index * NS + step; ring slot f % PF, LDS buffer f % 2
    i32x4v wr[PF][2];
    auto load_w = [&](int slot, int t, int st) {
        const bool ok = t < my_strips && st < ns;
        const uint32_t so = (uint32_t)(((int)blockIdx.x + t * (int)gridDim.x) * 16) * (uint32_t)p.ldbt + (uint32_t)(s0 + st) * kStep;
#pragma unroll
        for (int h = 0; h < 2; h++)
            wr[slot][h] = __builtin_bit_cast(i32x4v, __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, ok ? voff_w[h] : kOutOfRange, so, 2));
    };
    auto to_lds_w = [&](int slot, int buf) {
        char *dst = tb + buf * 2048 + lane * 16;
#pragma unroll
        for (int h = 0; h < 2; h++) *reinterpret_cast<i32x4v *>(dst + h * 1024) = wr[slot][h];
    };
#pragma unroll
    for (int r = 0; r < PF; r++) load_w(r, r / NS, r % NS);

    // per-token scales do not depend on the strip: wavefront t < MT finishes tile t of every strip
    const bool finisher = wave < MT;
    const int em = wave * 16 + c;
    const float ps = p.pertoken && finisher ? p.pertoken[min(em, p.M - 1)] : 1.0f;
    const float sc_one = p.scale_len != 1 ? 0.0f : p.qparam ? __uint_as_float((uint32_t)p.qparam[0]) : p.scale ? p.scale[0] : 0.0f;

    // turn the activation fragments around (a wavefront's LDS operations complete in order)
#pragma unroll
    for (int j = 0; j < NS; j++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            char *xb = tb + 4096 + mt * 2048;
#pragma unroll
            for (int h = 0; h < 2; h++) *reinterpret_cast<i32x4v *>(xb + h * 1024 + lane * 16) = xf[j][mt][h];
#pragma unroll
            for (int h = 0; h < 2; h++) xf[j][mt][h] = *reinterpret_cast<const i32x4v *>(xb + (t_rd ^ (64 * h)));
        }

    const uint32_t of_one = p.scale_len == 1 && p.qparam ? (uint32_t)(p.qparam[0] >> 32) : 0u;
    const bool has_ps = p.pertoken != nullptr;
    const bool has_bias = p.bias_kind == MI355_BIAS_BF16 || p.bias_kind == MI355_BIAS_FP32;
    to_lds_w(0, 0);
    for (int t = 0; t < my_strips; t++) {
        const int n0 = ((int)blockIdx.x + t * (int)gridDim.x) * 16;
        const int en = n0 + 4 * g;
        // dequantisation parameters of this strip, requested before its last weights are (wavefronts that finish no tile
        // get an out-of-range offset: no branch around loads)
        const uint32_t pn = finisher && en < p.N ? (uint32_t)en : kOutOfRange / 4;
        const uint32_t sc_off = p.scale_len == 1 || pn >= kOutOfRange / 4 ? kOutOfRange : pn * sc_elem;
        u32x4 scq = __builtin_amdgcn_raw_buffer_load_b128(rsrc_sc, sc_off, 0, 0);
        u32x4 ofq = u32x4{0u, 0u, 0u, 0u};                                // the high words: the offset of an int8 output
        if (p.qparam) {                                                   // columns 0, 1 | 2, 3: low words apart from high
            const u32x4 hi = __builtin_amdgcn_raw_buffer_load_b128(rsrc_sc, sc_off == kOutOfRange ? kOutOfRange : sc_off + 16u, 0, 0);
            ofq = u32x4{scq[1], scq[3], hi[1], hi[3]};
            scq = u32x4{scq[0], scq[2], hi[0], hi[2]};
        }
        const u32x4 bq = __builtin_amdgcn_raw_buffer_load_b128(rsrc_bias, bias_elem == 4u ? pn * 4u : kOutOfRange, 0, 0);
        const u32x2 bh = __builtin_amdgcn_raw_buffer_load_b64(rsrc_bias, bias_elem == 2u ? pn * 2u : kOutOfRange, 0, 0);

        i32x4v acc[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[mt] = i32x4v{0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < NS; j++) {
            const char *src = tb + (j & 1) * 2048;
            i32x4v wf[2];
#pragma unroll
            for (int h = 0; h < 2; h++) wf[h] = *reinterpret_cast<const i32x4v *>(src + (t_rd ^ (64 * h)));
            to_lds_w((j + 1) % PF, (j + 1) & 1);                          // the next step's registers take the other buffer
            __builtin_amdgcn_sched_barrier(0);
            load_w(j % PF, t + (j + PF) / NS, (j + PF) % NS);             // this step's registers are free again
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int mt = 0; mt < MT; mt++) acc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[h], xf[j][mt][h], acc[mt], 0, 0, 0);
        }

        // the eight partial sums of every tile meet in LDS (two areas in turn: one barrier per strip); wavefront t adds
        // those of tile t and writes it out while the others go on
        i32x4v *const rd = red + (t & 1) * (8 * MT * 64);
#pragma unroll
        for (int mt = 0; mt < MT; mt++) rd[(wave * MT + mt) * 64 + lane] = acc[mt];
        __syncthreads();
        if (finisher) {
            i32x4v sum = rd[wave * 64 + lane];
#pragma unroll
            for (int w = 1; w < 8; w++) sum += rd[(w * MT + wave) * 64 + lane];
            if (em < p.M && en < p.N && p.out_i32) {
                i32x4v o = sum;                                           // the accumulator itself, plus an int32 bias
                if (p.bias_kind == MI355_BIAS_INT32)
#pragma unroll
                    for (int r = 0; r < 4; r++) o[r] = (int32_t)((uint32_t)sum[r] + bq[r]);
                *reinterpret_cast<i32x4v *>(static_cast<int32_t *>(p.out) + (int64_t)em * p.ldc + en) = o;
            } else if (em < p.M && en < p.N && p.out_i8) {
                // clamp(rint((sum + int32 bias) * scale + offset)): each operation rounded to float32
                uint32_t w = 0;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int32_t bi = p.bias_kind == MI355_BIAS_INT32 ? (int32_t)bq[r] : 0;
                    float v = (float)(int32_t)((uint32_t)sum[r] + (uint32_t)bi);
                    v = v * (p.scale_len == 1 ? sc_one : __uint_as_float(scq[r]));
                    v = v + qparam_hi_offset(p.scale_len == 1 ? of_one : ofq[r]);
                    v = fminf(fmaxf(rintf(v), -128.0f), 127.0f);
                    w |= ((uint32_t)(int32_t)v & 0xffu) << (8 * r);
                }
                *reinterpret_cast<uint32_t *>(static_cast<int8_t *>(p.out) + (int64_t)em * p.ldc + en) = w;
            } else if (em < p.M && en < p.N) {
                float f[4];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int32_t bi = p.bias_kind == MI355_BIAS_INT32 ? (int32_t)bq[r] : 0;
                    float v = (float)(int32_t)((uint32_t)sum[r] + (uint32_t)bi);      // wraps like the hardware accumulator
                    if (has_ps) v = v * ps;
                    v = v * (p.scale_len == 1 ? sc_one : __uint_as_float(scq[r]));
                    if (has_bias) v = v + (bias_elem == 2u ? ((r & 1) ? bf16_hi(bh[r >> 1]) : bf16_lo(bh[r >> 1])) : __uint_as_float(bq[r]));
                    f[r] = v;
                }
                u32x2 pk;
                pk.x = p.out_f16 ? pack_f16x2(f[0], f[1]) : pack_bf16x2(f[0], f[1]);
                pk.y = p.out_f16 ? pack_f16x2(f[2], f[3]) : pack_bf16x2(f[2], f[3]);
                *reinterpret_cast<u32x2 *>(static_cast<uint16_t *>(p.out) + (int64_t)em * p.ldc + en) = pk;
            }
        }
    }
}

template <int MT, int NS, int PF>
int launch(const QmmDecodeArgs &p, hipStream_t s)
{
    constexpr int lds_bytes = 8 * (4096 + MT * 2048) + 2 * 8 * MT * 1024;
    auto kern = qmm_decode_kernel<MT, NS, PF>;
    static int attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (attr_status != hipSuccess) return MI355_ERR_LAUNCH;
    const int strips = (p.N + 15) / 16;
    hipLaunchKernelGGL(kern, dim3((unsigned)(strips < kMaxWorkgroups ? strips : kMaxWorkgroups)), dim3(512), lds_bytes, s, p);
    return check_launch();
}

} // namespace

bool qmm_decode_shape(int64_t M, int64_t N, int64_t K)
{
    if (knob(kKnobQmmDecodeOff) == 1 || M < 1 || M > 64 || K % kStep != 0 || K < 8 * kStep || N < 2048) return false;
    // The activations of a wavefront's eighth of K stay in registers: up to 16 steps with one tile of 16 rows, 8 with two,
    // 4 with four.  With four tiles and more than 1024 strips the tiled kernel's streaming loop is faster (measured at
    // K = 4096: N = 6144 11.8 against 15.1 us, N = 28672 27.7 against 25.8).
    const int64_t steps = (K / kStep + 7) / 8;
    if (M <= 16) return steps <= 16;
    if (M <= 32) return steps <= 8;
    return steps <= 4 && N <= 16384;
}

int launch_qmm_decode(const QmmDecodeArgs &p, hipStream_t s)
{
    if (!qmm_decode_shape(p.M, p.N, p.K)) return MI355_ERR_UNSUPPORTED;
    if ((p.lda & 15) != 0 || (p.ldbt & 15) != 0 || !aligned(p.a, 16) || !aligned(p.bt, 16) || p.ldbt < p.K)
        return MI355_ERR_UNSUPPORTED;
    // dequantisation parameters and results in pieces of four columns
    if ((p.N & 3) != 0 || (p.ldc & 3) != 0 || !aligned(p.out, p.out_i32 ? 16 : 8) || !aligned(p.qparam ? static_cast<const void *>(p.qparam) : static_cast<const void *>(p.scale), 16) ||
        (p.bias && !aligned(p.bias, p.bias_kind == MI355_BIAS_BF16 ? 8 : 16)))
        return MI355_ERR_UNSUPPORTED;
    // 32-bit buffer offsets over the whole weight and all activation rows
    if ((uint64_t)(p.N + 16) * (uint64_t)p.ldbt + (uint64_t)p.K >= (1ull << 31) || (uint64_t)p.M * (uint64_t)p.lda + (uint64_t)p.K >= (1ull << 31))
        return MI355_ERR_UNSUPPORTED;
    const int ns = (p.K / kStep + 7) / 8;                                 // steps of the busiest wavefront
    if (p.M <= 16) return ns <= 4 ? launch<1, 4, 4>(p, s) : ns <= 8 ? launch<1, 8, 4>(p, s) : launch<1, 16, 4>(p, s);
    if (p.M <= 32) return ns <= 4 ? launch<2, 4, 4>(p, s) : launch<2, 8, 4>(p, s);
    return launch<4, 4, 4>(p, s);
}

} // namespace mi355
