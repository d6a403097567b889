// npu_weight_quant_batchmatmul, int4 weights with their words along K (storage [N, K/8], the contrib module's layout,
// torch_npu/contrib/module/linear_weight_quant.py:71,106) and many activation rows: the register-expanding GEMM for
// words along N is 30-45 % faster than the kernel for this layout from 64 rows up, so from 256 rows up the weight is
// rewritten per call into the workspace with its words along N (a nibble transpose, bound by the 2 x K x N / 2 bytes it
// moves) and the parameters are gathered into row-major [G, N]; the repack costs less than the difference.
#include "common.h"
#include "weight_quant_repack.h"

namespace mi355 {
namespace {

// A workgroup turns 256 weight rows (n) x 32 words (256 k) into 256 rows (k) x 32 words (256 n).  Both sides move
// whole 128-byte row segments; in between a thread transposes 8 x 8 nibble blocks in registers.
__global__ __launch_bounds__(256) void repack_int4_k_to_n_kernel(const uint32_t *__restrict__ w_nk, int64_t ldw_n,
                                                                 uint32_t *__restrict__ w_kn, int64_t ldw_out, int N, int K)
{
    // one buffer, used twice: [n][word] with the 16-byte chunk c of row r at chunk c ^ (r & 7), then, after every thread
    // has its blocks in registers, [k][word (n block), rotated by the k word] with a pitch of 33
    __shared__ __attribute__((aligned(16))) uint32_t buf[256 * 33];
    uint32_t *const tin = buf, *const tout = buf;
    const int t = threadIdx.x;
    const int n0 = blockIdx.x * 256, j0 = blockIdx.y * 32;
    const int KW = K / 8, NWD = N / 8;
#pragma unroll
    for (int it = 0; it < 8; it++) {
        const int row = (t >> 3) + 32 * it, c = t & 7;
        u32x4 v = u32x4{0u, 0u, 0u, 0u};
        if (n0 + row < N && j0 + 4 * c < KW)                          // K is a multiple of 32: whole chunks
            v = *reinterpret_cast<const u32x4 *>(w_nk + (int64_t)(n0 + row) * ldw_n + j0 + 4 * c);
        *reinterpret_cast<u32x4 *>(tin + row * 32 + ((c ^ (row & 7)) << 2)) = v;
    }
    __syncthreads();
    const int j = t & 31;
    uint32_t blocks[4][8];                                            // 32 n blocks x 32 words = 1024 blocks, four per thread
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int nb = (t >> 5) + 8 * it;
        uint32_t(&r)[8] = blocks[it];
#pragma unroll
        for (int i = 0; i < 8; i++) r[i] = tin[(8 * nb + i) * 32 + ((((j >> 2) ^ i) << 2) | (j & 3))];
        // r[i] holds nibbles k = 0..7 of row i; three rounds of block swaps leave r[k] with nibbles n = 0..7 of k
#pragma unroll
        for (int round = 0; round < 3; round++) {
            const int d = 1 << round, sh = 4 << round;
            const uint32_t mask = round == 0 ? 0x0f0f0f0fu : round == 1 ? 0x00ff00ffu : 0x0000ffffu;
#pragma unroll
            for (int i = 0; i < 8; i++)
                if ((i & d) == 0) {
                    const uint32_t x = ((r[i] >> sh) ^ r[i + d]) & mask;
                    r[i + d] ^= x;
                    r[i] ^= x << sh;
                }
        }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int nb = (t >> 5) + 8 * it;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) tout[(8 * j + kk) * 33 + ((nb + j) & 31)] = blocks[it][kk];
    }
    __syncthreads();
    const bool vec = (ldw_out & 3) == 0 && aligned_dev(w_kn, 16);
#pragma unroll
    for (int it = 0; it < 8; it++) {
        const int lr = (t >> 3) + 32 * it, c = t & 7, jj = lr >> 3;
        const int k = 8 * j0 + lr;
        if (k >= K) continue;
        u32x4 v;
#pragma unroll
        for (int w = 0; w < 4; w++) v[w] = tout[lr * 33 + ((4 * c + w + jj) & 31)];
        uint32_t *o = w_kn + (int64_t)k * ldw_out + n0 / 8 + 4 * c;
        const int left = NWD - (n0 / 8 + 4 * c);                      // words of this row that exist
        if (vec && left >= 4) {
            *reinterpret_cast<u32x4 *>(o) = v;
        } else {
#pragma unroll
            for (int w = 0; w < 4; w++)
                if (w < left) o[w] = v[w];
        }
    }
}

__global__ __launch_bounds__(256) void gather_params_u16_kernel(const uint16_t *__restrict__ src, int64_t ld_g, int64_t ld_n,
                                                                uint16_t *__restrict__ dst, int G, int N)
{
    const int n = blockIdx.x * 256 + threadIdx.x, g = blockIdx.y;
    if (n < N) dst[(int64_t)g * N + n] = src[(int64_t)g * ld_g + (int64_t)n * ld_n];
}

} // namespace

int launch_repack_int4_k_to_n(const void *w_nk, int64_t ldw_n, void *w_kn, int64_t ldw_out, int64_t N, int64_t K, void *stream)
{
    const dim3 grid((unsigned)((N + 255) / 256), (unsigned)((K / 8 + 31) / 32));
    hipLaunchKernelGGL(repack_int4_k_to_n_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint32_t *>(w_nk), ldw_n, static_cast<uint32_t *>(w_kn), ldw_out, (int)N, (int)K);
    return check_launch();
}

int launch_gather_params_u16(const void *src, int64_t ld_g, int64_t ld_n, void *dst, int64_t G, int64_t N, void *stream)
{
    hipLaunchKernelGGL(gather_params_u16_kernel, dim3((unsigned)((N + 255) / 256), (unsigned)G), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(src), ld_g, ld_n, static_cast<uint16_t *>(dst),
                       (int)G, (int)N);
    return check_launch();
}

} // namespace mi355
