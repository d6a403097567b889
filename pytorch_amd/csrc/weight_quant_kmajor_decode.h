// Internal interface of the decode-shaped kernel for int8 weights stored [N, K] with one scale per column (at most 32
// activation rows); not part of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace mi355 {

struct WqKmDecodeArgs {
    const uint16_t *x;         // bf16 / fp16 [M, K], row pitch ldx elements
    const int8_t *w;           // [N, K], row pitch ldw bytes
    const uint16_t *scale;     // [N]
    const uint16_t *offset;    // [N] or null
    const uint16_t *bias;      // [N] or null
    uint16_t *out;             // [M, N], row pitch ldo elements
    int64_t ldx, ldw, ldo;
    int M, N, K;
};

// The part of the decision that depends on the shape alone (the kernel needs no workspace).
__attribute__((visibility("hidden"))) bool wq_kmajor_decode_shape(int64_t M, int64_t N, int64_t K, int64_t group_size);

// MI355_ERR_UNSUPPORTED when pointers or pitches do not fit the kernel: the caller then takes the tiled K-major kernel.
__attribute__((visibility("hidden"))) int launch_wq_kmajor_decode(const WqKmDecodeArgs &p, int act_f16, hipStream_t stream);

} // namespace mi355
