// Internal interface of the decode-shaped kernel for int4 weights packed along K (storage [N, K/8]) with scale groups of
// 128 (at most 32 activation rows); not part of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace mi355 {

struct WqKpDecodeArgs {
    const uint16_t *x;         // bf16 / fp16 [M, K], row pitch ldx elements
    const void *w;             // int32 words [N, K/8], row pitch ldw_bytes
    const uint16_t *scale;     // element (group, column) at group * ld_param_g + column * ld_param_n
    const uint16_t *offset;    // same strides, or null
    const uint16_t *bias;      // [N] or null
    uint16_t *out;             // [M, N], row pitch ldo elements
    int64_t ldx, ldo, ld_param_g, ld_param_n;
    uint32_t ldw_bytes;
    int M, N, K;
};

// The part of the decision that depends on the shape alone (the kernel needs no workspace).
__attribute__((visibility("hidden"))) bool wq_kpacked_decode_shape(int64_t M, int64_t N, int64_t K, int64_t group_size);

// MI355_ERR_UNSUPPORTED when pointers or pitches do not fit the kernel: the caller then takes the other K-packed kernel.
__attribute__((visibility("hidden"))) int launch_wq_kpacked_decode(const WqKpDecodeArgs &p, int act_f16, hipStream_t stream);

} // namespace mi355
