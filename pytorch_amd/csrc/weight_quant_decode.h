// Internal interface of the decode-shaped kernel for int4 weights packed along N (at most 32 activation rows); not part
// of the C ABI.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace mi355 {

struct WqDecodePlan {
    bool ok;                 // the kernel accepts this problem
    int mt;                  // m tiles (16 rows): 1 or 2
    int strips;              // 128-byte strips of a weight row (256 columns each)
    int S;                   // workgroups that share a strip, 1024 weight rows each
    bool grouped;
    size_t zone_bytes;       // bytes of the workspace's zero area (behind the arrival counters) used for the exchange
};

__attribute__((visibility("hidden"))) WqDecodePlan make_wq_decode_plan(int64_t M, int64_t N, int64_t K, int w_bits,
                                                                       int64_t group_size, int64_t ldw_k, int64_t ldx,
                                                                       const void *x, const void *w, const void *scale,
                                                                       const void *offset);

// `workspace`: the zero area of the shared workspace when plan.S > 1 (zero on entry, left zero)
__attribute__((visibility("hidden"))) int launch_wq_decode(const WqDecodePlan &plan, const void *x, int act_f16, const void *w,
                                                           const void *scale, const void *offset, const void *bias, void *out,
                                                           int64_t M, int64_t N, int64_t K, int64_t group_size, int64_t ldx,
                                                           int64_t ldw_k, int64_t ldo, void *workspace, void *stream);

} // namespace mi355
