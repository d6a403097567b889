// Internal interface of the register-expanding tiled kernel (int4 weights packed along N, int8 weights [K, N]; more than
// 32 activation rows); not part of the C ABI.  ldw_k: int32 words (int4) or bytes (int8) between weight rows.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace mi355 {

struct WqGemm4Plan {
    bool ok;                 // the kernel accepts this problem
    int bm;                  // activation rows per workgroup tile: 64 or 128
    int tiles_m, strips;     // workgroup tiles: row blocks x strips of 256 columns (128 bytes of an int4 row, 256 of an int8 row)
    int S;                   // workgroups that share a tile's K range
    int gstages;             // stages (128 rows of int4, 64 of int8) per scale group (per channel: all stages of a workgroup)
    size_t zone_bytes;       // bytes of the workspace's zero area used for the exchange (S > 1)
};

__attribute__((visibility("hidden"))) WqGemm4Plan make_wq_gemm4_plan(int64_t M, int64_t N, int64_t K, int w_bits,
                                                                     int64_t group_size, int64_t ldw_k, int64_t ldx,
                                                                     const void *x, const void *w, const void *scale,
                                                                     const void *offset);

__attribute__((visibility("hidden"))) int launch_wq_gemm4(const WqGemm4Plan &plan, const void *x, int act_f16, const void *w,
                                                          int w_bits, const void *scale, const void *offset, const void *bias, void *out,
                                                          int64_t M, int64_t N, int64_t K, int64_t group_size, int64_t ldx,
                                                          int64_t ldw_k, int64_t ldo, void *workspace, void *stream);

} // namespace mi355
