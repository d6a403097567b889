// Internal interface of the tiled weight-only GEMM (more than 32 activation rows); not part of the C ABI.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace mi355 {

struct WqGemmPlan {
    bool ok;                 // the tiled kernel accepts this problem
    int bm;                  // activation rows per workgroup tile (64 or 128)
    int tiles_m, tiles_n;    // workgroup tiles; a tile spans one 128-byte strip of the weight rows
    int S;                   // workgroups that share the K range of a tile
    int unit_stages;         // 64-row stages per unit of K: a scale group, or two stages per channel
    int n_units;
    bool grouped, accum;     // accum: a workgroup meets more than one scale group
    bool k_major;            // int8 weights stored [N, K]
    size_t counter_bytes, partial_bytes;   // workspace when S > 1: [arrival counters | partial sums]
};

// layout 1: weight rows contiguous along N, `ldw` elements (int8 bytes / int32 words) between k rows;
// layout 2: int8 stored [N, K], `ldw` bytes between columns; anything else: not eligible.
__attribute__((visibility("hidden"))) WqGemmPlan make_wq_gemm_plan(int64_t M, int64_t N, int64_t K, int w_bits,
                                                                   int64_t group_size, int layout, int64_t ldw,
                                                                   int64_t ldx, const void *x, const void *w,
                                                                   const void *scale, const void *offset);

// Launches the tiled kernel; `workspace` holds counter_bytes + partial_bytes when plan.S > 1.
__attribute__((visibility("hidden"))) int launch_wq_gemm(const WqGemmPlan &plan, const void *x, int act_f16, const void *w,
                                                         int w_bits, const void *scale, const void *offset, const void *bias,
                                                         void *out, int64_t M, int64_t N, int64_t K, int64_t ldx,
                                                         int64_t ldw, int64_t ldo, void *workspace, void *stream);

} // namespace mi355
