// Internal interface of the kernel for int4 weights packed along K (storage [N, K/8]); not part of the C ABI.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace mi355 {

struct WqKpackedPlan {
    bool ok;                 // the kernel accepts this problem
    int mt;                  // m tiles (16 rows) per workgroup: 1, 2 or 4
    int nw;                  // 16-column tiles per workgroup: 4 or 8
    int ntw;                 // column tiles per wavefront: 2 with four m tiles, else 1
    int ks;                  // slices of the workgroup's K range (nw * ks wavefronts): 1 or 2
    int mchunks, tiles;      // workgroups along M and N
    int S;                   // workgroups that share the K range of a tile
    int unit_steps, n_units; // K is split between workgroups in units of unit_steps * 256
    int unit_sub;            // sub-steps of 128 k per scale group (grouped only)
    bool grouped;
    size_t lds_bytes, counter_bytes, partial_bytes;   // workspace when S > 1: [arrival counters | partial sums]
};

// `ldw_n`: int32 words between the rows of two consecutive output columns
__attribute__((visibility("hidden"))) WqKpackedPlan make_wq_kpacked_plan(int64_t M, int64_t N, int64_t K, int64_t group_size,
                                                                         int64_t ldw_n, int64_t ldx, const void *x,
                                                                         const void *w);

// scale / offset element (group, column) at index group * ld_param_g + column * ld_param_n, any strides;
// `workspace` holds counter_bytes + partial_bytes when plan.S > 1
__attribute__((visibility("hidden"))) int launch_wq_kpacked(const WqKpackedPlan &plan, const void *x, int act_f16, const void *w,
                                                            const void *scale, const void *offset, const void *bias, void *out,
                                                            int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw_n,
                                                            int64_t ldo, int64_t ld_param_g, int64_t ld_param_n,
                                                            void *workspace, void *stream);

} // namespace mi355
