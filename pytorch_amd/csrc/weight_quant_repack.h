// Internal interface of the per-call repack of int4 weights stored with their words along K; not part of the C ABI.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace mi355 {

// int4 words along K ([N, K/8] words, rows ldw_n words apart) -> words along N ([K, ldw_out] words, N/8 of them used per row)
__attribute__((visibility("hidden"))) int launch_repack_int4_k_to_n(const void *w_nk, int64_t ldw_n, void *w_kn, int64_t ldw_out,
                                                                    int64_t N, int64_t K, void *stream);

// 16-bit parameters with element (g, n) at src[g * ld_g + n * ld_n] -> dense row-major [G, N]
__attribute__((visibility("hidden"))) int launch_gather_params_u16(const void *src, int64_t ld_g, int64_t ld_n, void *dst, int64_t G,
                                                                   int64_t N, void *stream);

} // namespace mi355
