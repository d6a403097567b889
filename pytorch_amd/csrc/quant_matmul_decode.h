// Internal interface of the decode-shaped int8 x int8 kernel (at most 64 activation rows, weight stored [N, K]); not part of
// the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace mi355 {

struct QmmDecodeArgs {
    const int8_t *a;           // [M, K], row pitch lda
    const int8_t *bt;          // [N, K], row pitch ldbt
    const float *pertoken;     // [M] or null
    const float *scale;        // [scale_len], or null when qparam is given or the output is int32
    const uint64_t *qparam;    // [scale_len] packed quantisation parameters (bits 0-31: the float32 scale), or null
    const void *bias;          // [N] of bias_kind, or null
    int bias_kind;             // MI355_BIAS_*
    int out_f16;               // round to fp16 instead of bf16
    int out_i8;                // re-quantise to int8 with the scale and offset of qparam (no pertoken, bias none or int32)
    int out_i32;               // the int32 accumulator (plus an int32 bias) itself: no scales
    void *out;                 // [M, N] 16-bit floats, int8 or int32, row pitch ldc in elements
    int64_t lda, ldbt, ldc;
    int M, N, K;
    int scale_len;             // 1 or N
};

// The part of the decision that depends on the shape alone (the workspace query uses it: the kernel needs no workspace).
__attribute__((visibility("hidden"))) bool qmm_decode_shape(int64_t M, int64_t N, int64_t K);

// MI355_ERR_UNSUPPORTED when pointers or pitches do not fit the kernel: the caller then takes the tiled kernel.
__attribute__((visibility("hidden"))) int launch_qmm_decode(const QmmDecodeArgs &p, hipStream_t stream);

} // namespace mi355
