// torch.ops.npu.* operator library for the quantized-inference path on MI355X.
//
// Mirrors what torchnpugen generates for torch_npu (schema registration with
// TORCH_LIBRARY(npu) and a backend wrapper per op that checks devices, guards the device and
// calls the adapter: torchnpugen/templates/CustomRegisterSchema.cpp:49-70,
// torchnpugen/custom_functions.py:94-255) and what the op-plugin adapter does (allocate the
// outputs, infer shapes, call the aclnn entry point).  Here the adapter calls the C ABI of
// include/mi355_quant.h on the current HIP stream.
//
// Dispatch keys: CUDA (PyTorch's name for the HIP device on ROCm builds) and Meta (shape
// inference for FakeTensor).  There is deliberately no CPU kernel: calling these ops with CPU
// tensors fails in the dispatcher.
#include <ATen/ATen.h>
#include <ATen/ExpandUtils.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <hip/hip_runtime_api.h>
#include <torch/library.h>

#include <map>
#include <mutex>

#include "mi355_quant.h"

namespace {

using at::Tensor;
using c10::optional;

void check_status(int status, const char *op)
{
    TORCH_CHECK(status == MI355_OK, op, ": ", mi355_status_string(status), " (status ", status, ")");
}

// Same text as the reference's generated wrapper check (asserted by
// test/custom_ops/test_npu_anti_quant.py:86-88).
void check_same_device(const char *op, std::initializer_list<const Tensor *> ts)
{
    const Tensor *first = nullptr;
    for (const Tensor *t : ts) {
        if (!t || !t->defined()) continue;
        if (!first) {
            first = t;
            continue;
        }
        TORCH_CHECK(t->device() == first->device(),
                    "Expected all tensors to be on the same device, but found at least two devices, ", first->device(),
                    " and ", t->device(), "! (when checking arguments for ", op, ")");
    }
}

const Tensor *opt(const optional<Tensor> &t) { return t.has_value() && t->defined() ? &*t : nullptr; }

void *stream_of(const Tensor &t)
{
    // PyTorch-ROCm names its HIP device type "cuda"; these are its stream/guard classes for that device type
    return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

// ---------------------------------------------------------------- npu_dynamic_quant

// Per-expert smooth scales: smooth_scales [E, H] with group_index [E], the running totals of the rows of each expert.
// `int4_ok`: the operator also packs int4 codes (dst_type torch.quint4x2).
void dynamic_quant_check(const Tensor &input, const optional<Tensor> &smooth_scales, const optional<Tensor> &group_index,
                         optional<at::ScalarType> dst_type, bool int4_ok = false)
{
    TORCH_CHECK(input.scalar_type() == at::kBFloat16 || input.scalar_type() == at::kHalf,
                "npu_dynamic_quant: input must be bfloat16 or float16, got ", input.scalar_type());
    TORCH_CHECK(input.dim() >= 1, "npu_dynamic_quant: input must have at least one dimension");
    TORCH_CHECK(!dst_type.has_value() || *dst_type == at::kChar || (int4_ok && *dst_type == at::kQUInt4x2),
                "npu_dynamic_quant: dst_type must be torch.int8", int4_ok ? " or torch.quint4x2" : "", ", got ", *dst_type);
    if (dst_type.has_value() && *dst_type == at::kQUInt4x2)
        TORCH_CHECK(input.size(-1) % 8 == 0, "npu_dynamic_quant: dst_type=torch.quint4x2 packs eight values per int32 word: the last "
                    "dimension must be a multiple of 8, got ", input.size(-1));
    if (const Tensor *g = opt(group_index)) {
        const Tensor *s = opt(smooth_scales);
        TORCH_CHECK(s, "npu_dynamic_quant: group_index needs smooth_scales of shape [experts, ", input.size(-1), "]");
        TORCH_CHECK(g->scalar_type() == at::kInt || g->scalar_type() == at::kLong,
                    "npu_dynamic_quant: group_index must be int32 or int64, got ", g->scalar_type());
        TORCH_CHECK(g->dim() == 1 && g->size(0) >= 1, "npu_dynamic_quant: group_index must have shape [experts]");
        TORCH_CHECK(s->scalar_type() == input.scalar_type(), "npu_dynamic_quant: smooth_scales must have the dtype of input");
        TORCH_CHECK(s->dim() == 2 && s->size(0) == g->size(0) && s->size(1) == input.size(-1),
                    "npu_dynamic_quant: with group_index, smooth_scales must have shape [", g->size(0), ", ", input.size(-1), "], got ",
                    s->sizes());
    } else if (const Tensor *s = opt(smooth_scales)) {
        TORCH_CHECK(s->scalar_type() == input.scalar_type(), "npu_dynamic_quant: smooth_scales must have the dtype of input");
        TORCH_CHECK(s->dim() == 1 && s->size(0) == input.size(-1),
                    "npu_dynamic_quant: smooth_scales must have shape [", input.size(-1), "]");
    }
}

// int4: an int32 result whose last dimension is an eighth of the input's
std::tuple<Tensor, Tensor> dynamic_quant_alloc(const Tensor &input, bool int4 = false)
{
    auto scale_shape = input.sizes().vec();
    scale_shape.pop_back();
    auto y_shape = input.sizes().vec();
    if (int4) y_shape.back() /= 8;
    return {at::empty(y_shape, input.options().dtype(int4 ? at::kInt : at::kChar)),
            at::empty(scale_shape, input.options().dtype(at::kFloat))};
}

std::tuple<Tensor, Tensor> dynamic_quant_meta(const Tensor &input, const optional<Tensor> &smooth_scales,
                                              const optional<Tensor> &group_index, optional<at::ScalarType> dst_type)
{
    dynamic_quant_check(input, smooth_scales, group_index, dst_type, true);
    return dynamic_quant_alloc(input, dst_type.has_value() && *dst_type == at::kQUInt4x2);
}

std::tuple<Tensor, Tensor> dynamic_quant_hip(const Tensor &input, const optional<Tensor> &smooth_scales,
                                             const optional<Tensor> &group_index, optional<at::ScalarType> dst_type)
{
    dynamic_quant_check(input, smooth_scales, group_index, dst_type, true);
    check_same_device("npu_dynamic_quant", {&input, opt(smooth_scales), opt(group_index)});
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    const bool int4 = dst_type.has_value() && *dst_type == at::kQUInt4x2;
    auto [y, scale] = dynamic_quant_alloc(input, int4);
    const int64_t cols = input.size(-1);
    const int64_t rows = cols ? input.numel() / cols : 0;
    if (rows == 0 || cols == 0) {
        scale.zero_();
        return {y, scale};
    }
    // rows must be addressable with one stride: a 2-D view with unit inner stride, else a packed copy
    Tensor x = input;
    int64_t row_stride = cols;
    if (x.dim() == 2 && x.stride(1) == 1 && x.stride(0) >= cols) {
        row_stride = x.stride(0);
    } else if (!x.is_contiguous()) {
        x = x.contiguous();
    }
    Tensor smooth;
    if (const Tensor *s = opt(smooth_scales)) smooth = s->contiguous();
    Tensor gi;                                             // a handful of totals: int64 ones are narrowed on the device
    if (const Tensor *g = opt(group_index)) gi = g->to(at::kInt).contiguous();
    if (int4) {
        check_status(mi355_dynamic_quant_int4(x.data_ptr(), x.scalar_type() == at::kBFloat16 ? MI355_DTYPE_BF16 : MI355_DTYPE_FP16,
                                              smooth.defined() ? smooth.data_ptr() : nullptr,
                                              gi.defined() ? gi.data_ptr<int32_t>() : nullptr, gi.defined() ? gi.numel() : 0,
                                              y.data_ptr(), scale.data_ptr<float>(), rows, cols, row_stride, stream_of(input)),
                     "npu_dynamic_quant");
        return {y, scale};
    }
    check_status(mi355_dynamic_quant_grouped(x.data_ptr(), x.scalar_type() == at::kBFloat16 ? MI355_DTYPE_BF16 : MI355_DTYPE_FP16,
                                             smooth.defined() ? smooth.data_ptr() : nullptr,
                                             gi.defined() ? gi.data_ptr<int32_t>() : nullptr, gi.defined() ? gi.numel() : 0,
                                             y.data_ptr<int8_t>(), scale.data_ptr<float>(), rows, cols, row_stride,
                                             stream_of(input)),
                 "npu_dynamic_quant");
    return {y, scale};
}

// ---------------------------------------------------------------- npu_dynamic_quant_asymmetric
// torch_npu.npu_dynamic_quant_asymmetric(input, *, smooth_scales=None, group_index=None, dst_type=None)
// -> (y int8, scale float32, offset float32)   (test/test_fake_tensor.py:1689-1709, test/torch_npu_schema.json:2147-2149)

std::tuple<Tensor, Tensor, Tensor> dynamic_quant_asym_alloc(const Tensor &input)
{
    auto [y, scale] = dynamic_quant_alloc(input);
    return {y, scale, at::empty_like(scale)};
}

std::tuple<Tensor, Tensor, Tensor> dynamic_quant_asym_meta(const Tensor &input, const optional<Tensor> &smooth_scales,
                                                           const optional<Tensor> &group_index,
                                                           optional<at::ScalarType> dst_type)
{
    dynamic_quant_check(input, smooth_scales, group_index, dst_type);
    return dynamic_quant_asym_alloc(input);
}

std::tuple<Tensor, Tensor, Tensor> dynamic_quant_asym_hip(const Tensor &input, const optional<Tensor> &smooth_scales,
                                                          const optional<Tensor> &group_index,
                                                          optional<at::ScalarType> dst_type)
{
    dynamic_quant_check(input, smooth_scales, group_index, dst_type);
    check_same_device("npu_dynamic_quant_asymmetric", {&input, opt(smooth_scales), opt(group_index)});
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    auto [y, scale, offset] = dynamic_quant_asym_alloc(input);
    const int64_t cols = input.size(-1);
    const int64_t rows = cols ? input.numel() / cols : 0;
    if (rows == 0 || cols == 0) {
        scale.zero_();
        offset.zero_();
        return {y, scale, offset};
    }
    Tensor x = input;
    int64_t row_stride = cols;
    if (x.dim() == 2 && x.stride(1) == 1 && x.stride(0) >= cols) {
        row_stride = x.stride(0);
    } else if (!x.is_contiguous()) {
        x = x.contiguous();
    }
    Tensor smooth;
    if (const Tensor *s = opt(smooth_scales)) smooth = s->contiguous();
    Tensor gi;
    if (const Tensor *g = opt(group_index)) gi = g->to(at::kInt).contiguous();
    check_status(mi355_dynamic_quant_asymmetric_grouped(x.data_ptr(),
                                                        x.scalar_type() == at::kBFloat16 ? MI355_DTYPE_BF16 : MI355_DTYPE_FP16,
                                                        smooth.defined() ? smooth.data_ptr() : nullptr,
                                                        gi.defined() ? gi.data_ptr<int32_t>() : nullptr, gi.defined() ? gi.numel() : 0,
                                                        y.data_ptr<int8_t>(), scale.data_ptr<float>(), offset.data_ptr<float>(), rows,
                                                        cols, row_stride, stream_of(input)),
                 "npu_dynamic_quant_asymmetric");
    return {y, scale, offset};
}

// The matmul kernels exchange split-K partial sums through a workspace whose leading zero area (arrival counters and
// the exchange zone, MI355_WORKSPACE_ZERO_BYTES) must be zero before a launch; the kernels leave it zero.  One
// zero-initialised buffer per (device, stream) is kept and reused; launches on one stream are ordered, so they never
// overlap.  Lifetime rules, because a captured HIP graph keeps the pointer it was recorded with:
//   * eager calls: a buffer that is superseded by a larger one is never released (it stays alive, zeroed, until the
//     process ends), so a graph recorded earlier replays on valid, quiescent memory;
//   * a call made while the stream is capturing uses the stream's eager buffer when there is one that is large enough
//     (the operator was run on this stream before the capture: nothing is allocated or filled inside the graph);
//     otherwise the capture gets a buffer of its own (keyed by the capture's id): it comes from the graph's private
//     memory pool and its zero fill is a node of that graph, so every replay starts from zeros and the memory lives
//     exactly as long as the graph.  Such a buffer is never handed to an eager call or to another capture; the cache
//     drops its reference when it sees the next capture (or an eager call) on that stream, which returns the block
//     to the pool of the graph that owns it.
struct WorkspaceCache {
    struct Captured {
        unsigned long long id = 0;
        Tensor ws;
    };
    std::mutex mu;
    std::map<std::pair<int, void *>, Tensor> eager;
    std::map<std::pair<int, void *>, Captured> captured;
    std::vector<std::pair<std::pair<int, void *>, Tensor>> retired;       // never freed: an earlier graph may point into them
};

WorkspaceCache &workspace_cache()
{
    static WorkspaceCache *c = new WorkspaceCache();                      // intentionally never destroyed
    return *c;
}

// A kernel that gave up waiting for partial sums has said so in the workspace's status word (and put NaN where the sums
// belonged).  Reading the word needs the stream to drain, so it is read where that costs nothing extra: before a
// workspace is retired, and on request (mi355_npu_check_workspaces, pytorch_amd.check_device_status()), the way the
// reference reports a failed device task at the caller's next synchronisation (OpParamMaker.cpp:541-571).
void check_workspace(const Tensor &ws, void *stream, const char *when)
{
    const int st = mi355_workspace_status(ws.data_ptr(), (size_t)ws.numel(), 1, stream);
    TORCH_CHECK(st == MI355_OK, "mi355: ", mi355_status_string(st), " (found ", when,
                "; the outputs of that launch hold NaN, the workspace has been cleared and is usable again)");
}

Tensor zeroed_workspace(const Tensor &like, size_t bytes)
{
    WorkspaceCache &wc = workspace_cache();
    std::lock_guard<std::mutex> lock(wc.mu);
    const auto key = std::make_pair((int)like.device().index(), stream_of(like));
    int64_t want = (int64_t)std::max<size_t>(bytes, (size_t)MI355_WORKSPACE_ZERO_BYTES + ((size_t)1 << 20));
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    unsigned long long capture_id = 0;
    TORCH_CHECK(hipStreamGetCaptureInfo(static_cast<hipStream_t>(key.second), &capturing, &capture_id) == hipSuccess,
                "hipStreamGetCaptureInfo failed");
    if (capturing != hipStreamCaptureStatusNone) {
        const auto eager = wc.eager.find(key);
        if (eager != wc.eager.end() && eager->second.defined() && (size_t)eager->second.numel() >= bytes) return eager->second;
        WorkspaceCache::Captured &c = wc.captured[key];
        if (!c.ws.defined() || c.id != capture_id || (size_t)c.ws.numel() < bytes) {
            c.ws = at::zeros({want}, like.options().dtype(at::kChar));      // the fill is recorded into this capture
            c.id = capture_id;
        }
        return c.ws;
    }
    wc.captured.erase(key);
    Tensor &ws = wc.eager[key];
    if (!ws.defined() || (size_t)ws.numel() < bytes) {
        if (ws.defined()) {
            // geometric growth bounds the buffers a stream can retire (a handful between 17 MiB and the largest problem)
            want = std::max<int64_t>(want, 2 * ws.numel());
            Tensor old = ws;
            wc.retired.emplace_back(key, old);
            ws = at::zeros({want}, like.options().dtype(at::kChar));
            check_workspace(old, key.second, "when its workspace was outgrown");
        } else {
            ws = at::zeros({want}, like.options().dtype(at::kChar));
        }
    }
    return ws;
}

// ---------------------------------------------------------------- npu_trans_quant_param
// torch_npu.npu_trans_quant_param(scale, offset=None) (linear_quant.py:104-108; shapes test/test_fake_tensor.py:1929-1943:
// the result is int64 and takes the shape of whichever argument has more elements)

std::vector<int64_t> trans_quant_param_shape(const Tensor &scale, const optional<Tensor> &offset)
{
    TORCH_CHECK(scale.scalar_type() == at::kFloat, "npu_trans_quant_param: scale must be float32, got ", scale.scalar_type());
    TORCH_CHECK(scale.dim() >= 1 && scale.dim() <= 2, "npu_trans_quant_param: scale must have 1 or 2 dimensions");
    const Tensor *o = opt(offset);
    if (!o) return scale.sizes().vec();
    TORCH_CHECK(o->scalar_type() == at::kFloat, "npu_trans_quant_param: offset must be float32, got ", o->scalar_type());
    TORCH_CHECK(o->dim() >= 1 && o->dim() <= 2, "npu_trans_quant_param: offset must have 1 or 2 dimensions");
    TORCH_CHECK(scale.numel() == o->numel() || scale.numel() == 1 || o->numel() == 1,
                "npu_trans_quant_param: scale and offset must have the same number of elements, or one of them a single one");
    return (o->numel() > scale.numel() ? *o : scale).sizes().vec();
}

Tensor trans_quant_param_meta(const Tensor &scale, const optional<Tensor> &offset)
{
    return at::empty(trans_quant_param_shape(scale, offset), scale.options().dtype(at::kLong));
}

Tensor trans_quant_param_hip(const Tensor &scale, const optional<Tensor> &offset)
{
    check_same_device("npu_trans_quant_param", {&scale, opt(offset)});
    Tensor out = trans_quant_param_meta(scale, offset);
    if (out.numel() == 0) return out;
    c10::hip::HIPGuardMasqueradingAsCUDA guard(scale.device());
    Tensor sc = scale.contiguous();
    Tensor of = opt(offset) ? opt(offset)->contiguous() : Tensor();
    check_status(mi355_trans_quant_param(sc.data_ptr<float>(), sc.numel(), of.defined() ? of.data_ptr<float>() : nullptr,
                                         of.defined() ? of.numel() : 0, reinterpret_cast<uint64_t *>(out.data_ptr<int64_t>()),
                                         out.numel(), stream_of(scale)),
                 "npu_trans_quant_param");
    return out;
}

// ---------------------------------------------------------------- npu_quant_matmul

struct QmmPlan {
    std::vector<int64_t> out_shape;
    std::vector<int64_t> batch;      // broadcast batch shape
    int64_t M, N, K;
    at::ScalarType out_dtype;
    bool a4w4;                       // both inputs int32 words of eight int4 values
    bool x2_packed_k;                // a4w4: x2 is [K/8, N] (words along K) instead of [K, N/8]
    bool packed_scale;               // scale is the int64 result of npu_trans_quant_param
};

QmmPlan quant_matmul_plan(const Tensor &x1, const Tensor &x2, const Tensor &scale, const optional<Tensor> &offset,
                          const optional<Tensor> &pertoken_scale, const optional<Tensor> &bias,
                          optional<at::ScalarType> output_dtype)
{
    const bool a4w4 = x1.scalar_type() == at::kInt && x2.scalar_type() == at::kInt;
    TORCH_CHECK(a4w4 || (x1.scalar_type() == at::kChar && x2.scalar_type() == at::kChar),
                "npu_quant_matmul: x1 and x2 must both be int8, or both int32 holding eight int4 values per word, got ",
                x1.scalar_type(), " and ", x2.scalar_type());
    TORCH_CHECK(x1.dim() >= 2 && x2.dim() >= 2, "npu_quant_matmul: x1 and x2 must have at least 2 dimensions");
    QmmPlan p;
    p.a4w4 = a4w4;
    p.x2_packed_k = false;
    p.M = x1.size(-2);
    p.K = x1.size(-1) * (a4w4 ? 8 : 1);
    p.N = x2.size(-1);
    if (a4w4 && x2.size(-2) == p.K) {
        // x2 [K, N/8]: words run along N (test/test_fake_tensor.py:1917-1923)
        p.N = x2.size(-1) * 8;
    } else if (a4w4) {
        // x2 [K/8, N]: the transposed view of a weight stored [N, K/8] (linear_quant.py:40-50, :110)
        TORCH_CHECK(x2.size(-2) * 8 == p.K, "npu_quant_matmul: int4 inner dimensions differ: x1 [..., ", p.M, ", ", x1.size(-1),
                    "] words (K = ", p.K, ") against x2 [..., ", x2.size(-2), ", ", x2.size(-1),
                    "] words; x2 must be [K, N/8] or [K/8, N]");
        p.x2_packed_k = true;
    } else {
        TORCH_CHECK(x2.size(-2) == p.K, "npu_quant_matmul: inner dimensions differ: x1 [..., ", p.M, ", ", p.K,
                    "] x2 [..., ", x2.size(-2), ", ", p.N, "]");
    }
    // output_dtype=None is the re-quantised int8 output (linear_quant.py:60-72)
    p.out_dtype = output_dtype.value_or(at::kChar);
    TORCH_CHECK(p.out_dtype == at::kBFloat16 || p.out_dtype == at::kHalf || p.out_dtype == at::kInt || p.out_dtype == at::kChar,
                "npu_quant_matmul: output_dtype must be torch.int8, torch.bfloat16, torch.float16 or torch.int32, got ", p.out_dtype);
    p.packed_scale = scale.scalar_type() == at::kLong;        // the result of npu_trans_quant_param
    if (p.out_dtype == at::kChar) {
        TORCH_CHECK(p.packed_scale || scale.scalar_type() == at::kFloat,
                    "npu_quant_matmul: scale must be int64 (npu_trans_quant_param) or float32 for int8 output, got ", scale.scalar_type());
        TORCH_CHECK(scale.dim() <= 2 && (scale.numel() == 1 || scale.numel() == p.N),
                    "npu_quant_matmul: scale must have 1 or ", p.N, " elements");
        TORCH_CHECK(!opt(pertoken_scale), "npu_quant_matmul: pertoken_scale is not applicable to int8 output");
        if (const Tensor *o = opt(offset)) {
            TORCH_CHECK(o->scalar_type() == at::kFloat, "npu_quant_matmul: offset must be float32, got ", o->scalar_type());
            TORCH_CHECK(o->numel() == 1 || o->numel() == p.N, "npu_quant_matmul: offset must have 1 or ", p.N, " elements");
        }
        if (const Tensor *b = opt(bias)) {
            TORCH_CHECK(b->scalar_type() == at::kInt, "npu_quant_matmul: bias must be int32 for int8 output, got ", b->scalar_type());
            TORCH_CHECK(b->numel() == p.N && b->size(-1) == p.N, "npu_quant_matmul: bias must have shape [", p.N, "]");
        }
    } else {
        TORCH_CHECK(!opt(offset), "npu_quant_matmul: offset is only meaningful for int8 output");
    }
    if (p.out_dtype == at::kChar) {
        // checked above
    } else
    if (p.out_dtype != at::kInt) {
        TORCH_CHECK(scale.scalar_type() == at::kFloat || scale.scalar_type() == at::kBFloat16 || p.packed_scale,
                    "npu_quant_matmul: scale must be float32, bfloat16 or int64 (npu_trans_quant_param) for a floating-point "
                    "output, got ", scale.scalar_type());
        TORCH_CHECK((scale.dim() == 1 || (p.packed_scale && scale.dim() == 2)) && (scale.numel() == 1 || scale.numel() == p.N),
                    "npu_quant_matmul: scale must have shape [1] or [", p.N, "]");
        TORCH_CHECK(!(p.packed_scale && opt(pertoken_scale)), "npu_quant_matmul: an int64 scale excludes pertoken_scale");
        if (const Tensor *ps = opt(pertoken_scale)) {
            TORCH_CHECK(ps->scalar_type() == at::kFloat, "npu_quant_matmul: pertoken_scale must be float32");
            TORCH_CHECK(ps->dim() == 1 && ps->size(0) == p.M, "npu_quant_matmul: pertoken_scale must have shape [", p.M, "]");
        }
        if (const Tensor *b = opt(bias)) {
            // int32: added to the accumulator (LinearQuant's default bias dtype, linear_quant.py:92); bf16 / float32:
            // added after dequantisation
            TORCH_CHECK(b->scalar_type() == at::kInt || b->scalar_type() == at::kFloat ||
                            (b->scalar_type() == at::kBFloat16 && p.out_dtype == at::kBFloat16),
                        "npu_quant_matmul: bias must be int32, float32 or (for bfloat16 output) bfloat16, got ", b->scalar_type());
            TORCH_CHECK(b->numel() == p.N && b->size(-1) == p.N, "npu_quant_matmul: bias must have shape [", p.N, "]");
        }
    } else {
        if (const Tensor *b = opt(bias)) {
            TORCH_CHECK(b->scalar_type() == at::kInt, "npu_quant_matmul: bias must be int32 for int32 output, got ", b->scalar_type());
            TORCH_CHECK(b->numel() == p.N && b->size(-1) == p.N, "npu_quant_matmul: bias must have shape [", p.N, "]");
        }
        TORCH_CHECK(!opt(pertoken_scale), "npu_quant_matmul: pertoken_scale is not applicable to int32 output");
    }
    auto b1 = x1.sizes().slice(0, x1.dim() - 2), b2 = x2.sizes().slice(0, x2.dim() - 2);
    p.batch = at::infer_size(b1, b2);
    p.out_shape = p.batch;
    p.out_shape.push_back(p.M);
    p.out_shape.push_back(p.N);
    return p;
}

Tensor quant_matmul_meta(const Tensor &x1, const Tensor &x2, const Tensor &scale, const optional<Tensor> &offset,
                         const optional<Tensor> &pertoken_scale, const optional<Tensor> &bias,
                         optional<at::ScalarType> output_dtype)
{
    QmmPlan p = quant_matmul_plan(x1, x2, scale, offset, pertoken_scale, bias, output_dtype);
    return at::empty(p.out_shape, x1.options().dtype(p.out_dtype));
}

// A 2-D int8 matrix the kernel can address: one of its strides is 1 and the other covers a row.
Tensor as_matrix(const Tensor &t)
{
    const bool row_major = t.stride(1) == 1 && t.stride(0) >= t.size(1);
    const bool col_major = t.stride(0) == 1 && t.stride(1) >= t.size(0);
    return (row_major || col_major) ? t : t.contiguous();
}

// int32 words of eight int4 values along the last dimension -> int8 of eight times that last dimension
// (contiguous result; the input is made contiguous first if its rows are not)
Tensor unpack_int4_rows(const Tensor &t)
{
    Tensor src = t.contiguous();
    auto shape = src.sizes().vec();
    const int64_t words = shape.back();
    shape.back() = words * 8;
    Tensor dst = at::empty(shape, src.options().dtype(at::kChar));
    const int64_t rows = words ? src.numel() / words : 0;
    check_status(mi355_unpack_int4(src.data_ptr(), dst.data_ptr<int8_t>(), rows, words * 8, words, words * 8, stream_of(t)),
                 "npu_quant_matmul (int4 operands)");
    return dst;
}

Tensor quant_matmul_hip(const Tensor &x1, const Tensor &x2, const Tensor &scale, const optional<Tensor> &offset,
                        const optional<Tensor> &pertoken_scale, const optional<Tensor> &bias,
                        optional<at::ScalarType> output_dtype)
{
    QmmPlan p = quant_matmul_plan(x1, x2, scale, offset, pertoken_scale, bias, output_dtype);
    check_same_device("npu_quant_matmul", {&x1, &x2, &scale, opt(pertoken_scale), opt(bias)});
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x1.device());
    Tensor out = at::empty(p.out_shape, x1.options().dtype(p.out_dtype));
    if (out.numel() == 0) return out;
    Tensor xa = x1, xb = x2;
    if (p.a4w4) {
        xa = unpack_int4_rows(x1);                                              // [..., M, K] int8
        xb = p.x2_packed_k ? unpack_int4_rows(x2.transpose(-2, -1)).transpose(-2, -1)   // stored [..., N, K]
                           : unpack_int4_rows(x2);                              // [..., K, N]
    }
    const bool i8 = p.out_dtype == at::kChar;
    const bool bf16 = p.out_dtype != at::kInt && !i8;     // a floating-point (dequantised) output
    Tensor scale_f, ps, b, qp;
    if (p.packed_scale) {
        qp = scale.reshape({-1}).contiguous();            // an int64 scale carries its offset (any `offset` repeats it)
    } else if (i8) {
        // float32 scale with int8 output: packed here the way the reference's module does it with
        // npu_trans_quant_param (linear_quant.py:104-108)
        qp = trans_quant_param_hip(scale, offset).reshape({-1});
    } else if (bf16) {
        scale_f = scale.to(at::kFloat).contiguous();
        if (const Tensor *t = opt(pertoken_scale)) ps = t->contiguous();
    }
    if (const Tensor *t = opt(bias)) b = t->reshape({p.N}).contiguous();
    const int bias_dtype = !b.defined() ? MI355_BIAS_NONE
                           : b.scalar_type() == at::kInt ? MI355_BIAS_INT32
                           : b.scalar_type() == at::kFloat ? MI355_BIAS_FP32 : MI355_BIAS_BF16;
    const int out_dtype = i8 ? MI355_OUT_INT8
                          : p.out_dtype == at::kInt ? MI355_OUT_INT32 : p.out_dtype == at::kHalf ? MI355_OUT_FP16 : MI355_OUT_BF16;
    int64_t nb = 1;
    for (auto d : p.batch) nb *= d;
    // x1 with batch dimensions against a single weight matrix is one tall matmul
    bool x2_single = true;
    for (int64_t d = 0; d < xb.dim() - 2; d++) x2_single = x2_single && xb.size(d) == 1;
    std::vector<std::pair<Tensor, Tensor>> jobs; // (a [m,K], b [K,N]) pairs writing consecutive rows of out
    Tensor out2d = out.view({-1, p.N});
    if (x2_single) {
        Tensor w2 = xb.dim() == 2 ? xb : xb.as_strided({p.K, p.N}, {xb.stride(-2), xb.stride(-1)});
        jobs.emplace_back(xa.reshape({-1, p.K}), w2);
        // the [M] per-token scales apply to every matrix of the batch: one copy per matrix of the tall matmul
        if (ps.defined() && p.M > 0 && jobs.back().first.size(0) != p.M) ps = ps.repeat({jobs.back().first.size(0) / p.M});
    } else {
        auto x1s = p.batch, x2s = p.batch;
        x1s.push_back(p.M), x1s.push_back(p.K), x2s.push_back(p.K), x2s.push_back(p.N);
        Tensor x1e = xa.expand(x1s).reshape({nb, p.M, p.K});
        Tensor x2e = xb.expand(x2s);
        x2e = x2e.reshape({nb, p.K, p.N});
        for (int64_t i = 0; i < nb; i++) jobs.emplace_back(x1e[i], x2e[i]);
    }
    int64_t row0 = 0;
    for (auto &job : jobs) {
        Tensor a = job.first.stride(1) == 1 && job.first.stride(0) >= p.K ? job.first : job.first.contiguous();
        Tensor w = as_matrix(job.second);
        const int64_t m = a.size(0);
        Tensor ws;
        const size_t ws_bytes = mi355_quant_matmul_workspace(m, p.N, p.K, w.stride(0), w.stride(1));
        if (ws_bytes) ws = zeroed_workspace(xa, ws_bytes);
        Tensor o = out2d.narrow(0, row0, m);
        const int st = qp.defined()
            ? mi355_quant_matmul_qparam(a.data_ptr<int8_t>(), w.data_ptr<int8_t>(), reinterpret_cast<const uint64_t *>(qp.data_ptr<int64_t>()),
                                        qp.numel(), b.defined() ? b.data_ptr() : nullptr, bias_dtype, o.data_ptr(), out_dtype, m, p.N,
                                        p.K, a.stride(0), w.stride(0), w.stride(1), o.stride(0),
                                        ws.defined() ? ws.data_ptr() : nullptr, ws_bytes, stream_of(x1))
            : mi355_quant_matmul(a.data_ptr<int8_t>(), w.data_ptr<int8_t>(), ps.defined() ? ps.data_ptr<float>() : nullptr,
                                 bf16 ? scale_f.data_ptr<float>() : nullptr, bf16 ? scale_f.numel() : 0,
                                 b.defined() ? b.data_ptr() : nullptr, bias_dtype, o.data_ptr(), out_dtype, m, p.N, p.K,
                                 a.stride(0), w.stride(0), w.stride(1), o.stride(0), ws.defined() ? ws.data_ptr() : nullptr,
                                 ws_bytes, stream_of(x1));
        check_status(st, "npu_quant_matmul");
        row0 += m;
    }
    return out;
}

// ---------------------------------------------------------------- npu_weight_quant_batchmatmul

struct WqPlan {
    std::vector<int64_t> out_shape;
    int64_t M, N, K, groups;
    int bits;
    bool packed_k;       // int4 words along K: weight [K/8, N], the transposed view of [N, K/8]
};

WqPlan weight_quant_plan(const Tensor &x, const Tensor &weight, const Tensor &antiquant_scale,
                         const optional<Tensor> &antiquant_offset, const optional<Tensor> &quant_scale,
                         const optional<Tensor> &quant_offset, const optional<Tensor> &bias, int64_t group_size,
                         int64_t inner_precise, optional<at::ScalarType> weight_dtype)
{
    const char *op = "npu_weight_quant_batchmatmul";
    TORCH_CHECK(x.scalar_type() == at::kBFloat16 || x.scalar_type() == at::kHalf, op, ": x must be bfloat16 or float16, got ",
                x.scalar_type());
    TORCH_CHECK(weight.scalar_type() == at::kChar || weight.scalar_type() == at::kInt, op,
                ": weight must be int8, or int32 holding 8 int4 values per word, got ", weight.scalar_type());
    TORCH_CHECK(x.dim() >= 2 && weight.dim() == 2, op, ": x must be [..., K] with at least 2 dimensions and weight 2-D");
    TORCH_CHECK(opt(quant_scale) || !opt(quant_offset), op, ": quant_offset needs quant_scale");
    // inner_precise: 0 = high precision, 1 = the vendor's faster, less precise accumulation.  Every kernel here accumulates in
    // float32, so both values give the high-precision result.
    TORCH_CHECK(inner_precise == 0 || inner_precise == 1, op, ": inner_precise must be 0 or 1, got ", inner_precise);
    TORCH_CHECK(!weight_dtype.has_value(), op, ": weight_dtype is not supported");
    WqPlan p;
    p.bits = weight.scalar_type() == at::kInt ? 4 : 8;
    p.K = x.size(-1);
    p.M = p.K ? x.numel() / p.K : 0;
    // int4: [K, N/8] holds the words along N; [K/8, N] - what the contrib module passes, the transposed view of its
    // [out_features, in_features/8] parameter (linear_weight_quant.py:71,106) - holds them along K
    p.packed_k = p.bits == 4 && weight.size(0) != p.K && weight.size(0) * 8 == p.K;
    p.N = weight.size(1) * (p.bits == 4 && !p.packed_k ? 8 : 1);
    TORCH_CHECK(weight.size(0) == p.K || p.packed_k, op, ": inner dimensions differ: x [..., ", p.K, "] weight [", weight.size(0),
                ", ...]", p.bits == 4 ? " (int4 weights are [K, N/8] or [K/8, N])" : "");
    TORCH_CHECK(group_size >= 0, op, ": antiquant_group_size must be >= 0");
    if (group_size > 0)
        TORCH_CHECK(p.K % group_size == 0 && group_size % 32 == 0, op,
                    ": antiquant_group_size must be a multiple of 32 that divides K=", p.K);
    p.groups = group_size > 0 ? p.K / group_size : 1;
    auto check_param = [&](const Tensor &t, const char *name) {
        TORCH_CHECK(t.scalar_type() == x.scalar_type(), op, ": ", name, " must have the dtype of x (", x.scalar_type(), "), got ",
                    t.scalar_type());
        const bool ok1 = t.dim() == 1 && t.size(0) == p.N && p.groups == 1;
        const bool ok2 = t.dim() == 2 && t.size(0) == p.groups && t.size(1) == p.N;
        TORCH_CHECK(ok1 || ok2, op, ": ", name, " must have shape [", p.N, "] (per channel) or [", p.groups, ", ", p.N,
                    "] (per group), got ", t.sizes());
    };
    check_param(antiquant_scale, "antiquant_scale");
    if (const Tensor *o = opt(antiquant_offset)) check_param(*o, "antiquant_offset");
    if (const Tensor *b = opt(bias)) {
        TORCH_CHECK(b->scalar_type() == x.scalar_type(), op, ": bias must have the dtype of x (", x.scalar_type(), "), got ",
                    b->scalar_type());
        TORCH_CHECK(b->numel() == p.N && b->size(-1) == p.N, op, ": bias must have shape [", p.N, "]");
    }
    // quant_scale (float32, or the int64 words of npu_trans_quant_param, which hold the offset as well) and quant_offset
    // (float32): one value or one per output column; they turn the output into int8
    auto check_requant = [&](const Tensor &t, const char *name, bool may_be_packed) {
        TORCH_CHECK(t.scalar_type() == at::kFloat || (may_be_packed && t.scalar_type() == at::kLong), op, ": ", name, " must be float32",
                    may_be_packed ? " or int64 (npu_trans_quant_param)" : "", ", got ", t.scalar_type());
        TORCH_CHECK((t.dim() == 1 || (t.dim() == 2 && t.size(0) == 1)) && (t.size(-1) == p.N || t.size(-1) == 1), op, ": ", name,
                    " must have shape [", p.N, "], [1, ", p.N, "] or one element, got ", t.sizes());
    };
    if (const Tensor *q = opt(quant_scale)) {
        check_requant(*q, "quant_scale", true);
        if (const Tensor *o = opt(quant_offset)) {
            TORCH_CHECK(q->scalar_type() == at::kFloat, op, ": an int64 quant_scale already holds the offset; pass quant_offset=None");
            check_requant(*o, "quant_offset", false);
        }
    }
    p.out_shape = x.sizes().vec();
    p.out_shape.back() = p.N;
    return p;
}

Tensor weight_quant_meta(const Tensor &x, const Tensor &weight, const Tensor &antiquant_scale,
                         const optional<Tensor> &antiquant_offset, const optional<Tensor> &quant_scale,
                         const optional<Tensor> &quant_offset, const optional<Tensor> &bias, int64_t group_size,
                         int64_t inner_precise, optional<at::ScalarType> weight_dtype)
{
    WqPlan p = weight_quant_plan(x, weight, antiquant_scale, antiquant_offset, quant_scale, quant_offset, bias, group_size,
                                 inner_precise, weight_dtype);
    return at::empty(p.out_shape, opt(quant_scale) ? x.options().dtype(at::kChar) : x.options());
}

Tensor weight_quant_hip(const Tensor &x, const Tensor &weight, const Tensor &antiquant_scale,
                        const optional<Tensor> &antiquant_offset, const optional<Tensor> &quant_scale,
                        const optional<Tensor> &quant_offset, const optional<Tensor> &bias, int64_t group_size,
                        int64_t inner_precise, optional<at::ScalarType> weight_dtype)
{
    WqPlan p = weight_quant_plan(x, weight, antiquant_scale, antiquant_offset, quant_scale, quant_offset, bias, group_size,
                                 inner_precise, weight_dtype);
    check_same_device("npu_weight_quant_batchmatmul",
                      {&x, &weight, &antiquant_scale, opt(antiquant_offset), opt(quant_scale), opt(quant_offset), opt(bias)});
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    Tensor out = at::empty(p.out_shape, x.options());
    if (out.numel() == 0) return out;
    Tensor x2 = x.reshape({p.M, p.K});
    if (x2.stride(1) != 1 || x2.stride(0) < p.K) x2 = x2.contiguous();
    Tensor w;
    int64_t ldw_k, ldw_n;
    if (p.packed_k) {
        // columns of K/8 consecutive words; a K of 8 would make both strides 1, which the C ABI reads as words along N
        TORCH_CHECK(p.K >= 16, "npu_weight_quant_batchmatmul: int4 weights packed along K need K >= 16");
        w = weight.stride(0) == 1 && weight.stride(1) >= weight.size(0) ? weight : weight.t().contiguous().t();
        ldw_k = 1, ldw_n = w.stride(1);
    } else if (p.bits == 4) {
        w = weight.stride(1) == 1 && weight.stride(0) >= weight.size(1) ? weight : weight.contiguous();
        ldw_k = w.stride(0), ldw_n = 1;
    } else {
        w = as_matrix(weight);
        ldw_k = w.stride(0), ldw_n = w.stride(1);
    }
    // The contrib module hands 2-D parameters over as transposed views of [N, G] (linear_weight_quant.py:98-109).  The
    // kernel for words along K reads them with their strides; the others want row-major [G, N].
    Tensor s = antiquant_scale, o;
    if (const Tensor *t = opt(antiquant_offset)) o = *t;
    if (!p.packed_k || (o.defined() && o.strides() != s.strides())) {
        s = s.contiguous();
        if (o.defined()) o = o.contiguous();
    }
    const int64_t ld_param_g = s.dim() == 2 ? s.stride(0) : 0, ld_param_n = s.dim() == 2 ? s.stride(1) : s.stride(0);
    Tensor bias_c;
    if (const Tensor *t = opt(bias)) bias_c = t->reshape({p.N}).contiguous();
    Tensor out2d = out.view({p.M, p.N});
    const size_t ws_bytes = mi355_weight_quant_matmul_workspace(p.M, p.N, p.K, p.bits, group_size);
    Tensor ws;
    if (ws_bytes) ws = zeroed_workspace(x, ws_bytes);
    check_status(mi355_weight_quant_matmul(x2.data_ptr(), x.scalar_type() == at::kHalf ? MI355_DTYPE_FP16 : MI355_DTYPE_BF16,
                                           w.data_ptr(), p.bits, s.data_ptr(), o.defined() ? o.data_ptr() : nullptr,
                                           bias_c.defined() ? bias_c.data_ptr() : nullptr,
                                           out2d.data_ptr(), p.M, p.N, p.K, group_size, ld_param_g, ld_param_n, x2.stride(0),
                                           ldw_k, ldw_n, out2d.stride(0),
                                           ws.defined() ? ws.data_ptr() : nullptr, ws.defined() ? (size_t)ws.numel() : 0,
                                           stream_of(x)),
                 "npu_weight_quant_batchmatmul");
    const Tensor *qs = opt(quant_scale);
    if (!qs) return out;
    // int8 output: y = clamp(rint(float(out) * quant_scale[n] + quant_offset[n]), -128, 127), the product rounded to the
    // dtype of x first (it is the operator's result without quant_scale), every later operation rounded to float32, and
    // the offset brought to the 9-bit integer range that the packed parameter words hold (round, clip to [-256, 255]: the
    // reference's own test helper f32_2_s9, test/contrib/test_linear_weight_quant.py:13-16).  The reference tree holds no
    // golden for this output; the formula is the re-quantisation of npu_quant_matmul's int8 output applied to the
    // rounded product.
    Tensor scale_f, offset_f;
    if (qs->scalar_type() == at::kLong) {
        const Tensor q = qs->reshape({-1});
        scale_f = q.bitwise_and((int64_t)0xffffffffLL).bitwise_xor((int64_t)0x80000000LL).sub((int64_t)0x80000000LL).to(at::kInt).view(at::kFloat);
        offset_f = q.bitwise_right_shift(37).bitwise_and(0x1ff).bitwise_xor(256).sub(256).to(at::kFloat);
    } else {
        scale_f = qs->reshape({-1}).contiguous();
        if (const Tensor *qo = opt(quant_offset)) offset_f = at::clamp(at::round(qo->reshape({-1})), -256.0, 255.0).contiguous();
    }
    Tensor out8 = at::empty(p.out_shape, x.options().dtype(at::kChar));
    check_status(mi355_quantize(out2d.data_ptr(), x.scalar_type() == at::kHalf ? MI355_DTYPE_FP16 : MI355_DTYPE_BF16,
                                scale_f.data_ptr<float>(), scale_f.numel(), offset_f.defined() ? offset_f.data_ptr() : nullptr,
                                MI355_DTYPE_FP32, offset_f.defined() ? offset_f.numel() : 0, out8.data_ptr(), MI355_Q_INT8, p.M, p.N, 1,
                                0, stream_of(x)),
                 "npu_weight_quant_batchmatmul (quant_scale)");
    return out8;
}

// ---------------------------------------------------------------- npu_swiglu

void swiglu_check(const Tensor &input, int64_t dim)
{
    TORCH_CHECK(input.scalar_type() == at::kBFloat16, "npu_swiglu: only bfloat16 is supported, got ", input.scalar_type());
    TORCH_CHECK(input.dim() >= 1, "npu_swiglu: input must have at least one dimension");
    TORCH_CHECK(dim == -1 || dim == input.dim() - 1, "npu_swiglu: only the last dimension is supported");
    TORCH_CHECK(input.size(-1) % 2 == 0, "npu_swiglu: the split dimension must be even");
}

Tensor swiglu_meta(const Tensor &input, int64_t dim)
{
    swiglu_check(input, dim);
    auto shape = input.sizes().vec();
    shape.back() /= 2;
    return at::empty(shape, input.options());
}

Tensor swiglu_hip(const Tensor &input, int64_t dim)
{
    Tensor out = swiglu_meta(input, dim);
    if (out.numel() == 0) return out;
    c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
    Tensor x = input.contiguous();
    const int64_t half = out.size(-1);
    check_status(mi355_swiglu(x.data_ptr(), out.data_ptr(), out.numel() / half, half, 2 * half, stream_of(input)), "npu_swiglu");
    return out;
}

// ---------------------------------------------------------------- npu_swiglu_quant

// The operator is only named in the reference tree (docs/zh/release_notes.md:303); the argument list follows the
// vendor's published Python signature.  Implemented: dynamic per-token quantisation (quant_mode = 1) of the SwiGLU
// of the last dimension, optionally with smooth scales - one set, or one per expert with group_index (the running totals
// of the rows of each expert, or with group_list_type = 1 their counts); no static offsets.
void swiglu_quant_check(const Tensor &x, const optional<Tensor> &smooth_scales, const optional<Tensor> &offsets,
                        const optional<Tensor> &group_index, int64_t quant_mode, int64_t group_list_type,
                        optional<at::ScalarType> dst_type)
{
    TORCH_CHECK(x.scalar_type() == at::kBFloat16, "npu_swiglu_quant: only bfloat16 input is supported, got ", x.scalar_type());
    TORCH_CHECK(x.dim() >= 1 && x.size(-1) % 2 == 0, "npu_swiglu_quant: the last dimension must be even");
    if (const Tensor *sm = opt(smooth_scales)) {
        TORCH_CHECK(sm->scalar_type() == at::kBFloat16, "npu_swiglu_quant: smooth_scales must be bfloat16 like x, got ",
                    sm->scalar_type());
        if (const Tensor *g = opt(group_index)) {
            TORCH_CHECK(sm->dim() == 2 && sm->size(0) == g->numel() && sm->size(1) == x.size(-1) / 2,
                        "npu_swiglu_quant: with group_index, smooth_scales must have shape [", g->numel(), ", ", x.size(-1) / 2,
                        "], got ", sm->sizes());
        } else {
            TORCH_CHECK(sm->dim() == 1 && sm->size(0) == x.size(-1) / 2, "npu_swiglu_quant: smooth_scales must have shape [",
                        x.size(-1) / 2, "] (one per output column), got ", sm->sizes());
        }
    }
    TORCH_CHECK(!opt(offsets), "npu_swiglu_quant: offsets (static quantisation) is not supported");
    if (const Tensor *g = opt(group_index)) {
        TORCH_CHECK(opt(smooth_scales), "npu_swiglu_quant: group_index needs smooth_scales of shape [experts, ", x.size(-1) / 2, "]");
        TORCH_CHECK((g->scalar_type() == at::kInt || g->scalar_type() == at::kLong) && g->dim() == 1 && g->numel() >= 1,
                    "npu_swiglu_quant: group_index must be an int32 or int64 vector [experts]");
    }
    TORCH_CHECK(quant_mode == 1, "npu_swiglu_quant: only quant_mode=1 (dynamic per-token quantisation) is supported, got ",
                quant_mode);
    TORCH_CHECK(group_list_type == 0 || group_list_type == 1, "npu_swiglu_quant: group_list_type must be 0 (running totals) or 1 (counts)");
    TORCH_CHECK(!dst_type.has_value() || *dst_type == at::kChar, "npu_swiglu_quant: only dst_type=torch.int8 is supported");
}

std::tuple<Tensor, Tensor> swiglu_quant_alloc(const Tensor &x)
{
    auto shape = x.sizes().vec();
    shape.back() /= 2;
    auto scale_shape = shape;
    scale_shape.pop_back();
    return {at::empty(shape, x.options().dtype(at::kChar)), at::empty(scale_shape, x.options().dtype(at::kFloat))};
}

std::tuple<Tensor, Tensor> swiglu_quant_meta(const Tensor &x, const optional<Tensor> &smooth_scales,
                                             const optional<Tensor> &offsets, const optional<Tensor> &group_index,
                                             bool activate_left, int64_t quant_mode, int64_t group_list_type,
                                             optional<at::ScalarType> dst_type)
{
    (void)activate_left;
    swiglu_quant_check(x, smooth_scales, offsets, group_index, quant_mode, group_list_type, dst_type);
    return swiglu_quant_alloc(x);
}

std::tuple<Tensor, Tensor> swiglu_quant_hip(const Tensor &x, const optional<Tensor> &smooth_scales,
                                            const optional<Tensor> &offsets, const optional<Tensor> &group_index,
                                            bool activate_left, int64_t quant_mode, int64_t group_list_type,
                                            optional<at::ScalarType> dst_type)
{
    swiglu_quant_check(x, smooth_scales, offsets, group_index, quant_mode, group_list_type, dst_type);
    check_same_device("npu_swiglu_quant", {&x, opt(smooth_scales), opt(group_index)});
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    auto [y, scale] = swiglu_quant_alloc(x);
    const int64_t half = x.size(-1) / 2;
    const int64_t rows = half ? y.numel() / half : 0;
    if (rows == 0 || half == 0) {
        scale.zero_();
        return {y, scale};
    }
    Tensor xin = x;
    int64_t row_stride = 2 * half;
    if (xin.dim() == 2 && xin.stride(1) == 1 && xin.stride(0) >= 2 * half) {
        row_stride = xin.stride(0);
    } else if (!xin.is_contiguous()) {
        xin = xin.contiguous();
    }
    if (const Tensor *g = opt(group_index)) {
        Tensor sm = opt(smooth_scales)->contiguous();
        Tensor gi = (group_list_type == 1 ? g->cumsum(0) : *g).to(at::kInt).contiguous();     // counts -> running totals
        check_status(mi355_swiglu_quant_grouped(xin.data_ptr(), activate_left ? 1 : 0, sm.data_ptr(), gi.data_ptr<int32_t>(),
                                                gi.numel(), y.data_ptr<int8_t>(), scale.data_ptr<float>(), rows, half, row_stride,
                                                stream_of(x)),
                     "npu_swiglu_quant");
        return {y, scale};
    }
    if (const Tensor *smp = opt(smooth_scales)) {
        Tensor sm = smp->contiguous();
        check_status(mi355_swiglu_quant_smooth(xin.data_ptr(), activate_left ? 1 : 0, sm.data_ptr(), y.data_ptr<int8_t>(),
                                               scale.data_ptr<float>(), rows, half, row_stride, stream_of(x)),
                     "npu_swiglu_quant");
        return {y, scale};
    }
    check_status(mi355_swiglu_quant(xin.data_ptr(), activate_left ? 1 : 0, y.data_ptr<int8_t>(), scale.data_ptr<float>(), rows,
                                    half, row_stride, stream_of(x)),
                 "npu_swiglu_quant");
    return {y, scale};
}

// ---------------------------------------------------------------- npu_anti_quant
// torch_npu.npu_anti_quant(x, scale, *, offset=None, dst_dtype=None, src_dtype=None)
// (test/torch_npu_schema.json:2117-2119; golden test/custom_ops/test_npu_anti_quant.py:29-42)

at::ScalarType anti_quant_check(const Tensor &x, const Tensor &scale, const optional<Tensor> &offset,
                                optional<at::ScalarType> dst_dtype, optional<at::ScalarType> src_dtype)
{
    TORCH_CHECK(x.scalar_type() == at::kChar || x.scalar_type() == at::kInt,
                "npu_anti_quant: x must be int8 or int32 (packed int4), got ", x.scalar_type());
    TORCH_CHECK(x.dim() >= 1, "npu_anti_quant: x must have at least one dimension");
    TORCH_CHECK(!src_dtype.has_value() || *src_dtype == at::kChar, "npu_anti_quant: src_dtype must be torch.int8");
    const at::ScalarType dst = dst_dtype.value_or(at::kHalf);
    TORCH_CHECK(dst == at::kHalf || dst == at::kBFloat16, "npu_anti_quant: dst_dtype must be torch.float16 or torch.bfloat16");
    const int64_t cols = x.size(-1) * (x.scalar_type() == at::kInt ? 8 : 1);
    TORCH_CHECK(scale.scalar_type() == at::kFloat, "npu_anti_quant: scale must be float32, got ", scale.scalar_type());
    TORCH_CHECK(scale.dim() <= 1 && (scale.numel() == cols || scale.numel() == 1),
                "npu_anti_quant: scale must have one element or one per element of the last dimension (", cols, ")");
    if (const Tensor *o = opt(offset)) {
        TORCH_CHECK(o->scalar_type() == at::kFloat, "npu_anti_quant: offset must be float32, got ", o->scalar_type());
        TORCH_CHECK(o->dim() <= 1 && (o->numel() == cols || o->numel() == 1),
                    "npu_anti_quant: offset must have one element or one per element of the last dimension (", cols, ")");
    }
    return dst;
}

Tensor anti_quant_meta(const Tensor &x, const Tensor &scale, const optional<Tensor> &offset,
                       optional<at::ScalarType> dst_dtype, optional<at::ScalarType> src_dtype)
{
    const at::ScalarType dst = anti_quant_check(x, scale, offset, dst_dtype, src_dtype);
    auto shape = x.sizes().vec();
    if (x.scalar_type() == at::kInt) shape.back() *= 8;
    return at::empty(shape, x.options().dtype(dst));
}

Tensor anti_quant_hip(const Tensor &x, const Tensor &scale, const optional<Tensor> &offset,
                      optional<at::ScalarType> dst_dtype, optional<at::ScalarType> src_dtype)
{
    check_same_device("npu_anti_quant", {&x, &scale, opt(offset)});
    Tensor out = anti_quant_meta(x, scale, offset, dst_dtype, src_dtype);
    if (out.numel() == 0) return out;
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    Tensor xin = x.contiguous(), sc = scale.contiguous();
    Tensor of = opt(offset) ? opt(offset)->contiguous() : Tensor();
    const int64_t cols = out.size(-1), rows = out.numel() / cols;
    const bool int4 = x.scalar_type() == at::kInt;
    check_status(mi355_anti_quant(xin.data_ptr(), int4 ? 4 : 8, sc.data_ptr<float>(), sc.numel(),
                                  of.defined() ? of.data_ptr<float>() : nullptr, of.defined() ? of.numel() : 0, out.data_ptr(),
                                  out.scalar_type() == at::kHalf ? MI355_DTYPE_FP16 : MI355_DTYPE_BF16, rows, cols,
                                  int4 ? cols / 8 : cols, cols, stream_of(x)),
                 "npu_anti_quant");
    return out;
}


// ---------------------------------------------------------------- npu_quantize
// torch_npu.npu_quantize(inputs, scales, zero_points, dtype, axis, div_mode=True)
// (test/torch_npu_schema.json:2273-2275; torch_npu/onnx/wrapper_onnx_ops.py:855-877 names the output types:
// torch.qint8 -> int8, torch.quint8 -> uint8, torch.qint32 -> int32)

struct QuantizePlan {
    at::ScalarType out;
    int out_code;
    int64_t axis, outer, channels, inner;
};

QuantizePlan quantize_check(const Tensor &x, const Tensor &scales, const optional<Tensor> &zero_points, at::ScalarType dtype,
                            int64_t axis)
{
    QuantizePlan pl{};
    TORCH_CHECK(x.scalar_type() == at::kBFloat16 || x.scalar_type() == at::kHalf || x.scalar_type() == at::kFloat,
                "npu_quantize: inputs must be float32, float16 or bfloat16, got ", x.scalar_type());
    if (dtype == at::kQInt8 || dtype == at::kChar) pl.out = at::kChar, pl.out_code = MI355_Q_INT8;
    else if (dtype == at::kQUInt8 || dtype == at::kByte) pl.out = at::kByte, pl.out_code = MI355_Q_UINT8;
    else if (dtype == at::kQInt32 || dtype == at::kInt) pl.out = at::kInt, pl.out_code = MI355_Q_INT32;
    else TORCH_CHECK(false, "npu_quantize: dtype must be torch.qint8, torch.quint8 or torch.qint32, got ", dtype);
    const int64_t nd = x.dim();
    TORCH_CHECK(nd >= 1, "npu_quantize: inputs must have at least one dimension");
    TORCH_CHECK(axis >= -nd && axis < nd, "npu_quantize: axis ", axis, " out of range for ", nd, " dimensions");
    pl.axis = axis < 0 ? axis + nd : axis;
    pl.channels = x.size(pl.axis);
    pl.outer = 1;
    pl.inner = 1;
    for (int64_t d = 0; d < pl.axis; d++) pl.outer *= x.size(d);
    for (int64_t d = pl.axis + 1; d < nd; d++) pl.inner *= x.size(d);
    TORCH_CHECK(scales.dim() <= 1 && (scales.numel() == 1 || scales.numel() == pl.channels),
                "npu_quantize: scales must have one element or one per element of dimension ", pl.axis, " (", pl.channels, ")");
    TORCH_CHECK(at::isFloatingType(scales.scalar_type()), "npu_quantize: scales must be a floating-point tensor");
    if (const Tensor *z = opt(zero_points)) {
        TORCH_CHECK(z->dim() <= 1 && (z->numel() == 1 || z->numel() == pl.channels),
                    "npu_quantize: zero_points must have one element or one per element of dimension ", pl.axis, " (",
                    pl.channels, ")");
        TORCH_CHECK(z->scalar_type() != at::kBool && !at::isComplexType(z->scalar_type()),
                    "npu_quantize: zero_points must be an integer or floating-point tensor");
    }
    return pl;
}

Tensor quantize_meta(const Tensor &x, const Tensor &scales, const optional<Tensor> &zero_points, at::ScalarType dtype,
                     int64_t axis, bool div_mode)
{
    (void)div_mode;
    const QuantizePlan pl = quantize_check(x, scales, zero_points, dtype, axis);
    return at::empty(x.sizes(), x.options().dtype(pl.out));
}

Tensor quantize_hip(const Tensor &x, const Tensor &scales, const optional<Tensor> &zero_points, at::ScalarType dtype,
                    int64_t axis, bool div_mode)
{
    check_same_device("npu_quantize", {&x, &scales, opt(zero_points)});
    const QuantizePlan pl = quantize_check(x, scales, zero_points, dtype, axis);
    Tensor out = at::empty(x.sizes(), x.options().dtype(pl.out));
    if (out.numel() == 0) return out;
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    Tensor xin = x.contiguous();
    Tensor sc = scales.to(at::kFloat).contiguous();            // a few hundred to a few thousand elements
    Tensor zp;                                                 // int32 and float32 zero points go to the kernel as they are
    if (const Tensor *z = opt(zero_points))
        zp = (z->scalar_type() == at::kInt || z->scalar_type() == at::kFloat ? *z : z->to(at::kFloat)).contiguous();
    const int in_code = x.scalar_type() == at::kBFloat16 ? MI355_DTYPE_BF16
                        : x.scalar_type() == at::kHalf   ? MI355_DTYPE_FP16
                                                         : MI355_DTYPE_FP32;
    check_status(mi355_quantize(xin.data_ptr(), in_code, sc.data_ptr<float>(), sc.numel(),
                                zp.defined() ? zp.data_ptr() : nullptr,
                                zp.defined() && zp.scalar_type() == at::kInt ? MI355_DTYPE_INT32 : MI355_DTYPE_FP32,
                                zp.defined() ? zp.numel() : 0, out.data_ptr(),
                                pl.out_code, pl.outer, pl.channels, pl.inner, div_mode ? 1 : 0, stream_of(x)),
                 "npu_quantize");
    return out;
}

} // namespace

TORCH_LIBRARY_FRAGMENT(npu, m)
{
    m.def("npu_dynamic_quant(Tensor input, *, Tensor? smooth_scales=None, Tensor? group_index=None, "
          "ScalarType? dst_type=None) -> (Tensor, Tensor)");
    m.def("npu_dynamic_quant_asymmetric(Tensor input, *, Tensor? smooth_scales=None, Tensor? group_index=None, "
          "ScalarType? dst_type=None) -> (Tensor, Tensor, Tensor)");
    m.def("npu_quant_matmul(Tensor x1, Tensor x2, Tensor scale, *, Tensor? offset=None, Tensor? pertoken_scale=None, "
          "Tensor? bias=None, ScalarType? output_dtype=None) -> Tensor");
    m.def("npu_weight_quant_batchmatmul(Tensor x, Tensor weight, Tensor antiquant_scale, Tensor? antiquant_offset=None, "
          "Tensor? quant_scale=None, Tensor? quant_offset=None, Tensor? bias=None, int antiquant_group_size=0, "
          "int inner_precise=0, *, ScalarType? weight_dtype=None) -> Tensor");
    m.def("npu_swiglu(Tensor input, int dim=-1) -> Tensor");
    m.def("npu_swiglu_quant(Tensor x, *, Tensor? smooth_scales=None, Tensor? offsets=None, Tensor? group_index=None, "
          "bool activate_left=False, int quant_mode=0, int group_list_type=0, ScalarType? dst_type=None) -> (Tensor, Tensor)");
    m.def("npu_anti_quant(Tensor x, Tensor scale, *, Tensor? offset=None, ScalarType? dst_dtype=None, "
          "ScalarType? src_dtype=None) -> Tensor");
    m.def("npu_trans_quant_param(Tensor scale, Tensor? offset=None) -> Tensor");
    m.def("npu_quantize(Tensor inputs, Tensor scales, Tensor? zero_points, ScalarType dtype, int axis=1, "
          "bool div_mode=True) -> Tensor");
}

TORCH_LIBRARY_IMPL(npu, CUDA, m)
{
    m.impl("npu_dynamic_quant", TORCH_FN(dynamic_quant_hip));
    m.impl("npu_dynamic_quant_asymmetric", TORCH_FN(dynamic_quant_asym_hip));
    m.impl("npu_quant_matmul", TORCH_FN(quant_matmul_hip));
    m.impl("npu_weight_quant_batchmatmul", TORCH_FN(weight_quant_hip));
    m.impl("npu_swiglu", TORCH_FN(swiglu_hip));
    m.impl("npu_swiglu_quant", TORCH_FN(swiglu_quant_hip));
    m.impl("npu_anti_quant", TORCH_FN(anti_quant_hip));
    m.impl("npu_quantize", TORCH_FN(quantize_hip));
    m.impl("npu_trans_quant_param", TORCH_FN(trans_quant_param_hip));
}

TORCH_LIBRARY_IMPL(npu, Meta, m)
{
    m.impl("npu_dynamic_quant", TORCH_FN(dynamic_quant_meta));
    m.impl("npu_dynamic_quant_asymmetric", TORCH_FN(dynamic_quant_asym_meta));
    m.impl("npu_quant_matmul", TORCH_FN(quant_matmul_meta));
    m.impl("npu_weight_quant_batchmatmul", TORCH_FN(weight_quant_meta));
    m.impl("npu_swiglu", TORCH_FN(swiglu_meta));
    m.impl("npu_swiglu_quant", TORCH_FN(swiglu_quant_meta));
    m.impl("npu_anti_quant", TORCH_FN(anti_quant_meta));
    m.impl("npu_quantize", TORCH_FN(quantize_meta));
    m.impl("npu_trans_quant_param", TORCH_FN(trans_quant_param_meta));
}

// Reads the status word of every workspace kept for eager launches (synchronises their streams); throws c10::Error if a
// kernel reported a failure.  Exported with C linkage for the Python package (pytorch_amd.check_device_status()).
extern "C" int mi355_npu_check_workspaces(void)
{
    WorkspaceCache &wc = workspace_cache();
    std::vector<std::pair<std::pair<int, void *>, Tensor>> all;
    {
        std::lock_guard<std::mutex> lock(wc.mu);
        for (auto &kv : wc.eager)
            if (kv.second.defined()) all.emplace_back(kv.first, kv.second);
        for (auto &kv : wc.retired) all.push_back(kv);
    }
    int failures = 0;
    for (auto &kv : all) {
        c10::hip::HIPGuardMasqueradingAsCUDA guard(kv.second.device());
        if (mi355_workspace_status(kv.second.data_ptr(), (size_t)kv.second.numel(), 1, kv.first.second) != MI355_OK) failures++;
    }
    return failures;
}
