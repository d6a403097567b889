// Tuning knobs of the planners.  A knob is an integer, 0 = let the planner decide.  Each knob takes its initial value
// from the environment variable of the same name once, when the library is loaded; afterwards only
// mi355_set_tuning() changes it, so no launch ever reads the environment.
#include "common.h"
#include <atomic>
#include <stdlib.h>
#include <string.h>

namespace mi355 {
namespace {
const char *const kKnobNames[kKnobCount] = {"MI355_WQ_SPLIT", "MI355_WQ_W",    "MI355_WQG_SPLIT", "MI355_WQG_BM",   "MI355_WQ_GEMM_OFF",
                                            "MI355_WQK_MT",   "MI355_WQK_NW",  "MI355_WQK_KS",    "MI355_QMM_SPLIT", "MI355_QMM_TILE",
                                            "MI355_WQ_DECODE_OFF", "MI355_QMM_DEEP_OFF", "MI355_WQ_GEMM4_OFF",
                                            "MI355_QMM_DECODE_OFF", "MI355_QMM_LOOP", "MI355_WQ_MAX_POLLS", "MI355_WQ_ONLY_CHUNK",
                                            "MI355_QMM_STREAM_OUT"};
std::atomic<int> g_knobs[kKnobCount];
const bool g_knobs_loaded = []() {
    for (int i = 0; i < kKnobCount; i++) {
        const char *e = getenv(kKnobNames[i]);
        int v = 0;
        if (e) {
            int bm = 0, bn = 0;
            v = (i == kKnobQmmTile && sscanf(e, "%dx%d", &bm, &bn) == 2) ? bm * 1000 + bn : atoi(e);
        }
        g_knobs[i].store(v, std::memory_order_relaxed);
    }
    return true;
}();
} // namespace

int knob(Knob k) { return g_knobs[k].load(std::memory_order_relaxed); }
} // namespace mi355

extern "C" int mi355_set_tuning(const char *name, int value)
{
    using namespace mi355;
    if (!name) return MI355_ERR_BAD_ARGUMENT;
    for (int i = 0; i < kKnobCount; i++)
        if (strcmp(name, kKnobNames[i]) == 0) {
            g_knobs[i].store(value, std::memory_order_relaxed);
            return MI355_OK;
        }
    return MI355_ERR_BAD_ARGUMENT;
}

// Identifier of the capture `stream` is part of (0 when it is not capturing): lets a host layer keep one workspace per
// capture without reaching into the HIP runtime itself.
extern "C" int mi355_stream_capture_id(void *stream, unsigned long long *id)
{
    if (!id) return MI355_ERR_BAD_ARGUMENT;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long cid = 0;
    if (hipStreamGetCaptureInfo(static_cast<hipStream_t>(stream), &status, &cid) != hipSuccess) return MI355_ERR_LAUNCH;
    *id = status == hipStreamCaptureStatusNone ? 0ull : cid;
    return MI355_OK;
}

extern "C" size_t mi355_workspace_zero_bytes(void) { return mi355::kWorkspaceZeroBytes; }

// The sticky status word of a workspace (common.h): read it once the stream has drained; with `reset`, clear the whole zero
// area of a workspace that reported a failure, because late stores of the producers the collector gave up on may have
// left non-zero words in the exchange zone.
extern "C" int mi355_workspace_status(void *workspace, size_t workspace_bytes, int reset, void *stream)
{
    using namespace mi355;
    if (!workspace || workspace_bytes < kWorkspaceCounterCapacity) return MI355_ERR_BAD_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint32_t word = 0;
    if (hipMemcpyAsync(&word, static_cast<char *>(workspace) + kWorkspaceStatusOffset, sizeof(word), hipMemcpyDeviceToHost, s) != hipSuccess)
        return MI355_ERR_LAUNCH;
    if (hipStreamSynchronize(s) != hipSuccess) return MI355_ERR_LAUNCH;
    if (word == 0) return MI355_OK;
    if (reset) {
        const size_t n = workspace_bytes < kWorkspaceZeroBytes ? workspace_bytes : kWorkspaceZeroBytes;
        if (hipMemsetAsync(workspace, 0, n, s) != hipSuccess || hipStreamSynchronize(s) != hipSuccess) return MI355_ERR_LAUNCH;
    }
    return MI355_ERR_DEVICE;
}
