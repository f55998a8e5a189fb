// Benchmark driver loops (built into libopscv_bench.so, used by bench.py only).
//
// Each loop issues `steps` full two-phase calls through the public C-ABI back to back on one stream, rotating
// over `sets` independent tensor sets so that consecutive steps do not find their operands in the last-level
// cache, and brackets the whole sequence with HIP events recorded on that same stream.
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstdint>

#include "aclnn_grid_sampler2d.h"
#include "aclnn_grid_sampler2d_backward.h"
#include "aclnn_grid_sampler3d_backward.h"
#include "aclnn_grid_sampler3d.h"
#include "aclnn_resize.h"
#include "aclnn_upsample_bilinear_2d.h"
#include "aclnn_upsample_bilinear_2d_backward.h"

namespace {

// host time spent inside the two phases by the last loop, and the per-launch event timings of its last pass
double g_phase1_us = 0.0, g_phase2_us = 0.0;

struct EventPair {
    hipEvent_t e0 = nullptr, e1 = nullptr;
    bool ok = false;
    EventPair() { ok = hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess; }
    ~EventPair()
    {
        if (e0 != nullptr) {
            (void)hipEventDestroy(e0);
        }
        if (e1 != nullptr) {
            (void)hipEventDestroy(e1);
        }
    }
};

// Issues `warm` untimed steps, waits for the stream to drain, and then times `steps` steps: plan(i) + run(executor)
// for step k on tensor set i = k % sets between two events on `stream`.  The warm-up runs inside this call so that
// nothing but the synchronisation lies between it and the timed region (instruction caches of the host path warm,
// clocks of the device up).
// Returns 0 on success, else the failing aclnn status (or -1 for a HIP error).
// event_ms: GPU time between the two events; wall_ms: host time from first call to completed sync.
// The host time inside the first phase (validation and planning) and inside the second phase (kernel launches, which
// return before the kernels run) is accumulated per step and kept for opscv_bench_host_us().
template <typename Plan, typename Run>
int timed_loop(int sets, int warm, int steps, void* stream, double* event_ms, double* wall_ms, Plan plan, Run run)
{
    using clock = std::chrono::steady_clock;
    hipStream_t s = (hipStream_t)stream;
    EventPair ev;  // destroyed on every return path
    if (!ev.ok) {
        return -1;
    }
    for (int k = 0; k < warm; k++) {
        aclOpExecutor* ex = nullptr;
        aclnnStatus st = plan((steps + k) % sets, &ex);
        if (st == ACLNN_SUCCESS) {
            st = run(ex);
        }
        if (st != ACLNN_SUCCESS) {
            return st;
        }
    }
    if (hipStreamSynchronize(s) != hipSuccess) {
        return -1;
    }
    std::chrono::nanoseconds in_plan{0}, in_run{0};
    auto t0 = clock::now();
    (void)hipEventRecord(ev.e0, s);
    for (int k = 0; k < steps; k++) {
        aclOpExecutor* ex = nullptr;
        const auto ta = clock::now();
        aclnnStatus st = plan(k % sets, &ex);
        const auto tb = clock::now();
        if (st != ACLNN_SUCCESS) {
            return st;
        }
        st = run(ex);
        const auto tc = clock::now();
        if (st != ACLNN_SUCCESS) {
            return st;
        }
        in_plan += tb - ta;
        in_run += tc - tb;
    }
    (void)hipEventRecord(ev.e1, s);
    if (hipEventSynchronize(ev.e1) != hipSuccess) {
        return -1;
    }
    auto t1 = clock::now();
    float ms = 0.0f;
    (void)hipEventElapsedTime(&ms, ev.e0, ev.e1);
    *event_ms = ms;
    *wall_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    g_phase1_us = std::chrono::duration<double, std::micro>(in_plan).count() / (steps > 0 ? steps : 1);
    g_phase2_us = std::chrono::duration<double, std::micro>(in_run).count() / (steps > 0 ? steps : 1);
    return 0;
}

}  // namespace

#define OPSCV_BENCH_API extern "C" __attribute__((visibility("default")))

OPSCV_BENCH_API int opscv_bench_grid_sampler2d(const aclTensor* const* inputs, const aclTensor* const* grids,
                                               aclTensor* const* outs, int sets, int64_t interp, int64_t pad,
                                               bool align, void* workspace, uint64_t workspace_size, int warm, int steps,
                                               void* stream, double* event_ms, double* wall_ms)
{
    return timed_loop(
        sets, warm, steps, stream, event_ms, wall_ms,
        [&](int i, aclOpExecutor** ex) {
            uint64_t ws = 0;
            return aclnnGridSampler2DGetWorkspaceSize(inputs[i], grids[i], interp, pad, align, outs[i], &ws, ex);
        },
        [&](aclOpExecutor* ex) { return aclnnGridSampler2D(workspace, workspace_size, ex, stream); });
}

OPSCV_BENCH_API int opscv_bench_grid_sampler2d_backward(const aclTensor* const* gouts, const aclTensor* const* inputs,
                                                        const aclTensor* const* grids, aclTensor* const* dxs,
                                                        aclTensor* const* dgrids, int sets, int64_t interp,
                                                        int64_t pad, bool align, const aclBoolArray* mask,
                                                        void* workspace, uint64_t workspace_size, int warm, int steps,
                                                        void* stream, double* event_ms, double* wall_ms)
{
    return timed_loop(
        sets, warm, steps, stream, event_ms, wall_ms,
        [&](int i, aclOpExecutor** ex) {
            uint64_t ws = 0;
            return aclnnGridSampler2DBackwardGetWorkspaceSize(gouts[i], inputs[i], grids[i], interp, pad, align,
                                                                    mask, dxs[i], dgrids[i], &ws, ex);
        },
        [&](aclOpExecutor* ex) { return aclnnGridSampler2DBackward(workspace, workspace_size, ex, stream); });
}

OPSCV_BENCH_API int opscv_bench_grid_sampler3d_backward(const aclTensor* const* gouts, const aclTensor* const* inputs,
                                                        const aclTensor* const* grids, aclTensor* const* dxs,
                                                        aclTensor* const* dgrids, int sets, int64_t interp,
                                                        int64_t pad, bool align, const aclBoolArray* mask,
                                                        void* workspace, uint64_t workspace_size, int warm, int steps,
                                                        void* stream, double* event_ms, double* wall_ms)
{
    return timed_loop(
        sets, warm, steps, stream, event_ms, wall_ms,
        [&](int i, aclOpExecutor** ex) {
            uint64_t ws = 0;
            return aclnnGridSampler3DBackwardGetWorkspaceSize(gouts[i], inputs[i], grids[i], interp, pad, align,
                                                                    mask, dxs[i], dgrids[i], &ws, ex);
        },
        [&](aclOpExecutor* ex) { return aclnnGridSampler3DBackward(workspace, workspace_size, ex, stream); });
}

OPSCV_BENCH_API int opscv_bench_grid_sampler3d(const aclTensor* const* inputs, const aclTensor* const* grids,
                                               aclTensor* const* outs, int sets, int64_t interp, int64_t pad,
                                               bool align, void* workspace, uint64_t workspace_size, int warm, int steps,
                                               void* stream, double* event_ms, double* wall_ms)
{
    return timed_loop(
        sets, warm, steps, stream, event_ms, wall_ms,
        [&](int i, aclOpExecutor** ex) {
            uint64_t ws = 0;
            return aclnnGridSampler3DGetWorkspaceSize(inputs[i], grids[i], interp, pad, align, outs[i], &ws, ex);
        },
        [&](aclOpExecutor* ex) { return aclnnGridSampler3D(workspace, workspace_size, ex, stream); });
}

OPSCV_BENCH_API int opscv_bench_upsample_bilinear2d(const aclTensor* const* selfs, aclTensor* const* outs, int sets,
                                                    const aclIntArray* output_size, bool align, double scales_h,
                                                    double scales_w, void* workspace, uint64_t workspace_size,
                                                    int warm, int steps, void* stream, double* event_ms,
                                                    double* wall_ms)
{
    return timed_loop(
        sets, warm, steps, stream, event_ms, wall_ms,
        [&](int i, aclOpExecutor** ex) {
            uint64_t ws = 0;
            return aclnnUpsampleBilinear2dGetWorkspaceSize(selfs[i], output_size, align, scales_h, scales_w,
                                                                 outs[i], &ws, ex);
        },
        [&](aclOpExecutor* ex) { return aclnnUpsampleBilinear2d(workspace, workspace_size, ex, stream); });
}

OPSCV_BENCH_API int opscv_bench_upsample_bilinear2d_backward(const aclTensor* const* grads, aclTensor* const* outs,
                                                             int sets, const aclIntArray* output_size,
                                                             const aclIntArray* input_size, bool align,
                                                             double scales_h, double scales_w, void* workspace,
                                                             uint64_t workspace_size, int warm, int steps, void* stream,
                                                             double* event_ms, double* wall_ms)
{
    return timed_loop(
        sets, warm, steps, stream, event_ms, wall_ms,
        [&](int i, aclOpExecutor** ex) {
            uint64_t ws = 0;
            return aclnnUpsampleBilinear2dBackwardGetWorkspaceSize(grads[i], output_size, input_size, align,
                                                                         scales_h, scales_w, outs[i], &ws, ex);
        },
        [&](aclOpExecutor* ex) { return aclnnUpsampleBilinear2dBackward(workspace, workspace_size, ex, stream); });
}

OPSCV_BENCH_API int opscv_bench_resize(const aclTensor* const* selfs, aclTensor* const* outs, int sets,
                                       const aclFloatArray* scales, const char* mode, void* workspace,
                                       uint64_t workspace_size, int warm, int steps, void* stream, double* event_ms,
                                       double* wall_ms)
{
    return timed_loop(
        sets, warm, steps, stream, event_ms, wall_ms,
        [&](int i, aclOpExecutor** ex) {
            uint64_t ws = 0;
            return aclnnResizeGetWorkspaceSize(selfs[i], scales, mode, outs[i], &ws, ex);
        },
        [&](aclOpExecutor* ex) { return aclnnResize(workspace, workspace_size, ex, stream); });
}

// Host microseconds per call spent inside the first phase (GetWorkspaceSize: validation + plan) and inside the second
// phase (the launches; the kernels themselves run asynchronously) during the last loop of this library.
OPSCV_BENCH_API void opscv_bench_host_us(double* phase1_us, double* phase2_us)
{
    *phase1_us = g_phase1_us;
    *phase2_us = g_phase2_us;
}
