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

// Runs call(i) for step k on tensor set i = k % sets between two events on `stream`.
// Returns 0 on success, else the failing aclnn status (or -1 for a HIP error).
// event_ms: GPU time between the two events; wall_ms: host time from first call to completed sync.
template <typename Call>
int timed_loop(int sets, int steps, void* stream, double* event_ms, double* wall_ms, Call call)
{
    hipStream_t s = (hipStream_t)stream;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        return -1;
    }
    if (hipStreamSynchronize(s) != hipSuccess) {
        return -1;
    }
    auto t0 = std::chrono::steady_clock::now();
    (void)hipEventRecord(e0, s);
    for (int k = 0; k < steps; k++) {
        const aclnnStatus st = call(k % sets);
        if (st != ACLNN_SUCCESS) {
            return st;
        }
    }
    (void)hipEventRecord(e1, s);
    if (hipEventSynchronize(e1) != hipSuccess) {
        return -1;
    }
    auto t1 = std::chrono::steady_clock::now();
    float ms = 0.0f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    *event_ms = ms;
    *wall_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return 0;
}

}  // namespace

#define OPSCV_BENCH_API extern "C" __attribute__((visibility("default")))

OPSCV_BENCH_API int opscv_bench_grid_sampler2d(const aclTensor* const* inputs, const aclTensor* const* grids,
                                               aclTensor* const* outs, int sets, int64_t interp, int64_t pad,
                                               bool align, void* workspace, uint64_t workspace_size, int steps,
                                               void* stream, double* event_ms, double* wall_ms)
{
    return timed_loop(sets, steps, stream, event_ms, wall_ms, [&](int i) {
        uint64_t ws = 0;
        aclOpExecutor* ex = nullptr;
        aclnnStatus st = aclnnGridSampler2DGetWorkspaceSize(inputs[i], grids[i], interp, pad, align, outs[i], &ws, &ex);
        return st != ACLNN_SUCCESS ? st : aclnnGridSampler2D(workspace, workspace_size, ex, stream);
    });
}

OPSCV_BENCH_API int opscv_bench_grid_sampler2d_backward(const aclTensor* const* gouts, const aclTensor* const* inputs,
                                                        const aclTensor* const* grids, aclTensor* const* dxs,
                                                        aclTensor* const* dgrids, int sets, int64_t interp,
                                                        int64_t pad, bool align, const aclBoolArray* mask,
                                                        void* workspace, uint64_t workspace_size, int steps,
                                                        void* stream, double* event_ms, double* wall_ms)
{
    return timed_loop(sets, steps, stream, event_ms, wall_ms, [&](int i) {
        uint64_t ws = 0;
        aclOpExecutor* ex = nullptr;
        aclnnStatus st = aclnnGridSampler2DBackwardGetWorkspaceSize(gouts[i], inputs[i], grids[i], interp, pad, align,
                                                                    mask, dxs[i], dgrids[i], &ws, &ex);
        return st != ACLNN_SUCCESS ? st : aclnnGridSampler2DBackward(workspace, workspace_size, ex, stream);
    });
}

OPSCV_BENCH_API int opscv_bench_grid_sampler3d_backward(const aclTensor* const* gouts, const aclTensor* const* inputs,
                                                        const aclTensor* const* grids, aclTensor* const* dxs,
                                                        aclTensor* const* dgrids, int sets, int64_t interp,
                                                        int64_t pad, bool align, const aclBoolArray* mask,
                                                        void* workspace, uint64_t workspace_size, int steps,
                                                        void* stream, double* event_ms, double* wall_ms)
{
    return timed_loop(sets, steps, stream, event_ms, wall_ms, [&](int i) {
        uint64_t ws = 0;
        aclOpExecutor* ex = nullptr;
        aclnnStatus st = aclnnGridSampler3DBackwardGetWorkspaceSize(gouts[i], inputs[i], grids[i], interp, pad, align,
                                                                    mask, dxs[i], dgrids[i], &ws, &ex);
        return st != ACLNN_SUCCESS ? st : aclnnGridSampler3DBackward(workspace, workspace_size, ex, stream);
    });
}

OPSCV_BENCH_API int opscv_bench_grid_sampler3d(const aclTensor* const* inputs, const aclTensor* const* grids,
                                               aclTensor* const* outs, int sets, int64_t interp, int64_t pad,
                                               bool align, void* workspace, uint64_t workspace_size, int steps,
                                               void* stream, double* event_ms, double* wall_ms)
{
    return timed_loop(sets, steps, stream, event_ms, wall_ms, [&](int i) {
        uint64_t ws = 0;
        aclOpExecutor* ex = nullptr;
        aclnnStatus st = aclnnGridSampler3DGetWorkspaceSize(inputs[i], grids[i], interp, pad, align, outs[i], &ws, &ex);
        return st != ACLNN_SUCCESS ? st : aclnnGridSampler3D(workspace, workspace_size, ex, stream);
    });
}

OPSCV_BENCH_API int opscv_bench_upsample_bilinear2d(const aclTensor* const* selfs, aclTensor* const* outs, int sets,
                                                    const aclIntArray* output_size, bool align, double scales_h,
                                                    double scales_w, void* workspace, uint64_t workspace_size,
                                                    int steps, void* stream, double* event_ms, double* wall_ms)
{
    return timed_loop(sets, steps, stream, event_ms, wall_ms, [&](int i) {
        uint64_t ws = 0;
        aclOpExecutor* ex = nullptr;
        aclnnStatus st = aclnnUpsampleBilinear2dGetWorkspaceSize(selfs[i], output_size, align, scales_h, scales_w,
                                                                 outs[i], &ws, &ex);
        return st != ACLNN_SUCCESS ? st : aclnnUpsampleBilinear2d(workspace, workspace_size, ex, stream);
    });
}

OPSCV_BENCH_API int opscv_bench_upsample_bilinear2d_backward(const aclTensor* const* grads, aclTensor* const* outs,
                                                             int sets, const aclIntArray* output_size,
                                                             const aclIntArray* input_size, bool align,
                                                             double scales_h, double scales_w, void* workspace,
                                                             uint64_t workspace_size, int steps, void* stream,
                                                             double* event_ms, double* wall_ms)
{
    return timed_loop(sets, steps, stream, event_ms, wall_ms, [&](int i) {
        uint64_t ws = 0;
        aclOpExecutor* ex = nullptr;
        aclnnStatus st = aclnnUpsampleBilinear2dBackwardGetWorkspaceSize(grads[i], output_size, input_size, align,
                                                                         scales_h, scales_w, outs[i], &ws, &ex);
        return st != ACLNN_SUCCESS ? st : aclnnUpsampleBilinear2dBackward(workspace, workspace_size, ex, stream);
    });
}

OPSCV_BENCH_API int opscv_bench_resize(const aclTensor* const* selfs, aclTensor* const* outs, int sets,
                                       const aclFloatArray* scales, const char* mode, void* workspace,
                                       uint64_t workspace_size, int steps, void* stream, double* event_ms,
                                       double* wall_ms)
{
    return timed_loop(sets, steps, stream, event_ms, wall_ms, [&](int i) {
        uint64_t ws = 0;
        aclOpExecutor* ex = nullptr;
        aclnnStatus st = aclnnResizeGetWorkspaceSize(selfs[i], scales, mode, outs[i], &ws, &ex);
        return st != ACLNN_SUCCESS ? st : aclnnResize(workspace, workspace_size, ex, stream);
    });
}
