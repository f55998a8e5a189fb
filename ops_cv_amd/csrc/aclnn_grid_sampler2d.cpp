// aclnnGridSampler2D: parameter validation, planning and the second-phase entry.
//
// Mirrors the checks, their order and their status codes of the reference implementation
// image/grid_sample/op_api/aclnn_grid_sampler2d.cpp:55-175,263-351.
#include <memory>
#include <new>

#include "aclnn_grid_sampler2d.h"
#include "executor.hpp"
#include "options.hpp"
#include "opscv_ext.h"

using namespace opscv;

namespace {

constexpr int64_t kSpatialDims = 4;

// aclnn_grid_sampler2d.cpp:78-92 : grid and out must match input's dtype; input's dtype must be in the list
bool check_dtypes(const aclTensor* input, const aclTensor* grid, const aclTensor* out)
{
    if (grid->dtype != input->dtype) {
        set_error("aclnnGridSampler2D: grid dtype %d differs from input dtype %d", (int)grid->dtype,
                  (int)input->dtype);
        return false;
    }
    if (out->dtype != input->dtype) {
        set_error("aclnnGridSampler2D: out dtype %d differs from input dtype %d", (int)out->dtype,
                  (int)input->dtype);
        return false;
    }
    switch (input->dtype) {
        case ACL_FLOAT:
        case ACL_FLOAT16:
        case ACL_BF16:
        case ACL_DOUBLE: return true;
        default: break;
    }
    set_error("aclnnGridSampler2D: dtype %d is not in {FLOAT, FLOAT16, BF16, DOUBLE}", (int)input->dtype);
    return false;
}

// aclnn_grid_sampler2d.cpp:94-110
// (N,C,H,W) view whose elements lie in memory as a dense (N,H,W,C) array
bool channels_last_dense(const aclTensor* t)
{
    const int64_t C = t->dims[1], H = t->dims[2], W = t->dims[3];
    const int64_t want[4] = {H * W * C, 1, W * C, C};
    for (int i = 0; i < 4; i++) {
        if (t->dims[i] != 1 && t->strides[i] != want[i]) {
            return false;
        }
    }
    return true;
}

bool check_attrs(int64_t interp, int64_t pad)
{
    if (interp < 0 || interp > 2) {
        set_error("interpolationMode %lld should be in support list {0(bilinear), 1(nearest), 2(bicubic)}.",
                  (long long)interp);
        return false;
    }
    if (pad < 0 || pad > 2) {
        set_error("paddingMode %lld should be in support list {0(zeros), 1(border), 2(reflection)}.",
                  (long long)pad);
        return false;
    }
    return true;
}

// aclnn_grid_sampler2d.cpp:112-157
bool check_shapes(const aclTensor* input, const aclTensor* grid, const aclTensor* out)
{
    if (input->ndim != kSpatialDims || grid->ndim != kSpatialDims || out->ndim != kSpatialDims) {
        set_error("aclnnGridSampler2D: input, grid and out must be 4-D, got %lld, %lld, %lld dims",
                  (long long)input->ndim, (long long)grid->ndim, (long long)out->ndim);
        return false;
    }
    if (input->dims[0] != grid->dims[0] || input->dims[0] != out->dims[0]) {
        set_error("expect input, grid and out to have same batch size");
        return false;
    }
    if (input->dims[1] != out->dims[1]) {
        set_error("expect input and out to have same channel size");
        return false;
    }
    if (grid->dims[1] != out->dims[2] || grid->dims[2] != out->dims[3]) {
        set_error("expect grid and out to have same H and W size");
        return false;
    }
    if (input->dims[2] == 0 || input->dims[3] == 0) {
        set_error("expect input to have non-empty spatial dimensions");
        return false;
    }
    if (grid->dims[3] != 2) {
        set_error("expect grid to have size 2 in last dimension");
        return false;
    }
    return true;
}

}  // namespace

namespace {

// Everything the first phase does except creating the executor: validation in the reference's order
// (aclnn_grid_sampler2d.cpp:159-175) and the plan, written into `ex`.
aclnnStatus plan_grid_sampler2d(const aclTensor* input, const aclTensor* grid, int64_t interpolationMode,
                                int64_t paddingMode, bool alignCorners, aclTensor* out, aclOpExecutor* ex)
{
    // 1. null pointers (aclnn_grid_sampler2d.cpp:55-61)
    if (input == nullptr || grid == nullptr || out == nullptr) {
        set_error("aclnnGridSampler2D: input, grid and out must not be NULL");
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    // 2. dtypes, 3. attributes, 4. shapes
    if (!check_dtypes(input, grid, out) || !check_attrs(interpolationMode, paddingMode) ||
        !check_shapes(input, grid, out)) {
        return ACLNN_ERR_PARAM_INVALID;
    }
    // empty tensors are a successful no-op that still hands out an executor (aclnn_grid_sampler2d.cpp:280-285)
    if (input->empty() || grid->empty()) {
        return ACLNN_SUCCESS;
    }
    // The reference routes DOUBLE to a host-CPU kernel that is not part of its tree; it does not exist here.
    Elem elem;
    if (!elem_of(input->dtype, &elem)) {
        set_error("aclnnGridSampler2D: DOUBLE tensors are not supported by the MI355X implementation");
        return ACLNN_ERR_PARAM_INVALID;
    }
    for (int i = 0; i < 4; i++) {
        if (input->dims[i] > INT32_MAX || grid->dims[i] > INT32_MAX) {
            set_error("aclnnGridSampler2D: every extent must fit in int32");
            return ACLNN_ERR_PARAM_INVALID;
        }
    }
    if (input->dims[2] * input->dims[3] > INT32_MAX) {
        set_error("aclnnGridSampler2D: Hin*Win must fit in int32");
        return ACLNN_ERR_PARAM_INVALID;
    }

    ex->kind = OpKind::GridSampler2D;
    GridSamplerArgs& a = ex->gs;
    // the process-wide options as they are now; the second phase runs with these whatever is set in between
    const Options opt = current_options();
    a.force_variant = opt.gs_variant;
    // the second coordinate rule exists for the bilinear mode only (the reference's arch35 GridSample kernel is
    // bilinear; its nearest and bicubic modes take other kernels, which are not mirrored)
    a.rule = (interpolationMode == 0) ? opt.grid_sampler2d_rule : kRuleGridSampler2D;
    a.elem = elem;
    a.interp = (int)interpolationMode;
    a.pad = (int)paddingMode;
    a.align = alignCorners ? 1 : 0;
    a.N = input->dims[0];
    a.C = input->dims[1];
    a.Hin = input->dims[2];
    a.Win = input->dims[3];
    a.Hout = grid->dims[1];
    a.Wout = grid->dims[2];
    const int esz = elem_size(elem);
    // Views that are dense in channels-last order (what a framework hands over for its channels_last memory
    // format) are sampled in place by the channels-last kernel instead of being repacked to NCHW and back.
    // (the channels-last kernel implements the first coordinate rule only: under the second, such views are packed)
    if (a.rule == kRuleGridSampler2D && !input->contiguous() && !out->contiguous() && channels_last_dense(input) &&
        channels_last_dense(out)) {
        a.channels_last = 1;
        ex->in0.direct = (input->data == nullptr) ? nullptr : (char*)input->data + input->offset * (int64_t)esz;
        ex->out0.direct = (out->data == nullptr) ? nullptr : (char*)out->data + out->offset * (int64_t)esz;
    } else {
        ex->in0 = plan_view(ex, input, esz, false);
        ex->out0 = plan_view(ex, out, esz, true);
    }
    ex->in1 = plan_view(ex, grid, esz, false);
    // what is known of the operands' addresses already now (a workspace slice is 256-byte aligned, like null): the
    // kernel choice depends on their alignment, and opscvExecutorVariant reports it from this plan
    a.x = ex->in0.in_workspace ? nullptr : ex->in0.direct;
    a.grid = ex->in1.in_workspace ? nullptr : ex->in1.direct;
    a.y = ex->out0.in_workspace ? nullptr : ex->out0.direct;
    return plan_status(ex, "aclnnGridSampler2D");
}

}  // namespace

extern "C" {

aclnnStatus aclnnGridSampler2DGetWorkspaceSize(const aclTensor* input, const aclTensor* grid,
                                               int64_t interpolationMode, int64_t paddingMode, bool alignCorners,
                                               aclTensor* out, uint64_t* workspaceSize, aclOpExecutor** executor)
{
    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) {
        set_error("aclnnGridSampler2D: cannot allocate the executor");
        return ACLNN_ERR_INNER_CREATE_EXECUTOR;
    }
    if (input != nullptr && grid != nullptr && out != nullptr && (workspaceSize == nullptr || executor == nullptr)) {
        set_error("aclnnGridSampler2D: workspaceSize and executor must not be NULL");
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    const aclnnStatus st =
        plan_grid_sampler2d(input, grid, interpolationMode, paddingMode, alignCorners, out, ex.get());
    if (st != ACLNN_SUCCESS) {
        return st;
    }
    *workspaceSize = ex->workspace_bytes;
    *executor = ex.release();
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnGridSampler2D(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream)
{
    return run_executor(workspace, workspaceSize, executor, stream, OpKind::GridSampler2D, "aclnnGridSampler2D");
}

// Both phases in one call, with the library's static scratch array in the place of the caller's workspace.  The plan
// lives on the stack (its packing lists have fixed storage), so the call allocates nothing on either side.
aclnnStatus opscvGridSampler2DNoAlloc(const aclTensor* input, const aclTensor* grid, int64_t interpolationMode,
                                      int64_t paddingMode, bool alignCorners, aclTensor* out, aclrtStream stream)
{
    aclOpExecutor ex;
    const aclnnStatus st = plan_grid_sampler2d(input, grid, interpolationMode, paddingMode, alignCorners, out, &ex);
    if (st != ACLNN_SUCCESS) {
        return st;
    }
    void* scratch = nullptr;
    if (ex.workspace_bytes > 0) {
        uint64_t capacity = 0;
        const hipError_t e = static_scratch(&scratch, &capacity);
        if (e != hipSuccess) {
            set_error("opscvGridSampler2DNoAlloc: the static scratch array is not available: %s",
                      hipGetErrorString(e));
            return ACLNN_ERR_RUNTIME_ERROR;
        }
        if (ex.workspace_bytes > capacity) {
            set_error("opscvGridSampler2DNoAlloc: packing the non-contiguous views needs %llu bytes, the static "
                      "scratch array holds %llu; use aclnnGridSampler2D with a workspace",
                      (unsigned long long)ex.workspace_bytes, (unsigned long long)capacity);
            return ACLNN_ERR_PARAM_INVALID;
        }
    }
    return execute_plan(scratch, &ex, stream, "opscvGridSampler2DNoAlloc");
}

}  // extern "C"
