// aclnnResize: parameter validation, planning and the second-phase entry.
//
// Mirrors the checks, their order and their status codes of the reference implementation
// image/resize_bilinear_v2/op_api/aclnn_resize.cpp:60-212, on the branch it takes on its newest parts
// (:274-293): sizes derived from the scales, ResizeNearestNeighborV2 / ResizeBilinearV2 on plain 4-D tensors
// with align_corners = false and no user scale.
#include <cstring>
#include <memory>
#include <new>

#include "aclnn_resize.h"
#include "executor.hpp"
#include "resize_plan.hpp"

using namespace opscv;

namespace {

constexpr const char* kApi = "aclnnResize";
constexpr double kEpsilon = 1e-5;  // aclnn_resize.cpp:51

// aclnn_resize.cpp:100-118: the output extent must lie between trunc(in * (scale - eps)) and trunc(in * (scale + eps))
bool extent_matches(int64_t in, double scale, int64_t out)
{
    const int64_t hi = (int64_t)((double)in * (scale + kEpsilon));
    const int64_t lo = (int64_t)((double)in * (scale - kEpsilon));
    return out >= lo && out <= hi;
}

}  // namespace

extern "C" {

aclnnStatus aclnnResizeGetWorkspaceSize(const aclTensor* self, const aclFloatArray* scales, const char* mode,
                                        aclTensor* out, uint64_t* workspaceSize, aclOpExecutor** executor)
{
    if (workspaceSize == nullptr || executor == nullptr) {
        set_error("%s: workspaceSize and executor must not be NULL", kApi);
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    // 1. null arguments, the mode string included (aclnn_resize.cpp:123-133,190)
    if (self == nullptr || scales == nullptr || out == nullptr || mode == nullptr) {
        set_error("%s: self, scales, mode and out must not be NULL", kApi);
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    // 2. mode: prefix match (aclnn_resize.cpp:147-155)
    const bool nearest = strncmp(mode, "nearest", strlen("nearest")) == 0;
    const bool bilinear = strncmp(mode, "bilinear", strlen("bilinear")) == 0;
    if (!nearest && !bilinear) {
        set_error("%s: CheckModeStr failed, mode:%s", kApi, mode);
        return ACLNN_ERR_PARAM_INVALID;
    }
    // 3. dtypes (aclnn_resize.cpp:135-145)
    if (self->dtype != ACL_FLOAT16 && self->dtype != ACL_FLOAT && self->dtype != ACL_BF16) {
        set_error("%s: dtype %d is not in {FLOAT16, FLOAT, BF16}", kApi, (int)self->dtype);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (self->dtype != out->dtype) {
        set_error("%s: self dtype %d differs from out dtype %d", kApi, (int)self->dtype, (int)out->dtype);
        return ACLNN_ERR_PARAM_INVALID;
    }
    // 4. formats (aclnn_resize.cpp:157-180)
    if (self->format != out->format) {
        set_error("%s: The format of self and out must be same.", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (self->format != ACL_FORMAT_NCHW && self->format != ACL_FORMAT_NHWC) {
        set_error("%s: The format of self must be NCHW or NHWC.", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    // 5./6. ranks, scale count, N/C and extents (aclnn_resize.cpp:60-121); the rank is tested first here because
    // the element checks index four dimensions
    if (self->ndim != 4 || out->ndim != 4) {
        set_error("%s: The selfShape and outShape must be 4 dim.", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (scales->v.size() != 4) {
        set_error("%s: scales must hold 4 values, got %zu", kApi, scales->v.size());
        return ACLNN_ERR_PARAM_INVALID;
    }
    const bool nhwc = (self->format == ACL_FORMAT_NHWC);
    const int dn = 0, dc = nhwc ? 3 : 1, dh = nhwc ? 1 : 2, dw = nhwc ? 2 : 3;
    if (self->dims[dn] != out->dims[dn] || self->dims[dc] != out->dims[dc]) {
        set_error("%s: The dim of batch or channel is not matched.", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (!extent_matches(self->dims[dh], (double)scales->v[dh], out->dims[dh])) {
        set_error("%s: The dim of height is not matched.", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (!extent_matches(self->dims[dw], (double)scales->v[dw], out->dims[dw])) {
        set_error("%s: The dim of width is not matched.", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }

    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) {
        set_error("%s: cannot allocate the executor", kApi);
        return ACLNN_ERR_INNER_CREATE_EXECUTOR;
    }
    if (self->empty() || out->empty()) {
        *workspaceSize = 0;
        *executor = ex.release();
        return ACLNN_SUCCESS;
    }
    Elem elem;
    if (!elem_of(self->dtype, &elem)) {
        set_error("%s: unsupported dtype %d", kApi, (int)self->dtype);
        return ACLNN_ERR_PARAM_INVALID;
    }
    for (int i = 0; i < 4; i++) {
        if (self->dims[i] > INT32_MAX || out->dims[i] > INT32_MAX) {
            set_error("%s: every extent must fit in int32", kApi);
            return ACLNN_ERR_PARAM_INVALID;
        }
    }
    ex->kind = OpKind::Resize;
    ResizeArgs& a = ex->rs;
    a.elem = elem;
    a.channels_last = nhwc ? 1 : 0;
    a.N = self->dims[dn];
    a.C = self->dims[dc];
    a.Hs = self->dims[dh];
    a.Ws = self->dims[dw];
    a.Hd = out->dims[dh];
    a.Wd = out->dims[dw];
    if (nhwc && (a.Wd * a.C > INT32_MAX || a.Ws * a.C > INT32_MAX)) {
        set_error("%s: W*C must fit in int32 for NHWC tensors", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (nearest) {
        plan_resize_nearest(&a);
    } else {
        plan_resize(&a, false, 0.0f, 0.0f);
    }
    const int esz = elem_size(elem);
    ex->in0 = plan_view(ex.get(), self, esz, false);
    ex->out0 = plan_view(ex.get(), out, esz, true);
    if (const aclnnStatus ps = plan_status(ex.get(), "aclnnResize"); ps != ACLNN_SUCCESS) {
        return ps;
    }
    *workspaceSize = ex->workspace_bytes;
    *executor = ex.release();
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnResize(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream)
{
    return run_executor(workspace, workspaceSize, executor, stream, OpKind::Resize, kApi);
}

}  // extern "C"
