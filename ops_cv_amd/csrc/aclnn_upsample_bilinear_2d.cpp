// aclnnUpsampleBilinear2d: parameter validation, planning and the second-phase entry.
//
// Mirrors the checks, their order and their status codes of the reference implementation
// image/upsample_bilinear2d/op_host/op_api/aclnn_upsample_bilinear_2d.cpp:62-195,384-467.  The computation is
// the branch that reference takes on its newest parts (:423-426): ResizeBilinearV2 on plain 4-D tensors with
// half_pixel_centers = !alignCorners (image/resize_bilinear_v2/op_api/resize_bilinear_v2.cpp:96-110).
#include <memory>
#include <new>

#include "aclnn_upsample_bilinear_2d.h"
#include "executor.hpp"
#include "resize_plan.hpp"

using namespace opscv;

namespace {

constexpr const char* kApi = "aclnnUpsampleBilinear2d";

// aclnn_upsample_bilinear_2d.cpp:85-111
bool check_format(const aclTensor* self, const aclTensor* out)
{
    if (self->format != out->format) {
        set_error("%s: Format of input and output should be equal, self [%d], out [%d].", kApi, (int)self->format,
                  (int)out->format);
        return false;
    }
    if (self->format != ACL_FORMAT_NCHW && self->format != ACL_FORMAT_NHWC) {
        set_error("%s: Do not support this format(%d) of input and output.", kApi, (int)self->format);
        return false;
    }
    if (self->ndim != 4 || out->ndim != 4) {
        set_error("%s: self and out must be 4-D, got %lld and %lld dims", kApi, (long long)self->ndim,
                  (long long)out->ndim);
        return false;
    }
    if (self->format == ACL_FORMAT_NCHW && self->dtype == ACL_DOUBLE) {
        set_error("%s: When dtype is DOUBLE, only support NHWC format", kApi);
        return false;
    }
    return true;
}

// common/stub/op_api/aclnn_kernels/common/op_error_check.h:108-135
bool check_nc(const aclTensor* self, const aclTensor* out)
{
    const int c_dim = (self->format == ACL_FORMAT_NCHW) ? 1 : 3;
    if (self->dims[0] != out->dims[0] || self->dims[c_dim] != out->dims[c_dim]) {
        set_error("%s: The selfDimN[%lld]/outDimN[%lld] or selfDimC[%lld]/outDimC[%lld] not equal.", kApi,
                  (long long)self->dims[0], (long long)out->dims[0], (long long)self->dims[c_dim],
                  (long long)out->dims[c_dim]);
        return false;
    }
    return true;
}

// aclnn_upsample_bilinear_2d.cpp:137-168
bool check_output_size(const aclTensor* out, const aclIntArray* output_size)
{
    if (output_size == nullptr) {
        set_error("%s: outputSize must not be null.", kApi);
        return false;
    }
    if (output_size->v.size() != 2) {
        set_error("%s: outputSize size must be 2, but got %zu.", kApi, output_size->v.size());
        return false;
    }
    const int h_dim = (out->format == ACL_FORMAT_NCHW) ? 2 : 1;
    if (output_size->v[0] != out->dims[h_dim] || output_size->v[1] != out->dims[h_dim + 1]) {
        set_error("%s: Expected output size (H: %lld, W: %lld), but got output tensor size (H: %lld, W: %lld).",
                  kApi, (long long)output_size->v[0], (long long)output_size->v[1], (long long)out->dims[h_dim],
                  (long long)out->dims[h_dim + 1]);
        return false;
    }
    return true;
}

}  // namespace

extern "C" {

aclnnStatus aclnnUpsampleBilinear2dGetWorkspaceSize(const aclTensor* self, const aclIntArray* outputSize,
                                                    const bool alignCorners, const double scalesH,
                                                    const double scalesW, aclTensor* out, uint64_t* workspaceSize,
                                                    aclOpExecutor** executor)
{
    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) {
        set_error("%s: cannot allocate the executor", kApi);
        return ACLNN_ERR_INNER_CREATE_EXECUTOR;
    }
    // 1. null tensors are reported as an inner error by this operator (aclnn_upsample_bilinear_2d.cpp:175)
    if (self == nullptr || out == nullptr) {
        set_error("%s: self and out must not be NULL", kApi);
        return ACLNN_ERR_INNER_NULLPTR;
    }
    if (workspaceSize == nullptr || executor == nullptr) {
        set_error("%s: workspaceSize and executor must not be NULL", kApi);
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    // 2. dtype list
    if (self->dtype != ACL_FLOAT16 && self->dtype != ACL_FLOAT && self->dtype != ACL_DOUBLE &&
        self->dtype != ACL_BF16) {
        set_error("%s: dtype %d is not in {FLOAT16, FLOAT, DOUBLE, BF16}", kApi, (int)self->dtype);
        return ACLNN_ERR_PARAM_INVALID;
    }
    // 3. equal dtypes
    if (self->dtype != out->dtype) {
        set_error("%s: self dtype %d differs from out dtype %d", kApi, (int)self->dtype, (int)out->dtype);
        return ACLNN_ERR_PARAM_INVALID;
    }
    // 4. formats and ranks, 5. N and C, 6. scales, 7. outputSize
    if (!check_format(self, out) || !check_nc(self, out)) {
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (scalesW < 0 || scalesH < 0) {
        set_error("%s: w scales and h scales cannot be negative , w_scales [%f], h_scales [%f].", kApi, scalesW,
                  scalesH);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (!check_output_size(out, outputSize)) {
        return ACLNN_ERR_PARAM_INVALID;
    }
    // empty tensors: successful no-op (aclnn_upsample_bilinear_2d.cpp:398-403)
    if (self->empty() || out->empty()) {
        *workspaceSize = 0;
        *executor = ex.release();
        return ACLNN_SUCCESS;
    }
    Elem elem;
    if (!elem_of(self->dtype, &elem)) {
        // the reference sends DOUBLE to a host-CPU kernel that is not part of its tree
        set_error("%s: DOUBLE tensors are not supported by the MI355X implementation", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    for (int i = 0; i < 4; i++) {
        if (self->dims[i] > INT32_MAX || out->dims[i] > INT32_MAX) {
            set_error("%s: every extent must fit in int32", kApi);
            return ACLNN_ERR_PARAM_INVALID;
        }
    }

    const bool nhwc = (self->format == ACL_FORMAT_NHWC);
    ex->kind = OpKind::Resize;
    ResizeArgs& a = ex->rs;
    a.elem = elem;
    a.channels_last = nhwc ? 1 : 0;
    a.N = self->dims[0];
    a.C = self->dims[nhwc ? 3 : 1];
    a.Hs = self->dims[nhwc ? 1 : 2];
    a.Ws = self->dims[nhwc ? 2 : 3];
    a.Hd = out->dims[nhwc ? 1 : 2];
    a.Wd = out->dims[nhwc ? 2 : 3];
    if (nhwc && a.Wd * a.C > INT32_MAX) {
        set_error("%s: Wout*C must fit in int32 for NHWC tensors", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    // the user scales reach the kernel narrowed to float (aclnn_upsample_bilinear_2d.cpp:411-412)
    plan_resize(&a, alignCorners, (float)scalesH, (float)scalesW);
    const int esz = elem_size(elem);
    ex->in0 = plan_view(ex.get(), self, esz, false);
    ex->out0 = plan_view(ex.get(), out, esz, true);

    if (const aclnnStatus ps = plan_status(ex.get(), "aclnnUpsampleBilinear2d"); ps != ACLNN_SUCCESS) {
        return ps;
    }
    *workspaceSize = ex->workspace_bytes;
    *executor = ex.release();
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnUpsampleBilinear2d(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                    aclrtStream stream)
{
    return run_executor(workspace, workspaceSize, executor, stream, OpKind::Resize, kApi);
}

}  // extern "C"
