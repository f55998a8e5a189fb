// aclnnUpsampleBilinear2dBackward: parameter validation, planning and the second-phase entry.
//
// Mirrors the checks, their order and their status codes of the reference implementation
// image/resize_bilinear_v2_grad/op_api/aclnn_upsample_bilinear_2d_backward.cpp:48-230, on the branch it takes on
// its newest parts (:251-265): ResizeBilinearV2Grad on plain 4-D tensors with half_pixel_centers = !alignCorners.
// Scales follow resize_bilinear_v2_grad_tiling_arch35.cpp:352-394 (the deterministic template).
#include <cfloat>
#include <cmath>
#include <memory>
#include <new>

#include "aclnn_upsample_bilinear_2d_backward.h"
#include "executor.hpp"

using namespace opscv;

namespace {

constexpr const char* kApi = "aclnnUpsampleBilinear2dBackward";

// resize_bilinear_v2_grad_tiling_arch35.cpp:352-394 with isDetermine = true
float grad_scale(int64_t len_src, int64_t len_dst, bool align_corners, float user_scale)
{
    if (align_corners) {
        if (len_src > 1 && len_dst > 1) {
            return (float)(len_src - 1) / (float)(len_dst - 1);
        }
        return (float)len_src / (float)len_dst;
    }
    if (user_scale > 0.0f) {
        return 1.0f / user_scale;
    }
    return (float)len_src / (float)len_dst;
}

}  // namespace

extern "C" {

aclnnStatus aclnnUpsampleBilinear2dBackwardGetWorkspaceSize(const aclTensor* gradOut, const aclIntArray* outputSize,
                                                            const aclIntArray* inputSize, bool alignCorners,
                                                            double scalesH, double scalesW, aclTensor* out,
                                                            uint64_t* workspaceSize, aclOpExecutor** executor)
{
    if (workspaceSize == nullptr || executor == nullptr) {
        set_error("%s: workspaceSize and executor must not be NULL", kApi);
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) {
        set_error("%s: cannot allocate the executor", kApi);
        return ACLNN_ERR_INNER_CREATE_EXECUTOR;
    }
    // 1. null arguments (aclnn_upsample_bilinear_2d_backward.cpp:48-56)
    if (gradOut == nullptr || outputSize == nullptr || inputSize == nullptr || out == nullptr) {
        set_error("%s: gradOut, outputSize, inputSize and out must not be NULL", kApi);
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    // 2. shapes (:143-198)
    if (gradOut->ndim != 4) {
        set_error("%s: gradOut must be 4-D, got %lld dims", kApi, (long long)gradOut->ndim);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (outputSize->v.size() != 2) {
        set_error("%s: It is expected output_size equals to 2, but got size %zu", kApi, outputSize->v.size());
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (inputSize->v.size() != 4) {
        set_error("%s: It is expected input_size equals to 4, but got size %zu", kApi, inputSize->v.size());
        return ACLNN_ERR_PARAM_INVALID;
    }
    const bool nhwc = (out->format != ACL_FORMAT_NCHW);  // the reference reads every other format as N,H,W,C here
    const int dc = nhwc ? 3 : 1, dh = nhwc ? 1 : 2, dw = nhwc ? 2 : 3;
    const int64_t N = inputSize->v[0], C = inputSize->v[dc], inH = inputSize->v[dh], inW = inputSize->v[dw];
    const int64_t outH = outputSize->v[0], outW = outputSize->v[1];
    if (inH <= 0 || inW <= 0 || outH <= 0 || outW <= 0) {
        set_error("%s: Size of H and W must be greater than 0, but got input (H: %lld, W: %lld), output (H: %lld, W: %lld)",
                  kApi, (long long)inH, (long long)inW, (long long)outH, (long long)outW);
        return ACLNN_ERR_PARAM_INVALID;
    }
    int64_t full_out[4], full_in[4];
    full_out[0] = full_in[0] = N;
    full_out[dc] = full_in[dc] = C;
    full_out[dh] = outH;
    full_out[dw] = outW;
    full_in[dh] = inH;
    full_in[dw] = inW;
    if (out->ndim != 4) {
        set_error("%s: out must be 4-D, got %lld dims", kApi, (long long)out->ndim);
        return ACLNN_ERR_PARAM_INVALID;
    }
    for (int i = 0; i < 4; i++) {
        if (gradOut->dims[i] != full_out[i]) {
            set_error("%s: The dim %d of gradOut should be %lld, but got %lld", kApi, i, (long long)full_out[i],
                      (long long)gradOut->dims[i]);
            return ACLNN_ERR_PARAM_INVALID;
        }
        if (out->dims[i] != full_in[i]) {
            set_error("%s: The dim %d of out should be %lld, but got %lld", kApi, i, (long long)full_in[i],
                      (long long)out->dims[i]);
            return ACLNN_ERR_PARAM_INVALID;
        }
    }
    // 3. dtypes (:104-125)
    bool same_sizes = true;
    for (int i = 0; i < 4; i++) {
        same_sizes = same_sizes && gradOut->dims[i] == inputSize->v[i];
    }
    const bool in_list = gradOut->dtype == ACL_FLOAT16 || gradOut->dtype == ACL_FLOAT || gradOut->dtype == ACL_BF16;
    const bool out_in_list = out->dtype == ACL_FLOAT16 || out->dtype == ACL_FLOAT || out->dtype == ACL_BF16;
    if (!same_sizes) {
        if (!in_list) {
            set_error("%s: gradOut dtype %d is not in {FLOAT16, FLOAT, BF16}", kApi, (int)gradOut->dtype);
            return ACLNN_ERR_PARAM_INVALID;
        }
        if (gradOut->dtype != ACL_FLOAT ? out->dtype != gradOut->dtype : !out_in_list) {
            set_error("%s: out dtype %d does not go with gradOut dtype %d", kApi, (int)out->dtype, (int)gradOut->dtype);
            return ACLNN_ERR_PARAM_INVALID;
        }
    } else if (out->dtype != gradOut->dtype) {
        set_error("%s: out dtype %d differs from gradOut dtype %d", kApi, (int)out->dtype, (int)gradOut->dtype);
        return ACLNN_ERR_PARAM_INVALID;
    }
    // 4./5. covered by the shape check above (the reference repeats it on gradOut and compares N and C);
    // 6. formats (:127-135)
    if (gradOut->format != out->format) {
        set_error("%s: The gradOut and out must have same format", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (out->format != ACL_FORMAT_NCHW && out->format != ACL_FORMAT_NHWC) {
        set_error("%s: The format must be NCHW or NHWC", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (gradOut->empty()) {
        *workspaceSize = 0;
        *executor = ex.release();
        return ACLNN_SUCCESS;
    }
    Elem ein, eout;
    if (!elem_of(gradOut->dtype, &ein) || !elem_of(out->dtype, &eout)) {
        set_error("%s: unsupported dtype", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    for (int i = 0; i < 4; i++) {
        if (gradOut->dims[i] > INT32_MAX || out->dims[i] > INT32_MAX) {
            set_error("%s: every extent must fit in int32", kApi);
            return ACLNN_ERR_PARAM_INVALID;
        }
    }
    ex->kind = OpKind::ResizeGrad;
    ResizeGradArgs& a = ex->rg;
    a.elem_in = ein;
    a.elem_out = eout;
    a.channels_last = nhwc ? 1 : 0;
    a.half_pixel = alignCorners ? 0 : 1;
    a.N = N;
    a.C = C;
    a.Hs = inH;
    a.Ws = inW;
    a.Hd = outH;
    a.Wd = outW;
    a.copy = same_sizes ? 1 : 0;
    a.scale_h = grad_scale(inH, outH, alignCorners, (float)scalesH);
    a.scale_w = grad_scale(inW, outW, alignCorners, (float)scalesW);
    a.inv_scale_h = 1.0f / a.scale_h;
    a.inv_scale_w = 1.0f / a.scale_w;
    // resize_bilinear_v2_grad_tiling_arch35.cpp:422-436: a user scale that is not the ratio of the sizes selects the
    // "determine_scales" template
    a.user_scales = (!alignCorners && (std::fabs((float)inH / (float)outH - a.scale_h) >= FLT_EPSILON ||
                                       std::fabs((float)inW / (float)outW - a.scale_w) >= FLT_EPSILON))
                        ? 1
                        : 0;
    ex->in0 = plan_view(ex.get(), gradOut, elem_size(ein), false);
    ex->out0 = plan_view(ex.get(), out, elem_size(eout), true);
    if (const aclnnStatus ps = plan_status(ex.get(), "aclnnUpsampleBilinear2dBackward"); ps != ACLNN_SUCCESS) {
        return ps;
    }
    *workspaceSize = ex->workspace_bytes;
    *executor = ex.release();
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnUpsampleBilinear2dBackward(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                            aclrtStream stream)
{
    return run_executor(workspace, workspaceSize, executor, stream, OpKind::ResizeGrad, kApi);
}

}  // extern "C"
