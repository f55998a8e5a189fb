// aclnnGridSampler2DBackward: parameter validation, planning and the second-phase entry.
//
// Mirrors the checks, their order and their status codes of the reference implementation
// image/grid_sampler2_d_grad/op_host/op_api/aclnn_grid_sampler2d_backward.cpp:77-240.
#include <memory>
#include <new>

#include "aclnn_grid_sampler2d_backward.h"
#include "executor.hpp"
#include "kernels.hpp"

using namespace opscv;

namespace {

const char* const kApi = "aclnnGridSampler2DBackward";

// aclnn_grid_sampler2d_backward.cpp:77-90
bool check_dtypes(const aclTensor* gout, const aclTensor* input, const aclTensor* grid, const aclTensor* dx,
                  const aclTensor* dgrid)
{
    const aclTensor* others[4] = {gout, grid, dx, dgrid};
    const char* names[4] = {"gradOutput", "grid", "inputGrad", "gridGrad"};
    for (int i = 0; i < 4; i++) {
        if (others[i]->dtype != input->dtype) {
            set_error("%s: %s dtype %d differs from input dtype %d", kApi, names[i], (int)others[i]->dtype,
                      (int)input->dtype);
            return false;
        }
    }
    switch (input->dtype) {
        case ACL_FLOAT:
        case ACL_FLOAT16:
        case ACL_DOUBLE:
        case ACL_BF16: return true;
        default: break;
    }
    set_error("%s: dtype %d is not in {FLOAT, FLOAT16, DOUBLE, BF16}", kApi, (int)input->dtype);
    return false;
}

// aclnn_grid_sampler2d_backward.cpp:92-108 (interpolation first)
bool check_attrs(int64_t interp, int64_t pad)
{
    if (interp < 0 || interp > 2) {
        set_error("interpolationMode %lld should be in range [0, 2].", (long long)interp);
        return false;
    }
    if (pad < 0 || pad > 2) {
        set_error("paddingMode %lld should be in range [0, 2].", (long long)pad);
        return false;
    }
    return true;
}

bool same_shape(const aclTensor* a, const aclTensor* b)
{
    if (a->ndim != b->ndim) {
        return false;
    }
    for (int64_t i = 0; i < a->ndim; i++) {
        if (a->dims[i] != b->dims[i]) {
            return false;
        }
    }
    return true;
}

// aclnn_grid_sampler2d_backward.cpp:120-172
bool check_shapes(const aclTensor* gout, const aclTensor* input, const aclTensor* grid, const aclTensor* dx,
                  const aclTensor* dgrid, const aclBoolArray* mask)
{
    if (input->ndim != 4 || grid->ndim != 4 || gout->ndim != 4) {
        set_error("%s: input, grid and gradOutput must be 4-D, got %lld, %lld, %lld dims", kApi,
                  (long long)input->ndim, (long long)grid->ndim, (long long)gout->ndim);
        return false;
    }
    if (input->dims[0] != grid->dims[0] || input->dims[0] != gout->dims[0]) {
        set_error("expect input grid and gradOutput to have same batch size");
        return false;
    }
    if (input->dims[1] != gout->dims[1]) {
        set_error("expect input and gradOutput to have same channel size");
        return false;
    }
    if (input->dims[2] == 0 || input->dims[3] == 0) {
        set_error("expect input to have non-empty spatial dimensions");
        return false;
    }
    if (grid->dims[1] != gout->dims[2] || grid->dims[2] != gout->dims[3]) {
        set_error("expect grid and gradOutput to have same H and W size");
        return false;
    }
    if (grid->dims[3] != 2) {
        set_error("expect grid to have size 2 in last dimension");
        return false;
    }
    if (!same_shape(dx, input)) {
        set_error("%s: inputGrad must have the shape of input", kApi);
        return false;
    }
    if (!same_shape(dgrid, grid)) {
        set_error("%s: gridGrad must have the shape of grid", kApi);
        return false;
    }
    if (mask->v.size() != 2) {
        set_error("Expected aclnnGridSampler2DBackward outputMask len to be 2, but got %zu.", mask->v.size());
        return false;
    }
    return true;
}

}  // namespace

extern "C" {

aclnnStatus aclnnGridSampler2DBackwardGetWorkspaceSize(const aclTensor* gradOutput, const aclTensor* input,
                                                       const aclTensor* grid, int64_t interpolationMode,
                                                       int64_t paddingMode, bool alignCorners,
                                                       const aclBoolArray* outputMask, aclTensor* inputGrad,
                                                       aclTensor* gridGrad, uint64_t* workspaceSize,
                                                       aclOpExecutor** executor)
{
    // aclnn_grid_sampler2d_backward.cpp:221
    if (workspaceSize == nullptr || executor == nullptr) {
        set_error("%s: workspaceSize and executor must not be NULL", kApi);
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) {
        set_error("%s: cannot allocate the executor", kApi);
        return ACLNN_ERR_INNER_CREATE_EXECUTOR;
    }
    // a missing mask is a successful no-op, before any other check (aclnn_grid_sampler2d_backward.cpp:229-233)
    if (outputMask == nullptr) {
        *workspaceSize = 0;
        *executor = ex.release();
        return ACLNN_SUCCESS;
    }
    if (gradOutput == nullptr || input == nullptr || grid == nullptr || inputGrad == nullptr || gridGrad == nullptr) {
        set_error("%s: gradOutput, input, grid, inputGrad and gridGrad must not be NULL", kApi);
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    if (!check_dtypes(gradOutput, input, grid, inputGrad, gridGrad) || !check_attrs(interpolationMode, paddingMode) ||
        !check_shapes(gradOutput, input, grid, inputGrad, gridGrad, outputMask)) {
        return ACLNN_ERR_PARAM_INVALID;
    }
    const bool want_dx = outputMask->v[0] != 0, want_dgrid = outputMask->v[1] != 0;
    // aclnn_grid_sampler2d_backward.cpp:238-243
    if (gradOutput->empty() || input->empty() || grid->empty() || (!want_dx && !want_dgrid)) {
        *workspaceSize = 0;
        *executor = ex.release();
        return ACLNN_SUCCESS;
    }
    // The reference routes DOUBLE to a host-CPU kernel that is not part of its tree; it does not exist here.
    Elem elem;
    if (!elem_of(input->dtype, &elem)) {
        set_error("%s: DOUBLE tensors are not supported by the MI355X implementation", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }
    for (int i = 0; i < 4; i++) {
        if (input->dims[i] > INT32_MAX || grid->dims[i] > INT32_MAX) {
            set_error("%s: every extent must fit in int32", kApi);
            return ACLNN_ERR_PARAM_INVALID;
        }
    }
    // the walk over chunks of 256 grid points runs up to a chunk past the last point
    if (input->dims[2] * input->dims[3] > INT32_MAX || grid->dims[1] * grid->dims[2] > INT32_MAX - 1024 ||
        input->dims[0] > 65535 || input->dims[1] > 65535) {
        set_error("%s: Hin*Win and Hout*Wout must fit in int32, N and C in 16 bits", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }

    ex->kind = OpKind::GridSampler2DGrad;
    GridSamplerGradArgs& a = ex->gsg;
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
    ex->in0 = plan_view(ex.get(), gradOutput, esz, false);
    ex->in1 = plan_view(ex.get(), input, esz, false);
    ex->in2 = plan_view(ex.get(), grid, esz, false);
    // known now unless packed into the workspace (whose slices are 256-byte aligned): lets the variant query see the
    // alignment the launch will see
    a.x = ex->in1.in_workspace ? nullptr : ex->in1.direct;
    a.gout = ex->in0.in_workspace ? nullptr : ex->in0.direct;
    ex->want_out0 = want_dx ? 1 : 0;
    ex->want_out1 = want_dgrid ? 1 : 0;
    if (want_dx) {
        ex->out0 = plan_view(ex.get(), inputGrad, esz, true);
    }
    if (want_dgrid) {
        ex->out1 = plan_view(ex.get(), gridGrad, esz, true);
    }
    if (want_dx) {
        // scratch of the input gradient's list variant (0 words when the shape does not qualify)
        const int64_t words = gs2d_grad_csr_words(a);
        if (words > 0) {
            ex->scratch.in_workspace = true;
            ex->scratch.ws_offset = (ex->workspace_bytes + 255) / 256 * 256;
            ex->workspace_bytes = ex->scratch.ws_offset + (uint64_t)words * 4;
        }
    }
    if (const aclnnStatus ps = plan_status(ex.get(), "aclnnGridSampler2DBackward"); ps != ACLNN_SUCCESS) {
        return ps;
    }
    *workspaceSize = ex->workspace_bytes;
    *executor = ex.release();
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnGridSampler2DBackward(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                       aclrtStream stream)
{
    return run_executor(workspace, workspaceSize, executor, stream, OpKind::GridSampler2DGrad, kApi);
}

}  // extern "C"
