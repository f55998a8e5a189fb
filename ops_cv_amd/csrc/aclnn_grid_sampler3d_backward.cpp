// aclnnGridSampler3DBackward: parameter validation, planning and the second-phase entry.
//
// Mirrors the checks, their order and their status codes of the reference implementation
// image/grid_sampler3_d_grad/op_host/op_api/aclnn_grid_sampler3d_backward.cpp:64-236.
#include <memory>
#include <new>

#include "aclnn_grid_sampler3d_backward.h"
#include "executor.hpp"
#include "options.hpp"
#include "kernels.hpp"
#include "resize_plan.hpp"

using namespace opscv;

namespace {

const char* const kApi = "aclnnGridSampler3DBackward";

// aclnn_grid_sampler3d_backward.cpp:64-76
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
        case ACL_BF16:
        case ACL_DOUBLE: return true;
        default: break;
    }
    set_error("%s: dtype %d is not in {FLOAT, FLOAT16, BF16, DOUBLE}", kApi, (int)input->dtype);
    return false;
}

// aclnn_grid_sampler3d_backward.cpp:78-94 (padding first)
bool check_attrs(int64_t interp, int64_t pad)
{
    if (pad < 0 || pad > 2) {
        set_error("paddingMode %lld should be in range [0, 2].", (long long)pad);
        return false;
    }
    if (interp < 0 || interp > 1) {
        set_error("interpolationMode %lld should be in range [0, 1].", (long long)interp);
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

// aclnn_grid_sampler3d_backward.cpp:117-172; the layout of input decides how gradOutput is read
bool check_shapes(const aclTensor* gout, const aclTensor* input, const aclTensor* grid, const aclTensor* dx,
                  const aclTensor* dgrid)
{
    if (input->ndim != 5 || grid->ndim != 5 || gout->ndim != 5) {
        set_error("%s: input, grid and gradOutput must be 5-D, got %lld, %lld, %lld dims", kApi,
                  (long long)input->ndim, (long long)grid->ndim, (long long)gout->ndim);
        return false;
    }
    const bool ndhwc = input->format == ACL_FORMAT_NDHWC;
    const int ci = ndhwc ? 4 : 1, di = ndhwc ? 1 : 2, hi = ndhwc ? 2 : 3, wi = ndhwc ? 3 : 4;
    if (input->dims[0] != grid->dims[0] || input->dims[0] != gout->dims[0]) {
        set_error("expect input grid and gradOutput to have same batch size");
        return false;
    }
    if (input->dims[ci] != gout->dims[ci]) {
        set_error("expect input and gradOutput to have same channel size");
        return false;
    }
    if (grid->dims[1] != gout->dims[di] || grid->dims[2] != gout->dims[hi] || grid->dims[3] != gout->dims[wi]) {
        set_error("expect grid and gradOutput to have same D, H and W size");
        return false;
    }
    if (grid->dims[4] != 3) {
        set_error("expect grid to have size 3 in last dimension");
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
    return true;
}

}  // namespace

extern "C" {

aclnnStatus aclnnGridSampler3DBackwardGetWorkspaceSize(const aclTensor* gradOutput, const aclTensor* input,
                                                       const aclTensor* grid, int64_t interpolationMode,
                                                       int64_t paddingMode, bool alignCorners,
                                                       const aclBoolArray* outputMask, aclTensor* inputGrad,
                                                       aclTensor* gridGrad, uint64_t* workspaceSize,
                                                       aclOpExecutor** executor)
{
    // aclnn_grid_sampler3d_backward.cpp:212
    if (workspaceSize == nullptr || executor == nullptr) {
        set_error("%s: workspaceSize and executor must not be NULL", kApi);
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) {
        set_error("%s: cannot allocate the executor", kApi);
        return ACLNN_ERR_INNER_CREATE_EXECUTOR;
    }
    // a missing mask is a successful no-op, before any other check (aclnn_grid_sampler3d_backward.cpp:221-226)
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
        !check_shapes(gradOutput, input, grid, inputGrad, gridGrad)) {
        return ACLNN_ERR_PARAM_INVALID;
    }
    // aclnn_grid_sampler3d_backward.cpp:105-113
    if (outputMask->v.size() != 2) {
        set_error("Expected aclnnGridSampler3DBackward outputMask len to be 2, but got %zu.", outputMask->v.size());
        return ACLNN_ERR_PARAM_INVALID;
    }
    const bool want_dx = outputMask->v[0] != 0, want_dgrid = outputMask->v[1] != 0;
    // aclnn_grid_sampler3d_backward.cpp:232-238
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
    const bool ndhwc = input->format == ACL_FORMAT_NDHWC;
    const int ci = ndhwc ? 4 : 1, di = ndhwc ? 1 : 2, hi = ndhwc ? 2 : 3, wi = ndhwc ? 3 : 4;
    for (int i = 0; i < 5; i++) {
        if (input->dims[i] > INT32_MAX || grid->dims[i] > INT32_MAX) {
            set_error("%s: every extent must fit in int32", kApi);
            return ACLNN_ERR_PARAM_INVALID;
        }
    }
    if (input->dims[di] * input->dims[hi] > INT32_MAX ||
        input->dims[di] * input->dims[hi] * input->dims[wi] > INT32_MAX ||
        grid->dims[1] * grid->dims[2] > INT32_MAX ||
        grid->dims[1] * grid->dims[2] * grid->dims[3] > INT32_MAX - 1024 ||  // chunk arithmetic runs a chunk past it
        input->dims[0] > 65535 || input->dims[ci] > 65535) {
        set_error("%s: Din*Hin*Win and Dout*Hout*Wout must fit in int32, N and C in 16 bits", kApi);
        return ACLNN_ERR_PARAM_INVALID;
    }

    ex->kind = OpKind::GridSampler3DGrad;
    GridSampler3DGradArgs& a = ex->gsg3;
    a.elem = elem;
    a.interp = (int)interpolationMode;
    a.pad = (int)paddingMode;
    a.align = alignCorners ? 1 : 0;
    a.N = input->dims[0];
    a.C = input->dims[ci];
    a.Din = input->dims[di];
    a.Hin = input->dims[hi];
    a.Win = input->dims[wi];
    a.Dout = grid->dims[1];
    a.Hout = grid->dims[2];
    a.Wout = grid->dims[3];
    // batch items a core of the reference device walks as one run of grid points
    // (image/grid_sampler3_d_grad/op_host/grid_sampler3_d_grad_tiling.cpp:183-191)
    const int64_t cores = reference_vector_cores();
    a.items_per_core = (a.N > cores) ? (a.N + cores - 1) / cores : 1;
    a.force_variant = current_options().gs3d_grad_variant;
    const int esz = elem_size(elem);
    // The kernels work on (N,C,D,H,W) operands.  Channels-last tensors are those operands seen through a permuted
    // view, packed (and the gradient scattered) like any other non-contiguous view.
    static const int kToNcdhw[5] = {0, 4, 1, 2, 3};
    const int* perm = ndhwc ? kToNcdhw : nullptr;
    ex->in0 = plan_view(ex.get(), gradOutput, esz, false, perm);
    ex->in1 = plan_view(ex.get(), input, esz, false, perm);
    ex->in2 = plan_view(ex.get(), grid, esz, false);
    ex->want_out0 = want_dx ? 1 : 0;
    ex->want_out1 = want_dgrid ? 1 : 0;
    if (want_dx) {
        ex->out0 = plan_view(ex.get(), inputGrad, esz, true, perm);
    }
    if (want_dgrid) {
        ex->out1 = plan_view(ex.get(), gridGrad, esz, true);
    }
    if (want_dx) {
        // scratch of the input-gradient kernels: the voxel span of every chunk of grid points, then (from the next
        // 256-byte boundary) the cell slots and corner weights of the gather variant
        const int64_t range_words = gs3d_grad_range_words(a);
        const int64_t list_words = gs3d_grad_list_words(a);
        if (range_words > 0 || list_words > 0) {
            ex->scratch.in_workspace = true;
            ex->scratch.ws_offset = (ex->workspace_bytes + 255) / 256 * 256;
            ex->workspace_bytes = ex->scratch.ws_offset + (list_words > 0 ? gs3d_grad_lists_offset(range_words) +
                                                                                 (uint64_t)list_words * 4
                                                                           : (uint64_t)range_words * 4);
        }
    }
    if (const aclnnStatus ps = plan_status(ex.get(), "aclnnGridSampler3DBackward"); ps != ACLNN_SUCCESS) {
        return ps;
    }
    *workspaceSize = ex->workspace_bytes;
    *executor = ex.release();
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnGridSampler3DBackward(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                       aclrtStream stream)
{
    return run_executor(workspace, workspaceSize, executor, stream, OpKind::GridSampler3DGrad, kApi);
}

}  // extern "C"
