// aclnnGridSampler3D: parameter validation, planning and the second-phase entry.
//
// Mirrors the checks, their order and their status codes of the reference implementation
// image/grid_sample/op_api/aclnn_grid_sampler3d.cpp:60-208,314-380.
#include <memory>
#include <new>

#include "aclnn_grid_sampler3d.h"
#include "executor.hpp"

using namespace opscv;

namespace {

constexpr int64_t kVolumetricDims = 5;

// aclnn_grid_sampler3d.cpp:83-93
bool check_dtypes(const aclTensor* input, const aclTensor* grid, const aclTensor* out)
{
    if (grid->dtype != input->dtype) {
        set_error("aclnnGridSampler3D: grid dtype %d differs from input dtype %d", (int)grid->dtype,
                  (int)input->dtype);
        return false;
    }
    if (out->dtype != input->dtype) {
        set_error("aclnnGridSampler3D: out dtype %d differs from input dtype %d", (int)out->dtype,
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
    set_error("aclnnGridSampler3D: dtype %d is not in {FLOAT16, FLOAT, DOUBLE, BF16}", (int)input->dtype);
    return false;
}

bool volumetric_format(aclFormat f)
{
    return f == ACL_FORMAT_NCDHW || f == ACL_FORMAT_NDHWC || f == ACL_FORMAT_ND;
}

// aclnn_grid_sampler3d.cpp:101-118
bool check_formats(const aclTensor* input, const aclTensor* out)
{
    if (!volumetric_format(input->format)) {
        set_error("Input format only supports [NCDHW, NDHWC, ND] format, but format is [%d]", (int)input->format);
        return false;
    }
    if (!volumetric_format(out->format)) {
        set_error("Out format only supports [NCDHW, NDHWC, ND] format, but format is [%d]", (int)out->format);
        return false;
    }
    return true;
}

// aclnn_grid_sampler3d.cpp:121-136 (padding first)
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

// aclnn_grid_sampler3d.cpp:138-192
bool check_shapes(const aclTensor* input, const aclTensor* grid, const aclTensor* out)
{
    if (input->ndim != kVolumetricDims || grid->ndim != kVolumetricDims || out->ndim != kVolumetricDims) {
        set_error("aclnnGridSampler3D: input, grid and out must be 5-D, got %lld, %lld, %lld dims",
                  (long long)input->ndim, (long long)grid->ndim, (long long)out->ndim);
        return false;
    }
    if (input->dims[0] != grid->dims[0] || input->dims[0] != out->dims[0]) {
        set_error("expect input grid and out to have same batch size");
        return false;
    }
    const bool ndhwc = input->format == ACL_FORMAT_NDHWC;
    const int ci = ndhwc ? 4 : 1, di = ndhwc ? 1 : 2, hi = ndhwc ? 2 : 3, wi = ndhwc ? 3 : 4;
    if (input->dims[ci] != out->dims[ci]) {
        set_error("expect input and out to have same channel size");
        return false;
    }
    if (grid->dims[1] != out->dims[di] || grid->dims[2] != out->dims[hi] || grid->dims[3] != out->dims[wi]) {
        set_error("expect grid and out to have same D H W size");
        return false;
    }
    if (input->dims[3] == 0 || input->dims[4] == 0) {
        set_error("expect input to have non-empty spatial dimensions");
        return false;
    }
    if (grid->dims[4] != 3) {
        set_error("expect grid to have size 3 in last dimension");
        return false;
    }
    return true;
}

}  // namespace

extern "C" {

aclnnStatus aclnnGridSampler3DGetWorkspaceSize(const aclTensor* input, const aclTensor* grid,
                                               int64_t interpolationMode, int64_t paddingMode, bool alignCorners,
                                               aclTensor* out, uint64_t* workspaceSize, aclOpExecutor** executor)
{
    std::unique_ptr<aclOpExecutor> ex(new (std::nothrow) aclOpExecutor());
    if (!ex) {
        set_error("aclnnGridSampler3D: cannot allocate the executor");
        return ACLNN_ERR_INNER_CREATE_EXECUTOR;
    }
    // aclnn_grid_sampler3d.cpp:60-66
    if (input == nullptr || grid == nullptr || out == nullptr) {
        set_error("aclnnGridSampler3D: input, grid and out must not be NULL");
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    if (workspaceSize == nullptr || executor == nullptr) {
        set_error("aclnnGridSampler3D: workspaceSize and executor must not be NULL");
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    if (!check_dtypes(input, grid, out) || !check_formats(input, out) ||
        !check_attrs(interpolationMode, paddingMode) || !check_shapes(input, grid, out)) {
        return ACLNN_ERR_PARAM_INVALID;
    }
    // aclnn_grid_sampler3d.cpp:323-327
    if (input->empty() || grid->empty()) {
        *workspaceSize = 0;
        *executor = ex.release();
        return ACLNN_SUCCESS;
    }
    // The reference routes DOUBLE to a host-CPU kernel that is not part of its tree; it does not exist here.
    Elem elem;
    if (!elem_of(input->dtype, &elem)) {
        set_error("aclnnGridSampler3D: DOUBLE tensors are not supported by the MI355X implementation");
        return ACLNN_ERR_PARAM_INVALID;
    }
    const bool ndhwc = input->format == ACL_FORMAT_NDHWC;
    const int ci = ndhwc ? 4 : 1, di = ndhwc ? 1 : 2, hi = ndhwc ? 2 : 3, wi = ndhwc ? 3 : 4;
    for (int i = 0; i < 5; i++) {
        if (input->dims[i] > INT32_MAX || grid->dims[i] > INT32_MAX) {
            set_error("aclnnGridSampler3D: every extent must fit in int32");
            return ACLNN_ERR_PARAM_INVALID;
        }
    }
    if (input->dims[hi] * input->dims[wi] > INT32_MAX) {
        set_error("aclnnGridSampler3D: Hin*Win must fit in int32");
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (grid->dims[1] * grid->dims[2] * grid->dims[3] > (int64_t)INT32_MAX * 256) {
        set_error("aclnnGridSampler3D: Dout*Hout*Wout is too large");
        return ACLNN_ERR_PARAM_INVALID;
    }

    ex->kind = OpKind::GridSampler3D;
    GridSampler3DArgs& a = ex->gs3;
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
    const int esz = elem_size(elem);
    // The kernel works on (N,C,D,H,W) operands.  A channels-last tensor is that operand seen through a permuted
    // view, which is packed (and the result scattered) like any other non-contiguous view; this takes the place of
    // the reference's transposes around its kernel (aclnn_grid_sampler3d.cpp:247-274).
    // Dense NDHWC tensors on both sides are sampled in place by the channels-last kernel.
    static const int kToNcdhw[5] = {0, 4, 1, 2, 3};
    if (ndhwc && input->contiguous() && out->contiguous()) {
        a.channels_last = 1;
        ex->in0 = plan_view(ex.get(), input, esz, false);
        ex->out0 = plan_view(ex.get(), out, esz, true);
    } else {
        ex->in0 = plan_view(ex.get(), input, esz, false, ndhwc ? kToNcdhw : nullptr);
        ex->out0 = plan_view(ex.get(), out, esz, true, ndhwc ? kToNcdhw : nullptr);
    }
    ex->in1 = plan_view(ex.get(), grid, esz, false);

    if (const aclnnStatus ps = plan_status(ex.get(), "aclnnGridSampler3D"); ps != ACLNN_SUCCESS) {
        return ps;
    }
    *workspaceSize = ex->workspace_bytes;
    *executor = ex.release();
    return ACLNN_SUCCESS;
}

aclnnStatus aclnnGridSampler3D(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor, aclrtStream stream)
{
    return run_executor(workspace, workspaceSize, executor, stream, OpKind::GridSampler3D, "aclnnGridSampler3D");
}

}  // extern "C"
