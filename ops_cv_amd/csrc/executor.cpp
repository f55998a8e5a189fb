// Second-phase runner and view-packing plan shared by the aclnn entry points.
#include "executor.hpp"

#include <hip/hip_runtime_api.h>

#include "kernels.hpp"

namespace opscv {

namespace {
uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }
}  // namespace

PlannedPtr plan_view(aclOpExecutor* ex, const aclTensor* t, int elem_bytes, bool is_output, const int* perm)
{
    PlannedPtr p;
    char* base = (t->data == nullptr) ? nullptr : (char*)t->data + t->offset * (int64_t)elem_bytes;
    aclOpExecutor::Pack pk;
    pk.view.base = base;
    const int n = (int)t->ndim;
    const int lead = kViewDims - n;
    for (int i = 0; i < lead; i++) {
        pk.view.dims[i] = 1;
        pk.view.strides[i] = 0;
    }
    for (int i = 0; i < n; i++) {
        const int src = (perm != nullptr) ? perm[i] : i;
        pk.view.dims[lead + i] = t->dims[src];
        pk.view.strides[lead + i] = t->strides[src];
    }
    bool dense = true;
    int64_t expect = 1;
    for (int i = kViewDims - 1; i >= 0; i--) {
        if (pk.view.dims[i] != 1 && pk.view.strides[i] != expect) {
            dense = false;
        }
        expect *= pk.view.dims[i];
    }
    if (dense) {
        p.direct = base;
        return p;
    }
    pk.elem_bytes = elem_bytes;
    pk.ws_offset = align_up(ex->workspace_bytes, 256);
    ex->workspace_bytes = pk.ws_offset + (uint64_t)t->numel() * (uint64_t)elem_bytes;
    p.in_workspace = true;
    p.ws_offset = pk.ws_offset;
    if (!(is_output ? ex->unpack_out.push_back(pk) : ex->pack_in.push_back(pk))) {
        ex->pack_overflow = true;
    }
    return p;
}

aclnnStatus plan_status(const aclOpExecutor* ex, const char* api)
{
    if (ex->pack_overflow) {
        set_error("%s: more strided views than the plan can pack", api);
        return ACLNN_ERR_INNER;
    }
    return ACLNN_SUCCESS;
}

aclnnStatus run_executor(void* workspace, uint64_t workspace_size, aclOpExecutor* ex, aclrtStream stream,
                         OpKind expected, const char* api)
{
    if (ex == nullptr) {
        set_error("%s: executor is NULL", api);
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    if (ex->magic != kExecutorMagic) {
        set_error("%s: executor is not live (already consumed?)", api);
        return ACLNN_ERR_PARAM_INVALID;
    }
    std::unique_ptr<aclOpExecutor> owner(ex);  // consumed whatever happens below
    ex->magic = 0;
    if (ex->kind != OpKind::Nop && ex->kind != expected) {
        set_error("%s: executor was created by a different operator", api);
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (ex->workspace_bytes > 0) {
        if (workspace == nullptr) {
            set_error("%s: workspace is NULL but %llu bytes are required", api,
                      (unsigned long long)ex->workspace_bytes);
            return ACLNN_ERR_PARAM_NULLPTR;
        }
        if (workspace_size < ex->workspace_bytes) {
            set_error("%s: workspace of %llu bytes is smaller than the %llu required", api,
                      (unsigned long long)workspace_size, (unsigned long long)ex->workspace_bytes);
            return ACLNN_ERR_PARAM_INVALID;
        }
        // the slices handed to the kernels are cut at multiples of 256 bytes from the workspace's start and are read
        // and written with 16-byte vector accesses and 32-bit atomics
        if (reinterpret_cast<uintptr_t>(workspace) % kWorkspaceAlignment != 0) {
            set_error("%s: the workspace must start on a %d-byte boundary", api, (int)kWorkspaceAlignment);
            return ACLNN_ERR_PARAM_INVALID;
        }
    }
    return execute_plan(workspace, ex, stream, api);
}

aclnnStatus execute_plan(void* workspace, const aclOpExecutor* ex, aclrtStream stream, const char* api)
{
    if (ex->kind == OpKind::Nop) {
        return ACLNN_SUCCESS;
    }
    if (ex->pack_overflow) {
        set_error("%s: more strided views than the plan can pack", api);
        return ACLNN_ERR_INNER;
    }
    hipStream_t s = (hipStream_t)stream;
    for (const auto& pk : ex->pack_in) {
        if (pk.view.base == nullptr) {
            set_error("%s: tensor data pointer is NULL", api);
            return ACLNN_ERR_PARAM_NULLPTR;
        }
        hipError_t e = launch_strided_copy(pk.view, (char*)workspace + pk.ws_offset, pk.elem_bytes, true, s);
        if (e != hipSuccess) {
            set_error("%s: packing a strided input failed: %s", api, hipGetErrorString(e));
            return ACLNN_ERR_RUNTIME_ERROR;
        }
    }
    hipError_t e = hipSuccess;
    if (ex->kind == OpKind::GridSampler2D) {
        GridSamplerArgs a = ex->gs;
        a.x = resolve(ex->in0, workspace);
        a.grid = resolve(ex->in1, workspace);
        a.y = resolve(ex->out0, workspace);
        if (a.x == nullptr || a.grid == nullptr || a.y == nullptr) {
            set_error("%s: tensor data pointer is NULL", api);
            return ACLNN_ERR_PARAM_NULLPTR;
        }
        e = launch_grid_sampler2d(a, s);
    } else if (ex->kind == OpKind::GridSampler2DGrad) {
        GridSamplerGradArgs a = ex->gsg;
        a.gout = resolve(ex->in0, workspace);
        a.x = resolve(ex->in1, workspace);
        a.grid = resolve(ex->in2, workspace);
        a.dx = ex->want_out0 ? resolve(ex->out0, workspace) : nullptr;
        a.dgrid = ex->want_out1 ? resolve(ex->out1, workspace) : nullptr;
        a.scratch = ex->scratch.in_workspace ? resolve(ex->scratch, workspace) : nullptr;
        if (a.gout == nullptr || a.x == nullptr || a.grid == nullptr || (ex->want_out0 && a.dx == nullptr) ||
            (ex->want_out1 && a.dgrid == nullptr)) {
            set_error("%s: tensor data pointer is NULL", api);
            return ACLNN_ERR_PARAM_NULLPTR;
        }
        e = launch_grid_sampler2d_grad(a, s);
    } else if (ex->kind == OpKind::GridSampler3DGrad) {
        GridSampler3DGradArgs a = ex->gsg3;
        a.gout = resolve(ex->in0, workspace);
        a.x = resolve(ex->in1, workspace);
        a.grid = resolve(ex->in2, workspace);
        a.dx = ex->want_out0 ? resolve(ex->out0, workspace) : nullptr;
        a.dgrid = ex->want_out1 ? resolve(ex->out1, workspace) : nullptr;
        if (ex->scratch.in_workspace) {
            char* scratch = static_cast<char*>(resolve(ex->scratch, workspace));
            const int64_t range_words = gs3d_grad_range_words(a);
            a.chunk_ranges = range_words > 0 ? scratch : nullptr;
            a.lists = gs3d_grad_list_words(a) > 0 ? scratch + gs3d_grad_lists_offset(range_words) : nullptr;
        }
        if (a.gout == nullptr || a.x == nullptr || a.grid == nullptr || (ex->want_out0 && a.dx == nullptr) ||
            (ex->want_out1 && a.dgrid == nullptr)) {
            set_error("%s: tensor data pointer is NULL", api);
            return ACLNN_ERR_PARAM_NULLPTR;
        }
        e = launch_grid_sampler3d_grad(a, s);
    } else if (ex->kind == OpKind::GridSampler3D) {
        GridSampler3DArgs a = ex->gs3;
        a.x = resolve(ex->in0, workspace);
        a.grid = resolve(ex->in1, workspace);
        a.y = resolve(ex->out0, workspace);
        if (a.x == nullptr || a.grid == nullptr || a.y == nullptr) {
            set_error("%s: tensor data pointer is NULL", api);
            return ACLNN_ERR_PARAM_NULLPTR;
        }
        e = launch_grid_sampler3d(a, s);
    } else if (ex->kind == OpKind::ResizeGrad) {
        ResizeGradArgs a = ex->rg;
        a.x = resolve(ex->in0, workspace);
        a.y = resolve(ex->out0, workspace);
        if (a.x == nullptr || a.y == nullptr) {
            set_error("%s: tensor data pointer is NULL", api);
            return ACLNN_ERR_PARAM_NULLPTR;
        }
        e = launch_resize_grad(a, s);
    } else {
        ResizeArgs a = ex->rs;
        a.x = resolve(ex->in0, workspace);
        a.y = resolve(ex->out0, workspace);
        if (a.x == nullptr || a.y == nullptr) {
            set_error("%s: tensor data pointer is NULL", api);
            return ACLNN_ERR_PARAM_NULLPTR;
        }
        e = launch_resize(a, s);
    }
    if (e != hipSuccess) {
        set_error("%s: kernel launch failed: %s", api, hipGetErrorString(e));
        return ACLNN_ERR_RUNTIME_ERROR;
    }
    for (const auto& pk : ex->unpack_out) {
        if (pk.view.base == nullptr) {
            set_error("%s: tensor data pointer is NULL", api);
            return ACLNN_ERR_PARAM_NULLPTR;
        }
        e = launch_strided_copy(pk.view, (char*)workspace + pk.ws_offset, pk.elem_bytes, false, s);
        if (e != hipSuccess) {
            set_error("%s: scattering the strided output failed: %s", api, hipGetErrorString(e));
            return ACLNN_ERR_RUNTIME_ERROR;
        }
    }
    return ACLNN_SUCCESS;
}

}  // namespace opscv
