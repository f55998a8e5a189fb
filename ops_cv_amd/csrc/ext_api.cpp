// Introspection entry points (no counterpart in the reference).
#include "opscv_ext.h"

#include <hip/hip_runtime_api.h>

#include <cstring>

#include "acl_types.hpp"
#include "kernels.hpp"
#include "options.hpp"

using namespace opscv;

static_assert(sizeof(opscvTapRecord) == sizeof(TapRecord), "tap record layouts must match");
static_assert(sizeof(opscvBicubicTapRecord) == sizeof(BicubicTapRecord), "tap record layouts must match");

extern "C" {

aclnnStatus opscvGridSampler2DTaps(const void* grid, aclDataType dataType, int64_t N, int64_t Hin, int64_t Win,
                                   int64_t Hout, int64_t Wout, int64_t interpolationMode, int64_t paddingMode,
                                   bool alignCorners, opscvTapRecord* taps, aclrtStream stream)
{
    if (grid == nullptr || taps == nullptr) {
        set_error("opscvGridSampler2DTaps: grid and taps must not be NULL");
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    GridSamplerArgs a;
    if (!elem_of(dataType, &a.elem) || interpolationMode < 0 || interpolationMode > 1 || paddingMode < 0 ||
        paddingMode > 2) {
        set_error("opscvGridSampler2DTaps: unsupported dtype or mode");
        return ACLNN_ERR_PARAM_INVALID;
    }
    a.interp = (int)interpolationMode;
    a.pad = (int)paddingMode;
    a.align = alignCorners ? 1 : 0;
    a.N = N;
    a.C = 1;
    a.Hin = Hin;
    a.Win = Win;
    a.Hout = Hout;
    a.Wout = Wout;
    a.grid = grid;
    hipError_t e = launch_grid_sampler2d_taps(a, (TapRecord*)taps, (hipStream_t)stream);
    if (e == hipErrorInvalidValue) {
        set_error("opscvGridSampler2DTaps: shapes out of range");
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (e != hipSuccess) {
        set_error("opscvGridSampler2DTaps: launch failed: %s", hipGetErrorString(e));
        return ACLNN_ERR_RUNTIME_ERROR;
    }
    return ACLNN_SUCCESS;
}

aclnnStatus opscvGridSampler2DBicubicTaps(const void* grid, aclDataType dataType, int64_t N, int64_t Hin, int64_t Win,
                                          int64_t Hout, int64_t Wout, int64_t paddingMode, bool alignCorners,
                                          opscvBicubicTapRecord* taps, aclrtStream stream)
{
    if (grid == nullptr || taps == nullptr) {
        set_error("opscvGridSampler2DBicubicTaps: grid and taps must not be NULL");
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    GridSamplerArgs a;
    if (!elem_of(dataType, &a.elem) || paddingMode < 0 || paddingMode > 2) {
        set_error("opscvGridSampler2DBicubicTaps: unsupported dtype or mode");
        return ACLNN_ERR_PARAM_INVALID;
    }
    a.interp = 2;
    a.pad = (int)paddingMode;
    a.align = alignCorners ? 1 : 0;
    a.N = N;
    a.C = 1;
    a.Hin = Hin;
    a.Win = Win;
    a.Hout = Hout;
    a.Wout = Wout;
    a.grid = grid;
    hipError_t e = launch_grid_sampler2d_bicubic_taps(a, (BicubicTapRecord*)taps, (hipStream_t)stream);
    if (e == hipErrorInvalidValue) {
        set_error("opscvGridSampler2DBicubicTaps: shapes out of range");
        return ACLNN_ERR_PARAM_INVALID;
    }
    if (e != hipSuccess) {
        set_error("opscvGridSampler2DBicubicTaps: launch failed: %s", hipGetErrorString(e));
        return ACLNN_ERR_RUNTIME_ERROR;
    }
    return ACLNN_SUCCESS;
}

const char* opscvExecutorVariant(const aclOpExecutor* executor)
{
    if (executor == nullptr || executor->magic != kExecutorMagic) {
        return "";
    }
    switch (executor->kind) {
        case OpKind::GridSampler2D: return grid_sampler2d_variant(executor->gs);
        case OpKind::Resize: return resize_variant(executor->rs);
        case OpKind::ResizeGrad: return executor->rg.copy ? "copy" : resize_grad_variant(executor->rg);
        case OpKind::GridSampler2DGrad:
            // the grid gradient has a variant that stages the input planes through LDS
        {
            // input gradient: elections or lists; grid gradient: one lane per point or the LDS-ring variant
            const bool lists = executor->want_out0 && executor->scratch.in_workspace;
            const bool rings = executor->want_out1 && gs2d_grad_grid_uses_lds(executor->gsg);
            return lists ? (rings ? "gs2d_grad_lists_lds" : "gs2d_grad_lists")
                         : (rings ? "gs2d_grad_ordered_lds" : "gs2d_grad_ordered");
        }
        case OpKind::GridSampler3DGrad:
            // input gradient: a gather over every voxel's contributions, or elections in their order
            return (executor->want_out0 && gs3d_grad_list_words(executor->gsg3) > 0) ? "gs3d_grad_lists"
                                                                                      : "gs3d_grad_ordered";
        case OpKind::GridSampler3D:
            if (executor->gs3.channels_last) {
                return executor->gs3.interp == 0 ? "gs3d_ndhwc_bilinear" : "gs3d_ndhwc_nearest";
            }
            return executor->gs3.interp == 0 ? "gs3d_bilinear" : "gs3d_nearest";
        default: break;
    }
    return "";
}

aclnnStatus opscvSetOption(const char* name, int64_t value)
{
    if (name == nullptr) {
        set_error("opscvSetOption: name must not be NULL");
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    if (!set_option(name, value)) {
        set_error("opscvSetOption: unknown option '%s' or value %lld out of its range", name, (long long)value);
        return ACLNN_ERR_PARAM_INVALID;
    }
    return ACLNN_SUCCESS;
}

aclnnStatus opscvGetOption(const char* name, int64_t* value)
{
    if (name == nullptr || value == nullptr) {
        set_error("opscvGetOption: name and value must not be NULL");
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    if (!get_option(name, value)) {
        set_error("opscvGetOption: unknown option '%s'", name);
        return ACLNN_ERR_PARAM_INVALID;
    }
    return ACLNN_SUCCESS;
}

int32_t opscvVariantRevision(const char* variant)
{
    // longest matching prefix wins; bump an entry with the change that alters the variant's memory traffic
    static const struct {
        const char* prefix;
        int32_t revision;
    } table[] = {
        // 2 (ring and pair variants): streaming stores and grid loads, batch-fastest block order; ring: 5:3 channel split
        {"lds_ring", 4},
        {"lds_ring_pairs", 1},
        {"lds_pair", 2},       {"lds_pair_bicubic", 2}, {"box_lds", 1},          {"direct", 1},          {"direct_arch35", 1},          {"nhwc", 1},
        {"nchw_band_lds", 1},  {"nchw_flat_lds", 1},    {"nchw_band", 1},       {"nchw_generic", 1},
        {"nhwc_", 1},          {"nearest_", 1},         {"copy", 1},            {"point_copy", 1},
        {"broadcast", 1},      {"first_pixel", 1},      {"resize_grad", 1},     {"gs2d_grad", 4},
        {"gs3d_grad", 1},      {"gs3d_", 1},
    };
    if (variant == nullptr) {
        return 0;
    }
    int32_t best = 0;
    size_t best_len = 0;
    for (const auto& e : table) {
        const size_t n = strlen(e.prefix);
        if (strncmp(variant, e.prefix, n) == 0 && n >= best_len) {
            best = e.revision;
            best_len = n;
        }
    }
    return best;
}

const char* opscvVersion(void) { return "opscv-amd 0.1 (gfx950)"; }

}  // extern "C"
