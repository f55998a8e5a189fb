#include "resize_plan.hpp"

#include "options.hpp"

#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstdlib>

namespace opscv {

float resize_axis_scale(int64_t len_src, int64_t len_dst, bool align_corners, float user_scale)
{
    if (!align_corners) {
        if (user_scale > 0.0f) {
            return 1.0f / user_scale;
        }
        return (float)len_src / (float)len_dst;
    }
    if (len_dst > 1) {
        return (float)(len_src - 1) / (float)(len_dst - 1);
    }
    return (float)len_src / (float)len_dst;
}

// resize_bilinear_v2_tiling_arch35.cpp:254-303 (MatchPointCopyCondition, IsMatchPointCopy): channels-last data
// with runs of at least 128 bytes, shrunk by whole factors whose sampling points fall exactly on source pixels
// (always with align_corners; with half-pixel centres only for odd factors).  Every destination pixel is then a
// copy of one source pixel, and the reference copies instead of interpolating.
static bool point_copy_steps(const ResizeArgs& a, bool align_corners, int64_t* step_h, int64_t* step_w)
{
    if (!a.channels_last || a.C * elem_size(a.elem) < 128) {
        return false;
    }
    if (a.scale_h < 1.0f || a.scale_w < 1.0f) {
        return false;
    }
    const int64_t fh = (int64_t)(a.scale_h + FLT_EPSILON), fw = (int64_t)(a.scale_w + FLT_EPSILON);
    if (std::fabs(a.scale_h - (float)fh) >= FLT_EPSILON || std::fabs(a.scale_w - (float)fw) >= FLT_EPSILON) {
        return false;
    }
    *step_h = fh;
    *step_w = fw;
    if (align_corners) {
        return true;
    }
    if (!a.half_pixel) {
        return true;
    }
    return fh % 2 == 1 && fw % 2 == 1;
}

void plan_resize(ResizeArgs* a, bool align_corners, float user_scale_h, float user_scale_w)
{
    const Options opt = current_options();
    a->force_variant = opt.resize_variant;
    a->force_nearest = opt.nearest_variant;
    a->half_pixel = align_corners ? 0 : 1;
    a->scale_h = resize_axis_scale(a->Hs, a->Hd, align_corners, user_scale_h);
    a->scale_w = resize_axis_scale(a->Ws, a->Wd, align_corners, user_scale_w);
    const int64_t esz = elem_size(a->elem);
    constexpr int64_t kMinRunBytes = 128;  // MIN_C_SIZE of the reference tiling
    const bool one_src = (a->Hs == 1 && a->Ws == 1);
    const bool one_dst = (a->Hd == 1 && a->Wd == 1);
    // contiguous run the broadcast template copies per source element
    const int64_t run_bytes = a->channels_last ? a->C * esz : a->Hd * a->Wd * esz;
    a->mode = ResizeMode::Bilinear;
    if (a->Hs == a->Hd && a->Ws == a->Wd) {
        a->mode = ResizeMode::Copy;
    } else if (point_copy_steps(*a, align_corners, &a->point_step_h, &a->point_step_w)) {
        a->mode = ResizeMode::PointCopy;
    } else if (one_src && run_bytes >= kMinRunBytes) {
        a->mode = ResizeMode::Broadcast;
    } else if (a->channels_last && a->C * esz >= kMinRunBytes && a->scale_w >= 2.0f && a->scale_h >= 2.0f) {
        // resize_bilinear_v2_tiling_arch35.cpp:337-352,604 (IsMatchCParallel): long channel runs shrunk to half or less
        // go to the template that sums four weighted taps (resize_bilinear_v2_c_parallel.h:122-232); it comes before
        // the per-element template and its special cases
        a->mode = ResizeMode::FourWeights;
    } else if (one_src && align_corners) {
        a->mode = ResizeMode::Broadcast;
    } else if (one_dst && align_corners) {
        a->mode = ResizeMode::FirstPixel;
    }
    // resize_bilinear_v2_tiling_arch35.cpp:592-595,606-615: NCHW outputs of at least cores * 1024 pixels (cores * 512
    // when a tensor needs 64-bit indices) go to the template that splits H*W over the cores; it takes the fraction from
    // the unclamped source coordinate (see axis_tap), which only differs with half-pixel centres
    a->raw_lambda = 0;
    if (a->mode == ResizeMode::Bilinear && !a->channels_last && a->half_pixel) {
        const int64_t x_elems = a->N * a->C * a->Hs * a->Ws, y_elems = a->N * a->C * a->Hd * a->Wd;
        const bool idx32 = y_elems < (int64_t)UINT32_MAX && x_elems < (int64_t)UINT32_MAX;
        const int64_t threshold = reference_vector_cores() * (idx32 ? 1024 : 512);
        if (x_elems != 1 && a->Hd * a->Wd >= threshold) {
            a->raw_lambda = 1;
        }
    }
}

// option "reference_cores" (options.hpp): 64 unless set, the core count of the reference's tiling unit test
int64_t reference_vector_cores() { return current_options().reference_cores; }

// bytes of the reference device's unified buffer, option "reference_ub_bytes": 253952 unless set, that of the
// reference's tiling unit test
static int64_t reference_ub_bytes() { return current_options().reference_ub_bytes; }

// Whether the reference resizes this channels-last tensor with the template that replicates every source pixel a
// whole number of times (IsMatchTiling_NHWC_UB2UB, resize_nearest_neighbor_v2_tiling_base.cpp:640-665, called with
// align_corners = half_pixel_centers = false and no scales, aclnn_resize.cpp:278): an upscale by whole factors, 128
// bytes of channels or more per pixel, a source row and an output row that fit the unified buffer twice, tensors under
// 2^32 elements.  That template's index is destination / factor in integer arithmetic
// (resize_nearest_neighbor_v2_data_copy_nhwc.h:205-231); floor(float(destination) * scale), the rule of every other
// template, first differs from it at a factor of 41.
static bool nearest_replicates(const ResizeArgs& a)
{
    if (!a.channels_last || a.Wd <= a.Ws || a.Hd < a.Hs || a.Wd % a.Ws != 0 || a.Hd % a.Hs != 0) {
        return false;
    }
    const int64_t esz = elem_size(a.elem), block = 32;
    const int64_t c_bytes = a.C * esz;
    const bool whole_blocks = c_bytes % block == 0;
    const int64_t c_padded = (c_bytes + block - 1) / block * block / esz;  // channels rounded up to whole blocks
    if (whole_blocks ? c_padded * a.Ws * esz < 256 : c_bytes < 128) {
        return false;
    }
    if ((a.Ws + a.Wd) * c_padded * esz * 2 > reference_ub_bytes()) {
        return false;
    }
    if (a.N * a.C * a.Hs * a.Ws >= (int64_t)UINT32_MAX || a.N * a.C * a.Hd * a.Wd >= (int64_t)UINT32_MAX) {
        return false;
    }
    if (whole_blocks && a.Wd * c_bytes < 4096) {
        return false;
    }
    return a.Hd / a.Hs <= INT32_MAX && a.Wd / a.Ws <= INT32_MAX;
}

void plan_resize_nearest(ResizeArgs* a)
{
    const Options opt = current_options();
    a->force_variant = opt.resize_variant;
    a->force_nearest = opt.nearest_variant;
    a->half_pixel = 0;
    a->scale_h = (float)a->Hs / (float)a->Hd;
    a->scale_w = (float)a->Ws / (float)a->Wd;
    a->rep_h = a->rep_w = 0;
    if (nearest_replicates(*a)) {
        a->rep_h = (int32_t)(a->Hd / a->Hs);
        a->rep_w = (int32_t)(a->Wd / a->Ws);
    }
    a->mode = ResizeMode::Nearest;
    if (a->Hs == a->Hd && a->Ws == a->Wd) {
        a->mode = ResizeMode::Copy;  // every index maps to itself: floor(i * 1.0f) = i
    } else if (a->Hs == 1 && a->Ws == 1) {
        a->mode = ResizeMode::Broadcast;
    }
}

}  // namespace opscv
