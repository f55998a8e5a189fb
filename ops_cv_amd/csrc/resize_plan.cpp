#include "resize_plan.hpp"

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

void plan_resize(ResizeArgs* a, bool align_corners, float user_scale_h, float user_scale_w)
{
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
    } else if (one_src && (run_bytes >= kMinRunBytes || align_corners)) {
        a->mode = ResizeMode::Broadcast;
    } else if (one_dst && align_corners) {
        a->mode = ResizeMode::FirstPixel;
    }
}

void plan_resize_nearest(ResizeArgs* a)
{
    a->half_pixel = 0;
    a->scale_h = (float)a->Hs / (float)a->Hd;
    a->scale_w = (float)a->Ws / (float)a->Wd;
    a->mode = ResizeMode::Nearest;
    if (a->Hs == a->Hd && a->Ws == a->Wd) {
        a->mode = ResizeMode::Copy;  // every index maps to itself: floor(i * 1.0f) = i
    } else if (a->Hs == 1 && a->Ws == 1) {
        a->mode = ResizeMode::Broadcast;
    }
}

}  // namespace opscv
