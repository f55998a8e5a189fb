// Per-axis source coordinate of the bilinear resize, usable on host and device (the file is always compiled
// with -ffp-contract=off, so both sides round every operation separately and agree bit for bit).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace opscv {

struct AxisTap {
    int32_t i0, i1;
    float lambda;
};

// image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_simt_nchw.h:108-134 for one axis.
//
// raw_lambda selects the arithmetic of the reference's template for large outputs
// (image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_simt_hw.h:79-86): it does not clamp the source
// coordinate at zero before taking the fraction, so the first rows and columns of a half-pixel upscale (coordinate
// in [-0.5, 0)) blend the border pixel with itself, (1-l)*v + l*v with l = coordinate + 1, instead of passing it
// through with l = 0.  Its taps are the same: floor and ceil converted to an unsigned index and capped at size-1,
// a negative floor taken as index 0 (the conversion is undefined in C++; zero is what the clamp the reference
// writes around it intends).
template <bool HALF_PIXEL>
__host__ __device__ __forceinline__ AxisTap axis_tap(int32_t d, float scale, int32_t len_src, int raw_lambda = 0)
{
    float orig;
    if (HALF_PIXEL) {
        orig = ((float)d + 0.5f) * scale - 0.5f;
    } else {
        orig = (float)d * scale;
    }
    const float raw = orig;
    if (orig < 0.0f) {
        orig = 0.0f;
    }
    const float fl = __builtin_floorf(orig);
    const float lo = (orig > 0.0f) ? fl : 0.0f;
    const float hi = (orig > 0.0f) ? __builtin_ceilf(orig) : 0.0f;
    const float last = (float)(len_src - 1);
    AxisTap t;
    t.i0 = (lo < last) ? (int32_t)lo : len_src - 1;
    t.i1 = (hi < last) ? (int32_t)hi : len_src - 1;
    t.lambda = orig - fl;
    if (HALF_PIXEL && raw_lambda != 0) {
        t.lambda = raw - __builtin_floorf(raw);
    }
    return t;
}

}  // namespace opscv
