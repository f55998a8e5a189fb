// Device-side arithmetic of the grid-sampler backward pass.
//
// Mirrors, operation for operation, the reference helpers
//   image/grid_sampler3_d_grad/op_kernel/arch35/grid_sampler3_d_grad_simt_base.h:50-311
// and the per-point code of
//   image/grid_sampler2_d_grad/op_kernel/arch35/grid_sampler2_d_grad_simt_det.h:103-355.
// The reference keeps several intermediates in the tensor's element type T; rt<T>() marks every place where a
// value is rounded to T (a no-op for float).  Products and sums are rounded separately (the translation unit is
// compiled with -ffp-contract=off).
#pragma once

#include <hip/hip_runtime.h>

#include "sampler_math.hpp"

namespace opscv {

template <typename T>
__device__ __forceinline__ float rt(float v)
{
    T t;
    ElemIO<T>::store(&t, v);
    return ElemIO<T>::load(&t);
}
template <>
__device__ __forceinline__ float rt<float>(float v)
{
    return v;
}

// grid_sampler3_d_grad_simt_base.h:50-66
template <typename T>
__device__ __forceinline__ float unnormalize_set_grad(float coord, int32_t size, int align, float* mult)
{
    float c;
    if (align == 1) {
        c = (coord + 1.0f) / 2.0f * (float)(size - 1);
        *mult = rt<T>((float)(size - 1) / 2.0f);
    } else {
        c = ((coord + 1.0f) * (float)size - 1.0f) / 2.0f;
        *mult = rt<T>((float)size / 2.0f);
    }
    // the fp32 result is pinned before it is rounded to T: product and conversion merged into one instruction would
    // round once where the reference rounds twice
    return rt<T>(as_fp32_value(c));
}

// grid_sampler3_d_grad_simt_base.h:68-86
template <typename T>
__device__ __forceinline__ float clip_set_grad(float coord, int32_t limit, float* g)
{
    if (coord <= 0.0f) {
        *g = 0.0f;
        return 0.0f;
    }
    const float mx = rt<T>((float)(limit - 1));
    if (coord >= mx) {
        *g = 0.0f;
        return mx;
    }
    *g = 1.0f;
    return coord;
}

// grid_sampler3_d_grad_simt_base.h:88-118.  span2 = twiceHigh - twiceLow.  The parity of floor(coord / span) is
// taken from the float: floats of 2^24 and more are even integers, a NaN quotient counts as even.
template <typename T>
__device__ __forceinline__ float reflect_set_grad(float coord, int32_t low2, int64_t span2, float* g)
{
    if (span2 == 0) {
        *g = 0.0f;
        return 0.0f;
    }
    const float mn = (float)low2 / 2.0f;
    const float span = (float)span2 / 2.0f;
    coord = rt<T>(coord - mn);
    float m;
    if (coord < 0.0f) {
        m = -1.0f;
        coord = -coord;
    } else {
        m = 1.0f;
    }
    const float extra = __builtin_fmodf(coord, span);
    const float fl = __builtin_floorf(coord / span);
    const bool odd = (fl < 16777216.0f) && (((int32_t)fl & 1) != 0);
    if (!odd) {
        *g = m;
        return rt<T>(extra + mn);
    }
    *g = -m;
    return rt<T>(span - extra + mn);
}

// grid_sampler3_d_grad_simt_base.h:159-185
template <typename T>
__device__ __forceinline__ float source_index_set_grad(float coord, int32_t size, int pad, int align, float* mult)
{
    float gc = 0.0f, gr = 0.0f;
    coord = unnormalize_set_grad<T>(coord, size, align, mult);
    if (pad == 1) {
        coord = clip_set_grad<T>(coord, size, &gc);
        *mult = rt<T>(*mult * gc);
    } else if (pad == 2) {
        if (align) {
            coord = reflect_set_grad<T>(coord, 0, 2 * ((int64_t)size - 1), &gr);
        } else {
            coord = reflect_set_grad<T>(coord, -1, 2 * (int64_t)size, &gr);
        }
        coord = clip_set_grad<T>(coord, size, &gc);
        *mult = rt<T>(*mult * gr * gc);
    }
    if (nan_or_inf(coord)) {
        return -100.0f;
    }
    return coord;
}

// grid_sampler3_d_grad_simt_base.h:216-246: derivatives of the four cubic coefficients with respect to t
__device__ __forceinline__ void cubic_coefficients_grad(float c[4], float t)
{
    const float A = -0.75f;
    float x = t + 1.0f;
    c[0] = (3.0f * A * x - 10.0f * A) * x + 8.0f * A;
    x = t;
    c[1] = (3.0f * (A + 2.0f) * x - 2.0f * (A + 3.0f)) * x;
    x = 1.0f - t;
    c[2] = -((3.0f * (A + 2.0f) * x - 2.0f * (A + 3.0f)) * x);
    x = 2.0f - t;
    c[3] = -((3.0f * A * x - 10.0f * A) * x + 8.0f * A);
}

// grid_sampler3_d_grad_simt_base.h:198-214
__device__ __forceinline__ void cubic_coefficients(float c[4], float t)
{
    c[0] = cubic_convolution2(t + 1.0f, -0.75f);
    c[1] = cubic_convolution1(t, -0.75f);
    c[2] = cubic_convolution1(1.0f - t, -0.75f);
    c[3] = cubic_convolution2(2.0f - t, -0.75f);
}

// Plane offset of the bicubic tap at float coordinates (x, y) after padding, or -1 when the tap falls outside
// (grid_sampler3_d_grad_simt_base.h:249-311 and grid_sampler2_d_grad_simt_det.h:239-277: the same rule for reading
// x and for adding into its gradient).
__device__ __forceinline__ int32_t bicubic_bounded_offset(float x, float y, int32_t W, int32_t H, int pad, int align)
{
    if (pad == 0) {
        if (x < 0.0f || x >= (float)W || y < 0.0f || y >= (float)H) {
            return -1;
        }
    } else if (pad == 1) {
        x = (x < 0.0f) ? 0.0f : ((x >= (float)W) ? (float)W - 1.0f : x);
        y = (y < 0.0f) ? 0.0f : ((y >= (float)H) ? (float)H - 1.0f : y);
    } else {
        float g;
        if (align) {
            x = reflect_set_grad<float>(x, 0, 2 * ((int64_t)W - 1), &g);
            y = reflect_set_grad<float>(y, 0, 2 * ((int64_t)H - 1), &g);
        } else {
            x = reflect_set_grad<float>(x, -1, 2 * (int64_t)W, &g);
            y = reflect_set_grad<float>(y, -1, 2 * (int64_t)H, &g);
        }
        x = clip_set_grad<float>(x, W, &g);
        y = clip_set_grad<float>(y, H, &g);
    }
    const int32_t ix = float_to_i32(nan_or_inf(x) ? -100.0f : x);
    const int32_t iy = float_to_i32(nan_or_inf(y) ? -100.0f : y);
    if (ix >= 0 && ix < W && iy >= 0 && iy < H) {
        return iy * W + ix;
    }
    return -1;
}

// Per grid point: where its contributions land in the (H, W) plane and with what weight.
//   INTERP 0: four corners nw, ne, sw, se; weight = rt<T>(product of the two distances)
//   INTERP 1: one tap, weight 1
//   INTERP 2: sixteen taps, index i * 4 + j with i along x and j along y; weight = cx[i] * cy[j]
// off[k] = -1 marks a tap outside the plane.  fx/fy receive the source coordinates, mx/my the chain-rule
// multipliers of the grid gradient.
template <typename T, int INTERP>
struct GradTaps {
    static constexpr int NT = (INTERP == 0) ? 4 : ((INTERP == 1) ? 1 : 16);
    int32_t off[NT];
    float w[NT];
    float fx, fy, mx, my;
    int32_t x0, y0;  // bilinear: north-west corner
};

template <typename T, int INTERP>
__device__ __forceinline__ void decide_grad_taps(GradTaps<T, INTERP>& t, float gx, float gy, int32_t H, int32_t W,
                                                 int pad, int align)
{
    if (INTERP == 2) {
        // grid_sampler2_d_grad_simt_det.h:378-381: only unnormalized; padding applies to every tap
        t.fy = unnormalize_set_grad<T>(gy, H, align, &t.my);
        t.fx = unnormalize_set_grad<T>(gx, W, align, &t.mx);
        const float xf = __builtin_floorf(t.fx), yf = __builtin_floorf(t.fy);
        float cx[4], cy[4];
        cubic_coefficients(cy, t.fy - yf);
        cubic_coefficients(cx, t.fx - xf);
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float nx = xf - 1.0f + (float)i;
                const float ny = yf - 1.0f + (float)j;
                t.off[i * 4 + j] = bicubic_bounded_offset(nx, ny, W, H, pad, align);
                t.w[i * 4 + j] = cx[i] * cy[j];
            }
        }
        t.x0 = t.y0 = 0;
        return;
    }
    t.fy = source_index_set_grad<T>(gy, H, pad, align, &t.my);
    t.fx = source_index_set_grad<T>(gx, W, pad, align, &t.mx);
    if (INTERP == 1) {
        const int32_t xi = float_to_i32(__builtin_rintf(t.fx));
        const int32_t yi = float_to_i32(__builtin_rintf(t.fy));
        t.off[0] = within(yi, xi, H, W) ? yi * W + xi : -1;
        t.w[0] = 1.0f;
        t.x0 = xi;
        t.y0 = yi;
        return;
    }
    const int32_t x0 = float_to_i32(__builtin_floorf(t.fx));
    const int32_t y0 = float_to_i32(__builtin_floorf(t.fy));
    t.x0 = x0;
    t.y0 = y0;
    const int32_t x1 = (x0 == INT32_MAX) ? x0 : x0 + 1, y1 = (y0 == INT32_MAX) ? y0 : y0 + 1;
    const float dxe = (float)x1 - t.fx, dxw = t.fx - (float)x0;
    const float dys = (float)y1 - t.fy, dyn = t.fy - (float)y0;
    t.w[0] = rt<T>(dxe * dys);
    t.w[1] = rt<T>(dxw * dys);
    t.w[2] = rt<T>(dxe * dyn);
    t.w[3] = rt<T>(dxw * dyn);
    t.off[0] = within(y0, x0, H, W) ? y0 * W + x0 : -1;
    t.off[1] = within(y0, x1, H, W) ? y0 * W + x1 : -1;
    t.off[2] = within(y1, x0, H, W) ? y1 * W + x0 : -1;
    t.off[3] = within(y1, x1, H, W) ? y1 * W + x1 : -1;
}

}  // namespace opscv
