// Device-side coordinate arithmetic shared by the grid-sampler kernels.
//
// Every function mirrors, operation for operation, the scalar code of the reference SIMT kernel
// image/grid_sampler2_d/op_kernel/arch35/grid_sampler2_d_simt.h.  The translation unit is compiled with
// -ffp-contract=off, so a*b+c is two roundings everywhere except the single explicit fused multiply-add
// in unnormalize(), exactly as in the reference (grid_sampler2_d_simt.h:74,131).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace opscv {

// ---- element <-> float conversion (round to nearest even on the way out) ----
template <typename T>
struct ElemIO;

template <>
struct ElemIO<float> {
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};

template <>
struct ElemIO<_Float16> {
    static __device__ __forceinline__ float load(const _Float16* p) { return (float)*p; }
    static __device__ __forceinline__ void store(_Float16* p, float v) { *p = (_Float16)v; }
};

template <>
struct ElemIO<__bf16> {
    static __device__ __forceinline__ float load(const __bf16* p)
    {
        // the object is read as what it is and its bits reinterpreted afterwards (reading it through a
        // uint16_t lvalue would let the compiler reorder the read against writes of the __bf16 object)
        return __builtin_bit_cast(float, (uint32_t)__builtin_bit_cast(uint16_t, *p) << 16);
    }
    static __device__ __forceinline__ void store(__bf16* p, float v) { *p = (__bf16)v; }
};

// Store of one element with the non-temporal hint (same rounding as ElemIO<T>::store): for results that are written
// once and not read again by the kernel, so that they are written through instead of staying dirty in L2.
template <typename T>
__device__ __forceinline__ void store_streaming(T* p, float v)
{
    T e;
    ElemIO<T>::store(&e, v);
    if constexpr (sizeof(T) == 4) {
        __builtin_nontemporal_store(__builtin_bit_cast(uint32_t, e), reinterpret_cast<uint32_t*>(p));
    } else {
        __builtin_nontemporal_store(__builtin_bit_cast(uint16_t, e), reinterpret_cast<uint16_t*>(p));
    }
}

// grid_sampler2_d_simt.h:125-132
template <bool ALIGN>
__device__ __forceinline__ float unnormalize(float coord, int32_t size)
{
    if (ALIGN) {
        return ((coord + 1.0f) / 2.0f) * (float)(size - 1);
    }
    float scaling = (float)size / 2.0f;
    return __builtin_fmaf(scaling, coord + 1.0f, -0.5f);
}

// grid_sampler2_d_simt.h:136-143
__device__ __forceinline__ float clip_coordinates(float coord, int32_t size)
{
    float max_val = (float)(size - 1);
    if (__builtin_isnan(coord)) {
        return 0.0f;
    }
    return __builtin_fminf(__builtin_fmaxf(coord, 0.0f), max_val);
}

// grid_sampler2_d_simt.h:171-185 (product and difference are rounded separately)
__device__ __forceinline__ float reflect_coordinates(float coord, float low, float twice_span)
{
    if (twice_span == 0.0f) {
        return 0.0f;
    }
    float abs_in = __builtin_fabsf(coord - low);
    float flips = __builtin_truncf(abs_in / twice_span);
    float product = flips * twice_span;
    float extra = abs_in - product;
    float complement = twice_span - extra;
    return __builtin_fminf(extra, complement) + low;
}

// grid_sampler2_d_simt.h:187-200
template <int PAD, bool ALIGN>
__device__ __forceinline__ float compute_coordinates(float coord, int32_t size)
{
    if (PAD == 1) {
        coord = clip_coordinates(coord, size);
    } else if (PAD == 2) {
        if (ALIGN) {
            coord = reflect_coordinates(coord, 0.0f, 2.0f * (float)(size - 1));
        } else {
            coord = reflect_coordinates(coord, -0.5f, 2.0f * (float)size);
        }
        coord = clip_coordinates(coord, size);
    }
    return coord;
}

// grid_sampler2_d_simt.h:202-207
template <int PAD, bool ALIGN>
__device__ __forceinline__ float compute_source_index(float coord, int32_t size)
{
    return compute_coordinates<PAD, ALIGN>(unnormalize<ALIGN>(coord, size), size);
}

// The same with padding mode and align_corners as run-time, wave-uniform values (kernel arguments): each branch is the
// instantiation above, so the arithmetic is identical; the branches are scalar.
__device__ __forceinline__ float unnormalize_rt(float coord, int32_t size, bool align)
{
    return align ? unnormalize<true>(coord, size) : unnormalize<false>(coord, size);
}

__device__ __forceinline__ float compute_coordinates_rt(float coord, int32_t size, int32_t pad, bool align)
{
    if (pad == 1) {
        coord = clip_coordinates(coord, size);
    } else if (pad == 2) {
        coord = align ? reflect_coordinates(coord, 0.0f, 2.0f * (float)(size - 1))
                      : reflect_coordinates(coord, -0.5f, 2.0f * (float)size);
        coord = clip_coordinates(coord, size);
    }
    return coord;
}

__device__ __forceinline__ float compute_source_index_rt(float coord, int32_t size, int32_t pad, bool align)
{
    return compute_coordinates_rt(unnormalize_rt(coord, size, align), size, pad, align);
}

__device__ __forceinline__ bool nan_or_inf(float x) { return __builtin_isnan(x) || __builtin_isinf(x); }

// grid_sampler2_d_simt.h:209-215
__device__ __forceinline__ float safe_downgrade(float x)
{
    if (x > 2147483646.0f || x < -2147483648.0f || nan_or_inf(x)) {
        return -100.0f;
    }
    return x;
}

// float -> int32 with saturation: values from 2^31 up give INT32_MAX, values below -2^31 give INT32_MIN (either is out
// of bounds for every caller) and NaN gives 0.  This is what the hardware conversion does by itself; spelled with
// comparisons in C++ (where the out-of-range cast is undefined) it compiles to branches around the same instruction.
__device__ __forceinline__ int32_t float_to_i32(float v)
{
    int32_t r;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(v));
    return r;
}

// grid_sampler2_d_simt.h:219-234
__device__ __forceinline__ int32_t banker_round(float x)
{
    float fl = __builtin_floorf(x);
    float frac = x - fl;
    int32_t fi = float_to_i32(fl);
    int32_t up = (fi == INT32_MAX) ? fi : fi + 1;
    if (frac < 0.5f) {
        return fi;
    }
    if (frac > 0.5f) {
        return up;
    }
    return ((fi & 1) == 0) ? fi : up;
}

// What the sampler decides per output pixel, before the channel loop.
struct PixelTap {
    int32_t x0, y0;  // bilinear: north-west corner; nearest: the selected texel
    float w[4];      // nw, ne, sw, se (bilinear only)
    int32_t flag;    // 1: write NaN to every channel (non-finite source coordinate, bilinear only)
};

// grid_sampler2_d_simt.h:479-498 and :307-316
template <int INTERP, int PAD, bool ALIGN>
__device__ __forceinline__ PixelTap decide_pixel(float gx, float gy, int32_t H, int32_t W)
{
    PixelTap t;
    float ix = compute_source_index<PAD, ALIGN>(gx, W);
    float iy = compute_source_index<PAD, ALIGN>(gy, H);
    t.flag = 0;
    t.w[0] = t.w[1] = t.w[2] = t.w[3] = 0.0f;
    if (INTERP == 0) {
        if (nan_or_inf(ix) || nan_or_inf(iy)) {
            t.flag = 1;
            t.x0 = 0;
            t.y0 = 0;
            return t;
        }
        ix = safe_downgrade(ix);
        iy = safe_downgrade(iy);
        float ixf = __builtin_floorf(ix);
        float iyf = __builtin_floorf(iy);
        t.x0 = float_to_i32(ixf);
        t.y0 = float_to_i32(iyf);
        t.w[0] = (ixf + 1.0f - ix) * (iyf + 1.0f - iy);
        t.w[1] = (ix - ixf) * (iyf + 1.0f - iy);
        t.w[2] = (ixf + 1.0f - ix) * (iy - iyf);
        t.w[3] = (ix - ixf) * (iy - iyf);
    } else {
        ix = safe_downgrade(ix);
        iy = safe_downgrade(iy);
        t.x0 = banker_round(ix);
        t.y0 = banker_round(iy);
    }
    return t;
}

// ---- bicubic mode (A = -0.75), grid_sampler2_d_simt.h:271-298 and :375-412 ----

// every product, sum and difference rounds separately (the translation unit has contraction off)
__device__ __forceinline__ float cubic_convolution1(float x, float a)
{
    float t0 = (a + 2.0f) * x;
    float t1 = t0 - (a + 3.0f);
    float t2 = t1 * x;
    float t3 = t2 * x;
    return t3 + 1.0f;
}

__device__ __forceinline__ float cubic_convolution2(float x, float a)
{
    float t0 = a * x;
    float t1 = t0 - 5.0f * a;
    float t2 = t1 * x;
    float t3 = t2 + 8.0f * a;
    float t4 = t3 * x;
    return t4 - 4.0f * a;
}

__device__ __forceinline__ int32_t safe_float_to_i32(float f)
{
    if (f >= 0.0f && f < 2147483648.0f) {
        return (int32_t)f;
    }
    return -1;
}

// Pins a value as an fp32 register.  The reference rounds the last fused multiply-add of the bicubic sum to fp32
// and then converts to the 16-bit output type (two roundings); without this the compiler merges that
// multiply-add and the conversion into one instruction that rounds once, which differs on exact ties.
__device__ __forceinline__ float as_fp32_value(float v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// grid_sampler2_d_simt.h:362-371: a plain product, then three explicit fused multiply-adds
__device__ __forceinline__ float bicubic_weighted_sum(float c0, float c1, float c2, float c3, float v0, float v1,
                                                      float v2, float v3)
{
    float r = c0 * v0;
    r = __builtin_fmaf(c1, v1, r);
    r = __builtin_fmaf(c2, v2, r);
    r = __builtin_fmaf(c3, v3, r);
    return as_fp32_value(r);
}

struct BicubicTap {
    int32_t bx[4], by[4];  // tap columns / rows after padding; -1 = outside
    float cx[4], cy[4];    // column / row coefficients
    int32_t flag;          // 1: write NaN to every channel (non-finite source coordinate)
};

// grid_sampler2_d_simt.h:499-503 (the coordinate is only unnormalized; padding applies to every tap) and :379-412
template <int PAD, bool ALIGN>
__device__ __forceinline__ BicubicTap decide_bicubic(float gx, float gy, int32_t H, int32_t W)
{
    constexpr float A = -0.75f;
    BicubicTap t;
    const float ix = unnormalize<ALIGN>(gx, W);
    const float iy = unnormalize<ALIGN>(gy, H);
    t.flag = 0;
    if (nan_or_inf(ix) || nan_or_inf(iy)) {
        t.flag = 1;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            t.bx[k] = t.by[k] = 0;
            t.cx[k] = t.cy[k] = 0.0f;
        }
        return t;
    }
    const float ixf = __builtin_floorf(ix);
    const float iyf = __builtin_floorf(iy);
    const float tx = ix - ixf;
    const float ty = iy - iyf;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        t.bx[k] = safe_float_to_i32(compute_coordinates<PAD, ALIGN>(ixf + (float)(k - 1), W));
        t.by[k] = safe_float_to_i32(compute_coordinates<PAD, ALIGN>(iyf + (float)(k - 1), H));
    }
    t.cx[0] = cubic_convolution2(tx + 1.0f, A);
    t.cx[1] = cubic_convolution1(tx, A);
    t.cx[2] = cubic_convolution1(1.0f - tx, A);
    t.cx[3] = cubic_convolution2(2.0f - tx, A);
    t.cy[0] = cubic_convolution2(ty + 1.0f, A);
    t.cy[1] = cubic_convolution1(ty, A);
    t.cy[2] = cubic_convolution1(1.0f - ty, A);
    t.cy[3] = cubic_convolution2(2.0f - ty, A);
    return t;
}

// decide_bicubic with run-time padding mode and align_corners (see compute_coordinates_rt)
__device__ __forceinline__ BicubicTap decide_bicubic_rt(float gx, float gy, int32_t H, int32_t W, int32_t pad, bool align)
{
    constexpr float A = -0.75f;
    BicubicTap t;
    const float ix = unnormalize_rt(gx, W, align);
    const float iy = unnormalize_rt(gy, H, align);
    t.flag = 0;
    if (nan_or_inf(ix) || nan_or_inf(iy)) {
        t.flag = 1;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            t.bx[k] = t.by[k] = 0;
            t.cx[k] = t.cy[k] = 0.0f;
        }
        return t;
    }
    const float ixf = __builtin_floorf(ix);
    const float iyf = __builtin_floorf(iy);
    const float tx = ix - ixf;
    const float ty = iy - iyf;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        t.bx[k] = safe_float_to_i32(compute_coordinates_rt(ixf + (float)(k - 1), W, pad, align));
        t.by[k] = safe_float_to_i32(compute_coordinates_rt(iyf + (float)(k - 1), H, pad, align));
    }
    t.cx[0] = cubic_convolution2(tx + 1.0f, A);
    t.cx[1] = cubic_convolution1(tx, A);
    t.cx[2] = cubic_convolution1(1.0f - tx, A);
    t.cx[3] = cubic_convolution2(2.0f - tx, A);
    t.cy[0] = cubic_convolution2(ty + 1.0f, A);
    t.cy[1] = cubic_convolution1(ty, A);
    t.cy[2] = cubic_convolution1(1.0f - ty, A);
    t.cy[3] = cubic_convolution2(2.0f - ty, A);
    return t;
}

// ---- the coordinate rule of the reference's GridSample operator on its arch35 part ----
// (the 3-D sampler follows it; the 2-D sampler offers it as its second rule: the kernel that the reference's
// aclnnGridSampler2D launches there, image/grid_sample/op_kernel/arch35/grid_sampler_2d_bilinear_smit.h:109-153)

// grid_sampler_bilinear_smit_common.h:37-46 (size is an unsigned index type there: size - 1 is converted to
// float for the comparison, the replacement value is float(size) - 1)
__device__ __forceinline__ float clip3_coordinates(float coord, int32_t size)
{
    coord = (coord < 0.0f) ? 0.0f : coord;
    coord = (coord > (float)(size - 1)) ? (float)size - 1.0f : coord;
    if (__builtin_isnan(coord) || __builtin_isinf(coord)) {
        return 0.0f;
    }
    return coord;
}

// grid_sampler_bilinear_smit_common.h:48-66.  `low2` is twiceLow (0 or -1), `span2` is twiceHigh - twiceLow.
// The parity of floor(coord / span) is taken from the float itself: every float of 2^24 or more is an even
// integer, below that the conversion to an integer is exact.
__device__ __forceinline__ float reflect3_coordinates(float coord, int32_t low2, int64_t span2)
{
    if (span2 == 0) {
        return 0.0f;
    }
    const float mn = (float)low2 / 2.0f;
    const float span = (float)span2 / 2.0f;
    coord = __builtin_fabsf(coord - mn);
    const float extra = __builtin_fmodf(coord, span);
    const float fl = __builtin_floorf(coord / span);
    const bool odd = (fl < 16777216.0f) && (((int32_t)fl & 1) != 0);
    if (!odd) {
        return extra + mn;
    }
    return span - extra + mn;
}

// grid_sampler_bilinear_smit_common.h:76-92
template <int PAD, bool ALIGN>
__device__ __forceinline__ float clip3(float coord, int32_t size)
{
    if (PAD == 1) {
        coord = clip3_coordinates(coord, size);
    } else if (PAD == 2) {
        if (ALIGN) {
            coord = reflect3_coordinates(coord, 0, 2 * ((int64_t)size - 1));
        } else {
            coord = reflect3_coordinates(coord, -1, 2 * (int64_t)size);
        }
        coord = clip3_coordinates(coord, size);
    }
    if (nan_or_inf(coord)) {
        return -100.0f;
    }
    return coord;
}

// grid_sampler_3d_bilinear_smit.h:171-179
template <bool ALIGN>
__device__ __forceinline__ float unnormalize3(float g, int32_t size)
{
    if (ALIGN) {
        return (g + 1.0f) / 2.0f * (float)(size - 1);
    }
    return ((g + 1.0f) * (float)size - 1.0f) / 2.0f;
}

__device__ __forceinline__ bool within(int32_t h, int32_t w, int32_t H, int32_t W)
{
    return h >= 0 && h < H && w >= 0 && w < W;
}

}  // namespace opscv
