// Dispatch helpers shared by the grid-sampler translation units.
#pragma once

#include <hip/hip_runtime.h>

#include "kernels.hpp"

namespace opscv {

// Expands the run-time (interp, pad, align) triple into the template instantiation.
template <typename T, typename F>
inline hipError_t dispatch_modes(const GridSamplerArgs& a, F&& f)
{
#define OPSCV_CASE(I, P, A)                                   \
    if (a.interp == I && a.pad == P && (a.align != 0) == A) { \
        return f.template operator()<T, I, P, A>();           \
    }
    OPSCV_CASE(0, 0, false)
    OPSCV_CASE(0, 0, true)
    OPSCV_CASE(0, 1, false)
    OPSCV_CASE(0, 1, true)
    OPSCV_CASE(0, 2, false)
    OPSCV_CASE(0, 2, true)
    OPSCV_CASE(1, 0, false)
    OPSCV_CASE(1, 0, true)
    OPSCV_CASE(1, 1, false)
    OPSCV_CASE(1, 1, true)
    OPSCV_CASE(1, 2, false)
    OPSCV_CASE(1, 2, true)
    OPSCV_CASE(2, 0, false)
    OPSCV_CASE(2, 0, true)
    OPSCV_CASE(2, 1, false)
    OPSCV_CASE(2, 1, true)
    OPSCV_CASE(2, 2, false)
    OPSCV_CASE(2, 2, true)
#undef OPSCV_CASE
    return hipErrorInvalidValue;
}

template <typename F>
inline hipError_t dispatch_elem(const GridSamplerArgs& a, F&& f)
{
    switch (a.elem) {
        case Elem::F32: return dispatch_modes<float>(a, f);
        case Elem::F16: return dispatch_modes<_Float16>(a, f);
        case Elem::BF16: return dispatch_modes<__bf16>(a, f);
    }
    return hipErrorInvalidValue;
}

// Shape limits shared by every variant (the reference tiling enforces the same ones,
// grid_sampler2_d_tiling.cpp:92-156): every extent and the input plane fit in int32.
inline bool gs_shapes_ok(const GridSamplerArgs& a)
{
    if (a.N < 0 || a.C < 0 || a.Hout < 0 || a.Wout < 0 || a.Hin <= 0 || a.Win <= 0) {
        return false;
    }
    const int64_t lim = INT32_MAX;
    if (a.N > lim || a.C > lim || a.Hin > lim || a.Win > lim || a.Hout > lim || a.Wout > lim) {
        return false;
    }
    if (a.Hin * a.Win > lim) {
        return false;
    }
    if (a.Hout != 0 && a.Wout != 0 && a.Hout > INT64_MAX / a.Wout / (a.N > 0 ? a.N : 1) / 2) {
        return false;
    }
    return true;
}


// LDS-staged variant (gs2d_lds.hip).  Sets *handled to false, launching nothing, when the shape does not fit
// its assumptions (input plane too large for LDS); the caller then falls back to the direct variant.
hipError_t run_gs2d_lds(const GridSamplerArgs& a, hipStream_t stream, bool* handled);
const char* gs2d_lds_variant_name(const GridSamplerArgs& a);
// whether that variant would stage two channels at a time, interleaved (gs2d_lds_kernel.hpp, CHANNEL_PAIRS)
bool gs2d_lds_channel_pairs(const GridSamplerArgs& a);
// ... and the average number of channels that a channel block then takes (0 where it stages single channels)
int64_t gs2d_lds_channel_pairs_per_block(const GridSamplerArgs& a);

// Pair-layout LDS variant (gs2d_pair.hip): bilinear, 16-bit elements, several output pixels per input pixel; same
// convention as run_gs2d_lds.
hipError_t run_gs2d_pair(const GridSamplerArgs& a, hipStream_t stream, bool* handled);
const char* gs2d_pair_variant_name(const GridSamplerArgs& a);
// ... and its bicubic counterpart (gs2d_bicubic_pair.hip); both are reached through the two functions above
hipError_t run_gs2d_bicubic_pair(const GridSamplerArgs& a, hipStream_t stream, bool* handled);
const char* gs2d_bicubic_pair_variant_name(const GridSamplerArgs& a);

// Box variant (gs2d_box.hip): bilinear, 16-bit elements, planes beyond the LDS variants; the box of input pixels that a
// tile of output pixels reads goes through LDS.  Same convention as run_gs2d_lds.
hipError_t run_gs2d_box(const GridSamplerArgs& a, hipStream_t stream, bool* handled);
const char* gs2d_box_variant_name(const GridSamplerArgs& a);

// Channels-last variant (gs2d_nhwc.hip): a.x is (N,Hin,Win,C), a.y is (N,Hout,Wout,C).
hipError_t run_gs2d_nhwc(const GridSamplerArgs& a, hipStream_t stream);

// CUs of the current device (256 on MI355X; also the answer where no device can be asked); gs2d_lds.hip
int compute_unit_count();

}  // namespace opscv
