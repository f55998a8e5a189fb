// Bilinear resize, NCHW, LDS-staged row-band variant: plan and launch (device code in
// resize_band_lds_kernel.hpp).
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "kernels.hpp"
#include "resize_band_lds_kernel.hpp"

namespace opscv {

namespace {

constexpr int kBand = 12;               // output rows per workgroup (measured best on the 4K x2 upscale)
constexpr int kLdsBudget = 64 * 1024;   // per workgroup, so that at least two are resident per CU
constexpr int64_t kStreamingBytes = 128ll << 20;  // outputs beyond this are written with non-temporal stores

struct BandPlan {
    bool ok = false;
    BandLdsParams p{};
    uint32_t lds_bytes = 0;
    int threads = 256;
    dim3 grid;
};

// Exact maxima over all bands / column blocks of the staged extent, using the same tap arithmetic as the
// kernel (host and device round identically).
template <typename T, bool HALF_PIXEL>
void staged_extent(const ResizeArgs& a, int gran, int kThreads, int32_t* max_rows, int32_t* max_seg_elems)
{
    constexpr int V = 16 / (int)sizeof(T);
    const int32_t ge = gran / (int)sizeof(T);
    const int32_t Wd = (int32_t)a.Wd, Hd = (int32_t)a.Hd, Ws = (int32_t)a.Ws, Hs = (int32_t)a.Hs;
    int32_t mr = 0, ms = 0;
    for (int32_t hb = 0; hb < Hd; hb += kBand) {
        const int32_t he = (hb + kBand < Hd) ? hb + kBand : Hd;
        const int32_t lo = axis_tap<HALF_PIXEL>(hb, a.scale_h, Hs).i0;
        const int32_t hi = axis_tap<HALF_PIXEL>(he - 1, a.scale_h, Hs).i1;
        mr = (hi - lo + 1 > mr) ? hi - lo + 1 : mr;
    }
    for (int32_t cb = 0; cb < Wd; cb += kThreads * V) {
        const int32_t cl = ((cb + kThreads * V < Wd) ? cb + kThreads * V : Wd) - 1;
        const int32_t lo = axis_tap<HALF_PIXEL>(cb, a.scale_w, Ws).i0;
        const int32_t hi = axis_tap<HALF_PIXEL>(cl, a.scale_w, Ws).i1;
        const int32_t c0 = lo / ge * ge;
        const int32_t se = (hi + 1 - c0 + ge - 1) / ge * ge;
        ms = (se > ms) ? se : ms;
    }
    *max_rows = mr;
    *max_seg_elems = ms;
}

template <typename T>
BandPlan make_plan(const ResizeArgs& a)
{
    BandPlan bp;
    constexpr int V = 16 / (int)sizeof(T);
    if (a.channels_last || a.mode != ResizeMode::Bilinear) {
        return bp;
    }
    // whole 16-byte output vectors, 16-byte aligned output, 32-bit row byte offsets
    if (a.Wd % V != 0 || reinterpret_cast<uintptr_t>(a.y) % 16 != 0 || a.Wd * (int64_t)sizeof(T) >= (1ll << 31)) {
        return bp;
    }
    const uintptr_t xa = reinterpret_cast<uintptr_t>(a.x);
    int gran;
    if ((a.Ws * sizeof(T)) % 16 == 0 && xa % 16 == 0) {
        gran = 16;
    } else if ((a.Ws * sizeof(T)) % 4 == 0 && xa % 4 == 0) {
        gran = 4;
    } else {
        return bp;
    }
    // one workgroup spans the whole output row when it fits in 512 lanes (fewer, longer row segments)
    const int kThreads = (a.Wd / V > 256) ? 512 : 256;
    bp.threads = kThreads;
    int32_t rows = 0, seg = 0;
    if (a.half_pixel) {
        staged_extent<T, true>(a, gran, kThreads, &rows, &seg);
    } else {
        staged_extent<T, false>(a, gran, kThreads, &rows, &seg);
    }
    const int64_t pitch = ((int64_t)seg * sizeof(T) + 15) / 16 * 16;
    const int64_t bytes = pitch * rows;
    if (bytes > kLdsBudget || bytes <= 0) {
        return bp;  // strong down-scaling: the band touches too many source rows/columns
    }
    const int64_t bands = (a.Hd + kBand - 1) / kBand;
    const int64_t cblocks = (a.Wd + kThreads * V - 1) / (kThreads * V);
    const int64_t planes = a.N * a.C;
    if (bands > 65535 || cblocks > INT32_MAX) {
        return bp;
    }
    bp.p.planes = planes;
    bp.p.Hs = (int32_t)a.Hs;
    bp.p.Ws = (int32_t)a.Ws;
    bp.p.Hd = (int32_t)a.Hd;
    bp.p.Wd = (int32_t)a.Wd;
    bp.p.scale_h = a.scale_h;
    bp.p.scale_w = a.scale_w;
    bp.p.lds_pitch = (int32_t)pitch;
    bp.p.lds_rows = rows;
    bp.p.gran = gran;
    bp.p.neg_zero = -0.0f;
    bp.p.streaming = (a.N * a.C * a.Hd * a.Wd * (int64_t)sizeof(T) >= kStreamingBytes) ? 1 : 0;
    bp.lds_bytes = (uint32_t)bytes;
    bp.grid = dim3((unsigned)cblocks, (unsigned)bands, (unsigned)(planes < 65535 ? planes : 65535));
    const char* v = getenv("OPSCV_RESIZE_VARIANT");
    bp.ok = !(v != nullptr && (v[0] == 'g' || v[0] == 'r'));  // generic / register-band forced (benchmark knob)
    return bp;
}

template <typename T>
hipError_t run_typed(const ResizeArgs& a, hipStream_t stream, bool* handled)
{
    const BandPlan bp = make_plan<T>(a);
    if (!bp.ok) {
        return hipSuccess;
    }
    *handled = true;
    if (bp.threads == 512) {
        if (a.half_pixel) {
            hipLaunchKernelGGL((resize_band_lds_kernel<T, true, 512, kBand>), bp.grid, dim3(512), bp.lds_bytes, stream,
                               (const T*)a.x, (T*)a.y, bp.p);
        } else {
            hipLaunchKernelGGL((resize_band_lds_kernel<T, false, 512, kBand>), bp.grid, dim3(512), bp.lds_bytes,
                               stream, (const T*)a.x, (T*)a.y, bp.p);
        }
    } else {
        if (a.half_pixel) {
            hipLaunchKernelGGL((resize_band_lds_kernel<T, true, 256, kBand>), bp.grid, dim3(256), bp.lds_bytes, stream,
                               (const T*)a.x, (T*)a.y, bp.p);
        } else {
            hipLaunchKernelGGL((resize_band_lds_kernel<T, false, 256, kBand>), bp.grid, dim3(256), bp.lds_bytes,
                               stream, (const T*)a.x, (T*)a.y, bp.p);
        }
    }
    return hipGetLastError();
}

}  // namespace

bool resize_band_lds_applicable(const ResizeArgs& a)
{
    switch (a.elem) {
        case Elem::F32: return make_plan<float>(a).ok;
        case Elem::F16: return make_plan<_Float16>(a).ok;
        case Elem::BF16: return make_plan<__bf16>(a).ok;
    }
    return false;
}

hipError_t run_resize_band_lds(const ResizeArgs& a, hipStream_t stream, bool* handled)
{
    *handled = false;
    switch (a.elem) {
        case Elem::F32: return run_typed<float>(a, stream, handled);
        case Elem::F16: return run_typed<_Float16>(a, stream, handled);
        case Elem::BF16: return run_typed<__bf16>(a, stream, handled);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
