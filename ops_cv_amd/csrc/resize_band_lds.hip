// Bilinear resize, NCHW, LDS-staged row-band variant: plan and launch (device code in
// resize_band_lds_kernel.hpp).
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "kernels.hpp"
#include "options.hpp"
#include "resize_band_lds_kernel.hpp"
#include "resize_flat_lds_kernel.hpp"

namespace opscv {

namespace {

constexpr int kBand = 12;               // output rows per workgroup (measured best on the 4K x2 upscale)
constexpr int kLdsBudget = 64 * 1024;   // per workgroup, so that at least two are resident per CU
// outputs from this size on are written with non-temporal stores (written through instead of left dirty in L2 for the
// end of the kernel to write back)
constexpr int64_t kStreamingBytes = 1ll << 20;

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
    const int32_t ge = (gran == 1) ? 1 : gran / (int)sizeof(T);
    const int32_t Wd = (int32_t)a.Wd, Hd = (int32_t)a.Hd, Ws = (int32_t)a.Ws, Hs = (int32_t)a.Hs;
    const int32_t ci = a.channels_last ? (int32_t)a.C : 1;  // row elements per pixel
    const int32_t Wde = Wd * ci;
    int32_t mr = 0, ms = 0;
    for (int32_t hb = 0; hb < Hd; hb += kBand) {
        const int32_t he = (hb + kBand < Hd) ? hb + kBand : Hd;
        const int32_t lo = axis_tap<HALF_PIXEL>(hb, a.scale_h, Hs).i0;
        const int32_t hi = axis_tap<HALF_PIXEL>(he - 1, a.scale_h, Hs).i1;
        mr = (hi - lo + 1 > mr) ? hi - lo + 1 : mr;
    }
    for (int32_t cb = 0; cb < Wde; cb += kThreads * V) {
        const int32_t cl = ((cb + kThreads * V < Wde) ? cb + kThreads * V : Wde) - 1;
        const int32_t lo = axis_tap<HALF_PIXEL>(cb / ci, a.scale_w, Ws).i0 * ci;
        const int32_t hi = axis_tap<HALF_PIXEL>(cl / ci, a.scale_w, Ws).i1 * ci + ci - 1;
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
    if (a.mode != ResizeMode::Bilinear) {
        return bp;
    }
    // Channels-last images whose pixels are not whole 16-byte vectors are resized as planes with rows of Ws * C
    // elements (taps C elements apart); whole vectors per pixel have their own kernel.
    const int64_t ci = a.channels_last ? a.C : 1;
    // Staging pays when source rows are reused: images that at least double in area (3-channel fp16 1080p to 4K: 211 ->
    // 101 us; 224 -> 256 is faster without staging).
    if (a.channels_last && ((a.C * sizeof(T)) % 16 == 0 || a.Ws * ci > INT32_MAX || a.Wd * ci > INT32_MAX ||
                            a.Hd * a.Wd < 2 * a.Hs * a.Ws)) {
        return bp;
    }
    const int64_t Wse = a.Ws * ci, Wde = a.Wd * ci;
    // element-aligned output (the vector stores are), 32-bit row byte offsets
    if (reinterpret_cast<uintptr_t>(a.y) % sizeof(T) != 0 || Wde * (int64_t)sizeof(T) >= (1ll << 31)) {
        return bp;
    }

    const uintptr_t xa = reinterpret_cast<uintptr_t>(a.x);
    int gran;
    if ((Wse * sizeof(T)) % 16 == 0 && xa % 16 == 0) {
        gran = 16;
    } else if (xa % sizeof(T) == 0) {
        gran = 1;  // rows off the 16-byte grid: 16-byte copies in the shifted layout (see the kernel)
    } else {
        return bp;
    }
    // one workgroup spans the whole output row when it fits in 512 lanes (fewer, longer row segments)
    const int kThreads = ((Wde + V - 1) / V > 256) ? 512 : 256;
    bp.threads = kThreads;
    int32_t rows = 0, seg = 0;
    if (a.half_pixel) {
        staged_extent<T, true>(a, gran, kThreads, &rows, &seg);
    } else {
        staged_extent<T, false>(a, gran, kThreads, &rows, &seg);
    }
    const int64_t pitch = ((int64_t)seg * sizeof(T) + (gran == 1 ? 15 : 0) + 15) / 16 * 16;
    const int64_t bytes = pitch * rows;
    if (bytes > kLdsBudget || bytes <= 0) {
        return bp;  // strong down-scaling: the band touches too many source rows/columns
    }
    const int64_t bands = (a.Hd + kBand - 1) / kBand;
    const int64_t cblocks = (Wde + kThreads * V - 1) / (kThreads * V);
    const int64_t planes = a.channels_last ? a.N : a.N * a.C;
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
    bp.p.raw_lambda = a.raw_lambda;
    bp.p.interleave = (int32_t)ci;
    bp.p.streaming = (a.N * a.C * a.Hd * a.Wd * (int64_t)sizeof(T) >= kStreamingBytes) ? 1 : 0;
    bp.lds_bytes = (uint32_t)bytes;
    bp.grid = dim3((unsigned)cblocks, (unsigned)bands, (unsigned)(planes < 65535 ? planes : 65535));
    // generic / register-band forced (benchmark knob, option "resize_variant")
    bp.ok = !(a.force_variant == kResizeGeneric || a.force_variant == kResizeRegisterBand);
    return bp;
}

// ---- narrow images: 2-D lane arrangement (resize_flat_lds_kernel.hpp) ----
constexpr int kFlatThreads = 256;
constexpr int kFlatMaxColumnLanes = 128;   // wider rows keep at least half of the band variant's lanes busy
constexpr int kFlatLdsBudget = 32 * 1024;  // per workgroup: several workgroups per CU hide the staging latency
constexpr int64_t kFlatWantBlocks = 1024;

struct FlatPlan {
    bool ok = false;
    FlatLdsParams p{};
    uint32_t lds_bytes = 0;
    dim3 grid;
};

template <typename T, bool HALF_PIXEL>
int32_t flat_max_rows(const ResizeArgs& a, int32_t band_rows)
{
    const int32_t Hd = (int32_t)a.Hd, Hs = (int32_t)a.Hs;
    int32_t mr = 0;
    for (int32_t hb = 0; hb < Hd; hb += band_rows) {
        const int32_t he = (hb + band_rows < Hd) ? hb + band_rows : Hd;
        const int32_t lo = axis_tap<HALF_PIXEL>(hb, a.scale_h, Hs).i0;
        const int32_t hi = axis_tap<HALF_PIXEL>(he - 1, a.scale_h, Hs).i1;
        mr = (hi - lo + 1 > mr) ? hi - lo + 1 : mr;
    }
    return mr;
}

template <typename T>
FlatPlan make_flat_plan(const ResizeArgs& a)
{
    FlatPlan fp;
    constexpr int V = 16 / (int)sizeof(T);
    if (a.channels_last || a.mode != ResizeMode::Bilinear) {
        return fp;
    }
    // element-aligned output (the vector stores are), 32-bit byte offsets inside an output plane
    if (reinterpret_cast<uintptr_t>(a.y) % sizeof(T) != 0 || a.Hd * a.Wd * (int64_t)sizeof(T) >= (1ll << 31)) {
        return fp;
    }
    const int64_t cl = (a.Wd + V - 1) / V;
    if (cl > kFlatMaxColumnLanes) {
        return fp;
    }
    const uintptr_t xa = reinterpret_cast<uintptr_t>(a.x);
    int gran;
    if ((a.Ws * sizeof(T)) % 16 == 0 && xa % 16 == 0) {
        gran = 16;
    } else if (xa % sizeof(T) == 0) {
        gran = 1;  // rows off the 16-byte grid: 16-byte copies in the shifted layout (see the kernel)
    } else {
        return fp;
    }
    const int32_t rg_max = kFlatThreads / (int32_t)cl;
    const int64_t planes = a.N * a.C;
    // bands: enough workgroups to fill the chip several times over, each a whole number of row-group passes
    // bands: about four workgroups per CU, all resident at once (a second round of workgroups would wait out the
    // staging latency again while few stores flow: fp32 8x64 56x56 -> 112x112 10.6 us with 2048 workgroups, 8.8 with
    // 1024).  The rows of a plane are shared out evenly, and so are a band's rows among the row groups: with r rows
    // in `passes` turns, ceil(r / passes) groups are at work in every turn and the rest of the lanes sit idle, which
    // costs less than a last turn that one group walks alone.
    int64_t bands = (kFlatWantBlocks + planes - 1) / planes;
    if (bands > a.Hd) {
        bands = a.Hd;
    }
    int64_t band_rows = (a.Hd + bands - 1) / bands;
    int32_t rows = 0;
    for (;;) {
        rows = a.half_pixel ? flat_max_rows<T, true>(a, (int32_t)band_rows) : flat_max_rows<T, false>(a, (int32_t)band_rows);
        if ((int64_t)rows * a.Ws * (int64_t)sizeof(T) <= kFlatLdsBudget) {
            break;
        }
        if (band_rows <= 1) {
            return fp;  // even one output row touches more source rows than the budget holds
        }
        band_rows = (band_rows + 1) / 2;
    }
    const int64_t passes = (band_rows + rg_max - 1) / rg_max;
    const int32_t rg = (int32_t)((band_rows + passes - 1) / passes);
    bands = (a.Hd + band_rows - 1) / band_rows;
    if (bands > INT32_MAX) {
        return fp;
    }
    fp.p.planes = planes;
    fp.p.Hs = (int32_t)a.Hs;
    fp.p.Ws = (int32_t)a.Ws;
    fp.p.Hd = (int32_t)a.Hd;
    fp.p.Wd = (int32_t)a.Wd;
    fp.p.scale_h = a.scale_h;
    fp.p.scale_w = a.scale_w;
    fp.p.band_rows = (int32_t)band_rows;
    fp.p.cl = (int32_t)cl;
    fp.p.rg = rg;
    fp.p.gran = gran;
    fp.p.neg_zero = -0.0f;
    fp.p.raw_lambda = a.raw_lambda;
    fp.lds_bytes = (uint32_t)(((int64_t)rows * a.Ws * (int64_t)sizeof(T) + (gran == 1 ? 15 : 0) + 15) / 16 * 16);
    fp.grid = dim3((unsigned)bands, (unsigned)(planes < 65535 ? planes : 65535));
    // generic / register-band / LDS band forced (benchmark knob, option "resize_variant")
    fp.ok = a.force_variant == kResizeAuto;
    return fp;
}

template <typename T>
hipError_t run_flat_typed(const ResizeArgs& a, hipStream_t stream, bool* handled)
{
    const FlatPlan fp = make_flat_plan<T>(a);
    if (!fp.ok) {
        return hipSuccess;
    }
    *handled = true;
    if (a.half_pixel) {
        hipLaunchKernelGGL((resize_flat_lds_kernel<T, true, kFlatThreads>), fp.grid, dim3(kFlatThreads), fp.lds_bytes,
                           stream, (const T*)a.x, (T*)a.y, fp.p);
    } else {
        hipLaunchKernelGGL((resize_flat_lds_kernel<T, false, kFlatThreads>), fp.grid, dim3(kFlatThreads), fp.lds_bytes,
                           stream, (const T*)a.x, (T*)a.y, fp.p);
    }
    return hipGetLastError();
}

template <typename T>
hipError_t run_typed(const ResizeArgs& a, hipStream_t stream, bool* handled)
{
    const hipError_t e = run_flat_typed<T>(a, stream, handled);
    if (*handled || e != hipSuccess) {
        return e;
    }
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

const char* resize_lds_variant(const ResizeArgs& a)
{
    bool flat = false, band = false;
    switch (a.elem) {
        case Elem::F32: flat = make_flat_plan<float>(a).ok; band = make_plan<float>(a).ok; break;
        case Elem::F16: flat = make_flat_plan<_Float16>(a).ok; band = make_plan<_Float16>(a).ok; break;
        case Elem::BF16: flat = make_flat_plan<__bf16>(a).ok; band = make_plan<__bf16>(a).ok; break;
    }
    return flat ? "nchw_flat_lds" : (band ? (a.channels_last ? "nhwc_band_lds" : "nchw_band_lds") : nullptr);
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
