// Grid sampler 2-D forward, pair-layout LDS variant (device code in gs2d_pair_kernel.hpp): plan and launch.
#include <hip/hip_runtime.h>

#include "gs2d_common.hpp"
#include "gs2d_pair_kernel.hpp"

namespace opscv {

namespace {

constexpr int kPairSamplerWaves = 12;
constexpr int kPairLoaderWaves = 4;
constexpr int kPairPpt = 12;
constexpr int kPairRmax = 5;
constexpr int kPairPitches[4] = {36, 68, 100, 132};  // staged row length in dwords for W <= 32, 64, 96, 128

constexpr uint32_t pair_row_step(uint32_t pitch)
{
    return 2u * pitch * 4u + (((2u * pitch * 4u / 16u) & 1u) ? 0u : 16u);  // ROW_STEP of the kernel
}

struct PairPlan {
    bool ok = false;
    int cls = 0;
    uint32_t lds_bytes = 0;
    uint32_t tiles_per_n = 0, cblocks = 0;
    int32_t chans_per_block = 0;
    int xcd_swizzle = 0;
};

// The variant pays where the LDS reads of the taps bound the ring kernel: bilinear samples of 16-bit elements, several
// output pixels per input pixel (bf16 N8 C128 128x128 -> 256x256 at scattered positions: 81 us ring, 69 us pairs).  Its
// loader wants rows of whole 64-byte runs on the 16-byte grid, and a staged plane takes a little over twice the
// plane's bytes, two of which must fit the LDS.
PairPlan make_pair_plan(const GridSamplerArgs& a)
{
    PairPlan p;
    if (a.elem == Elem::F32 || a.interp != 0 || a.Win % 32 != 0 || a.Win > 128) {
        return p;
    }
    const int64_t out_plane = a.Hout * a.Wout, in_plane = a.Hin * a.Win;
    if (out_plane < 3 * in_plane || out_plane % 2 != 0 || out_plane * 2 >= ((int64_t)1 << 31)) {
        return p;
    }
    if (reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || reinterpret_cast<uintptr_t>(a.y) % 4 != 0) {
        return p;
    }
    p.cls = (int)(a.Win / 32) - 1;
    const uint32_t step = pair_row_step((uint32_t)kPairPitches[p.cls]);
    const int64_t lds = (a.Hin + 3) * (int64_t)step;
    // the loaders number their runs in blocks of sixteen rows: a last, partial block takes the numbers of a whole one
    const int64_t runs = (a.Hin + 15) / 16 * 16 * (a.Win / 32);
    if (lds > kLdsLimit || runs > (int64_t)kPairRmax * (kPairLoaderWaves / 2) * 64) {
        return p;
    }
    p.lds_bytes = (uint32_t)lds;
    const int64_t tile = (int64_t)kPairSamplerWaves * 64 * kPairPpt;
    p.tiles_per_n = (uint32_t)((out_plane + tile - 1) / tile);
    // one workgroup of sixteen wavefronts per CU at a time: aim at one round of 256 workgroups (or whole rounds), with
    // at least eight channels each so that the per-pixel decisions are worth their while
    const int64_t base = a.N * p.tiles_per_n;
    int64_t cblocks = (256 + base - 1) / base;
    if (cblocks > a.C / 8) {
        cblocks = a.C / 8;
    }
    if (cblocks < 1) {
        cblocks = 1;
    }
    const int64_t cpb = (a.C + cblocks - 1) / cblocks;
    cblocks = (a.C + cpb - 1) / cpb;
    p.chans_per_block = (int32_t)cpb;
    p.cblocks = (uint32_t)cblocks;
    if (a.N * p.tiles_per_n * cblocks > INT32_MAX) {
        return p;
    }
    p.xcd_swizzle = ((a.N * cblocks) % 8 == 0) ? 1 : 0;
    p.ok = true;
    return p;
}

template <typename T, int PITCH>
hipError_t pair_launch_one(const GridSamplerArgs& a, const PairPlan& p, hipStream_t stream)
{
    auto kernel = gs2d_pair_kernel<T, kPairSamplerWaves, kPairLoaderWaves, kPairPpt, PITCH, kPairRmax>;
    static std::atomic<uint32_t> lds_allowed{0};
    const hipError_t ea = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLdsLimit, lds_allowed);
    if (ea != hipSuccess) {
        return ea;
    }
    const int pair_aligned = (reinterpret_cast<uintptr_t>(a.grid) % 4 == 0);
    const uint32_t blocks = (uint32_t)(a.N * p.tiles_per_n * p.cblocks);
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3((kPairSamplerWaves + kPairLoaderWaves) * 64), p.lds_bytes, stream,
                       (const T*)a.x, (const T*)a.grid, (T*)a.y, make_fast_div((uint32_t)a.N), (int32_t)a.C,
                       (int32_t)a.Hin, (int32_t)a.Win, (int32_t)(a.Hout * a.Wout), make_fast_div(p.tiles_per_n),
                       p.chans_per_block, pair_aligned, p.xcd_swizzle, (int32_t)a.pad, (int32_t)(a.align != 0), -0.0f);
    return hipGetLastError();
}

template <typename T>
hipError_t pair_launch_typed(const GridSamplerArgs& a, const PairPlan& p, hipStream_t stream)
{
    switch (p.cls) {
        case 0: return pair_launch_one<T, kPairPitches[0]>(a, p, stream);
        case 1: return pair_launch_one<T, kPairPitches[1]>(a, p, stream);
        case 2: return pair_launch_one<T, kPairPitches[2]>(a, p, stream);
        case 3: return pair_launch_one<T, kPairPitches[3]>(a, p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

const char* gs2d_pair_variant_name(const GridSamplerArgs& a)
{
    if (a.interp == 2) {
        return gs2d_bicubic_pair_variant_name(a);
    }
    const PairPlan p = make_pair_plan(a);
    if (!p.ok) {
        return nullptr;
    }
    static const char* names[4] = {"lds_pair_w32", "lds_pair_w64", "lds_pair_w96", "lds_pair_w128"};
    return names[p.cls];
}

hipError_t run_gs2d_pair(const GridSamplerArgs& a, hipStream_t stream, bool* handled)
{
    if (a.interp == 2) {
        return run_gs2d_bicubic_pair(a, stream, handled);
    }
    *handled = false;
    const PairPlan p = make_pair_plan(a);
    if (!p.ok) {
        return hipSuccess;
    }
    *handled = true;
    if (a.pad < 0 || a.pad > 2) {
        return hipErrorInvalidValue;
    }
    if (a.elem == Elem::F16) {
        return pair_launch_typed<_Float16>(a, p, stream);
    }
    return pair_launch_typed<__bf16>(a, p, stream);
}

}  // namespace opscv
