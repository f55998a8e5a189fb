// Grid sampler 2-D forward, bicubic pair-layout LDS variant (device code in gs2d_bicubic_pair_kernel.hpp): plan and
// launch.
#include <hip/hip_runtime.h>

#include "gs2d_bicubic_pair_kernel.hpp"
#include "gs2d_common.hpp"

namespace opscv {

namespace {

constexpr int kSamplerWaves = 8;
constexpr int kLoaderWaves = 4;
constexpr int kPitches[4] = {40, 72, 104, 136};  // staged row length in dwords for W = 32, 64, 96, 128 (W + 8)
constexpr int kRunsPerLane[3] = {1, 2, 5};       // 32-element runs a loader lane takes per plane, by plane size

// Distance between consecutive rows of one slot: the rows of the two slots and 112 bytes, which shifts consecutive
// rows by 12 banks (every pitch above is 8 modulo 32 dwords) and makes the step an odd number of 16-byte units; see the
// kernel's header for what the shift is worth.
constexpr uint32_t row_step(uint32_t pitch)
{
    return 2u * pitch * 4u + 112u;
}

struct BicubicPairPlan {
    bool ok = false;
    int cls = 0;    // row length class
    int rcls = 0;   // index into kRunsPerLane
    int ppt = 2;
    uint32_t lds_bytes = 0;
    uint32_t tiles_per_n = 0, cblocks = 0;
    int32_t chans_per_block = 0;
    // as in the ring kernel's plan (gs2d_lds_launch.hpp): the first `wide_blocks` channel blocks take `chans_wide`
    // channels each, and channels are dealt out in turn, `chan_stride` apart, when that is not 0
    uint32_t wide_blocks = 0;
    int32_t chans_wide = 0;
    int32_t chan_stride = 0;
    int xcd_swizzle = 0;
    uint32_t row_step = 0;
};

// The variant takes bicubic samples of 16-bit elements under zeros or border padding whenever its loader can stage the
// planes: rows of whole 64-byte runs on the 16-byte grid, two staged planes (a little over twice the plane's bytes
// each) in LDS.
BicubicPairPlan make_plan(const GridSamplerArgs& a)
{
    BicubicPairPlan p;
    if (a.elem == Elem::F32 || a.interp != 2 || a.pad == 2 || a.Win % 32 != 0 || a.Win > 128 || a.Hin < 1) {
        return p;
    }
    const int64_t out_plane = a.Hout * a.Wout, in_plane = a.Hin * a.Win;
    if (out_plane * 2 < in_plane || out_plane % 2 != 0 || out_plane * 2 >= ((int64_t)1 << 31)) {
        return p;
    }
    if (reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || reinterpret_cast<uintptr_t>(a.y) % 4 != 0) {
        return p;
    }
    p.cls = (int)(a.Win / 32) - 1;
    const uint32_t step = row_step((uint32_t)kPitches[p.cls]);
    p.row_step = step;
    const int64_t lds = (a.Hin + 1) * (int64_t)step;
    // the loaders number their runs in blocks of sixteen rows (gs2d_bicubic_pair_kernel.hpp): a last, partial block
    // takes the run numbers of a whole one
    const int64_t runs = (a.Hin + 15) / 16 * 16 * (a.Win / 32);
    constexpr int64_t group_lanes = (kLoaderWaves / 2) * 64;
    if (lds > kLdsLimit || runs > (int64_t)kRunsPerLane[2] * group_lanes) {
        return p;
    }
    p.rcls = runs <= kRunsPerLane[0] * group_lanes ? 0 : (runs <= kRunsPerLane[1] * group_lanes ? 1 : 2);
    p.lds_bytes = (uint32_t)lds;
    // two pixels per lane where two workgroups share a CU; four where the staged planes leave room for one only, and
    // the registers of four pixels cost no occupancy (bf16 N8 C128 128x128 -> 256x256: 309 us with two, 187 with four)
    p.ppt = (p.lds_bytes > kLdsLimit / 2 && out_plane >= (int64_t)8 * kSamplerWaves * 64) ? 4 : 2;
    const int64_t tile = (int64_t)kSamplerWaves * 64 * p.ppt;
    p.tiles_per_n = (uint32_t)((out_plane + tile - 1) / tile);
    // two workgroups per CU where two fit, with at least eight channels each so that the per-pixel decisions are worth
    // their while
    const int64_t want_blocks = (p.lds_bytes > kLdsLimit / 2) ? 256 : 512;
    const int64_t base = a.N * p.tiles_per_n;
    int64_t cblocks = (want_blocks + base - 1) / base;
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
    // Exactly two workgroups per CU: the first to reach a CU runs ahead of the second (gs2d_lds.hip), so the lower half
    // of the channel blocks takes 5 channels for every 3 of the upper half; and channels are dealt out in turn where
    // every block's count is exact (fp16 N16 C256 64x64: 35.6 us with 32 + 32 in contiguous ranges, 35.5 dealt out,
    // 35.2 with 36 + 28, 34.8 with 40 + 24, 34.9 with 44 + 20, 35.8 with 48 + 16: the LDS, not the schedule, bounds
    // this kernel).
    if (a.C == cblocks * cpb && cblocks > 1) {
        if (cblocks % 2 == 0 && cpb >= 8 && a.N * p.tiles_per_n * cblocks == 2 * (int64_t)compute_unit_count() &&
            (a.N * cblocks / 2) % 8 == 0) {
            const int64_t wide = (cpb * 5 + 2) / 4;
            const int64_t narrow = 2 * cpb - wide;
            if (narrow >= 1) {
                p.wide_blocks = (uint32_t)(cblocks / 2);
                p.chans_wide = (int32_t)wide;
                p.chans_per_block = (int32_t)narrow;
            }
        }
        p.chan_stride = (int32_t)cblocks;
    }
    p.xcd_swizzle = ((a.N * cblocks) % 8 == 0) ? 1 : 0;
    p.ok = true;
    return p;
}

template <typename T, int PPT, int PITCH, int RMAX>
hipError_t launch_one(const GridSamplerArgs& a, const BicubicPairPlan& p, hipStream_t stream)
{
    auto kernel = gs2d_bicubic_pair_kernel<T, kSamplerWaves, kLoaderWaves, PPT, PITCH, RMAX, 1>;
    static std::atomic<uint32_t> lds_allowed{0};
    const hipError_t ea = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLdsLimit, lds_allowed);
    if (ea != hipSuccess) {
        return ea;
    }
    const int pair_aligned = (reinterpret_cast<uintptr_t>(a.grid) % 4 == 0);
    const uint32_t blocks = (uint32_t)(a.N * p.tiles_per_n * p.cblocks);
    // A wavefront's 64 pixels are a block of 16 columns by 4 rows of the output where its size allows, not 64
    // consecutive pixels: under a smooth grid the lanes' taps then lie in a compact patch of the plane, many lanes
    // read the same pair (one bank access serves them all) and the patch's rows fall on different banks, where the
    // taps of 64 pixels in a row are strung along a slanted line through half the plane (fp16 N16 C256 64x64,
    // rotations of up to 30 degrees: 34.8 us in rows, 35.9 with 32 x 2, 31.9 with 16 x 4, 37.5 with 8 x 8 whose stores
    // are 16-byte pieces, 56.1 with 4 x 16; the row step of 12 banks stays the best one: 31.8 us, as 20; 4 and 28: 40).
    int32_t bw_shift = 0, blocks_per_row = 0;
    if (a.Wout % 16 == 0 && a.Hout % 4 == 0) {
        bw_shift = 4;
        blocks_per_row = (int32_t)(a.Wout / 16);
    }
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3((kSamplerWaves + kLoaderWaves) * 64), p.lds_bytes, stream,
                       (const T*)a.x, (const T*)a.grid, (T*)a.y, make_fast_div((uint32_t)a.N), (int32_t)a.C,
                       (int32_t)a.Hin, (int32_t)a.Win, (int32_t)(a.Hout * a.Wout), make_fast_div(p.tiles_per_n),
                       p.chans_per_block, p.wide_blocks, p.chans_wide, p.chan_stride, pair_aligned, p.xcd_swizzle,
                       p.row_step, (int32_t)a.pad, (int32_t)(a.align != 0), bw_shift, blocks_per_row, -0.0f);
    return hipGetLastError();
}

template <typename T, int PPT, int PITCH>
hipError_t launch_runs(const GridSamplerArgs& a, const BicubicPairPlan& p, hipStream_t stream)
{
    switch (p.rcls) {
        case 0: return launch_one<T, PPT, PITCH, kRunsPerLane[0]>(a, p, stream);
        case 1: return launch_one<T, PPT, PITCH, kRunsPerLane[1]>(a, p, stream);
        default: return launch_one<T, PPT, PITCH, kRunsPerLane[2]>(a, p, stream);
    }
}

template <typename T, int PPT>
hipError_t launch_pitch(const GridSamplerArgs& a, const BicubicPairPlan& p, hipStream_t stream)
{
    switch (p.cls) {
        case 0: return launch_runs<T, PPT, kPitches[0]>(a, p, stream);
        case 1: return launch_runs<T, PPT, kPitches[1]>(a, p, stream);
        case 2: return launch_runs<T, PPT, kPitches[2]>(a, p, stream);
        case 3: return launch_runs<T, PPT, kPitches[3]>(a, p, stream);
        default: return hipErrorInvalidValue;
    }
}

template <typename T>
hipError_t launch_typed(const GridSamplerArgs& a, const BicubicPairPlan& p, hipStream_t stream)
{
    switch (p.ppt) {
        case 2: return launch_pitch<T, 2>(a, p, stream);
        case 4: return launch_pitch<T, 4>(a, p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

const char* gs2d_bicubic_pair_variant_name(const GridSamplerArgs& a)
{
    const BicubicPairPlan p = make_plan(a);
    if (!p.ok) {
        return nullptr;
    }
    static const char* names[4] = {"lds_pair_bicubic_w32", "lds_pair_bicubic_w64", "lds_pair_bicubic_w96",
                                   "lds_pair_bicubic_w128"};
    return names[p.cls];
}

hipError_t run_gs2d_bicubic_pair(const GridSamplerArgs& a, hipStream_t stream, bool* handled)
{
    *handled = false;
    const BicubicPairPlan p = make_plan(a);
    if (!p.ok) {
        return hipSuccess;
    }
    *handled = true;
    if (a.elem == Elem::F16) {
        return launch_typed<_Float16>(a, p, stream);
    }
    return launch_typed<__bf16>(a, p, stream);
}

}  // namespace opscv
