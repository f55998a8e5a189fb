// Grid sampler 2-D forward, LDS-staged variant: launch plan and the typed launch template.
// The element types, and for each the two plane layouts, are instantiated in separate translation units so that they
// compile in parallel.
#pragma once

#include <hip/hip_runtime.h>

#include "gs2d_common.hpp"
#include "gs2d_lds_kernel.hpp"

namespace opscv {

struct LdsPlan {
    bool ok = false;
    int cls = 0;  // index into kPitch / kCgs
    int ppt = 4;
    int adj = 1;  // neighbouring output pixels per store (2: pairs of 16-bit results as one dword)
    int copy_gran = 16;
    int xcd_swizzle = 0;
    int row_shift = 0;  // 7 | turn << 8 when the staged planes (128-byte rows) use the bank-spreading layout, else 0
    uint32_t lds_bytes = 0;
    uint32_t tiles_per_n = 0, cblocks = 0;
    int32_t chans_per_block = 0;
    // the first `wide_blocks` channel blocks take `chans_wide` channels each (0: all blocks alike)
    uint32_t wide_blocks = 0;
    int32_t chans_wide = 0;
    // != 0: channels are dealt out to the channel blocks in turn, this many apart (the number of blocks), instead of
    // a contiguous range per block
    int32_t chan_stride = 0;
    // elements per staged row: Win, or Win's row padded to a multiple of 128 bytes (gs2d_lds_kernel.hpp, loaders)
    int32_t lds_w = 0;
    // two neighbouring channels per stage, interleaved in LDS (gs2d_lds_kernel.hpp, CHANNEL_PAIRS); the channel counts
    // above stay in channels, the launch halves them
    bool chan_pairs = false;
    int32_t pairs_pitch = 0;  // kPairsPitch or kPairsPitchLarge
};

// the channel-pair kernels' LDS: two slots of two planes of the 8 KiB or of the 16 KiB class and the zeros
constexpr int kPairsPitch = 16400;
constexpr int kPairsPitchLarge = 32784;
constexpr int kPairsNbuf = 2;
constexpr int kPairsLoaderWaves = 4;

constexpr int kSamplerWaves = 8;  // 512 lanes own output pixels
// loader wavefronts per size class (the 16 KiB class as the 8 KiB one): enough that (NBUF-2) stages of one loader's copy instructions fit the
// 6-bit outstanding-operation counter (a 1 KiB chunk per instruction), and for the 8 KiB class four of them
// because one wavefront alone issues the copies of a stage too slowly to keep the ring full
constexpr int kLoaderWaves[5] = {1, 4, 4, 2, 4};
constexpr int kThreads = kSamplerWaves * 64;  // pixels per tile = kThreads * ppt
// plane pitch in LDS and planes per stage for the five size classes (the 16 KiB class keeps two workgroups per CU
// for planes a little over 8 KiB, which the 32 KiB class would run one per CU at a third of the speed)
constexpr int kPitch[5] = {2064, 8208, 16400, 32784, 81904};
// (8 KiB class: six single-plane stages measured a little better than four stages of two planes, 16.0 vs 16.3 us
// on fp16 N16 C256 64x64, with a quarter less LDS)
constexpr int kCgs[5] = {4, 1, 1, 1, 1};   // planes per stage
constexpr int kNbuf[5] = {4, 6, 4, 4, 2};  // ring slots (stages resident in LDS)

LdsPlan make_lds_plan(const GridSamplerArgs& a);

template <typename T, int I, int PPT, int ADJ, int CGS, int NBUF, int PITCH, int LWAVES, bool SHIFTED>
hipError_t launch_one(const GridSamplerArgs& a, const LdsPlan& p, hipStream_t stream)
{
    auto kernel = gs2d_lds_kernel<T, I, kSamplerWaves, LWAVES, PPT, ADJ, CGS, NBUF, PITCH, SHIFTED>;
    static std::atomic<uint32_t> lds_allowed{0};
    const hipError_t ea = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLdsLimit, lds_allowed);
    if (ea != hipSuccess) {
        return ea;
    }
    const int64_t esz = sizeof(T);
    const int pair_aligned = (reinterpret_cast<uintptr_t>(a.grid) % (2 * esz) == 0);
    const uint32_t blocks = (uint32_t)(a.N * p.tiles_per_n * p.cblocks);
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3((kSamplerWaves + LWAVES) * 64), p.lds_bytes, stream, (const T*)a.x, (const T*)a.grid,
                       (T*)a.y, make_fast_div((uint32_t)a.N), (int32_t)a.C, (int32_t)a.Hin, (int32_t)a.Win, (int32_t)(a.Hout * a.Wout),
                       make_fast_div(p.tiles_per_n), p.chans_per_block, p.wide_blocks, p.chans_wide, p.chan_stride, p.copy_gran,
                       pair_aligned, p.xcd_swizzle, p.row_shift, (int32_t)a.pad, (int32_t)(a.align != 0), (int32_t)a.rule, p.lds_w,
                       -0.0f);
    return hipGetLastError();
}

template <typename T, int I, int CLS, int PPT, bool SHIFTED>
hipError_t launch_cls(const GridSamplerArgs& a, const LdsPlan& p, hipStream_t stream)
{
    // pairs of neighbouring pixels per store exist for 16-bit elements with four or eight pixels per lane
    if constexpr (sizeof(T) == 2 && PPT >= 4) {
        if (p.adj == 2) {
            return launch_one<T, I, PPT, 2, kCgs[CLS], kNbuf[CLS], kPitch[CLS], kLoaderWaves[CLS], SHIFTED>(a, p,
                                                                                                                 stream);
        }
    }
    return launch_one<T, I, PPT, 1, kCgs[CLS], kNbuf[CLS], kPitch[CLS], kLoaderWaves[CLS], SHIFTED>(a, p, stream);
}

// Expands (interp, size class, pixels per lane) for one element type and launches; padding mode and align_corners are
// run-time arguments of the kernel.  Eight pixels per lane exist for the two large-plane classes only.
template <typename T, bool SHIFTED>
struct LdsTypedLauncher {
    const GridSamplerArgs& a;
    const LdsPlan& p;
    hipStream_t stream;
    template <int I>
    hipError_t run() const
    {
        if constexpr (I == 2) {
            // bicubic keeps sixteen tap offsets per pixel: one or two pixels per lane
            switch (p.cls * 16 + p.ppt) {
                case 0 * 16 + 1: return launch_cls<T, I, 0, 1, SHIFTED>(a, p, stream);
                case 0 * 16 + 2: return launch_cls<T, I, 0, 2, SHIFTED>(a, p, stream);
                case 1 * 16 + 1: return launch_cls<T, I, 1, 1, SHIFTED>(a, p, stream);
                case 1 * 16 + 2: return launch_cls<T, I, 1, 2, SHIFTED>(a, p, stream);
                case 2 * 16 + 1: return launch_cls<T, I, 2, 1, SHIFTED>(a, p, stream);
                case 2 * 16 + 2: return launch_cls<T, I, 2, 2, SHIFTED>(a, p, stream);
                case 3 * 16 + 1: return launch_cls<T, I, 3, 1, SHIFTED>(a, p, stream);
                case 3 * 16 + 2: return launch_cls<T, I, 3, 2, SHIFTED>(a, p, stream);
                case 4 * 16 + 1: return launch_cls<T, I, 4, 1, SHIFTED>(a, p, stream);
                case 4 * 16 + 2: return launch_cls<T, I, 4, 2, SHIFTED>(a, p, stream);
                default: return hipErrorInvalidValue;
            }
        }
        switch (p.cls * 16 + p.ppt) {
            case 0 * 16 + 1: return launch_cls<T, I, 0, 1, SHIFTED>(a, p, stream);
            case 0 * 16 + 4: return launch_cls<T, I, 0, 4, SHIFTED>(a, p, stream);
            case 1 * 16 + 1: return launch_cls<T, I, 1, 1, SHIFTED>(a, p, stream);
            case 1 * 16 + 4: return launch_cls<T, I, 1, 4, SHIFTED>(a, p, stream);
            case 2 * 16 + 1: return launch_cls<T, I, 2, 1, SHIFTED>(a, p, stream);
            case 2 * 16 + 4: return launch_cls<T, I, 2, 4, SHIFTED>(a, p, stream);
            case 2 * 16 + 8: return launch_cls<T, I, 2, 8, SHIFTED>(a, p, stream);
            case 3 * 16 + 1: return launch_cls<T, I, 3, 1, SHIFTED>(a, p, stream);
            case 3 * 16 + 4: return launch_cls<T, I, 3, 4, SHIFTED>(a, p, stream);
            case 3 * 16 + 8: return launch_cls<T, I, 3, 8, SHIFTED>(a, p, stream);
            case 4 * 16 + 1: return launch_cls<T, I, 4, 1, SHIFTED>(a, p, stream);
            case 4 * 16 + 4: return launch_cls<T, I, 4, 4, SHIFTED>(a, p, stream);
            case 4 * 16 + 8: return launch_cls<T, I, 4, 8, SHIFTED>(a, p, stream);
            default: return hipErrorInvalidValue;
        }
    }
};

// SHIFTED: the kernels for planes off the 16-byte grid (plan.copy_gran == 2)
template <typename T, bool SHIFTED>
hipError_t lds_launch_typed(const GridSamplerArgs& a, const LdsPlan& p, hipStream_t stream)
{
    const LdsTypedLauncher<T, SHIFTED> launcher{a, p, stream};
    switch (a.interp) {
        case 0: return launcher.template run<0>();
        case 1: return launcher.template run<1>();
        case 2: return launcher.template run<2>();
        default: return hipErrorInvalidValue;
    }
}

// the CHANNEL_PAIRS kernels (16-bit elements, bilinear, the 8 KiB class with four pixels per lane): gs2d_lds_pairs.hip
hipError_t lds_launch_channel_pairs(const GridSamplerArgs& a, const LdsPlan& p, hipStream_t stream);

extern template hipError_t lds_launch_typed<float, false>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);
extern template hipError_t lds_launch_typed<_Float16, false>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);
extern template hipError_t lds_launch_typed<__bf16, false>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);
extern template hipError_t lds_launch_typed<float, true>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);
extern template hipError_t lds_launch_typed<_Float16, true>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);
extern template hipError_t lds_launch_typed<__bf16, true>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);

}  // namespace opscv
