// LDS-staged grid sampler kernels with two channels per stage interleaved in LDS (16-bit elements, bilinear and bicubic).
#include "gs2d_lds_launch.hpp"

namespace opscv {

namespace {

template <typename T, int PPT, int ADJ, int PITCH, int INTERP = 0>
hipError_t launch_pairs(const GridSamplerArgs& a, const LdsPlan& p, hipStream_t stream)
{
    auto kernel = gs2d_lds_kernel<T, INTERP, kSamplerWaves, kPairsLoaderWaves, PPT, ADJ, 1, kPairsNbuf, PITCH, false, true>;
    static std::atomic<uint32_t> lds_allowed{0};
    const hipError_t ea = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLdsLimit, lds_allowed);
    if (ea != hipSuccess) {
        return ea;
    }
    const int pair_aligned = (reinterpret_cast<uintptr_t>(a.grid) % (2 * sizeof(T)) == 0);
    const uint32_t blocks = (uint32_t)(a.N * p.tiles_per_n * p.cblocks);
    // channel counts in pairs of channels
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3((kSamplerWaves + kPairsLoaderWaves) * 64), p.lds_bytes, stream,
                       (const T*)a.x, (const T*)a.grid, (T*)a.y, make_fast_div((uint32_t)a.N), (int32_t)(a.C / 2),
                       (int32_t)a.Hin, (int32_t)a.Win, (int32_t)(a.Hout * a.Wout), make_fast_div(p.tiles_per_n),
                       p.chans_per_block / 2, p.wide_blocks, p.chans_wide / 2, p.chan_stride, p.copy_gran, pair_aligned,
                       p.xcd_swizzle, p.row_shift, (int32_t)a.pad, (int32_t)(a.align != 0), (int32_t)a.rule, p.lds_w,
                       -0.0f);
    return hipGetLastError();
}

template <typename T, int PPT, int PITCH>
hipError_t launch_pairs_adj(const GridSamplerArgs& a, const LdsPlan& p, hipStream_t stream)
{
    return p.adj == 2 ? launch_pairs<T, PPT, 2, PITCH>(a, p, stream) : launch_pairs<T, PPT, 1, PITCH>(a, p, stream);
}

template <typename T>
hipError_t launch_pairs_typed(const GridSamplerArgs& a, const LdsPlan& p, hipStream_t stream)
{
    if (a.interp == 2) {  // bicubic: one or two pixels per lane, single stores
        if (p.pairs_pitch == kPairsPitch && p.ppt == 2) {
            return launch_pairs<T, 2, 1, kPairsPitch, 2>(a, p, stream);
        }
        if (p.pairs_pitch == kPairsPitch && p.ppt == 1) {
            return launch_pairs<T, 1, 1, kPairsPitch, 2>(a, p, stream);
        }
        if (p.pairs_pitch == kPairsPitchLarge && p.ppt == 2) {
            return launch_pairs<T, 2, 1, kPairsPitchLarge, 2>(a, p, stream);
        }
        if (p.pairs_pitch == kPairsPitchLarge && p.ppt == 1) {
            return launch_pairs<T, 1, 1, kPairsPitchLarge, 2>(a, p, stream);
        }
        return hipErrorInvalidValue;
    }
    if (p.pairs_pitch == kPairsPitch && p.ppt == 4) {
        return launch_pairs_adj<T, 4, kPairsPitch>(a, p, stream);
    }
    if (p.pairs_pitch == kPairsPitchLarge && p.ppt == 8) {
        return launch_pairs_adj<T, 8, kPairsPitchLarge>(a, p, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace

hipError_t lds_launch_channel_pairs(const GridSamplerArgs& a, const LdsPlan& p, hipStream_t stream)
{
    if (!p.chan_pairs) {
        return hipErrorInvalidValue;
    }
    switch (a.elem) {
        case Elem::F16: return launch_pairs_typed<_Float16>(a, p, stream);
        case Elem::BF16: return launch_pairs_typed<__bf16>(a, p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace opscv
