// Grid sampler 2-D forward kernels for gfx950 (bilinear, nearest and bicubic; zeros, border, reflection; align
// on/off).
//
// Replaces the reference device kernel image/grid_sampler2_d/op_kernel/arch35/grid_sampler2_d_simt.h:461-557 and
// its host tiling image/grid_sampler2_d/op_host/arch35/grid_sampler2_d_tiling.cpp:208-271.
//
// Common shape of every variant: one lane owns one output pixel (n, h, w); the wavefront therefore reads a
// contiguous run of grid values and writes a contiguous run of every output channel plane.  The source
// coordinate, the four tap offsets, the four weights and the bounds masks are computed once and stay in
// registers across the channel loop.
#include <hip/hip_runtime.h>

#include <type_traits>

#include <cstdlib>

#include "gs2d_common.hpp"
#include "kernels.hpp"
#include "options.hpp"
#include "sampler_math.hpp"

namespace opscv {

namespace {

constexpr int kDirectThreads = 256;

// ---------------------------------------------------------------------------------------------------------
// Direct variant: taps are read straight from global memory (through L1/L2).  Works for every shape.
// ---------------------------------------------------------------------------------------------------------
template <typename T, int INTERP, int PAD, bool ALIGN>
__global__ __launch_bounds__(kDirectThreads) void gs2d_direct_kernel(const T* __restrict__ x,
                                                                      const T* __restrict__ grid,
                                                                      T* __restrict__ y, int64_t total_pixels,
                                                                      int32_t C_all, int32_t H, int32_t W,
                                                                      int64_t out_plane, int32_t chan_chunk)
{
    // blockIdx.y selects a run of channels: with few output pixels the channels are what fills the GPU
    const int32_t c_first = (int32_t)blockIdx.y * chan_chunk;
    const int32_t C = (c_first + chan_chunk < C_all) ? chan_chunk : C_all - c_first;
    const int64_t in_plane = (int64_t)H * W;
    const int64_t stride = (int64_t)gridDim.x * kDirectThreads;
    for (int64_t p = (int64_t)blockIdx.x * kDirectThreads + threadIdx.x; p < total_pixels; p += stride) {
        const int64_t n = p / out_plane;
        const int64_t rem = p - n * out_plane;
        const float gx = ElemIO<T>::load(grid + 2 * p);
        const float gy = ElemIO<T>::load(grid + 2 * p + 1);
        const T* xp = x + (n * C_all + c_first) * in_plane;
        T* yp = y + (n * C_all + c_first) * out_plane + rem;
        if constexpr (INTERP == 2) {
            // grid_sampler2_d_simt.h:375-458
            const BicubicTap b = decide_bicubic<PAD, ALIGN>(gx, gy, H, W);
            if (b.flag) {
                const float nan_val = __builtin_nanf("");
                for (int32_t c = 0; c < C; c++) {
                    ElemIO<T>::store(yp, nan_val);
                    yp += out_plane;
                }
                continue;
            }
            bool col_in[4], row_in[4];
            int64_t row_off[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                col_in[k] = b.bx[k] >= 0 && b.bx[k] < W;
                row_in[k] = b.by[k] >= 0 && b.by[k] < H;
                row_off[k] = row_in[k] ? (int64_t)b.by[k] * W : 0;
            }
            // Away from the left and right edge the four columns of a row are neighbours in memory and inside the
            // image: one load of four elements (aligned to one element only) instead of four.  Taken when that holds
            // for every lane of the wavefront, so that the choice costs no divergence.
            const bool in_a_row = b.bx[0] >= 0 && b.bx[3] < W && b.bx[1] == b.bx[0] + 1 && b.bx[2] == b.bx[0] + 2 &&
                                  b.bx[3] == b.bx[0] + 3;
            if (__builtin_amdgcn_ballot_w64(!in_a_row) == 0) {
                for (int32_t c = 0; c < C; c++) {
                    float r[4];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        r[j] = 0.0f;
                        if (row_in[j]) {
                            uint64_t bits[sizeof(T) / 2];  // 8 bytes for 16-bit elements, 16 for fp32
                            __builtin_memcpy(bits, xp + row_off[j] + b.bx[0], 4 * sizeof(T));
                            T q[4];
                            __builtin_memcpy(q, bits, 4 * sizeof(T));
                            r[j] = bicubic_weighted_sum(b.cx[0], b.cx[1], b.cx[2], b.cx[3], ElemIO<T>::load(&q[0]),
                                                        ElemIO<T>::load(&q[1]), ElemIO<T>::load(&q[2]),
                                                        ElemIO<T>::load(&q[3]));
                        }
                    }
                    ElemIO<T>::store(yp,
                                     bicubic_weighted_sum(b.cy[0], b.cy[1], b.cy[2], b.cy[3], r[0], r[1], r[2], r[3]));
                    xp += in_plane;
                    yp += out_plane;
                }
                continue;
            }
            for (int32_t c = 0; c < C; c++) {
                float r[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    r[j] = 0.0f;
                    if (row_in[j]) {
                        float v[4];
#pragma unroll
                        for (int k = 0; k < 4; k++) {
                            v[k] = col_in[k] ? ElemIO<T>::load(xp + row_off[j] + b.bx[k]) : 0.0f;
                        }
                        r[j] = bicubic_weighted_sum(b.cx[0], b.cx[1], b.cx[2], b.cx[3], v[0], v[1], v[2], v[3]);
                    }
                }
                ElemIO<T>::store(yp, bicubic_weighted_sum(b.cy[0], b.cy[1], b.cy[2], b.cy[3], r[0], r[1], r[2], r[3]));
                xp += in_plane;
                yp += out_plane;
            }
            continue;
        }
        const PixelTap t = decide_pixel<(INTERP == 2 ? 0 : INTERP), PAD, ALIGN>(gx, gy, H, W);
        if (INTERP == 0) {
            if (t.flag) {
                const float nan_val = __builtin_nanf("");
                for (int32_t c = 0; c < C; c++) {
                    ElemIO<T>::store(yp, nan_val);
                    yp += out_plane;
                }
                continue;
            }
            const int32_t x0 = t.x0, y0 = t.y0;
            const int32_t x1 = (x0 == INT32_MAX) ? x0 : x0 + 1;
            const int32_t y1 = (y0 == INT32_MAX) ? y0 : y0 + 1;
            const bool in_nw = within(y0, x0, H, W), in_ne = within(y0, x1, H, W);
            const bool in_sw = within(y1, x0, H, W), in_se = within(y1, x1, H, W);
            // offsets are only dereferenced under their mask; clamp them to 0 so that they are always valid
            const int64_t o_nw = in_nw ? (int64_t)y0 * W + x0 : 0;
            const int64_t o_ne = in_ne ? (int64_t)y0 * W + x1 : 0;
            const int64_t o_sw = in_sw ? (int64_t)y1 * W + x0 : 0;
            const int64_t o_se = in_se ? (int64_t)y1 * W + x1 : 0;
            if (W >= 2) {
                // The west and east corner of a row are neighbours in memory: one load of two elements (aligned to
                // one element only, which global memory accesses allow) per row instead of two loads halves the
                // addresses the gather puts through the memory pipeline, which is what bounds it.  The pair sits at
                // column pb = clamp(x0, 0, W - 2), so it never leaves the row; which half is which corner follows
                // from pb.  Same sums in the same order.
                using PairBits = typename std::conditional<sizeof(T) == 2, uint32_t, uint64_t>::type;
                const int32_t pb = (x0 < 0) ? 0 : ((x0 > W - 2) ? W - 2 : x0);
                const bool lo_w = (x0 == pb), lo_e = (x1 == pb);
                const bool row_n = in_nw || in_ne, row_s = in_sw || in_se;
                const int64_t o_n = row_n ? (int64_t)y0 * W + pb : 0;
                const int64_t o_s = row_s ? (int64_t)y1 * W + pb : 0;
#pragma unroll 4
                for (int32_t c = 0; c < C; c++) {
                    PairBits north = 0, south = 0;
                    if (row_n) {
                        __builtin_memcpy(&north, xp + o_n, sizeof(PairBits));
                    }
                    if (row_s) {
                        __builtin_memcpy(&south, xp + o_s, sizeof(PairBits));
                    }
                    T n2[2], s2[2];
                    __builtin_memcpy(n2, &north, sizeof(PairBits));
                    __builtin_memcpy(s2, &south, sizeof(PairBits));
                    const float nlo = ElemIO<T>::load(&n2[0]), nhi = ElemIO<T>::load(&n2[1]);
                    const float slo = ElemIO<T>::load(&s2[0]), shi = ElemIO<T>::load(&s2[1]);
                    float out = 0.0f;
                    if (in_nw) {
                        out += (lo_w ? nlo : nhi) * t.w[0];
                    }
                    if (in_ne) {
                        out += (lo_e ? nlo : nhi) * t.w[1];
                    }
                    if (in_sw) {
                        out += (lo_w ? slo : shi) * t.w[2];
                    }
                    if (in_se) {
                        out += (lo_e ? slo : shi) * t.w[3];
                    }
                    ElemIO<T>::store(yp, out);
                    xp += in_plane;
                    yp += out_plane;
                }
                continue;
            }
#pragma unroll 4
            for (int32_t c = 0; c < C; c++) {
                // grid_sampler2_d_simt.h:321-338 : nw, ne, sw, se added in this order, skipped when outside
                float out = 0.0f;
                if (in_nw) {
                    out += ElemIO<T>::load(xp + o_nw) * t.w[0];
                }
                if (in_ne) {
                    out += ElemIO<T>::load(xp + o_ne) * t.w[1];
                }
                if (in_sw) {
                    out += ElemIO<T>::load(xp + o_sw) * t.w[2];
                }
                if (in_se) {
                    out += ElemIO<T>::load(xp + o_se) * t.w[3];
                }
                ElemIO<T>::store(yp, out);
                xp += in_plane;
                yp += out_plane;
            }
        } else {
            const bool in = within(t.y0, t.x0, H, W);
            const int64_t o = in ? (int64_t)t.y0 * W + t.x0 : 0;
#pragma unroll 4
            for (int32_t c = 0; c < C; c++) {
                // grid_sampler2_d_simt.h:341-360 : the value passes through fp32, exact for 16-bit types
                float out = 0.0f;
                if (in) {
                    out = ElemIO<T>::load(xp + o);
                }
                ElemIO<T>::store(yp, out);
                xp += in_plane;
                yp += out_plane;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// Bilinear sampling by the second coordinate rule (option "grid_sampler2d_rule" = 1), for every shape the LDS ring
// does not take: the arithmetic of the kernel that the reference's aclnnGridSampler2D launches for NCHW tensors on its
// arch35 part, image/grid_sample/op_kernel/arch35/grid_sampler_2d_bilinear_smit.h:67-153 with
// grid_sampler_bilinear_smit_common.h:36-90 -- unnormalise as ((g + 1) * size - 1) / 2, reflect with fmodf, a
// non-finite coordinate becomes -100 (a zero sample), weights (1 - dh)(1 - dw) ..., the sum starts with the bare first
// product, a corner outside the image counts as the value 0.  One lane per output pixel, decisions hoisted out of the
// channel loop (the reference repeats them per channel; they do not depend on it).
// ---------------------------------------------------------------------------------------------------------
template <typename T, int PAD, bool ALIGN>
__global__ __launch_bounds__(kDirectThreads) void gs2d_arch35_kernel(const T* __restrict__ x,
                                                                      const T* __restrict__ grid,
                                                                      T* __restrict__ y, int64_t total_pixels,
                                                                      int32_t C_all, int32_t H, int32_t W,
                                                                      int64_t out_plane, int32_t chan_chunk)
{
    const int32_t c_first = (int32_t)blockIdx.y * chan_chunk;
    const int32_t C = (c_first + chan_chunk < C_all) ? chan_chunk : C_all - c_first;
    const int64_t in_plane = (int64_t)H * W;
    const int64_t stride = (int64_t)gridDim.x * kDirectThreads;
    for (int64_t p = (int64_t)blockIdx.x * kDirectThreads + threadIdx.x; p < total_pixels; p += stride) {
        const int64_t n = p / out_plane;
        const int64_t rem = p - n * out_plane;
        const float gw = ElemIO<T>::load(grid + 2 * p);
        const float gh = ElemIO<T>::load(grid + 2 * p + 1);
        const float pw = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gw, W), W);
        const float ph = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gh, H), H);
        const float hf = __builtin_floorf(ph), wf = __builtin_floorf(pw);
        const float dh = ph - hf, dw = pw - wf;
        // corner indices from the floats floor and floor + 1 (saturating conversion: anything beyond int32 lies
        // outside every image, like the reference's out-of-range conversion)
        const int32_t h0 = float_to_i32(hf), w0 = float_to_i32(wf);
        const int32_t h1 = float_to_i32(hf + 1.0f), w1 = float_to_i32(wf + 1.0f);
        const bool in[4] = {within(h0, w0, H, W), within(h0, w1, H, W), within(h1, w0, H, W), within(h1, w1, H, W)};
        const int64_t off[4] = {in[0] ? (int64_t)h0 * W + w0 : 0, in[1] ? (int64_t)h0 * W + w1 : 0,
                                in[2] ? (int64_t)h1 * W + w0 : 0, in[3] ? (int64_t)h1 * W + w1 : 0};
        const float wt[4] = {(1.0f - dh) * (1.0f - dw), (1.0f - dh) * dw, dh * (1.0f - dw), dh * dw};
        const T* xp = x + (n * C_all + c_first) * in_plane;
        T* yp = y + (n * C_all + c_first) * out_plane + rem;
#pragma unroll 4
        for (int32_t c = 0; c < C; c++) {
            float v[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                v[k] = in[k] ? ElemIO<T>::load(xp + off[k]) : 0.0f;
            }
            float out = v[0] * wt[0];
            out += v[1] * wt[1];
            out += v[2] * wt[2];
            out += v[3] * wt[3];
            ElemIO<T>::store(yp, out);
            xp += in_plane;
            yp += out_plane;
        }
    }
}

template <typename T, int INTERP, int PAD, bool ALIGN>
__global__ __launch_bounds__(kDirectThreads) void gs2d_taps_kernel(const T* __restrict__ grid,
                                                                    TapRecord* __restrict__ taps,
                                                                    int64_t total_pixels, int32_t H, int32_t W)
{
    const int64_t stride = (int64_t)gridDim.x * kDirectThreads;
    for (int64_t p = (int64_t)blockIdx.x * kDirectThreads + threadIdx.x; p < total_pixels; p += stride) {
        const float gx = ElemIO<T>::load(grid + 2 * p);
        const float gy = ElemIO<T>::load(grid + 2 * p + 1);
        const PixelTap t = decide_pixel<INTERP, PAD, ALIGN>(gx, gy, H, W);
        TapRecord r;
        r.x0 = t.x0;
        r.y0 = t.y0;
        r.w[0] = t.w[0];
        r.w[1] = t.w[1];
        r.w[2] = t.w[2];
        r.w[3] = t.w[3];
        r.flag = t.flag;
        taps[p] = r;
    }
}

template <typename T, int PAD, bool ALIGN>
__global__ __launch_bounds__(kDirectThreads) void gs2d_bicubic_taps_kernel(const T* __restrict__ grid,
                                                                            BicubicTapRecord* __restrict__ taps,
                                                                            int64_t total_pixels, int32_t H, int32_t W)
{
    const int64_t stride = (int64_t)gridDim.x * kDirectThreads;
    for (int64_t p = (int64_t)blockIdx.x * kDirectThreads + threadIdx.x; p < total_pixels; p += stride) {
        const float gx = ElemIO<T>::load(grid + 2 * p);
        const float gy = ElemIO<T>::load(grid + 2 * p + 1);
        const BicubicTap t = decide_bicubic<PAD, ALIGN>(gx, gy, H, W);
        BicubicTapRecord r;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            r.bx[k] = t.bx[k];
            r.by[k] = t.by[k];
            r.cx[k] = t.cx[k];
            r.cy[k] = t.cy[k];
        }
        r.flag = t.flag;
        taps[p] = r;
    }
}

inline int blocks_for(int64_t items, int threads)
{
    int64_t b = (items + threads - 1) / threads;
    const int64_t cap = 256 * 64;  // 256 CUs; enough resident waves, the loops are grid-stride
    if (b > cap) {
        b = cap;
    }
    if (b < 1) {
        b = 1;
    }
    return (int)b;
}

template <typename T, int INTERP, int PAD, bool ALIGN>
hipError_t run_direct(const GridSamplerArgs& a, hipStream_t stream)
{
    const int64_t total = a.N * a.Hout * a.Wout;
    const int blocks = blocks_for(total, kDirectThreads);
    // a lane walks its channels one after the other, each step waiting for its loads: aim at 8192 workgroups (eight
    // wavefronts per SIMD) by giving runs of channels to different workgroups when the pixels alone are too few
    int64_t chunks = (8192 + blocks - 1) / blocks;
    chunks = chunks < a.C ? chunks : a.C;
    chunks = chunks < 1 ? 1 : chunks;
    const int64_t chan_chunk = (a.C + chunks - 1) / chunks;
    const int64_t grid_y = (a.C + chan_chunk - 1) / chan_chunk;
    if (grid_y > 65535) {
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL((gs2d_direct_kernel<T, INTERP, PAD, ALIGN>), dim3((unsigned)blocks, (unsigned)grid_y),
                       dim3(kDirectThreads), 0, stream, (const T*)a.x, (const T*)a.grid, (T*)a.y, total,
                       (int32_t)a.C, (int32_t)a.Hin, (int32_t)a.Win, a.Hout * a.Wout, (int32_t)chan_chunk);
    return hipGetLastError();
}

template <typename T, int PAD, bool ALIGN>
hipError_t run_arch35(const GridSamplerArgs& a, hipStream_t stream)
{
    const int64_t total = a.N * a.Hout * a.Wout;
    const int blocks = blocks_for(total, kDirectThreads);
    int64_t chunks = (8192 + blocks - 1) / blocks;  // as run_direct
    chunks = chunks < a.C ? chunks : a.C;
    chunks = chunks < 1 ? 1 : chunks;
    const int64_t chan_chunk = (a.C + chunks - 1) / chunks;
    const int64_t grid_y = (a.C + chan_chunk - 1) / chan_chunk;
    if (grid_y > 65535) {
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL((gs2d_arch35_kernel<T, PAD, ALIGN>), dim3((unsigned)blocks, (unsigned)grid_y),
                       dim3(kDirectThreads), 0, stream, (const T*)a.x, (const T*)a.grid, (T*)a.y, total,
                       (int32_t)a.C, (int32_t)a.Hin, (int32_t)a.Win, a.Hout * a.Wout, (int32_t)chan_chunk);
    return hipGetLastError();
}

template <typename T, int INTERP, int PAD, bool ALIGN>
hipError_t run_taps(const GridSamplerArgs& a, TapRecord* taps, hipStream_t stream)
{
    const int64_t total = a.N * a.Hout * a.Wout;
    if constexpr (INTERP == 2) {
        (void)taps;
        (void)stream;
        (void)total;
        return hipErrorInvalidValue;  // the bicubic record has its own entry point
    } else {
        hipLaunchKernelGGL((gs2d_taps_kernel<T, INTERP, PAD, ALIGN>), dim3(blocks_for(total, kDirectThreads)),
                           dim3(kDirectThreads), 0, stream, (const T*)a.grid, taps, total, (int32_t)a.Hin,
                           (int32_t)a.Win);
        return hipGetLastError();
    }
}

template <typename T, int INTERP, int PAD, bool ALIGN>
hipError_t run_bicubic_taps(const GridSamplerArgs& a, BicubicTapRecord* taps, hipStream_t stream)
{
    const int64_t total = a.N * a.Hout * a.Wout;
    hipLaunchKernelGGL((gs2d_bicubic_taps_kernel<T, PAD, ALIGN>), dim3(blocks_for(total, kDirectThreads)),
                       dim3(kDirectThreads), 0, stream, (const T*)a.grid, taps, total, (int32_t)a.Hin,
                       (int32_t)a.Win);
    return hipGetLastError();
}

struct DirectLauncher {
    const GridSamplerArgs& a;
    hipStream_t stream;
    template <typename T, int I, int P, bool A>
    hipError_t operator()() const
    {
        return run_direct<T, I, P, A>(a, stream);
    }
};

struct Arch35Launcher {
    const GridSamplerArgs& a;
    hipStream_t stream;
    template <typename T, int I, int P, bool A>
    hipError_t operator()() const
    {
        if constexpr (I == 0) {
            return run_arch35<T, P, A>(a, stream);
        } else {
            return hipErrorInvalidValue;
        }
    }
};

struct TapsLauncher {
    const GridSamplerArgs& a;
    TapRecord* taps;
    hipStream_t stream;
    template <typename T, int I, int P, bool A>
    hipError_t operator()() const
    {
        return run_taps<T, I, P, A>(a, taps, stream);
    }
};

struct BicubicTapsLauncher {
    const GridSamplerArgs& a;
    BicubicTapRecord* taps;
    hipStream_t stream;
    template <typename T, int I, int P, bool A>
    hipError_t operator()() const
    {
        return run_bicubic_taps<T, I, P, A>(a, taps, stream);
    }
};

}  // namespace

namespace {
// option "gs_variant" as captured by the first phase: the direct kernel forced, or the pair-layout variant kept out
// (benchmark and test knobs)
bool force_direct(const GridSamplerArgs& a) { return a.force_variant == kGsDirect; }
bool force_ring(const GridSamplerArgs& a) { return a.force_variant == kGsRing || a.force_variant == kGsRingSingle; }
// Bilinear samples that the ring kernel takes two channels at a time go there rather than to the pair-layout kernel,
// up to eight output pixels per input pixel (fp16 N16 C128 64x64 -> 128x128: 18.5 us against the pair layout's 21.9,
// -> 160x160 29.5 against 41.5, bf16 N8 C128 32x128 -> 80x320 16.4 against 25.2; beyond, the pair layout's twelve pixels
// per lane stage every plane less often: fp16 N16 C64 64x64 -> 192x192 26.2 against 20.6).
// Bicubic samples under zeros padding likewise where a plane is above 4 KiB and a channel block takes 32 channels or
// more, over which the sixteen tap offsets of a pixel are decided once (fp16 N16 C256 64x64 -> 64x64: 29.1 us
// against the bicubic pair layout's 31.5, 40x96 28.4 against 35.0, 128x32 31.4 against 38.9; planes of 32x64 19.0
// against 14.0, N8 C64 64x64 with eight channels per block 11.9 against 7.6).  Under border padding the pair layout's
// staged margins win (64x64: 43.9 against 31.0); reflection has no pair layout and comes here anyway.
constexpr int64_t kBicubicRingChannels = 32;  // 16 per block: 19.6 us against 17.5, 24: 24.1 against 24.3
bool ring_before_pair(const GridSamplerArgs& a)
{
    if (a.interp == 2) {
        // (planes above 8 KiB, whose pair layout leaves room for fewer workgroups: from 16 channels per block on -- fp16
        // N16 C128 96x64 -> 96x64, 21 per block, 27.2 us against 41.9)
        const int64_t plane_bytes = a.Hin * a.Win * 2;
        const int64_t enough = plane_bytes > 8192 ? kBicubicRingChannels / 2 : kBicubicRingChannels;
        return a.pad == 0 && plane_bytes > 4096 && gs2d_lds_channel_pairs_per_block(a) >= enough;
    }
    return a.interp == 0 && a.Hout * a.Wout <= 8 * a.Hin * a.Win && gs2d_lds_channel_pairs(a);
}
}  // namespace

// The second coordinate rule (bilinear only) is implemented by the LDS ring and by a direct kernel of its own.
static bool second_rule(const GridSamplerArgs& a) { return a.rule != kRuleGridSampler2D && a.interp == 0; }

const char* grid_sampler2d_variant(const GridSamplerArgs& a)
{
    if (second_rule(a)) {
        const char* n = force_direct(a) ? nullptr : gs2d_lds_variant_name(a);
        return n != nullptr ? n : "direct_arch35";
    }
    if (a.channels_last) {
        return "nhwc";
    }
    if (!force_direct(a)) {
        const char* n = (force_ring(a) || ring_before_pair(a)) ? nullptr : gs2d_pair_variant_name(a);
        if (n == nullptr) {
            n = gs2d_lds_variant_name(a);
        }
        if (n == nullptr) {
            n = gs2d_box_variant_name(a);
        }
        if (n != nullptr) {
            return n;
        }
    }
    return "direct";
}

hipError_t launch_grid_sampler2d(const GridSamplerArgs& a, hipStream_t stream)
{
    if (!gs_shapes_ok(a) || a.interp < 0 || a.interp > 2 || a.pad < 0 || a.pad > 2) {
        return hipErrorInvalidValue;
    }
    if (a.N == 0 || a.C == 0 || a.Hout == 0 || a.Wout == 0) {
        return hipSuccess;
    }
    if (a.x == nullptr || a.grid == nullptr || a.y == nullptr) {
        return hipErrorInvalidValue;
    }
    if (second_rule(a)) {
        if (a.channels_last) {
            return hipErrorInvalidValue;  // the first phase packs such views under this rule
        }
        if (!force_direct(a)) {
            bool handled = false;
            const hipError_t e = run_gs2d_lds(a, stream, &handled);
            if (handled || e != hipSuccess) {
                return e;
            }
        }
        return dispatch_elem(a, Arch35Launcher{a, stream});
    }
    if (a.channels_last) {
        return run_gs2d_nhwc(a, stream);
    }
    if (!force_direct(a)) {
        bool handled = false;
        hipError_t e = (force_ring(a) || ring_before_pair(a)) ? hipSuccess : run_gs2d_pair(a, stream, &handled);
        if (handled || e != hipSuccess) {
            return e;
        }
        e = run_gs2d_lds(a, stream, &handled);
        if (handled || e != hipSuccess) {
            return e;
        }
        e = run_gs2d_box(a, stream, &handled);
        if (handled || e != hipSuccess) {
            return e;
        }
    }
    return dispatch_elem(a, DirectLauncher{a, stream});
}

hipError_t launch_grid_sampler2d_taps(const GridSamplerArgs& a, TapRecord* taps, hipStream_t stream)
{
    if (!gs_shapes_ok(a) || a.interp < 0 || a.interp > 1 || a.pad < 0 || a.pad > 2) {
        return hipErrorInvalidValue;
    }
    if (a.N == 0 || a.Hout == 0 || a.Wout == 0) {
        return hipSuccess;
    }
    if (a.grid == nullptr || taps == nullptr) {
        return hipErrorInvalidValue;
    }
    return dispatch_elem(a, TapsLauncher{a, taps, stream});
}

hipError_t launch_grid_sampler2d_bicubic_taps(const GridSamplerArgs& a, BicubicTapRecord* taps, hipStream_t stream)
{
    if (!gs_shapes_ok(a) || a.interp != 2 || a.pad < 0 || a.pad > 2) {
        return hipErrorInvalidValue;
    }
    if (a.N == 0 || a.Hout == 0 || a.Wout == 0) {
        return hipSuccess;
    }
    if (a.grid == nullptr || taps == nullptr) {
        return hipErrorInvalidValue;
    }
    return dispatch_elem(a, BicubicTapsLauncher{a, taps, stream});
}

}  // namespace opscv
