// Grid sampler 2-D forward for channels-last tensors (input (N,Hin,Win,C) and output (N,Hout,Wout,C) in memory)
// on gfx950.
//
// Same arithmetic as the NCHW variants (see sampler_math.hpp; reference kernel
// image/grid_sampler2_d/op_kernel/arch35/grid_sampler2_d_simt.h:303-360,375-458).  With the channels innermost
// every tap of a pixel is one contiguous run of C elements, so the gather needs no staging:
//   * `lpp` neighbouring lanes (a power of two, at most 32) share one output pixel; each takes every lpp-th
//     16-byte run of channels, so a pixel's tap is read -- and its output written -- as contiguous 16*lpp bytes;
//   * every lane decides its pixel once (tap offsets, weights, bounds masks) and keeps that across its channel runs;
//   * a tap outside the image is replaced by zeros after the (clamped, always valid) load, which is the
//     reference's "skip the tap": 0 * w adds nothing.
// When C is not a multiple of the vector length, or a tensor is not 16-byte aligned, the same kernel runs with
// one element per lane and step.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "gs2d_common.hpp"
#include "gs2d_lds_kernel.hpp"
#include "kernels.hpp"
#include "sampler_math.hpp"

namespace opscv {

namespace {

constexpr int kNhwcThreads = 256;

// What a lane keeps per pixel: element offsets of the taps inside image n (0, always valid, when the tap is
// outside), their bounds masks and the weights.
template <int NT, int NW>
struct NhwcPixel {
    int64_t toff[NT];
    bool tin[NT];
    float tw[NW];
};

template <typename T, int INTERP, int PAD, bool ALIGN, int NT, int NW>
__device__ __forceinline__ void nhwc_decide(float gx, float gy, int32_t C, int32_t H, int32_t W, NhwcPixel<NT, NW>& px)
{
    if constexpr (INTERP == 2) {
        const BicubicTap b = decide_bicubic<PAD, ALIGN>(gx, gy, H, W);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const bool row_in = b.by[r] >= 0 && b.by[r] < H && !b.flag;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const bool in = row_in && b.bx[k] >= 0 && b.bx[k] < W;
                px.tin[4 * r + k] = in;
                px.toff[4 * r + k] = in ? ((int64_t)b.by[r] * W + b.bx[k]) * C : 0;
            }
            px.tw[r] = b.cx[r];
            px.tw[4 + r] = b.cy[r];
        }
        if (b.flag) {
            px.tw[0] = __builtin_nanf("");  // 0 * NaN: every channel becomes NaN, as the reference writes
        }
    } else if constexpr (INTERP == 0) {
        const PixelTap t = decide_pixel<0, PAD, ALIGN>(gx, gy, H, W);
        const int32_t x0 = t.x0, y0 = t.y0;
        const int32_t x1 = (x0 == INT32_MAX) ? x0 : x0 + 1;
        const int32_t y1 = (y0 == INT32_MAX) ? y0 : y0 + 1;
        const int32_t xs[4] = {x0, x1, x0, x1};
        const int32_t ys[4] = {y0, y0, y1, y1};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const bool in = within(ys[k], xs[k], H, W) && !t.flag;
            px.tin[k] = in;
            px.toff[k] = in ? ((int64_t)ys[k] * W + xs[k]) * C : 0;
            px.tw[k] = t.w[k];
        }
        if (t.flag) {
            px.tw[0] = __builtin_nanf("");
        }
    } else {
        const PixelTap t = decide_pixel<1, PAD, ALIGN>(gx, gy, H, W);
        const bool in = within(t.y0, t.x0, H, W);
        px.tin[0] = in;
        px.toff[0] = in ? ((int64_t)t.y0 * W + t.x0) * C : 0;
        px.tw[0] = px.tw[1] = px.tw[2] = px.tw[3] = 0.0f;
    }
}

// PIX pixels per lane group: pixel j of a group is  block_first + j * groups_per_block + group,  so neighbouring
// groups read neighbouring grid points.  All grid values of the PIX pixels are loaded before any is used, and per
// channel run all PIX * NT tap vectors are requested before the first blend: one wavefront keeps that many
// independent memory operations in flight, which is what hides the two dependent latencies (grid, then taps)
// of a gather.
template <typename T, int INTERP, int PAD, bool ALIGN, bool VEC, int PIX>
__global__ __launch_bounds__(kNhwcThreads) void gs2d_nhwc_kernel(const T* __restrict__ x, const T* __restrict__ grid,
                                                                  T* __restrict__ y, int64_t total_pixels, int32_t C,
                                                                  int32_t H, int32_t W, int64_t out_plane,
                                                                  int32_t lpp_shift, float neg_zero)
{
    constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
    constexpr int NT = (INTERP == 0) ? 4 : (INTERP == 1 ? 1 : 16);
    constexpr int NW = (INTERP == 2) ? 8 : 4;
    const int32_t lpp = 1 << lpp_shift;
    const int32_t sub = threadIdx.x & (lpp - 1);
    const int32_t groups = kNhwcThreads >> lpp_shift;
    const int64_t first = (int64_t)blockIdx.x * groups * PIX + (threadIdx.x >> lpp_shift);

    float gx[PIX], gy[PIX];
    bool live[PIX];
    int64_t pix[PIX];
#pragma unroll
    for (int j = 0; j < PIX; j++) {
        const int64_t p = first + (int64_t)j * groups;
        live[j] = p < total_pixels;
        pix[j] = live[j] ? p : total_pixels - 1;
        // grid points and results stream (non-temporal hint), the tap loads do not: see load_grid_points in
        // gs2d_lds_kernel.hpp
        typedef typename std::conditional<sizeof(T) == 2, uint16_t, uint32_t>::type bits_t;
        const bits_t* gp = reinterpret_cast<const bits_t*>(grid + 2 * pix[j]);
        const T ex = __builtin_bit_cast(T, __builtin_nontemporal_load(gp));
        const T ey = __builtin_bit_cast(T, __builtin_nontemporal_load(gp + 1));
        gx[j] = ElemIO<T>::load(&ex);
        gy[j] = ElemIO<T>::load(&ey);
    }
    NhwcPixel<NT, NW> px[PIX];
    const T* xn[PIX];
#pragma unroll
    for (int j = 0; j < PIX; j++) {
        nhwc_decide<T, INTERP, PAD, ALIGN, NT, NW>(gx[j], gy[j], C, H, W, px[j]);
        xn[j] = x + (pix[j] / out_plane) * (int64_t)H * W * C;
    }

    const int32_t runs = C / V;  // VEC: C % V == 0
    for (int32_t cv = sub; cv < runs; cv += lpp) {
        const int32_t c = cv * V;
        T tap[PIX][NT][V];
#pragma unroll
        for (int j = 0; j < PIX; j++) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                if constexpr (VEC) {
                    // the reference skips a tap outside the image: zeros, so that 0 * w adds nothing
                    uint4 raw = *reinterpret_cast<const uint4*>(xn[j] + px[j].toff[t] + c);
                    if (!px[j].tin[t]) {
                        raw = make_uint4(0u, 0u, 0u, 0u);
                    }
                    __builtin_memcpy(tap[j][t], &raw, 16);
                } else {
                    T v = xn[j][px[j].toff[t] + c];
                    if (!px[j].tin[t]) {
                        ElemIO<T>::store(&v, 0.0f);
                    }
                    tap[j][t][0] = v;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < PIX; j++) {
            T outv[V];
#pragma unroll
            for (int i = 0; i < V; i++) {
                T raw[NT];
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    raw[t] = tap[j][t][i];
                }
                ElemIO<T>::store(&outv[i], blend<T, INTERP>(raw, px[j].tw, neg_zero));
            }
            if (live[j]) {
                T* yp = y + pix[j] * C + c;
                if constexpr (VEC) {
                    typedef uint32_t dwordx4_t __attribute__((ext_vector_type(4)));
                    dwordx4_t packed;
                    __builtin_memcpy(&packed, outv, 16);
                    __builtin_nontemporal_store(packed, reinterpret_cast<dwordx4_t*>(yp));
                } else {
                    typedef typename std::conditional<sizeof(T) == 2, uint16_t, uint32_t>::type bits_t;
                    __builtin_nontemporal_store(__builtin_bit_cast(bits_t, outv[0]), reinterpret_cast<bits_t*>(yp));
                }
            }
        }
    }
}

struct NhwcLauncher {
    const GridSamplerArgs& a;
    hipStream_t stream;
    template <typename T, int I, int P, bool A>
    hipError_t operator()() const
    {
        constexpr int V = 16 / (int)sizeof(T);
        // one pixel per lane group measured best on MI355X (four: 24.0 us instead of 17.7 us on the fp16
        // N16 C256 64x64 case -- the wavefronts lost outweigh the loads gained per wavefront)
        constexpr int PIX = 1;
        const bool vec = a.C % V == 0 && reinterpret_cast<uintptr_t>(a.x) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(a.y) % 16 == 0;
        const int64_t runs = vec ? a.C / V : a.C;
        // lanes per pixel: the largest power of two not above the number of channel runs, at most 32
        int shift = 0;
        while (shift < 5 && (2ll << shift) <= runs) {
            shift++;
        }
        const int64_t total = a.N * a.Hout * a.Wout;
        const int64_t per_block = (int64_t)(kNhwcThreads >> shift) * PIX;
        const int64_t blocks = (total + per_block - 1) / per_block;
        if (blocks > INT32_MAX) {
            return hipErrorInvalidValue;
        }
        if (vec) {
            hipLaunchKernelGGL((gs2d_nhwc_kernel<T, I, P, A, true, PIX>), dim3((unsigned)blocks), dim3(kNhwcThreads), 0,
                               stream, (const T*)a.x, (const T*)a.grid, (T*)a.y, total, (int32_t)a.C, (int32_t)a.Hin,
                               (int32_t)a.Win, a.Hout * a.Wout, shift, -0.0f);
        } else {
            hipLaunchKernelGGL((gs2d_nhwc_kernel<T, I, P, A, false, PIX>), dim3((unsigned)blocks), dim3(kNhwcThreads),
                               0, stream, (const T*)a.x, (const T*)a.grid, (T*)a.y, total, (int32_t)a.C,
                               (int32_t)a.Hin, (int32_t)a.Win, a.Hout * a.Wout, shift, -0.0f);
        }
        return hipGetLastError();
    }
};

}  // namespace

hipError_t run_gs2d_nhwc(const GridSamplerArgs& a, hipStream_t stream)
{
    return dispatch_elem(a, NhwcLauncher{a, stream});
}

}  // namespace opscv
