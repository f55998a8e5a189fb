// Grid sampler 2-D forward, LDS-staged variant for gfx950.
//
// Same arithmetic as the direct variant (see sampler_math.hpp; reference kernel
// image/grid_sampler2_d/op_kernel/arch35/grid_sampler2_d_simt.h:461-514), different data movement:
//
//   * a workgroup owns (batch n, a tile of THREADS*PPT output pixels, a range of channels);
//   * every lane decides its PPT pixels once -- four LDS byte offsets and four weights per pixel stay in
//     registers for the whole channel range;
//   * the channel range is walked in stages of CGS whole input planes: the planes are streamed from HBM into
//     LDS with coalesced 16-byte loads (each input element is read from memory once per workgroup), then every
//     tap is a 2- or 4-byte LDS read, so the scattered part of the gather never leaves the CU;
//   * a tap outside the image points at a 16-byte slot of zeros behind each staged plane, which reproduces the
//     reference's "skip the tap" exactly (0 * w adds nothing) without per-channel selects;
//   * every output channel plane is written once, 64 consecutive pixels per wavefront store.
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "gs2d_common.hpp"
#include "sampler_math.hpp"

namespace opscv {

namespace {

constexpr int kLdsLimit = 160 * 1024;  // LDS bytes per CU on gfx950

__host__ __device__ constexpr uint32_t round_up16(uint32_t v) { return (v + 15u) & ~15u; }

template <typename T>
__device__ __forceinline__ void load_grid_pair(const T* gp, bool pair_aligned, float* gx, float* gy)
{
    if constexpr (sizeof(T) == 2) {
        if (pair_aligned) {
            const uint32_t raw = *reinterpret_cast<const uint32_t*>(gp);
            T lo = __builtin_bit_cast(T, (uint16_t)(raw & 0xFFFFu));
            T hi = __builtin_bit_cast(T, (uint16_t)(raw >> 16));
            *gx = ElemIO<T>::load(&lo);
            *gy = ElemIO<T>::load(&hi);
            return;
        }
    } else {
        if (pair_aligned) {
            const float2 raw = *reinterpret_cast<const float2*>(gp);
            *gx = raw.x;
            *gy = raw.y;
            return;
        }
    }
    *gx = ElemIO<T>::load(gp);
    *gy = ElemIO<T>::load(gp + 1);
}

// PITCH: compile-time byte distance between staged planes in LDS (>= padded plane size + 16); with CGS == 1 it
// is unused.  Compile-time so that the per-channel LDS address is "tap offset + immediate".
template <typename T, int INTERP, int PAD, bool ALIGN, int THREADS, int PPT, int CGS, int PITCH>
__global__ __launch_bounds__(THREADS) void gs2d_lds_kernel(const T* __restrict__ x, const T* __restrict__ grid,
                                                           T* __restrict__ y, int32_t C, int32_t H, int32_t W,
                                                           int32_t out_plane, uint32_t tiles_per_n,
                                                           uint32_t cblocks, int32_t chans_per_block,
                                                           int32_t vec_ok, int32_t pair_aligned)
{
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    constexpr int NT = (INTERP == 0) ? 4 : 1;
    const int tid = threadIdx.x;

    uint32_t b = blockIdx.x;
    const uint32_t tile = b % tiles_per_n;
    b /= tiles_per_n;
    const uint32_t cb = b % cblocks;
    const uint32_t n = b / cblocks;

    const int32_t plane_elems = H * W;
    const uint32_t plane_bytes = (uint32_t)plane_elems * (uint32_t)sizeof(T);
    const uint32_t zero_off = round_up16(plane_bytes);
    const int32_t c_begin = (int32_t)cb * chans_per_block;
    const int32_t c_end = (c_begin + chans_per_block < C) ? c_begin + chans_per_block : C;

    // the zero slots behind each staged plane; stage copies never touch them
    if (tid < CGS * 4) {
        reinterpret_cast<uint32_t*>(lds + (tid >> 2) * PITCH + zero_off)[tid & 3] = 0u;
    }

    // ---- per-pixel decisions, once for the whole channel range ----
    uint32_t toff[PPT][NT];
    float tw[PPT][4];
    bool valid[PPT];
    int32_t pixel[PPT];
#pragma unroll
    for (int j = 0; j < PPT; j++) {
        const int32_t pix = (int32_t)tile * (THREADS * PPT) + j * THREADS + tid;
        valid[j] = pix < out_plane;
        const int32_t pc = valid[j] ? pix : out_plane - 1;
        pixel[j] = pc;
        float gx, gy;
        load_grid_pair<T>(grid + ((int64_t)n * out_plane + pc) * 2, pair_aligned != 0, &gx, &gy);
        const PixelTap t = decide_pixel<INTERP, PAD, ALIGN>(gx, gy, H, W);
        if (INTERP == 0) {
            const int32_t x0 = t.x0, y0 = t.y0;
            const int32_t x1 = (x0 == INT32_MAX) ? x0 : x0 + 1;
            const int32_t y1 = (y0 == INT32_MAX) ? y0 : y0 + 1;
            const bool in_nw = within(y0, x0, H, W), in_ne = within(y0, x1, H, W);
            const bool in_sw = within(y1, x0, H, W), in_se = within(y1, x1, H, W);
            const uint32_t uw = (uint32_t)W, es = (uint32_t)sizeof(T);
            toff[j][0] = in_nw ? ((uint32_t)y0 * uw + (uint32_t)x0) * es : zero_off;
            toff[j][1] = in_ne ? ((uint32_t)y0 * uw + (uint32_t)x1) * es : zero_off;
            toff[j][2] = in_sw ? ((uint32_t)y1 * uw + (uint32_t)x0) * es : zero_off;
            toff[j][3] = in_se ? ((uint32_t)y1 * uw + (uint32_t)x1) * es : zero_off;
            tw[j][0] = t.w[0];
            tw[j][1] = t.w[1];
            tw[j][2] = t.w[2];
            tw[j][3] = t.w[3];
            if (t.flag) {
                // non-finite source coordinate: every channel becomes NaN (0 * NaN), as the reference writes
                toff[j][0] = toff[j][1] = toff[j][2] = toff[j][3] = zero_off;
                tw[j][0] = __builtin_nanf("");
            }
        } else {
            const bool in = within(t.y0, t.x0, H, W);
            toff[j][0] = in ? ((uint32_t)t.y0 * (uint32_t)W + (uint32_t)t.x0) * (uint32_t)sizeof(T) : zero_off;
            tw[j][0] = tw[j][1] = tw[j][2] = tw[j][3] = 0.0f;
        }
    }

    const T* xn = x + (int64_t)n * C * plane_elems;
    T* yn = y + (int64_t)n * C * out_plane;

    for (int32_t c0 = c_begin; c0 < c_end; c0 += CGS) {
        const int32_t nch = (c_end - c0 < CGS) ? c_end - c0 : CGS;
        __syncthreads();  // readers of the previous stage are done (and the zero slots are visible)
        if (vec_ok) {
            const uint4* src = reinterpret_cast<const uint4*>(xn + (int64_t)c0 * plane_elems);
            const uint32_t vpp = plane_bytes >> 4;
#pragma unroll
            for (int k = 0; k < CGS; k++) {
                if (k < nch) {
                    uint4* dst = reinterpret_cast<uint4*>(lds + k * PITCH);
                    for (uint32_t i = tid; i < vpp; i += THREADS) {
                        dst[i] = src[(uint32_t)k * vpp + i];
                    }
                }
            }
        } else {
            const T* src = xn + (int64_t)c0 * plane_elems;
#pragma unroll
            for (int k = 0; k < CGS; k++) {
                if (k < nch) {
                    T* dst = reinterpret_cast<T*>(lds + k * PITCH);
                    for (int32_t i = tid; i < plane_elems; i += THREADS) {
                        dst[i] = src[(int64_t)k * plane_elems + i];
                    }
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < CGS; k++) {
            if (k < nch) {
                const char* pl = lds + k * PITCH;
                T* yc = yn + (int64_t)(c0 + k) * out_plane;
#pragma unroll
                for (int j = 0; j < PPT; j++) {
                    if (INTERP == 0) {
                        // grid_sampler2_d_simt.h:321-338 : 0 + nw + ne + sw + se, products and sums rounded separately
                        float out = 0.0f;
                        out += ElemIO<T>::load(reinterpret_cast<const T*>(pl + toff[j][0])) * tw[j][0];
                        out += ElemIO<T>::load(reinterpret_cast<const T*>(pl + toff[j][1])) * tw[j][1];
                        out += ElemIO<T>::load(reinterpret_cast<const T*>(pl + toff[j][2])) * tw[j][2];
                        out += ElemIO<T>::load(reinterpret_cast<const T*>(pl + toff[j][3])) * tw[j][3];
                        if (valid[j]) {
                            ElemIO<T>::store(yc + pixel[j], out);
                        }
                    } else {
                        // grid_sampler2_d_simt.h:341-360 : value passes through fp32
                        const float out = ElemIO<T>::load(reinterpret_cast<const T*>(pl + toff[j][0]));
                        if (valid[j]) {
                            ElemIO<T>::store(yc + pixel[j], out);
                        }
                    }
                }
            }
        }
    }
}

// ---- host side: variant selection ----
struct LdsPlan {
    bool ok = false;
    int cls = 0;            // 0: pitch 2064 x8, 1: pitch 8208 x8, 2: pitch 32784 x2, 3: single plane
    int ppt = 8;
    uint32_t lds_bytes = 0;
    uint32_t tiles_per_n = 0, cblocks = 0;
    int32_t chans_per_block = 0;
    int cgs = 1;
};

constexpr int kThreads = 512;
constexpr int kPitch[3] = {2064, 8208, 32784};
constexpr int kCgs[4] = {8, 8, 2, 1};

LdsPlan make_plan(const GridSamplerArgs& a)
{
    LdsPlan p;
    const int64_t esz = elem_size(a.elem);
    const int64_t plane_bytes = a.Hin * a.Win * esz;
    const int64_t need = ((plane_bytes + 15) & ~(int64_t)15) + 16;
    const int64_t out_plane = a.Hout * a.Wout;
    if (out_plane > INT32_MAX || need > kLdsLimit - 1024) {
        return p;
    }
    if (need <= kPitch[0]) {
        p.cls = 0;
    } else if (need <= kPitch[1]) {
        p.cls = 1;
    } else if (need <= kPitch[2]) {
        p.cls = 2;
    } else {
        p.cls = 3;
    }
    p.cgs = kCgs[p.cls];
    p.lds_bytes = (p.cls == 3) ? (uint32_t)need : (uint32_t)(kPitch[p.cls] * p.cgs);
    p.ppt = (out_plane > 2 * kThreads) ? 8 : 2;
    const int64_t tile = (int64_t)kThreads * p.ppt;
    p.tiles_per_n = (uint32_t)((out_plane + tile - 1) / tile);
    // channels per workgroup: as many stages as possible (the pixel decisions are reused across them) while
    // still giving the 256 CUs at least two workgroups each
    const int64_t want_blocks = 512;
    int64_t base = a.N * p.tiles_per_n;
    int64_t cblocks = (want_blocks + base - 1) / base;
    const int64_t max_cblocks = (a.C + p.cgs - 1) / p.cgs;
    if (cblocks > max_cblocks) {
        cblocks = max_cblocks;
    }
    if (cblocks < 1) {
        cblocks = 1;
    }
    int64_t cpb = (a.C + cblocks - 1) / cblocks;
    cpb = (cpb + p.cgs - 1) / p.cgs * p.cgs;
    cblocks = (a.C + cpb - 1) / cpb;
    p.chans_per_block = (int32_t)cpb;
    p.cblocks = (uint32_t)cblocks;
    if (a.N * p.tiles_per_n * cblocks > INT32_MAX) {
        return p;
    }
    p.ok = true;
    return p;
}

template <typename T, int I, int P, bool A, int PPT, int CGS, int PITCH>
hipError_t launch_one(const GridSamplerArgs& a, const LdsPlan& p, hipStream_t stream)
{
    auto kernel = gs2d_lds_kernel<T, I, P, A, kThreads, PPT, CGS, PITCH>;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit);
        if (e != hipSuccess) {
            return e;
        }
        attr_set = true;
    }
    const int64_t esz = sizeof(T);
    const int64_t plane_bytes = a.Hin * a.Win * esz;
    const int vec_ok = (plane_bytes % 16 == 0) && (reinterpret_cast<uintptr_t>(a.x) % 16 == 0);
    const int pair_aligned = (reinterpret_cast<uintptr_t>(a.grid) % (2 * esz) == 0);
    const uint32_t blocks = (uint32_t)(a.N * p.tiles_per_n * p.cblocks);
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kThreads), p.lds_bytes, stream, (const T*)a.x, (const T*)a.grid,
                       (T*)a.y, (int32_t)a.C, (int32_t)a.Hin, (int32_t)a.Win, (int32_t)(a.Hout * a.Wout),
                       p.tiles_per_n, p.cblocks, p.chans_per_block, vec_ok, pair_aligned);
    return hipGetLastError();
}

template <typename T, int I, int P, bool A, int PPT>
hipError_t launch_class(const GridSamplerArgs& a, const LdsPlan& p, hipStream_t stream)
{
    switch (p.cls) {
        case 0: return launch_one<T, I, P, A, PPT, kCgs[0], kPitch[0]>(a, p, stream);
        case 1: return launch_one<T, I, P, A, PPT, kCgs[1], kPitch[1]>(a, p, stream);
        case 2: return launch_one<T, I, P, A, PPT, kCgs[2], kPitch[2]>(a, p, stream);
        default: return launch_one<T, I, P, A, PPT, 1, 0>(a, p, stream);
    }
}

struct LdsLauncher {
    const GridSamplerArgs& a;
    const LdsPlan& p;
    hipStream_t stream;
    template <typename T, int I, int P, bool A>
    hipError_t operator()() const
    {
        if (p.ppt == 8) {
            return launch_class<T, I, P, A, 8>(a, p, stream);
        }
        return launch_class<T, I, P, A, 2>(a, p, stream);
    }
};

}  // namespace

const char* gs2d_lds_variant_name(const GridSamplerArgs& a)
{
    const LdsPlan p = make_plan(a);
    if (!p.ok) {
        return nullptr;
    }
    static const char* names[4] = {"lds_planes_p2064x8", "lds_planes_p8208x8", "lds_planes_p32784x2",
                                   "lds_single_plane"};
    return names[p.cls];
}

hipError_t run_gs2d_lds(const GridSamplerArgs& a, hipStream_t stream, bool* handled)
{
    *handled = false;
    const LdsPlan p = make_plan(a);
    if (!p.ok) {
        return hipSuccess;
    }
    *handled = true;
    return dispatch_elem(a, LdsLauncher{a, p, stream});
}

}  // namespace opscv
