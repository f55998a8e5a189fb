// Backward of grid_sampler2d for gfx950: gradient of the input (scatter) and of the grid, both deterministic.
//
// Replaces the reference device kernels
//   image/grid_sampler2_d_grad/op_kernel/arch35/grid_sampler2_d_grad_simt_det.h (deterministic mode) and
//   image/grid_sampler2_d_grad/op_kernel/arch35/grid_sampler2_d_grad_simt.h      (atomic mode).
//
// Gradient of the input.  The reference's deterministic mode walks the grid points of one batch item in chunks of
// 256; within a chunk it adds, tap after tap (nw, ne, sw, se; or the 16 bicubic taps in index order), the 256
// contributions one by one in point order, each add rounding to the tensor's element type
// (grid_sampler2_d_grad_simt_det.h:75-101).  The sum that reaches one element of the gradient is therefore a fixed
// sequence: its contributions ordered by (chunk, tap, point).  Adds to different elements commute, so only that
// per-element order has to be kept.  Here a workgroup owns one (batch item, group of channels, band of the plane):
// the band of every channel of the group lives in LDS, the workgroup walks the chunks in order and, inside a chunk,
// the taps in order.  The contributions of one tap that land on the same element are applied in rounds: an LDS
// max-reduction elects, per element, the waiting contribution of the lowest point; the elected ones are added (to
// every channel's plane) and retire.  Distinct points of a chunk rarely share a corner texel, so a tap mostly needs
// a single round with all lanes at work.  The result does not depend on scheduling and equals the sequential order
// above bit for bit.
//
// Gradient of the grid.  One lane per grid point walks the channels in order, as the reference does
// (grid_sampler2_d_grad_simt_det.h:103-196,279-343); no atomics are involved.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "gs2d_grad_math.hpp"
#include "kernels.hpp"

namespace opscv {

namespace {

constexpr int kThreads = 256;         // also the chunk length of the accumulation order
constexpr uint32_t kKeyBits = 8;      // 256 points of a chunk
constexpr uint32_t kEpochMax = (1u << (32 - kKeyBits)) - 1;
constexpr int kTagsMax = 1024;        // election tags of a band

// Tag of a band element.  Elements that share a tag are elected as if they were one; folding the high bits in keeps
// neighbours along every axis (offsets 1, W, H * W, often powers of two) on different tags.
__device__ __forceinline__ int32_t tag_of(int32_t off, int32_t tag_mask)
{
    return (off ^ (off >> 10)) & tag_mask;
}

// What a tap adds: the incoming gradient times the tap weight, rounded to fp32 and then to the element type (two
// roundings, as the reference's float product followed by a cast).  The fp32 value is pinned in a register: left
// alone, the compiler merges product and conversion into one instruction that rounds once, which differs on ties.
template <typename T, int INTERP>
__device__ __forceinline__ float contribution(float go, float w)
{
    if (INTERP == 1) {
        return rt<T>(go);
    }
    return rt<T>(as_fp32_value(INTERP == 0 ? w * go : go * w));
}

struct GradParams {
    int32_t C, H, W, Ho, Wo;
    int32_t pad, align;
    int32_t band_px;  // plane elements per workgroup (dx kernel)
    int32_t tags;     // election tags of the dx kernel, a power of two (tag_of)
};

// CB channels of one batch item per workgroup: the grid points, their taps and the election of a round are the
// same for every channel, only the values added differ, so that work is shared by the CB planes held in LDS.
template <typename T, int INTERP, int CB>
__global__ __launch_bounds__(kThreads) void gs2d_grad_input_kernel(const T* __restrict__ gout,
                                                                    const T* __restrict__ grid, T* __restrict__ dx,
                                                                    GradParams p)
{
    using Taps = GradTaps<T, INTERP>;
    constexpr int NT = Taps::NT;
    extern __shared__ uint32_t smem_u32[];
    __shared__ uint32_t s_flag[2];
    uint32_t* owner = smem_u32;
    T* planes = reinterpret_cast<T*>(smem_u32 + p.tags);  // [CB][band_px], values already in the element type
    const int32_t tag_mask = p.tags - 1;

    const int t = threadIdx.x;
    const int32_t plane_px = p.H * p.W;
    const int32_t b0 = blockIdx.x * p.band_px;
    const int32_t b1 = (b0 + p.band_px < plane_px) ? b0 + p.band_px : plane_px;
    const int32_t c0 = blockIdx.y * CB;
    const int32_t nc = (c0 + CB <= p.C) ? CB : p.C - c0;
    const int64_t n = blockIdx.z;
    for (int32_t i = t; i < p.tags; i += kThreads) {
        owner[i] = 0u;
    }
    for (int32_t i = t; i < b1 - b0; i += kThreads) {
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            ElemIO<T>::store(planes + cb * p.band_px + i, 0.0f);
        }
    }
    if (t == 0) {
        s_flag[0] = s_flag[1] = 0u;
    }
    __syncthreads();
    const int32_t points = p.Ho * p.Wo;
    const T* g_n = grid + n * (int64_t)points * 2;
    const T* go_n = gout + (n * p.C + c0) * (int64_t)points;
    uint32_t epoch = 1;
    int fl = 0;
    // the grid point and incoming gradients of the next chunk are requested before the rounds of this one
    float gx_next = 0.0f, gy_next = 0.0f, go_next[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        go_next[cb] = 0.0f;
    }
    auto request = [&](int32_t pt) {
        gx_next = ElemIO<T>::load(g_n + 2 * (int64_t)pt);
        gy_next = ElemIO<T>::load(g_n + 2 * (int64_t)pt + 1);
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            if (cb < nc) {
                go_next[cb] = ElemIO<T>::load(go_n + (int64_t)cb * points + pt);
            }
        }
    };
    if (t < points) {
        request(t);
    }
    for (int32_t base = 0; base < points; base += kThreads) {
        const int32_t pt = base + t;
        const float gx = gx_next, gy = gy_next;
        float go[CB];
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            go[cb] = go_next[cb];
        }
        if (pt + kThreads < points) {
            request(pt + kThreads);
        }
        int32_t off[NT];
        float wt[NT];
        uint32_t pend = 0;
        if (pt < points) {
            Taps tp;
            decide_grad_taps<T, INTERP>(tp, gx, gy, p.H, p.W, p.pad, p.align);
#pragma unroll
            for (int k = 0; k < NT; k++) {
                off[k] = tp.off[k] - b0;
                wt[k] = tp.w[k];
                if (tp.off[k] >= b0 && tp.off[k] < b1) {
                    pend |= 1u << k;
                }
            }
        }
        // Tap after tap, as the order demands.  Contributions of one tap rarely collide (two grid points of a chunk
        // with the same corner texel), so a tap usually takes one round in which every lane is busy.  A flag word
        // holds the number of the last round for which a contribution of tap k is still waiting; round numbers only
        // grow, so a stale value never matches.
        if (epoch > kEpochMax - 2u * NT * kThreads) {  // uniform: start the election tags over
            __syncthreads();
            for (int32_t i = t; i < p.tags; i += kThreads) {
                owner[i] = 0u;
            }
            if (t == 0) {
                s_flag[0] = s_flag[1] = 0u;
            }
            epoch = 1;
            __syncthreads();
        }
#pragma unroll
        for (int k = 0; k < NT; k++) {
            bool waiting = (pend & (1u << k)) != 0;
            fl ^= 1;  // the other flag than the tap before: its last readers are behind this tap's first barrier
            if (waiting) {
                s_flag[fl] = epoch;
            }
            __syncthreads();
            while (s_flag[fl] == epoch) {
                const uint32_t key = (epoch << kKeyBits) | (uint32_t)(kThreads - 1 - t);
                if (waiting) {
                    atomicMax(&owner[tag_of(off[k], tag_mask)], key);
                }
                __syncthreads();
                if (waiting) {
                    if (owner[tag_of(off[k], tag_mask)] == key) {
                        // the contribution is rounded to the element type before it is added, and so is the sum
                        T* e = planes + off[k];
                        if (nc == CB) {
                            // all planes read before any is written: the channels' updates overlap
                            float cur[CB];
#pragma unroll
                            for (int cb = 0; cb < CB; cb++) {
                                cur[cb] = ElemIO<T>::load(e + cb * p.band_px);
                            }
#pragma unroll
                            for (int cb = 0; cb < CB; cb++) {
                                const float val =
                                    contribution<T, INTERP>(go[cb], wt[k]);
                                ElemIO<T>::store(e + cb * p.band_px, cur[cb] + val);
                            }
                        } else {
#pragma unroll
                            for (int cb = 0; cb < CB; cb++) {
                                if (cb < nc) {
                                    const float val =
                                        contribution<T, INTERP>(go[cb], wt[k]);
                                    ElemIO<T>::store(e + cb * p.band_px, ElemIO<T>::load(e + cb * p.band_px) + val);
                                }
                            }
                        }
                        waiting = false;
                    } else {
                        s_flag[fl] = epoch + 1;  // somebody is left for the next round
                    }
                }
                __syncthreads();
                epoch++;
            }
            epoch++;
        }
    }
    __syncthreads();
    for (int cb = 0; cb < nc; cb++) {
        T* dx_nc = dx + (n * p.C + c0 + cb) * (int64_t)plane_px + b0;
        const T* pl = planes + cb * p.band_px;
        for (int32_t i = t; i < b1 - b0; i += kThreads) {
            dx_nc[i] = pl[i];
        }
    }
}

template <typename T, int INTERP>
__global__ __launch_bounds__(kThreads) void gs2d_grad_grid_kernel(const T* __restrict__ gout, const T* __restrict__ x,
                                                                   const T* __restrict__ grid, T* __restrict__ dgrid,
                                                                   int64_t total, GradParams p, int32_t blocks_per_item)
{
    using Taps = GradTaps<T, INTERP>;
    // blocks_per_item > 0: workgroups are handed to the 8 XCDs round-robin by index; all workgroups of one batch item
    // go to one XCD, so that the planes of that item (every lane walks all of them) are fetched into one L2 once
    // instead of into all eight (fp16 N16 C256 64x64: 185.6 MB fetched for 67.1 MB of operands otherwise).  The launch
    // plan asks for it when the items divide evenly among the XCDs and the workgroups evenly among the items.
    uint32_t block = blockIdx.x;
    if (blocks_per_item > 0) {
        const uint32_t xcd = blockIdx.x & 7u, i = blockIdx.x >> 3;
        block = ((i / (uint32_t)blocks_per_item) * 8u + xcd) * (uint32_t)blocks_per_item + i % (uint32_t)blocks_per_item;
    }
    const int64_t idx = (int64_t)block * kThreads + threadIdx.x;
    if (idx >= total) {
        return;
    }
    const int32_t points = p.Ho * p.Wo;
    const int64_t n = idx / points;
    const int32_t pt = (int32_t)(idx - n * points);
    if (INTERP == 1) {
        ElemIO<T>::store(dgrid + 2 * idx, 0.0f);
        ElemIO<T>::store(dgrid + 2 * idx + 1, 0.0f);
        return;
    }
    Taps tp;
    decide_grad_taps<T, INTERP>(tp, ElemIO<T>::load(grid + 2 * idx), ElemIO<T>::load(grid + 2 * idx + 1), p.H, p.W,
                                p.pad, p.align);
    const int32_t plane_px = p.H * p.W;
    const T* x_n = x + n * p.C * (int64_t)plane_px;
    const T* go_n = gout + n * p.C * (int64_t)points + pt;
    float gix = 0.0f, giy = 0.0f;
    if (INTERP == 0) {
        const float dxe = (float)(tp.x0 == INT32_MAX ? tp.x0 : tp.x0 + 1) - tp.fx, dxw = tp.fx - (float)tp.x0;
        const float dys = (float)(tp.y0 == INT32_MAX ? tp.y0 : tp.y0 + 1) - tp.fy, dyn = tp.fy - (float)tp.y0;
        // The sums run over the channels in order; the loads do not depend on them, so they are issued a group of
        // channels ahead (a lane has one grid point and would otherwise wait out every load in turn).
        constexpr int U = 8;
        const bool ok0 = tp.off[0] >= 0, ok1 = tp.off[1] >= 0, ok2 = tp.off[2] >= 0, ok3 = tp.off[3] >= 0;
        const int32_t o0 = ok0 ? tp.off[0] : 0, o1 = ok1 ? tp.off[1] : 0, o2 = ok2 ? tp.off[2] : 0,
                      o3 = ok3 ? tp.off[3] : 0;
        auto accumulate = [&](float go, float v0, float v1, float v2, float v3) {
            if (ok0) {
                gix -= v0 * dys * go;
                giy -= v0 * dxe * go;
            }
            if (ok1) {
                gix += v1 * dys * go;
                giy -= v1 * dxw * go;
            }
            if (ok2) {
                gix -= v2 * dyn * go;
                giy += v2 * dxe * go;
            }
            if (ok3) {
                gix += v3 * dyn * go;
                giy += v3 * dxw * go;
            }
        };
        int32_t c = 0;
        if (p.W >= 2) {
            // The west and east corner of a row are neighbours in memory: one load of two elements (aligned to one
            // element only) per row instead of two loads halves the addresses the gather puts through the memory
            // pipeline.  The pair sits at column pb = clamp(x0, 0, W - 2), so it never leaves the row; which half is
            // which corner follows from pb.  Corners outside the image are skipped by accumulate() as before.
            using PairBits = typename std::conditional<sizeof(T) == 2, uint32_t, uint64_t>::type;
            const int32_t x0 = tp.x0, x1 = (tp.x0 == INT32_MAX) ? tp.x0 : tp.x0 + 1;
            const int32_t y1 = (tp.y0 == INT32_MAX) ? tp.y0 : tp.y0 + 1;
            const int32_t pb = (x0 < 0) ? 0 : ((x0 > p.W - 2) ? p.W - 2 : x0);
            const bool lo_w = (x0 == pb), lo_e = (x1 == pb);
            const int32_t r0 = (tp.y0 >= 0 && tp.y0 < p.H) ? tp.y0 * p.W + pb : 0;
            const int32_t r1 = (y1 >= 0 && y1 < p.H) ? y1 * p.W + pb : 0;
            for (; c + U <= p.C; c += U) {
                float go[U];
                PairBits north[U], south[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const T* xc = x_n + (int64_t)(c + u) * plane_px;
                    go[u] = ElemIO<T>::load(go_n + (int64_t)(c + u) * points);
                    __builtin_memcpy(&north[u], xc + r0, sizeof(PairBits));
                    __builtin_memcpy(&south[u], xc + r1, sizeof(PairBits));
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    T n2[2], s2[2];
                    __builtin_memcpy(n2, &north[u], sizeof(PairBits));
                    __builtin_memcpy(s2, &south[u], sizeof(PairBits));
                    const float nlo = ElemIO<T>::load(&n2[0]), nhi = ElemIO<T>::load(&n2[1]);
                    const float slo = ElemIO<T>::load(&s2[0]), shi = ElemIO<T>::load(&s2[1]);
                    accumulate(go[u], lo_w ? nlo : nhi, lo_e ? nlo : nhi, lo_w ? slo : shi, lo_e ? slo : shi);
                }
            }
        }
        for (; c + U <= p.C; c += U) {
            float go[U], v[U][4];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const T* xc = x_n + (int64_t)(c + u) * plane_px;
                go[u] = ElemIO<T>::load(go_n + (int64_t)(c + u) * points);
                v[u][0] = ElemIO<T>::load(xc + o0);
                v[u][1] = ElemIO<T>::load(xc + o1);
                v[u][2] = ElemIO<T>::load(xc + o2);
                v[u][3] = ElemIO<T>::load(xc + o3);
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                accumulate(go[u], v[u][0], v[u][1], v[u][2], v[u][3]);
            }
        }
        for (; c < p.C; c++) {
            const T* xc = x_n + (int64_t)c * plane_px;
            accumulate(ElemIO<T>::load(go_n + (int64_t)c * points), ElemIO<T>::load(xc + o0),
                       ElemIO<T>::load(xc + o1), ElemIO<T>::load(xc + o2), ElemIO<T>::load(xc + o3));
        }
    } else {
        const float xf = __builtin_floorf(tp.fx), yf = __builtin_floorf(tp.fy);
        float cx[4], cy[4], cxg[4], cyg[4];
        cubic_coefficients(cy, tp.fy - yf);
        cubic_coefficients(cx, tp.fx - xf);
        cubic_coefficients_grad(cyg, tp.fy - yf);
        cubic_coefficients_grad(cxg, tp.fx - xf);
        for (int32_t c = 0; c < p.C; c++) {
            const float go = ElemIO<T>::load(go_n + (int64_t)c * points);
            const T* xc = x_n + (int64_t)c * plane_px;
#pragma unroll
            for (int i = 0; i < 4; i++) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int32_t o = tp.off[i * 4 + j];
                    const float v = (o >= 0) ? ElemIO<T>::load(xc + o) : 0.0f;
                    giy += v * cyg[j] * cx[i] * go;
                    gix += v * cxg[i] * cy[j] * go;
                }
            }
        }
    }
    // products in fp32 first, then the conversion (see contribution())
    ElemIO<T>::store(dgrid + 2 * idx, as_fp32_value(tp.mx * gix));
    ElemIO<T>::store(dgrid + 2 * idx + 1, as_fp32_value(tp.my * giy));
}

template <typename T, int INTERP>
hipError_t launch_interp(const GridSamplerGradArgs& a, hipStream_t stream)
{
    GradParams p;
    p.C = (int32_t)a.C;
    p.H = (int32_t)a.Hin;
    p.W = (int32_t)a.Win;
    p.Ho = (int32_t)a.Hout;
    p.Wo = (int32_t)a.Wout;
    p.pad = a.pad;
    p.align = a.align;
    const int64_t plane_px = a.Hin * a.Win;
    // bands of at most 4096 plane elements: election tags (4 bytes each) plus the planes of a channel group
    p.band_px = (int32_t)(plane_px < 4096 ? plane_px : 4096);
    // Elements that share a tag are elected as if they were one: never out of order, at worst a round more (they lie
    // 1024 elements apart, which a chunk of a smooth grid does not span).  1024 tags instead of one per element bring
    // the LDS of a workgroup from 48 KB to 36 KB, four workgroups per compute unit instead of three: the 1024
    // workgroups of the backward of C3 run side by side instead of in two turns (175 -> 127 us).
    p.tags = 64;
    while (p.tags < p.band_px && p.tags < kTagsMax) {
        p.tags *= 2;
    }
    // The grid gradient's LDS-ring kernel goes first where it runs: on its way it zeroes the words that the list
    // variant of the input gradient wants zeroed, which saves that one a launch (4.7 us).  Whichever of the two reads
    // gradOutput first reads it from HBM and leaves it in the last-level cache for the other; the grid gradient's
    // kernel loses more by going first (3.7 us) than the list variant's last kernel gains (1 us), still a net gain.
    bool dx_done = false, dgrid_done = false;
    if (INTERP == 0) {
        GradClear clear{};
        const bool lists = gs2d_grad_csr_clear(a, &clear);
        hipError_t e = run_gs2d_grad_grid_lds(a, stream, &dgrid_done, lists ? &clear : nullptr);
        if (e != hipSuccess) {
            return e;
        }
        if (lists) {
            e = run_gs2d_grad_input_csr(a, stream, &dx_done, dgrid_done);
            if (e != hipSuccess) {
                return e;
            }
        }
    }
    if (a.dx != nullptr && !dx_done) {
        const int64_t bands = (plane_px + p.band_px - 1) / p.band_px;
        // 8 bytes of planes per band element: 4 channels of a 16-bit type, 2 of fp32 (48 KB of LDS with the tags, three
        // workgroups per compute unit); fewer channels than that run one per workgroup
        constexpr int CBMAX = 8 / (int)sizeof(T);
        const bool grouped = a.C >= CBMAX;
        const int64_t cgroups = grouped ? (a.C + CBMAX - 1) / CBMAX : a.C;
        if (bands > INT32_MAX || cgroups > 65535 || a.N > 65535) {
            return hipErrorInvalidValue;
        }
        const dim3 grid((unsigned)bands, (unsigned)cgroups, (unsigned)a.N);
        static std::atomic<uint32_t> lds_allowed{0};  // more than the default 64 KB of dynamic LDS may be asked for
        const hipError_t ea =
            allow_dynamic_lds(reinterpret_cast<const void*>(gs2d_grad_input_kernel<T, INTERP, CBMAX>),
                              kTagsMax * 4 + 4096 * CBMAX * (int)sizeof(T), lds_allowed);
        if (ea != hipSuccess) {
            return ea;
        }
        if (grouped) {
            hipLaunchKernelGGL((gs2d_grad_input_kernel<T, INTERP, CBMAX>), grid, dim3(kThreads),
                               (size_t)p.tags * 4 + (size_t)p.band_px * CBMAX * sizeof(T), stream, (const T*)a.gout,
                               (const T*)a.grid, (T*)a.dx, p);
        } else {
            hipLaunchKernelGGL((gs2d_grad_input_kernel<T, INTERP, 1>), grid, dim3(kThreads),
                               (size_t)p.tags * 4 + (size_t)p.band_px * sizeof(T), stream, (const T*)a.gout,
                               (const T*)a.grid, (T*)a.dx, p);
        }
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            return e;
        }
    }
    if (a.dgrid != nullptr && !dgrid_done) {
        const int64_t total = a.N * a.Hout * a.Wout;
        const int64_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > INT32_MAX) {
            return hipErrorInvalidValue;
        }
        const int64_t points = a.Hout * a.Wout;
        const int32_t blocks_per_item =
            (points % kThreads == 0 && a.N % 8 == 0 && points / kThreads <= INT32_MAX) ? (int32_t)(points / kThreads) : 0;
        hipLaunchKernelGGL((gs2d_grad_grid_kernel<T, INTERP>), dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                           (const T*)a.gout, (const T*)a.x, (const T*)a.grid, (T*)a.dgrid, total, p, blocks_per_item);
        return hipGetLastError();
    }
    return hipSuccess;
}

template <typename T>
hipError_t launch_typed(const GridSamplerGradArgs& a, hipStream_t stream)
{
    switch (a.interp) {
        case 0: return launch_interp<T, 0>(a, stream);
        case 1: return launch_interp<T, 1>(a, stream);
        case 2: return launch_interp<T, 2>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t launch_grid_sampler2d_grad(const GridSamplerGradArgs& a, hipStream_t stream)
{
    if (a.gout == nullptr || a.x == nullptr || a.grid == nullptr || (a.dx == nullptr && a.dgrid == nullptr)) {
        return hipErrorInvalidValue;
    }
    if (a.pad < 0 || a.pad > 2 || a.N <= 0 || a.C <= 0 || a.Hin <= 0 || a.Win <= 0 || a.Hout <= 0 || a.Wout <= 0) {
        return hipErrorInvalidValue;
    }
    if (a.Hin * a.Win > INT32_MAX || a.Hout * a.Wout > INT32_MAX - 1024) {
        return hipErrorInvalidValue;
    }
    switch (a.elem) {
        case Elem::F32: return launch_typed<float>(a, stream);
        case Elem::F16: return launch_typed<_Float16>(a, stream);
        case Elem::BF16: return launch_typed<__bf16>(a, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
