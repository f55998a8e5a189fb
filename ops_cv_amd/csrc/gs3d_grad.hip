// Backward of the 3-D grid sampler for gfx950: gradient of the input volume (scatter) and of the grid, deterministic.
//
// Replaces the reference device kernel
//   image/grid_sampler3_d_grad/op_kernel/arch35/grid_sampler3_d_grad_simt_det.h (deterministic mode)
// and, up to the order of additions, its atomic mode (grid_sampler3_d_grad_simt.h).
//
// Gradient of the input.  The reference gives a core whole batch items and walks their grid points as one run of
// indices in chunks of 256; within a chunk it adds, channel after channel and corner after corner (tnw, tne, tsw, tse,
// bnw, bne, bsw, bse), the 256 contributions one by one in point order, each add rounding to the element type
// (grid_sampler3_d_grad_simt_det.h:63-96).  The sum that reaches one voxel of the gradient is therefore a fixed
// sequence: its contributions ordered by (chunk, corner, point).  Adds to different voxels commute.  A workgroup here
// owns one (batch item, group of channels, band of the volume) held in LDS and walks the chunks in order; the
// contributions of a chunk that land on the same voxel are applied in rounds, an LDS max-reduction electing per voxel
// the waiting contribution of the lowest (corner, point).  When a core of the reference holds several batch
// items, the chunk boundaries of its later items are shifted by (item * points) mod 256
// (grid_sampler3_d_grad_tiling.cpp:183-191); `items_per_core` carries that.
//
// Gradient of the grid.  One lane per grid point walks the channels in order (grid_sampler3_d_grad_simt_det.h:
// 98-330); no atomics are involved.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "gs2d_grad_math.hpp"
#include "gs3d_grad_math.hpp"
#include "kernels.hpp"

namespace opscv {

namespace {

constexpr int kThreads = kChunkPoints3;  // a workgroup walks a chunk of the accumulation order, a lane per point
constexpr uint32_t kLaneBits = 8;              // 256 points of a chunk
constexpr uint32_t kKeyBits = kLaneBits + 3;   // ... times eight corners
constexpr uint32_t kEpochMax = (1u << (32 - kKeyBits)) - 1;
constexpr int kTagsMax = 4096;  // election tags of a band (bands of 8192 voxels share them in pairs: two workgroups per CU)
constexpr int kBandMax = 8192;  // most voxels of the gradient a workgroup keeps in LDS

// Tag of a band element.  Elements that share a tag are elected as if they were one; folding the high bits in keeps
// neighbours along every axis (offsets 1, W, H * W, often powers of two) on different tags.
__device__ __forceinline__ int32_t tag_of(int32_t off, int32_t tag_mask)
{
    return (off ^ (off >> 10)) & tag_mask;
}

// Per (batch item, chunk): lowest and highest voxel any corner of the chunk's points lands on (lowest > highest for a
// chunk with none).  One workgroup per chunk.
template <typename T, int INTERP>
__global__ __launch_bounds__(kThreads) void gs3d_grad_range_kernel(const T* __restrict__ grid,
                                                                    int32_t* __restrict__ ranges, Grad3Params p)
{
    using Taps = GradTaps3<T, INTERP>;
    __shared__ int32_t s_lo[kThreads / 64], s_hi[kThreads / 64];
    const int t = threadIdx.x;
    const int64_t n = blockIdx.y;
    const int32_t pt = -chunk_phase(n, p) + (int32_t)blockIdx.x * kThreads + t;
    int32_t lo = INT32_MAX, hi = -1;
    if (pt >= 0 && pt < p.points) {
        const T* g = grid + (n * (int64_t)p.points + pt) * 3;
        Taps tp;
        decide_grad_taps3<T, INTERP>(tp, ElemIO<T>::load(g), ElemIO<T>::load(g + 1), ElemIO<T>::load(g + 2), p.D, p.H,
                                     p.W, p.pad, p.align);
#pragma unroll
        for (int k = 0; k < Taps::NT; k++) {
            if (tp.off[k] >= 0) {
                lo = tp.off[k] < lo ? tp.off[k] : lo;
                hi = tp.off[k] > hi ? tp.off[k] : hi;
            }
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const int32_t olo = __shfl_xor(lo, d), ohi = __shfl_xor(hi, d);
        lo = olo < lo ? olo : lo;
        hi = ohi > hi ? ohi : hi;
    }
    if ((t & 63) == 0) {
        s_lo[t >> 6] = lo;
        s_hi[t >> 6] = hi;
    }
    __syncthreads();
    if (t == 0) {
#pragma unroll
        for (int w = 1; w < kThreads / 64; w++) {
            lo = s_lo[w] < lo ? s_lo[w] : lo;
            hi = s_hi[w] > hi ? s_hi[w] : hi;
        }
        int32_t* r = ranges + (n * (int64_t)p.chunks + blockIdx.x) * 2;
        r[0] = lo;
        r[1] = hi;
    }
}

template <typename T, int INTERP, int CB>
__global__ __launch_bounds__(kThreads) void gs3d_grad_input_kernel(const T* __restrict__ gout,
                                                                    const T* __restrict__ grid, T* __restrict__ dx,
                                                                    const int32_t* __restrict__ ranges, Grad3Params p,
                                                                    const uint32_t* __restrict__ item_flags,
                                                                    uint32_t flag_stride)
{
    // with item flags: only the items the gather variant left over (the same answer for the whole workgroup)
    if (item_flags != nullptr && item_flags[(size_t)blockIdx.z * flag_stride] == 0u) {
        return;
    }
    using Taps = GradTaps3<T, INTERP>;
    constexpr int NT = Taps::NT;
    extern __shared__ uint32_t smem_u32[];
    __shared__ uint32_t s_flag[2];
    uint32_t* owner = smem_u32;
    T* planes = reinterpret_cast<T*>(smem_u32 + p.tags);  // [CB][band_px], values already in the element type
    const int32_t tag_mask = p.tags - 1;

    const int t = threadIdx.x;
    const int32_t vol = p.D * p.H * p.W;
    const int32_t b0 = blockIdx.x * p.band_px;
    const int32_t b1 = (b0 + p.band_px < vol) ? b0 + p.band_px : vol;
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
    const int32_t points = p.points;
    const T* g_n = grid + n * (int64_t)points * 3;
    const T* go_n = gout + (n * p.C + c0) * (int64_t)points;
    uint32_t epoch = 1;
    int fl = 0;
    // the grid point and incoming gradients of the next chunk are requested before the rounds of this one
    float gx_next = 0.0f, gy_next = 0.0f, gz_next = 0.0f, go_next[CB];
#pragma unroll
    for (int cb = 0; cb < CB; cb++) {
        go_next[cb] = 0.0f;
    }
    auto request = [&](int32_t pt) {
        gx_next = ElemIO<T>::load(g_n + 3 * (int64_t)pt);
        gy_next = ElemIO<T>::load(g_n + 3 * (int64_t)pt + 1);
        gz_next = ElemIO<T>::load(g_n + 3 * (int64_t)pt + 2);
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            if (cb < nc) {
                go_next[cb] = ElemIO<T>::load(go_n + (int64_t)cb * points + pt);
            }
        }
    };
    const int32_t first = -chunk_phase(n, p);
    // Chunks whose voxel span misses this band are passed over (the spans come from gs3d_grad_range_kernel; without
    // them every chunk is looked at).  The choice is the same for the whole workgroup.
    const int32_t* rng_n = (ranges != nullptr) ? ranges + n * 2 * (int64_t)p.chunks : nullptr;
    auto next_busy = [&](int32_t ci) {
        if (rng_n != nullptr) {
            while (ci < p.chunks && (rng_n[2 * ci + 1] < b0 || rng_n[2 * ci] >= b1)) {
                ci++;
            }
        }
        return ci;
    };
    auto request_chunk = [&](int32_t ci) {
        const int32_t pt = first + ci * kThreads + t;
        if (ci < p.chunks && pt >= 0 && pt < points) {
            request(pt);
        }
    };
    int32_t ci = next_busy(0);
    request_chunk(ci);
    while (ci < p.chunks) {
        const int32_t pt = first + ci * kThreads + t;
        const float gx = gx_next, gy = gy_next, gz = gz_next;
        float go[CB];
#pragma unroll
        for (int cb = 0; cb < CB; cb++) {
            go[cb] = go_next[cb];
        }
        ci = next_busy(ci + 1);
        request_chunk(ci);
        int32_t off[NT];
        float wt[NT];
        uint32_t pend = 0;
        if (pt >= 0 && pt < points) {
            Taps tp;
            decide_grad_taps3<T, INTERP>(tp, gx, gy, gz, p.D, p.H, p.W, p.pad, p.align);
#pragma unroll
            for (int k = 0; k < NT; k++) {
                off[k] = tp.off[k] - b0;
                wt[k] = tp.w[k];
                if (tp.off[k] >= b0 && tp.off[k] < b1) {
                    pend |= 1u << k;
                }
            }
        }
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
        // All corners of the chunk take part in one election: per voxel the waiting contribution with the lowest
        // (corner, point) wins the round, is added and retires, so a voxel receives its contributions in the order
        // corner after corner, point after point, and a chunk takes as many rounds as its busiest voxel has
        // contributions (mostly one or two) instead of at least one per corner.  The corners of one point are
        // different voxels, so a lane may win several of them in a round.  A flag word holds the number of the last
        // round for which a contribution is still waiting; round numbers only grow, so a stale value never matches.
        // A chunk none of whose points touches this band costs one barrier.
        fl ^= 1;  // the other flag than the chunk before: its last readers are behind this chunk's first barrier
        if (pend != 0) {
            s_flag[fl] = epoch;
        }
        __syncthreads();
        while (s_flag[fl] == epoch) {
            const uint32_t key = (epoch << kKeyBits) | (uint32_t)(kThreads - 1 - t);
#pragma unroll
            for (int k = 0; k < NT; k++) {
                if (pend & (1u << k)) {
                    atomicMax(&owner[tag_of(off[k], tag_mask)], key | ((uint32_t)(NT - 1 - k) << kLaneBits));
                }
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < NT; k++) {
                if ((pend & (1u << k)) && owner[tag_of(off[k], tag_mask)] == (key | ((uint32_t)(NT - 1 - k) << kLaneBits))) {
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
                            ElemIO<T>::store(e + cb * p.band_px, cur[cb] + contribution3<T, INTERP>(go[cb], wt[k]));
                        }
                    } else {
#pragma unroll
                        for (int cb = 0; cb < CB; cb++) {
                            if (cb < nc) {
                                const float val = contribution3<T, INTERP>(go[cb], wt[k]);
                                ElemIO<T>::store(e + cb * p.band_px, ElemIO<T>::load(e + cb * p.band_px) + val);
                            }
                        }
                    }
                    pend &= ~(1u << k);
                }
            }
            if (pend != 0) {
                s_flag[fl] = epoch + 1;  // somebody is left for the next round
            }
            __syncthreads();
            epoch++;
        }
        epoch++;
    }
    __syncthreads();
    for (int cb = 0; cb < nc; cb++) {
        T* dx_nc = dx + (n * p.C + c0 + cb) * (int64_t)vol + b0;
        const T* pl = planes + cb * p.band_px;
        for (int32_t i = t; i < b1 - b0; i += kThreads) {
            dx_nc[i] = pl[i];
        }
    }
}

template <typename T, int INTERP, int U>
__global__ __launch_bounds__(kThreads) void gs3d_grad_grid_kernel(const T* __restrict__ gout, const T* __restrict__ x,
                                                                   const T* __restrict__ grid, T* __restrict__ dgrid,
                                                                   int64_t total, Grad3Params p)
{
    using Taps = GradTaps3<T, INTERP>;
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) {
        return;
    }
    (void)gout;
    (void)x;
    if (INTERP == 1) {
        // grid_sampler3_d_grad_simt_det.h:354-356
        ElemIO<T>::store(dgrid + 3 * idx, 0.0f);
        ElemIO<T>::store(dgrid + 3 * idx + 1, 0.0f);
        ElemIO<T>::store(dgrid + 3 * idx + 2, 0.0f);
        return;
    }
    if constexpr (INTERP == 0) {
        const int32_t points = p.points;
        const int64_t n = idx / points;
        const int32_t pt = (int32_t)(idx - n * points);
        Taps tp;
        decide_grad_taps3<T, INTERP>(tp, ElemIO<T>::load(grid + 3 * idx), ElemIO<T>::load(grid + 3 * idx + 1),
                                     ElemIO<T>::load(grid + 3 * idx + 2), p.D, p.H, p.W, p.pad, p.align);
        gs3d_point_grid_gradient<T, U>(tp, gout, x, dgrid, idx, n, pt, p);
    }
}

// Voxels per band.  Every workgroup is a chain of dependent LDS round trips, so the chip is filled by workgroups
// next to each other: bands are halved (down to a quarter) until there are about two workgroups per compute unit.
// Measured on fp16 22x4x16x64x64 with an affine grid: 582 us with 8192 voxels, 383 with 4096, 280 with 2048.
int64_t band_voxels(const GridSampler3DGradArgs& a)
{
    const int64_t vol = a.Din * a.Hin * a.Win;
    const int cbmax = 8 / elem_size(a.elem);
    const int64_t cgroups = (a.C >= cbmax) ? (a.C + cbmax - 1) / cbmax : a.C;
    int64_t band = kBandMax;
    while (band > kBandMax / 4 && ((vol + band - 1) / band) * cgroups * a.N < 512) {
        band /= 2;
    }
    return vol < band ? vol : band;
}

template <typename T, int INTERP>
hipError_t launch_interp(const GridSampler3DGradArgs& a, hipStream_t stream)
{
    Grad3Params p;
    p.C = (int32_t)a.C;
    p.D = (int32_t)a.Din;
    p.H = (int32_t)a.Hin;
    p.W = (int32_t)a.Win;
    p.points = (int32_t)(a.Dout * a.Hout * a.Wout);
    p.pad = a.pad;
    p.align = a.align;
    p.items_per_core = (int32_t)(a.items_per_core > 0 ? a.items_per_core : 1);
    p.chunks = chunk_count(p.points, p.items_per_core);
    const int64_t vol = a.Din * a.Hin * a.Win;
    p.band_px = (int32_t)band_voxels(a);
    // voxels that share a tag are elected as if they were one: never out of order, at worst a round more
    p.tags = 64;
    while (p.tags < p.band_px && p.tags < kTagsMax) {
        p.tags *= 2;
    }
    bool dgrid_done = false;  // the gather variant's first kernel computes the grid gradient on its way
    if (a.dx != nullptr) {
        const int64_t bands = (vol + p.band_px - 1) / p.band_px;
        // 8 bytes of gradient per band voxel: 4 channels of a 16-bit type, 2 of fp32 (96 KB of LDS with the election
        // tags); fewer channels than that run one per workgroup
        constexpr int CBMAX = 8 / (int)sizeof(T);
        const bool grouped = a.C >= CBMAX;
        const int64_t cgroups = grouped ? (a.C + CBMAX - 1) / CBMAX : a.C;
        if (bands > INT32_MAX || cgroups > 65535 || a.N > 65535) {
            return hipErrorInvalidValue;
        }
        const dim3 grid((unsigned)bands, (unsigned)cgroups, (unsigned)a.N);
        const int32_t* ranges = nullptr;
        if (bands > 1 && a.chunk_ranges != nullptr) {
            if (p.chunks > 0x7fffffff / 2) {
                return hipErrorInvalidValue;
            }
            ranges = (const int32_t*)a.chunk_ranges;
        }
        // The gather variant first, where it runs: it does every item but those with crowded cells or voxels, flags
        // those, and notes the chunk spans on its way; the ordered kernel below then does the flagged items only.
        const uint32_t* item_flags = nullptr;
        uint32_t flag_stride = 0;
        if (INTERP == 0) {
            const hipError_t el = run_gs3d_grad_input_lists(a, p, const_cast<int32_t*>(ranges), stream, &item_flags,
                                                            &flag_stride, &dgrid_done);
            if (el != hipSuccess) {
                return el;
            }
        }
        if (ranges != nullptr && item_flags == nullptr) {
            hipLaunchKernelGGL((gs3d_grad_range_kernel<T, INTERP>), dim3((unsigned)p.chunks, (unsigned)a.N),
                               dim3(kThreads), 0, stream, (const T*)a.grid, (int32_t*)a.chunk_ranges, p);
        }
        // more than the default 64 KB of dynamic LDS
        static std::atomic<uint32_t> lds_allowed{0}, lds_allowed_single{0};
        hipError_t ea = allow_dynamic_lds(reinterpret_cast<const void*>(gs3d_grad_input_kernel<T, INTERP, CBMAX>),
                                          kTagsMax * 4 + kBandMax * CBMAX * (int)sizeof(T), lds_allowed);
        if (ea == hipSuccess) {
            ea = allow_dynamic_lds(reinterpret_cast<const void*>(gs3d_grad_input_kernel<T, INTERP, 1>),
                                   kTagsMax * 4 + kBandMax * (int)sizeof(T), lds_allowed_single);
        }
        if (ea != hipSuccess) {
            return ea;
        }
        if (grouped) {
            hipLaunchKernelGGL((gs3d_grad_input_kernel<T, INTERP, CBMAX>), grid, dim3(kThreads),
                               (size_t)p.tags * 4 + (size_t)p.band_px * CBMAX * sizeof(T), stream, (const T*)a.gout,
                               (const T*)a.grid, (T*)a.dx, ranges, p, item_flags, flag_stride);
        } else {
            hipLaunchKernelGGL((gs3d_grad_input_kernel<T, INTERP, 1>), grid, dim3(kThreads),
                               (size_t)p.tags * 4 + (size_t)p.band_px * sizeof(T), stream, (const T*)a.gout, (const T*)a.grid,
                               (T*)a.dx, ranges, p, item_flags, flag_stride);
        }
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            return e;
        }
    }
    if (a.dgrid != nullptr && !dgrid_done) {
        const int64_t total = a.N * (int64_t)p.points;
        const int64_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > INT32_MAX) {
            return hipErrorInvalidValue;
        }
        if (total < kGridGradFewPoints) {
            hipLaunchKernelGGL((gs3d_grad_grid_kernel<T, INTERP, 4>), dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                               (const T*)a.gout, (const T*)a.x, (const T*)a.grid, (T*)a.dgrid, total, p);
        } else {
            hipLaunchKernelGGL((gs3d_grad_grid_kernel<T, INTERP, 1>), dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                               (const T*)a.gout, (const T*)a.x, (const T*)a.grid, (T*)a.dgrid, total, p);
        }
        return hipGetLastError();
    }
    return hipSuccess;
}

template <typename T>
hipError_t launch_typed(const GridSampler3DGradArgs& a, hipStream_t stream)
{
    switch (a.interp) {
        case 0: return launch_interp<T, 0>(a, stream);
        case 1: return launch_interp<T, 1>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

int64_t gs3d_grad_range_words(const GridSampler3DGradArgs& a)
{
    if (a.Din * a.Hin * a.Win <= band_voxels(a)) {
        return 0;  // one band: every chunk concerns it
    }
    const int64_t per_core = a.items_per_core > 0 ? a.items_per_core : 1;
    return a.N * 2 * (int64_t)chunk_count(a.Dout * a.Hout * a.Wout, per_core);
}

hipError_t launch_grid_sampler3d_grad(const GridSampler3DGradArgs& a, hipStream_t stream)
{
    if (a.gout == nullptr || a.x == nullptr || a.grid == nullptr || (a.dx == nullptr && a.dgrid == nullptr)) {
        return hipErrorInvalidValue;
    }
    if (a.pad < 0 || a.pad > 2 || a.N <= 0 || a.C <= 0 || a.Din <= 0 || a.Hin <= 0 || a.Win <= 0 || a.Dout <= 0 ||
        a.Hout <= 0 || a.Wout <= 0) {
        return hipErrorInvalidValue;
    }
    if (a.Din * a.Hin * a.Win > INT32_MAX || a.Dout * a.Hout * a.Wout > INT32_MAX - 1024 || a.C > INT32_MAX) {
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
