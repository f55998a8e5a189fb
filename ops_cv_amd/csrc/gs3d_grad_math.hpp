// Backward of the 3-D grid sampler: what the kernels of gs3d_grad.hip and gs3d_grad_lists.hip share -- where a grid
// point's contributions land and with what weight, what a corner adds, and how the reference cuts the grid points of a
// batch item into chunks of 256 (image/grid_sampler3_d_grad/op_kernel/arch35/grid_sampler3_d_grad_simt_det.h,
// image/grid_sampler3_d_grad/op_host/grid_sampler3_d_grad_tiling.cpp:183-191).
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "acl_types.hpp"
#include "gs2d_grad_math.hpp"

namespace opscv {

constexpr int kChunkPoints3 = 256;  // the chunk length of the accumulation order

struct Grad3Params {
    int32_t C, D, H, W, points;
    int32_t pad, align;
    int32_t band_px;
    int32_t items_per_core;
    int32_t chunks;  // chunks a batch item is walked in, a possibly empty leading one included
    int32_t tags;    // election tags of the ordered kernel, a power of two
};

// Where the contributions of a grid point land in the (D, H, W) volume and with what weight.
//   INTERP 0: eight corners, index = x-high + 2 * y-high + 4 * z-high; weight = rt<T>(wx * wy * wz)
//   INTERP 1: one tap, weight 1
// off[k] = -1 marks a corner outside the volume.
template <typename T, int INTERP>
struct GradTaps3 {
    static constexpr int NT = (INTERP == 0) ? 8 : 1;
    int32_t off[NT];
    float w[NT];
    float wx[2], wy[2], wz[2];  // per axis: weight of the low and of the high corner
    int32_t x0, y0, z0;         // bilinear: the low corner
    float mx, my, mz;           // chain-rule multipliers of the grid gradient
};

__device__ __forceinline__ int32_t next_index(int32_t i)
{
    return (i == INT32_MAX) ? i : i + 1;
}

template <typename T, int INTERP>
__device__ __forceinline__ void decide_grad_taps3(GradTaps3<T, INTERP>& t, float gx, float gy, float gz, int32_t D,
                                                  int32_t H, int32_t W, int pad, int align)
{
    // grid_sampler3_d_grad_simt_det.h:381-383
    const float fx = source_index_set_grad<T>(gx, W, pad, align, &t.mx);
    const float fy = source_index_set_grad<T>(gy, H, pad, align, &t.my);
    const float fz = source_index_set_grad<T>(gz, D, pad, align, &t.mz);
    if (INTERP == 1) {
        // grid_sampler3_d_grad_simt_det.h:340-342
        const int32_t xi = float_to_i32(__builtin_rintf(fx));
        const int32_t yi = float_to_i32(__builtin_rintf(fy));
        const int32_t zi = float_to_i32(__builtin_rintf(fz));
        const bool in = (uint32_t)xi < (uint32_t)W && (uint32_t)yi < (uint32_t)H && (uint32_t)zi < (uint32_t)D;
        t.off[0] = in ? (zi * H + yi) * W + xi : -1;
        t.w[0] = 1.0f;
        return;
    }
    // grid_sampler3_d_grad_simt_det.h:281-297
    const int32_t x0 = float_to_i32(__builtin_floorf(fx));
    const int32_t y0 = float_to_i32(__builtin_floorf(fy));
    const int32_t z0 = float_to_i32(__builtin_floorf(fz));
    const int32_t x1 = next_index(x0), y1 = next_index(y0), z1 = next_index(z0);
    t.x0 = x0;
    t.y0 = y0;
    t.z0 = z0;
    t.wx[0] = (float)x1 - fx;
    t.wx[1] = fx - (float)x0;
    t.wy[0] = (float)y1 - fy;
    t.wy[1] = fy - (float)y0;
    t.wz[0] = (float)z1 - fz;
    t.wz[1] = fz - (float)z0;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const int xs = k & 1, ys = (k >> 1) & 1, zs = k >> 2;
        const int32_t cx = xs ? x1 : x0, cy = ys ? y1 : y0, cz = zs ? z1 : z0;
        const bool in = (uint32_t)cx < (uint32_t)W && (uint32_t)cy < (uint32_t)H && (uint32_t)cz < (uint32_t)D;
        t.off[k] = in ? (cz * H + cy) * W + cx : -1;
        // the fp32 product is pinned before it is rounded to T (one rounding each, as in the reference)
        t.w[k] = rt<T>(as_fp32_value(t.wx[xs] * t.wy[ys] * t.wz[zs]));
    }
}

// What a corner adds: weight times incoming gradient in fp32, then rounded to the element type
// (grid_sampler3_d_grad_simt_det.h:116-118,72-73).
template <typename T, int INTERP>
__device__ __forceinline__ float contribution3(float go, float w)
{
    if (INTERP == 1) {
        return rt<T>(go);
    }
    return rt<T>(as_fp32_value(w * go));
}

// Thread of the chunk that holds the first grid point of batch item n.
__device__ __forceinline__ int32_t chunk_phase(int64_t n, const Grad3Params& p)
{
    return (int32_t)(((n % p.items_per_core) * (int64_t)p.points) % kChunkPoints3);
}

// Chunks a batch item is walked in: with several items per core the first chunk of an item may start before its
// first point.
__host__ __device__ inline int32_t chunk_count(int64_t points, int64_t items_per_core)
{
    return (int32_t)(((items_per_core > 1 ? kChunkPoints3 - 1 : 0) + points + kChunkPoints3 - 1) / kChunkPoints3);
}

// The gradient of one grid point (bilinear): the sums over the channels of value times two distances times the
// incoming gradient for the eight corners, then the chain-rule multipliers (grid_sampler3_d_grad_simt_det.h:98-330).
// `idx` is the point's number among all points of the batch, n its batch item, pt its number within the item.
// U: channels whose loads are in flight together.  Four need about 150 vector registers (three wavefronts per SIMD),
// one about 76 (six): with grid points for four wavefronts per SIMD and more, the wavefronts hide the latency better
// than the unrolling does (fp16 22x4x16x64x64: 34.0 us with four, 29.1 us with one; 2x64x16x64x64: 32.0 and 41.5 us).
constexpr int64_t kGridGradFewPoints = 256 * 4 * 4 * 64;  // below: U = 4
template <typename T, int U>
__device__ __forceinline__ void gs3d_point_grid_gradient(const GradTaps3<T, 0>& tp, const T* __restrict__ gout,
                                                         const T* __restrict__ x, T* __restrict__ dgrid, int64_t idx,
                                                         int64_t n, int32_t pt, const Grad3Params& p)
{
    const int32_t points = p.points;
    const int32_t vol = p.D * p.H * p.W;
    const T* x_n = x + n * p.C * (int64_t)vol;
    const T* go_n = gout + n * p.C * (int64_t)points + pt;
    float gix = 0.0f, giy = 0.0f, giz = 0.0f;
    bool ok[8];
    int32_t o[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        ok[k] = tp.off[k] >= 0;
        o[k] = ok[k] ? tp.off[k] : 0;
    }
    // grid_sampler3_d_grad_simt_det.h:119-124 and the seven corners after it: value times two distances times the
    // incoming gradient, left to right, subtracted for a low corner of the axis and added for a high one
    auto accumulate = [&](float go, const float* v) {
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int xs = k & 1, ys = (k >> 1) & 1, zs = k >> 2;
            if (ok[k]) {
                const float tx = v[k] * tp.wy[ys] * tp.wz[zs] * go;
                const float ty = v[k] * tp.wx[xs] * tp.wz[zs] * go;
                const float tz = v[k] * tp.wx[xs] * tp.wy[ys] * go;
                gix = xs ? gix + tx : gix - tx;
                giy = ys ? giy + ty : giy - ty;
                giz = zs ? giz + tz : giz - tz;
            }
        }
    };
    // The sums run over the channels in order; the loads do not depend on them and are issued a group ahead.
    int32_t c = 0;
    if (p.W >= 2) {
        // The low and high corner along x are neighbours in memory: one load of two elements (aligned to one element
        // only) per row of corners instead of two halves the addresses the gather puts through the memory pipeline.
        // The pair sits at column pb = clamp(x0, 0, W - 2), so it never leaves the row; which half is which corner
        // follows from pb.  Corners outside the volume are skipped by accumulate() as before.
        using PairBits = typename std::conditional<sizeof(T) == 2, uint32_t, uint64_t>::type;
        const int32_t pb = (tp.x0 < 0) ? 0 : ((tp.x0 > p.W - 2) ? p.W - 2 : tp.x0);
        const bool lo_w = (tp.x0 == pb), lo_e = (next_index(tp.x0) == pb);
        int32_t rowoff[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int32_t cy = (r & 1) ? next_index(tp.y0) : tp.y0, cz = (r >> 1) ? next_index(tp.z0) : tp.z0;
            const bool in = (uint32_t)cy < (uint32_t)p.H && (uint32_t)cz < (uint32_t)p.D;
            rowoff[r] = in ? (cz * p.H + cy) * p.W + pb : 0;
        }
        for (; c + U <= p.C; c += U) {
            float go[U];
            PairBits pr[U][4];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const T* xc = x_n + (int64_t)(c + u) * vol;
                go[u] = ElemIO<T>::load(go_n + (int64_t)(c + u) * points);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    __builtin_memcpy(&pr[u][r], xc + rowoff[r], sizeof(PairBits));
                }
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                float v[8];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    T two[2];
                    __builtin_memcpy(two, &pr[u][r], sizeof(PairBits));
                    const float lo = ElemIO<T>::load(&two[0]), hi = ElemIO<T>::load(&two[1]);
                    v[2 * r] = lo_w ? lo : hi;
                    v[2 * r + 1] = lo_e ? lo : hi;
                }
                accumulate(go[u], v);
            }
        }
    }
    for (; c + U <= p.C; c += U) {
        float go[U], v[U][8];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const T* xc = x_n + (int64_t)(c + u) * vol;
            go[u] = ElemIO<T>::load(go_n + (int64_t)(c + u) * points);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                v[u][k] = ElemIO<T>::load(xc + o[k]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            accumulate(go[u], v[u]);
        }
    }
    for (; c < p.C; c++) {
        const T* xc = x_n + (int64_t)c * vol;
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            v[k] = ElemIO<T>::load(xc + o[k]);
        }
        accumulate(ElemIO<T>::load(go_n + (int64_t)c * points), v);
    }
    // grid_sampler3_d_grad_simt_det.h:324-326: product in fp32, then the conversion
    ElemIO<T>::store(dgrid + 3 * idx, as_fp32_value(tp.mx * gix));
    ElemIO<T>::store(dgrid + 3 * idx + 1, as_fp32_value(tp.my * giy));
    ElemIO<T>::store(dgrid + 3 * idx + 2, as_fp32_value(tp.mz * giz));
}

// The gather variant of the input gradient (gs3d_grad_lists.hip).  Runs when a.lists is set and the shape qualifies:
// *item_flags then points at a word per batch item, `*flag_stride` words apart, that is non-zero for the items it
// leaves to the ordered kernel, which has to run after it for those; otherwise *item_flags is null and nothing was
// launched.  `ranges` (may be null) receives the voxel span of every chunk, as from gs3d_grad_range_kernel.  When
// a.dgrid is set, its first kernel computes the gradient of the grid as well (*dgrid_done).
hipError_t run_gs3d_grad_input_lists(const GridSampler3DGradArgs& a, const Grad3Params& p, int32_t* ranges,
                                     hipStream_t stream, const uint32_t** item_flags, uint32_t* flag_stride,
                                     bool* dgrid_done);

}  // namespace opscv
