// Backward of the bilinear resize for gfx950, deterministic gather formulation.
//
// Replaces the reference device kernel
// image/resize_bilinear_v2_grad/op_kernel/arch35/resize_bilinear_v2_grad_simt_determine.h:56-117 and the scale rules
// of image/resize_bilinear_v2_grad/op_host/arch35/resize_bilinear_v2_grad_tiling_arch35.cpp:352-394.
//
// One lane per element (n, c, H, W) of the outgoing gradient.  It visits the incoming-gradient rows inY whose
// source coordinate outY = (inY + o) * scale - o lies in (H - 1, H + 1), starting at
// ceil((H - 1 + o) / scale - o) and advancing outY by repeated addition of the scale (as the reference does, so
// the rounding of every coordinate is the same), and likewise the columns; each visited element contributes
// g * (1 - |clamp(outY) - H|) * (1 - |clamp(outX) - W|), summed in fp32 in row-major visiting order.  No atomics:
// the result does not depend on scheduling.  The translation unit is compiled with -ffp-contract=off.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "kernels.hpp"
#include "sampler_math.hpp"

namespace opscv {

namespace {

constexpr int kGradThreads = 256;

// User-scale template (resize_bilinear_v2_grad_simt_determine_scales.h:77-305), for scales that are not the ratio
// of the sizes.  Same walk, but the source coordinate of every visited row/column is recomputed as
// scale * (i + o) - o instead of accumulated, and an element on the first or last row (column) of the outgoing
// gradient scans the incoming rows (columns) to the end and takes, per visited element, the weights of the taps
// that land on it (floor tap: 1 - |c - H|; next tap: c - floor(c)).
template <typename TI, typename TO, bool HALF_PIXEL, bool NHWC>
__global__ __launch_bounds__(kGradThreads) void resize_grad_scales_kernel(const TI* __restrict__ g, TO* __restrict__ y,
                                                                           int64_t total, int32_t C, int32_t Hs,
                                                                           int32_t Ws, int32_t Hd, int32_t Wd,
                                                                           float scale_h, float scale_w,
                                                                           float inv_scale_h, float inv_scale_w)
{
    const int64_t stride = (int64_t)gridDim.x * kGradThreads;
    const float offset = HALF_PIXEL ? 0.5f : 0.0f;
    const float last_y = (float)Hs - 1.0f, last_x = (float)Ws - 1.0f;
    auto source_index = [](float scale, int64_t i) {
        return HALF_PIXEL ? scale * ((float)i + 0.5f) - 0.5f : scale * (float)i;
    };
    for (int64_t idx = (int64_t)blockIdx.x * kGradThreads + threadIdx.x; idx < total; idx += stride) {
        int64_t t = idx;
        int32_t c, W, H;
        if (NHWC) {
            c = (int32_t)(t % C);
            t /= C;
            W = (int32_t)(t % Ws);
            t /= Ws;
            H = (int32_t)(t % Hs);
            t /= Hs;
        } else {
            W = (int32_t)(t % Ws);
            t /= Ws;
            H = (int32_t)(t % Hs);
            t /= Hs;
            c = (int32_t)(t % C);
            t /= C;
        }
        const int64_t n = t;
        const float fy0 = __builtin_ceilf(((float)H - 1.0f + offset) * inv_scale_h - offset);
        const float fx0 = __builtin_ceilf(((float)W - 1.0f + offset) * inv_scale_w - offset);
        const int64_t in_y_start = (fy0 > 0.0f) ? (int64_t)fy0 : 0;
        const int64_t in_x_start = (fx0 > 0.0f) ? (int64_t)fx0 : 0;
        const float out_y_start = ((float)in_y_start + offset) * scale_h - offset;
        const float out_x_start = ((float)in_x_start + offset) * scale_w - offset;
        const float fh = (float)H, fw = (float)W;
        const bool hb = (H == 0 || H == Hs - 1), wb = (W == 0 || W == Ws - 1);
        float acc = 0.0f;
        float out_y = out_y_start;
        for (int64_t in_y = in_y_start; (hb || out_y < fh + 1.0f) && in_y < Hd;) {
            const float yc = __builtin_fmaxf(0.0f, __builtin_fminf(out_y, last_y));
            const float y_lerp = 1.0f - __builtin_fabsf(yc - fh);
            const float yt = __builtin_fminf(__builtin_floorf(yc), last_y);
            const float lepy[2] = {y_lerp, yc - yt};
            float out_x = out_x_start;
            for (int64_t in_x = in_x_start; (wb || out_x < fw + 1.0f) && in_x < Wd;) {
                const int64_t gi = NHWC ? ((n * Hd + in_y) * Wd + in_x) * C + c : ((n * C + c) * Hd + in_y) * Wd + in_x;
                const float gv = ElemIO<TI>::load(g + gi);
                const float xc = __builtin_fmaxf(0.0f, __builtin_fminf(out_x, last_x));
                const float x_lerp = 1.0f - __builtin_fabsf(xc - fw);
                const float xt = __builtin_fminf(__builtin_floorf(xc), last_x);
                const float lepx[2] = {x_lerp, xc - xt};
                if (!hb && !wb) {
                    acc += gv * y_lerp * x_lerp;
                } else if (!hb) {
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        if (xt + (float)j == fw) {
                            acc += gv * lepx[j] * y_lerp;
                        }
                    }
                } else if (!wb) {
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        if (yt + (float)i == fh) {
                            acc += gv * lepy[i] * x_lerp;
                        }
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 2; i++) {
#pragma unroll
                        for (int j = 0; j < 2; j++) {
                            if (yt + (float)i == fh && xt + (float)j == fw) {
                                acc += gv * lepx[j] * lepy[i];
                            }
                        }
                    }
                }
                in_x++;
                out_x = source_index(scale_w, in_x);
            }
            in_y++;
            out_y = source_index(scale_h, in_y);
        }
        ElemIO<TO>::store(y + idx, acc);
    }
}

template <typename TI, typename TO, bool HALF_PIXEL, bool NHWC>
__global__ __launch_bounds__(kGradThreads) void resize_grad_kernel(const TI* __restrict__ g, TO* __restrict__ y,
                                                                    int64_t total, int32_t C, int32_t Hs, int32_t Ws,
                                                                    int32_t Hd, int32_t Wd, float scale_h,
                                                                    float scale_w, float inv_scale_h,
                                                                    float inv_scale_w)
{
    const int64_t stride = (int64_t)gridDim.x * kGradThreads;
    const float offset = HALF_PIXEL ? 0.5f : 0.0f;
    const float last_y = (float)Hs - 1.0f, last_x = (float)Ws - 1.0f;
    for (int64_t idx = (int64_t)blockIdx.x * kGradThreads + threadIdx.x; idx < total; idx += stride) {
        int64_t t = idx;
        int32_t c, W, H;
        if (NHWC) {
            c = (int32_t)(t % C);
            t /= C;
            W = (int32_t)(t % Ws);
            t /= Ws;
            H = (int32_t)(t % Hs);
            t /= Hs;
        } else {
            W = (int32_t)(t % Ws);
            t /= Ws;
            H = (int32_t)(t % Hs);
            t /= Hs;
            c = (int32_t)(t % C);
            t /= C;
        }
        const int64_t n = t;
        const float fy0 = __builtin_ceilf(((float)H - 1.0f + offset) * inv_scale_h - offset);
        const float fx0 = __builtin_ceilf(((float)W - 1.0f + offset) * inv_scale_w - offset);
        const int64_t in_y_start = (fy0 > 0.0f) ? (int64_t)fy0 : 0;
        const int64_t in_x_start = (fx0 > 0.0f) ? (int64_t)fx0 : 0;
        const float out_y_start = ((float)in_y_start + offset) * scale_h - offset;
        const float out_x_start = ((float)in_x_start + offset) * scale_w - offset;
        const float fh = (float)H, fw = (float)W;
        float acc = 0.0f;
        float out_y = out_y_start;
        for (int64_t in_y = in_y_start; out_y < fh + 1.0f && in_y < Hd; in_y++) {
            const float yc = __builtin_fmaxf(0.0f, __builtin_fminf(out_y, last_y));
            const float y_lerp = 1.0f - __builtin_fabsf(yc - fh);
            float out_x = out_x_start;
            for (int64_t in_x = in_x_start; out_x < fw + 1.0f && in_x < Wd; in_x++) {
                const int64_t gi = NHWC ? ((n * Hd + in_y) * Wd + in_x) * C + c : ((n * C + c) * Hd + in_y) * Wd + in_x;
                const float xc = __builtin_fmaxf(0.0f, __builtin_fminf(out_x, last_x));
                const float x_lerp = 1.0f - __builtin_fabsf(xc - fw);
                acc += ElemIO<TI>::load(g + gi) * y_lerp * x_lerp;
                out_x += scale_w;
            }
            out_y += scale_h;
        }
        ElemIO<TO>::store(y + idx, acc);
    }
}


// LDS-tiled variant of resize_grad_kernel for NCHW.  A workgroup owns (plane, tile of kTileRows x 128 elements of
// the outgoing gradient).  The incoming-gradient rows and columns the tile's lanes will visit form one rectangle
// (start of the first lane, largest end over all lanes, found with the very loops the lanes run later); it is
// copied into LDS with independent 4-byte loads -- all in flight together, where the gather variant waits for one
// two-byte load per visit -- and the lanes then run the unchanged visiting loops on LDS.  A rectangle that does not
// fit the LDS capacity is read from global memory instead (same loops, same result).
// The visiting loops of resize_grad_kernel over a row-major array whose element (y0, x0) is base[0].
template <typename TI>
__device__ __forceinline__ float visit_sum(const TI* base, int32_t pitch, int32_t y0, int32_t x0, int32_t in_y_start,
                                           int32_t in_x_start, float out_y_start, float out_x_start, float fh,
                                           float fw, float scale_h, float scale_w, float last_y, float last_x,
                                           int32_t Hd, int32_t Wd, int32_t ci = 1, int32_t ch = 0)
{
    // ci, ch: channels-last rows hold ci elements per pixel, this lane's channel is ch (x0 counts elements)
    float acc = 0.0f;
    float out_y = out_y_start;
    for (int32_t in_y = in_y_start; out_y < fh + 1.0f && in_y < Hd; in_y++) {
        const float yc = __builtin_fmaxf(0.0f, __builtin_fminf(out_y, last_y));
        const float y_lerp = 1.0f - __builtin_fabsf(yc - fh);
        const TI* row = base + (int64_t)(in_y - y0) * pitch;
        float out_x = out_x_start;
        for (int32_t in_x = in_x_start; out_x < fw + 1.0f && in_x < Wd; in_x++) {
            const float xc = __builtin_fmaxf(0.0f, __builtin_fminf(out_x, last_x));
            const float x_lerp = 1.0f - __builtin_fabsf(xc - fw);
            acc += ElemIO<TI>::load(row + ((int64_t)in_x * ci + ch - x0)) * y_lerp * x_lerp;
            out_x += scale_w;
        }
        out_y += scale_h;
    }
    return acc;
}

// The same sum with the column part of the loop taken out: a lane keeps the weights of the (at most KX) columns it
// visits -- computed once, by the same repeated additions -- and a row costs one LDS read, two products and an add
// per column.  Column k of a lane with fewer than k + 1 visits leaves the sum alone.
template <typename TI, int KX, int KMIN, bool IL = false>
__device__ __forceinline__ float visit_sum_fixed(const TI* tile_xy, int32_t pitch, int32_t y0, int32_t in_y_start,
                                                 int32_t nx, const float* xl, float out_y_start, float fh,
                                                 float scale_h, float last_y, int32_t Hd, float neg_zero,
                                                 int32_t ci = 1)
{
    const int32_t step = IL ? ci : 1;  // elements between the columns a lane visits
    float acc = 0.0f;
    float out_y = out_y_start;
    for (int32_t in_y = in_y_start; out_y < fh + 1.0f && in_y < Hd; in_y++) {
        // max(0, min(out_y, last_y)) as one median: out_y is never a NaN
        const float yc = __builtin_amdgcn_fmed3f(out_y, 0.0f, last_y);
        const float y_lerp = 1.0f - __builtin_fabsf(yc - fh);
        const TI* row = tile_xy + (in_y - y0) * pitch;
#pragma unroll
        for (int k = 0; k < KX; k++) {
            // fma(g, w, -0) is g * w bit for bit and lets a 16-bit element be converted by the multiply itself; the
            // read of a column past the lane's last one may fetch anything (it stays inside LDS) and is dropped.
            // Every lane of the workgroup visits at least KMIN columns: those need no test.
            const float t = __builtin_fmaf(ElemIO<TI>::load(row + k * step), y_lerp, neg_zero) * xl[k];
            acc = (k < KMIN || k < nx) ? acc + t : acc;
        }
        out_y += scale_h;
    }
    return acc;
}

// The same sum once more with the row part taken out as well.  The rows an outgoing row H visits, and their weights,
// do not depend on the plane or the column: a workgroup that walks over planes computes them once per H (by the very
// loop above) and keeps count and weights in registers.  H is the same for all lanes of a wavefront, so the count is
// a scalar and the row loop needs no lane masks.  A visited row then costs the LDS reads, one address add and, per
// column, two products and an add.
constexpr int kRowWeights = 6;  // visited rows per outgoing row kept in registers (more: the loops above)

template <int KX, int KMIN, int Q, bool IL = false>
__device__ __forceinline__ float tile_sum_fixed(const float* lane_rows, int32_t pitch, int32_t n_rows, float lerp_pack,
                                                int32_t nx, const float* xl, float neg_zero, int32_t ci = 1)
{
    const int32_t step = IL ? ci : 1;  // elements between the columns a lane visits
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < kRowWeights; j++) {
        if (j < n_rows) {  // n_rows is uniform over the wavefront
            // weight of visited row j of this wavefront's outgoing row Q: lane Q * kRowWeights + j of lerp_pack
            const float y_lerp = __builtin_bit_cast(
                float, __builtin_amdgcn_readlane(__builtin_bit_cast(int32_t, lerp_pack), Q * kRowWeights + j));
#pragma unroll
            for (int k = 0; k < KX; k++) {
                // fma(g, w, -0) is g * w bit for bit; the compiler may not fold it into the following product
                const float t = __builtin_fmaf(lane_rows[k * step], y_lerp, neg_zero) * xl[k];
                acc = (k < KMIN || k < nx) ? acc + t : acc;
            }
            lane_rows += pitch;
        }
    }
    return acc;
}

constexpr int kTileCols = 128;
constexpr int32_t kGradCapWords = 12288;  // at most 48 KB of LDS per workgroup (fp32 words, one per tile element)
constexpr int kTileGroups = kGradThreads / kTileCols;  // row groups of a workgroup

// IL: channels-last tensors, taken as planes whose rows are W * ci elements (element j of a row is channel j % ci of
// pixel j / ci); "columns" then count row elements, a lane's visited columns sit ci elements apart, and the column
// geometry (first visit, count, weights) is that of the lane's pixel.
template <typename TI, typename TO, bool HALF_PIXEL, bool IL>
__global__ __launch_bounds__(kGradThreads) void resize_grad_lds_kernel(const TI* __restrict__ g, TO* __restrict__ y,
                                                                        int64_t planes, int32_t Hs, int32_t Ws,
                                                                        int32_t Hd, int32_t Wd, float scale_h,
                                                                        float scale_w, float inv_scale_h,
                                                                        float inv_scale_w, int32_t tile_rows,
                                                                        int32_t cap_words, float neg_zero,
                                                                        uint32_t tiles_x, uint32_t tiles_y,
                                                                        uint32_t plane_slots, int32_t ci_arg)
{
    const int32_t ci = IL ? ci_arg : 1;
    const int32_t Wse = Ws * ci, Wde = Wd * ci;  // row elements
    // Workgroups are handed to the eight XCDs in turn, each with its own L2.  The launch is one-dimensional and padded
    // to a multiple of eight; workgroup L becomes tile (L % 8) * (count / 8) + L / 8, so that an XCD works through a
    // contiguous run of tiles and the rows and 128-byte lines that neighbouring tiles share are fetched from memory
    // once per XCD rather than once per tile.
    const uint32_t per_xcd = gridDim.x / 8u;
    const uint32_t tile_id = (blockIdx.x % 8u) * per_xcd + blockIdx.x / 8u;
    if (tile_id >= tiles_x * tiles_y * plane_slots) {
        return;
    }
    const uint32_t block_x = tile_id % tiles_x, block_y = (tile_id / tiles_x) % tiles_y;
    const uint32_t block_z = tile_id / (tiles_x * tiles_y);
    constexpr int EPW = 4 / (int)sizeof(TI);  // elements per 4-byte word
    extern __shared__ __attribute__((aligned(16))) uint32_t tile_words[];
    __shared__ int32_t s_x1, s_y1, s_nx, s_nx_min;
    const int tx = threadIdx.x % kTileCols, ty = threadIdx.x / kTileCols;
    const int32_t W0 = (int32_t)block_x * kTileCols, H0 = (int32_t)block_y * tile_rows;
    const float offset = HALF_PIXEL ? 0.5f : 0.0f;
    const float last_y = (float)Hs - 1.0f, last_x = (float)Ws - 1.0f;
    auto first_visit = [&](int32_t i, float inv_scale, int32_t len_dst) {
        const float f = __builtin_ceilf(((float)i - 1.0f + offset) * inv_scale - offset);
        // a start at or beyond the end visits nothing, whatever its exact value
        return (f > 0.0f) ? ((f < (float)len_dst) ? (int32_t)f : len_dst) : 0;
    };
    auto end_visit = [&](int32_t i, int32_t start, float scale, int32_t len_dst) {
        float out = ((float)start + offset) * scale - offset;
        int32_t in = start;
        for (; out < (float)i + 1.0f && in < len_dst; in++) {
            out += scale;
        }
        return in;
    };
    const int32_t W = W0 + tx;
    const bool col_ok = W < Wse;
    const int32_t px = IL ? (col_ok ? W : W0) / ci : (col_ok ? W : W0);  // pixel of this lane's column
    const int32_t ch = IL ? (col_ok ? W : W0) - px * ci : 0;               // and its channel
    const int32_t in_x_start = first_visit(px, inv_scale_w, Wd);
    const int32_t tile_x0 = first_visit(IL ? W0 / ci : W0, inv_scale_w, Wd) * ci / EPW * EPW;
    const int32_t tile_y0 = first_visit(H0, inv_scale_h, Hd);
    if (threadIdx.x == 0) {
        s_x1 = 0;
        s_y1 = 0;
        s_nx = 0;
        s_nx_min = INT32_MAX;
    }
    __syncthreads();
    int32_t nx = 0;
    {
        // largest end and largest visit count over the wavefront by a butterfly of lane exchanges, then one LDS atomic
        // per wavefront (an atomic per lane is serialised lane by lane on the scalar unit)
        int32_t x_end = 0;
        if (col_ok) {
            x_end = end_visit(px, in_x_start, scale_w, Wd);
            nx = x_end - in_x_start;
        }
        int32_t m_end = x_end, m_nx = nx, m_min = col_ok ? nx : INT32_MAX;  // lanes past the last column do not count
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            const int32_t o_end = __shfl_xor(m_end, d), o_nx = __shfl_xor(m_nx, d), o_min = __shfl_xor(m_min, d);
            m_end = (o_end > m_end) ? o_end : m_end;
            m_nx = (o_nx > m_nx) ? o_nx : m_nx;
            m_min = (o_min < m_min) ? o_min : m_min;
        }
        if ((threadIdx.x & 63) == 0) {
            atomicMax(&s_x1, m_end);
            atomicMax(&s_nx, m_nx);
            atomicMin(&s_nx_min, m_min);
        }
    }
    if (tx == 0) {
        for (int32_t H = H0 + ty; H < H0 + tile_rows && H < Hs; H += kTileGroups) {
            atomicMax(&s_y1, end_visit(H, first_visit(H, inv_scale_h, Hd), scale_h, Hd));
        }
    }
    __syncthreads();
    const int32_t tile_x1 = (s_x1 * ci + EPW - 1) / EPW * EPW;  // rows are multiples of EPW (host check): stays inside
    const int32_t tile_y1 = s_y1;
    const int32_t pitch_w = (tile_x1 > tile_x0) ? (tile_x1 - tile_x0) / EPW : 0;
    const int32_t rows = (tile_y1 > tile_y0) ? tile_y1 - tile_y0 : 0;
    // the tile holds fp32 values (16-bit gradients are widened by the copy, which is exact): a lane's run of columns
    // then starts on a 4-byte boundary whatever its parity, and LDS reads that straddle words are several times slower
    const int32_t pitch = pitch_w * EPW;
    const bool use_lds = (int64_t)rows * pitch <= cap_words;
    const float* tile = reinterpret_cast<const float*>(tile_words);
    const float out_x_start = ((float)in_x_start + offset) * scale_w - offset;
    const float fw = (float)px;

    // column weights of this lane, for the variants with a fixed column count
    constexpr int KMAX = 8;
    float xl[KMAX];
    {
        float out_x = out_x_start;
#pragma unroll
        for (int k = 0; k < KMAX; k++) {
            const float xc = __builtin_fmaxf(0.0f, __builtin_fminf(out_x, last_x));
            xl[k] = 1.0f - __builtin_fabsf(xc - fw);
            out_x += scale_w;
        }
    }
    const int32_t nx_max = s_nx, nx_min = s_nx_min;
    // starting position and step of this lane in the tile's (row, word) grid for the copy loop
    const int32_t pw1 = (pitch_w > 0) ? pitch_w : 1;
    const int32_t ld_r0 = (int32_t)threadIdx.x / pw1, ld_c0 = (int32_t)threadIdx.x % pw1;
    const int32_t ld_dr = kGradThreads / pw1, ld_dc = kGradThreads % pw1;
    const int32_t x_base = (nx > 0) ? in_x_start * ci + ch - tile_x0 : 0;

    // rows visited by each of this wavefront's outgoing rows, and their weights (see tile_sum_fixed)
    constexpr int HQ = 8 / kTileGroups;  // outgoing rows per lane at the largest tile height
    static_assert(HQ * kRowWeights <= 64, "the row weights of a wavefront are packed one per lane");
    float lerp_pack = 0.0f;  // lane q * kRowWeights + j: weight of visited row j of outgoing row q (a uniform table)
    int32_t meta_pack = -1;  // lane q: rows outgoing row q visits (-1: no such row in this tile); lane 8 + q: the first
    bool rows_fixed = true;
    const int32_t lane_id = (int32_t)threadIdx.x & 63;
#pragma unroll
    for (int q = 0; q < HQ; q++) {
        const int32_t H = __builtin_amdgcn_readfirstlane(H0 + ty + q * kTileGroups);
        if (H < H0 + tile_rows && H < Hs) {
            const int32_t start = first_visit(H, inv_scale_h, Hd);
            float out_y = ((float)start + offset) * scale_h - offset;
            const float fh = (float)H;
            int32_t n = 0;
            for (int32_t in_y = start; out_y < fh + 1.0f && in_y < Hd; in_y++) {
                const float w = 1.0f - __builtin_fabsf(__builtin_amdgcn_fmed3f(out_y, 0.0f, last_y) - fh);
                lerp_pack = (n < kRowWeights && lane_id == q * kRowWeights + n) ? w : lerp_pack;
                n++;
                out_y += scale_h;
            }
            meta_pack = (lane_id == q) ? n : ((lane_id == 8 + q) ? start : meta_pack);
            rows_fixed = rows_fixed && (__builtin_amdgcn_readfirstlane(n) <= kRowWeights);
        }
    }

    // Copy of the rectangle into LDS: word i of the tile is (row i / pitch_w, word i % pitch_w) of the rectangle.
    const int32_t total = rows * pitch_w;
    const int32_t row_words = Wde / EPW;

    for (int64_t pl = block_z; pl < planes; pl += plane_slots) {
        const TI* gp = g + pl * (int64_t)Hd * Wde;
        if (use_lds) {
            // the pair (row, word) is advanced instead of divided
            int32_t r = ld_r0, cw = ld_c0;
            const uint32_t* src = reinterpret_cast<const uint32_t*>(gp + (int64_t)tile_y0 * Wde + tile_x0);
#pragma unroll 8
            for (int32_t i = threadIdx.x; i < total; i += kGradThreads) {
                const uint32_t word = src[(int64_t)r * row_words + cw];
                if (EPW == 1) {
                    tile_words[i] = word;
                } else {
                    TI pair[2];
                    __builtin_memcpy(pair, &word, 4);
                    float2 wide;
                    wide.x = ElemIO<TI>::load(&pair[0]);
                    wide.y = ElemIO<TI>::load(&pair[1]);
                    reinterpret_cast<float2*>(tile_words)[i] = wide;
                }
                r += ld_dr;
                cw += ld_dc;
                if (cw >= pitch_w) {
                    cw -= pitch_w;
                    r++;
                }
            }
            __syncthreads();
        }
        if (col_ok && use_lds && rows_fixed && nx_max <= 6) {
            TO* yp = y + (pl * Hs + H0 + ty) * (int64_t)Wse + W;
            // -0 in a vector register: with the row weight in a scalar one, a second scalar operand would be copied
            // into a vector register before every product
            const float neg_zero_v = as_fp32_value(neg_zero);
            auto one_row = [&](auto qc) {
                constexpr int q = decltype(qc)::value;
                // read where they are used: kept in scalar registers from the set-up on, they would be spilled
                const int32_t n_rows = __builtin_amdgcn_readlane(meta_pack, q);
                if (n_rows >= 0) {
                    const int32_t first_row = __builtin_amdgcn_readlane(meta_pack, 8 + q);
                    const float* lane_rows = tile + (first_row - tile_y0) * pitch + x_base;
                    float acc;
#define OPSCV_TILE_SUM(KX, KMIN) \
    tile_sum_fixed<KX, KMIN, q, IL>(lane_rows, pitch, n_rows, lerp_pack, nx, xl, neg_zero_v, ci)
                    if (nx_max <= 4) {
                        acc = (nx_min >= 4) ? OPSCV_TILE_SUM(4, 4) : OPSCV_TILE_SUM(4, 0);
                    } else if (nx_max <= 5) {
                        acc = (nx_min >= 4) ? OPSCV_TILE_SUM(5, 4) : OPSCV_TILE_SUM(5, 0);
                    } else {
                        acc = (nx_min >= 4) ? OPSCV_TILE_SUM(6, 4) : OPSCV_TILE_SUM(6, 0);
                    }
#undef OPSCV_TILE_SUM
                    store_streaming<TO>(yp + (int64_t)q * kTileGroups * Wse, acc);
                }
            };
            static_assert(HQ == 4, "one call per outgoing row of a lane");
            one_row(std::integral_constant<int, 0>{});
            one_row(std::integral_constant<int, 1>{});
            one_row(std::integral_constant<int, 2>{});
            one_row(std::integral_constant<int, 3>{});
        } else if (col_ok) {
            for (int32_t H = H0 + ty; H < H0 + tile_rows && H < Hs; H += kTileGroups) {
                const int32_t in_y_start = first_visit(H, inv_scale_h, Hd);
                const float out_y_start = ((float)in_y_start + offset) * scale_h - offset;
                float acc;
                // separate call sites so that each is compiled for its own address space (LDS reads, global loads)
#define OPSCV_VISIT(KX, KMIN)                                                                                       \
    visit_sum_fixed<float, KX, KMIN, IL>(tile + x_base, pitch, tile_y0, in_y_start, nx, xl, out_y_start, (float)H,    \
                                         scale_h, last_y, Hd, neg_zero, ci)
                if (use_lds && nx_max <= 4) {
                    acc = (nx_min >= 4) ? OPSCV_VISIT(4, 4) : OPSCV_VISIT(4, 0);
                } else if (use_lds && nx_max <= 5) {
                    acc = (nx_min >= 4) ? OPSCV_VISIT(5, 4) : OPSCV_VISIT(5, 0);
                } else if (use_lds && nx_max <= 6) {
                    acc = (nx_min >= 4) ? OPSCV_VISIT(6, 4) : OPSCV_VISIT(6, 0);
                } else if (use_lds && nx_max <= 8) {
                    acc = OPSCV_VISIT(8, 0);
                } else if (use_lds) {
                    acc = visit_sum<float>(tile, pitch, tile_y0, tile_x0, in_y_start, in_x_start, out_y_start,
                                        out_x_start, (float)H, fw, scale_h, scale_w, last_y, last_x, Hd, Wd, ci, ch);
                } else {
                    acc = visit_sum<TI>(gp, Wde, 0, 0, in_y_start, in_x_start, out_y_start, out_x_start, (float)H, fw,
                                        scale_h, scale_w, last_y, last_x, Hd, Wd, ci, ch);
                }
#undef OPSCV_VISIT
                store_streaming<TO>(y + (pl * Hs + H) * (int64_t)Wse + W, acc);
            }
        }
        if (use_lds) {
            __syncthreads();  // the tile is overwritten by the next plane
        }
    }
}

// Output rows per workgroup for the LDS variant (0: use the gather kernel).  The estimate only sizes the launch;
// the kernel measures the rectangle itself.
template <typename TI>
int32_t lds_tile_rows(const ResizeGradArgs& a, int32_t cap_words, int32_t* need_words = nullptr)
{
    constexpr int EPW = 4 / (int)sizeof(TI);
    const int64_t ci = a.channels_last ? a.C : 1;  // row elements per pixel
    if (a.user_scales || (a.Wd * ci) % EPW != 0 || reinterpret_cast<uintptr_t>(a.x) % 4 != 0 ||
        a.Ws * ci > INT32_MAX || a.Wd * ci > INT32_MAX) {
        return 0;
    }
    const double per_col = (double)a.Wd / (double)a.Ws, per_row = (double)a.Hd / (double)a.Hs;
    // a tile of kTileCols outgoing elements visits that many times per_col incoming ones, plus two pixels either side
    const double cols = kTileCols * per_col + (2.0 * per_col + 2.0) * (double)ci + EPW;
    for (int32_t rows = 8; rows >= kTileGroups; rows /= 2) {
        const double need = (rows * per_row + 2.0 * per_row + 2.0) * cols;  // fp32 words: one per element
        if (need <= (double)cap_words) {
            if (need_words != nullptr) {
                *need_words = (int32_t)need + 1;
            }
            return rows;
        }
    }
    return 0;
}

template <typename TI, typename TO>
hipError_t run(const ResizeGradArgs& a, hipStream_t stream)
{
    constexpr int32_t kCapWords = kGradCapWords;
    int32_t lds_words = kCapWords;
    const int32_t tile_rows = lds_tile_rows<TI>(a, kCapWords, &lds_words);
    // the allocation follows the estimate so that more workgroups share a CU (their load and compute phases overlap);
    // a rectangle that turns out larger than the estimate is read from global memory by the kernel
    lds_words = (lds_words + 63) / 64 * 64;
    lds_words = lds_words < kCapWords ? lds_words : kCapWords;
    if (tile_rows > 0) {
        const int64_t ci = a.channels_last ? a.C : 1;
        const int64_t planes = a.channels_last ? a.N : a.N * a.C;
        const int64_t row_elems = a.Ws * ci;
        // A workgroup walks over several planes with the tile geometry and column weights it computed once; enough
        // workgroups are launched to keep every CU supplied (want_blocks), the rest of the planes are looped over.
        const int64_t tiles = ((row_elems + kTileCols - 1) / kTileCols) * ((a.Hs + tile_rows - 1) / tile_rows);
        const int64_t want_blocks = 8192;
        int64_t zdim = (want_blocks + tiles - 1) / tiles;
        zdim = zdim < planes ? zdim : planes;
        zdim = zdim < 65535 ? zdim : 65535;
        const int64_t tiles_x = (row_elems + kTileCols - 1) / kTileCols, tiles_y = (a.Hs + tile_rows - 1) / tile_rows;
        const int64_t blocks = (tiles * zdim + 7) / 8 * 8;  // padded for the XCD mapping of the kernel
        if (tiles_y <= 65535 && blocks <= (int64_t)INT32_MAX) {
            const dim3 grid((unsigned)blocks);
#define OPSCV_RGL(HP, IL)                                                                                            \
    hipLaunchKernelGGL((resize_grad_lds_kernel<TI, TO, HP, IL>), grid, dim3(kGradThreads), lds_words * 4, stream,     \
                       (const TI*)a.x, (TO*)a.y, planes, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, \
                       a.scale_h, a.scale_w, a.inv_scale_h, a.inv_scale_w, tile_rows, lds_words, -0.0f,              \
                       (uint32_t)tiles_x, (uint32_t)tiles_y, (uint32_t)zdim, (int32_t)ci)
            if (a.half_pixel) {
                if (a.channels_last) {
                    OPSCV_RGL(true, true);
                } else {
                    OPSCV_RGL(true, false);
                }
            } else {
                if (a.channels_last) {
                    OPSCV_RGL(false, true);
                } else {
                    OPSCV_RGL(false, false);
                }
            }
#undef OPSCV_RGL
            return hipGetLastError();
        }
    }
    const int64_t total = a.N * a.C * a.Hs * a.Ws;
    int64_t blocks = (total + kGradThreads - 1) / kGradThreads;
    if (blocks > 256 * 256) {
        blocks = 256 * 256;
    }
#define OPSCV_RG(HP, CL)                                                                                              \
    if (a.user_scales) {                                                                                              \
        hipLaunchKernelGGL((resize_grad_scales_kernel<TI, TO, HP, CL>), dim3((unsigned)blocks), dim3(kGradThreads),   \
                           0, stream, (const TI*)a.x, (TO*)a.y, total, (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws,    \
                           (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h, a.scale_w, a.inv_scale_h, a.inv_scale_w);         \
    } else {                                                                                                          \
        hipLaunchKernelGGL((resize_grad_kernel<TI, TO, HP, CL>), dim3((unsigned)blocks), dim3(kGradThreads), 0,       \
                           stream, (const TI*)a.x, (TO*)a.y, total, (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws,       \
                           (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h, a.scale_w, a.inv_scale_h, a.inv_scale_w);         \
    }
    if (a.half_pixel) {
        if (a.channels_last) {
            OPSCV_RG(true, true);
        } else {
            OPSCV_RG(true, false);
        }
    } else {
        if (a.channels_last) {
            OPSCV_RG(false, true);
        } else {
            OPSCV_RG(false, false);
        }
    }
#undef OPSCV_RG
    return hipGetLastError();
}

}  // namespace

const char* resize_grad_variant(const ResizeGradArgs& a)
{
    if (a.user_scales) {
        return "resize_grad_gather_scales";
    }
    constexpr int32_t kCapWords = kGradCapWords;
    const int32_t rows = (a.elem_in == Elem::F32) ? lds_tile_rows<float>(a, kCapWords)
                                                  : lds_tile_rows<uint16_t>(a, kCapWords);
    return (rows > 0 && (a.Hs + rows - 1) / rows <= 65535) ? "resize_grad_lds" : "resize_grad_gather";
}

hipError_t launch_resize_grad(const ResizeGradArgs& a, hipStream_t stream)
{
    const int64_t lim = INT32_MAX;
    if (a.N < 0 || a.C < 0 || a.Hs <= 0 || a.Ws <= 0 || a.Hd <= 0 || a.Wd <= 0 || a.Hs > lim || a.Ws > lim ||
        a.Hd > lim || a.Wd > lim || a.C > lim || a.N > lim) {
        return hipErrorInvalidValue;
    }
    if (a.N == 0 || a.C == 0) {
        return hipSuccess;
    }
    if (a.x == nullptr || a.y == nullptr) {
        return hipErrorInvalidValue;
    }
    if (a.copy) {
        if (a.elem_in != a.elem_out) {
            return hipErrorInvalidValue;
        }
        return hipMemcpyAsync(a.y, a.x, (size_t)(a.N * a.C * a.Hs * a.Ws) * elem_size(a.elem_in),
                              hipMemcpyDeviceToDevice, stream);
    }
    if (a.elem_in == Elem::F32) {
        switch (a.elem_out) {
            case Elem::F32: return run<float, float>(a, stream);
            case Elem::F16: return run<float, _Float16>(a, stream);
            case Elem::BF16: return run<float, __bf16>(a, stream);
        }
    }
    if (a.elem_in == Elem::F16 && a.elem_out == Elem::F16) {
        return run<_Float16, _Float16>(a, stream);
    }
    if (a.elem_in == Elem::BF16 && a.elem_out == Elem::BF16) {
        return run<__bf16, __bf16>(a, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
