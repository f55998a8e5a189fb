// Bilinear resize / upsample forward kernels for gfx950.
//
// Replaces the reference device kernels image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_simt_nchw.h:77-146
// (and the copy / broadcast templates selected in image/resize_bilinear_v2/op_kernel/resize_bilinear_v2_apt.cpp:42-115)
// and the host tiling image/resize_bilinear_v2/op_host/arch35/resize_bilinear_v2_tiling_arch35.cpp:175-243,592-623.
//
// Per axis: src = (dst + 0.5) * scale - 0.5 (half-pixel) or dst * scale (align corners), clamped at 0;
// taps floor/ceil clamped to size-1; lambda = src - floor(src);
// out = (1-dy) * ((1-dx)*TL + dx*TR) + dy * ((1-dx)*BL + dx*BR), every product and sum rounded separately
// (the file is compiled with -ffp-contract=off).
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "kernels.hpp"
#include "options.hpp"
#include "resize_band_lds_kernel.hpp"
#include "resize_math.hpp"
#include "sampler_math.hpp"

namespace opscv {

namespace {

constexpr int kThreads = 256;

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// 16-byte store that bypasses the caches (for outputs much larger than them)
// Outputs from this size on are written with non-temporal stores: the lines are written through instead of staying
// dirty in L2 until the end of the kernel writes them back (fp32 8x64x56x56 -> 112x112, 25.7 MB of output: 8.7 -> 6.7 us).
constexpr int64_t kResizeStreamingBytes = 1ll << 20;

__device__ __forceinline__ void store_streaming(uint4* dst, uint4 v)
{
    u32x4_t t;
    __builtin_memcpy(&t, &v, 16);
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4_t*>(dst));
}

// Generic NCHW variant: one lane per output pixel of a row, rows and planes on the other grid axes.
template <typename T, bool HALF_PIXEL>
__global__ __launch_bounds__(kThreads) void resize_nchw_generic_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                        int64_t planes, int32_t Hs, int32_t Ws,
                                                                        int32_t Hd, int32_t Wd, float scale_h,
                                                                        float scale_w, int raw_lambda)
{
    const int64_t rows = planes * Hd;
    const int32_t w = blockIdx.x * kThreads + threadIdx.x;
    if (w >= Wd) {
        return;
    }
    const AxisTap tx = axis_tap<HALF_PIXEL>(w, scale_w, Ws, raw_lambda);
    const float dx = tx.lambda;
    for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
        const int64_t pl = r / Hd;
        const int32_t h = (int32_t)(r - pl * Hd);
        const AxisTap ty = axis_tap<HALF_PIXEL>(h, scale_h, Hs, raw_lambda);
        const float dy = ty.lambda;
        const T* top = x + (pl * Hs + ty.i0) * (int64_t)Ws;
        const T* bot = x + (pl * Hs + ty.i1) * (int64_t)Ws;
        const float tl = ElemIO<T>::load(top + tx.i0);
        const float tr = ElemIO<T>::load(top + tx.i1);
        const float bl = ElemIO<T>::load(bot + tx.i0);
        const float br = ElemIO<T>::load(bot + tx.i1);
        const float out = (1.0f - dy) * ((1.0f - dx) * tl + dx * tr) + dy * ((1.0f - dx) * bl + dx * br);
        ElemIO<T>::store(y + r * Wd + w, out);
    }
}

// Row-band variant for NCHW, any width.
//
// A lane owns V = 16/sizeof(T) consecutive output columns and walks down a band of output rows.  The column
// taps (two source offsets and the lambda per column) are computed once per lane.  The reference formula
//     out = (1-dy) * ((1-dx)*TL + dx*TR) + dy * ((1-dx)*BL + dx*BR)
// is separable as written: the two inner terms depend on the source row only, so the horizontally blended
// source row  Hrow(y)[col] = (1-dx)*x[y,x0] + dx*x[y,x1]  is kept in registers and reused by every output row
// that touches source row y (two of them for a x2 upscale) -- same operations, same order, same bits.
// The two taps of a column are the same element or neighbours: they are fetched as one load of two elements
// (aligned to one element only, which global memory accesses allow) at column min(x0, Ws - 2).  Each lane writes
// one 16-byte vector per output row, at whatever alignment the row has (again element-aligned: rows of a width that
// is not a multiple of V start anywhere); the lane that holds the ragged end of a row stores its elements singly.
template <typename T, bool HALF_PIXEL, int BAND>
__global__ __launch_bounds__(kThreads) void resize_nchw_band_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                     int64_t planes, int32_t Hs, int32_t Ws,
                                                                     int32_t Hd, int32_t Wd, float scale_h,
                                                                     float scale_w, int raw_lambda)
{
    constexpr int V = 16 / (int)sizeof(T);
    using PairBits = typename std::conditional<sizeof(T) == 2, uint32_t, uint64_t>::type;
    const int32_t chunk = blockIdx.x * kThreads + threadIdx.x;
    const int32_t col0 = chunk * V;
    if (col0 >= Wd) {
        return;
    }
    const int32_t nvalid = (Wd - col0 < V) ? Wd - col0 : V;
    const bool pairs = Ws >= 2;
    int32_t xo0[V], xo1[V];  // pairs: xo0 = column of the pair; else the two tap columns
    uint32_t left_is_lo = 0, right_is_lo = 0;
    float dx[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        const int32_t c = (col0 + i < Wd) ? col0 + i : Wd - 1;
        const AxisTap t = axis_tap<HALF_PIXEL>(c, scale_w, Ws, raw_lambda);
        xo0[i] = t.i0;
        xo1[i] = t.i1;
        dx[i] = t.lambda;
        if (pairs) {
            const int32_t pb = (t.i0 < Ws - 2) ? t.i0 : Ws - 2;
            left_is_lo |= (uint32_t)(t.i0 == pb) << i;
            right_is_lo |= (uint32_t)(t.i1 == pb) << i;
            xo0[i] = pb;
        }
    }
    const int32_t h_begin = blockIdx.y * BAND;
    const int32_t h_end = (h_begin + BAND < Hd) ? h_begin + BAND : Hd;

    for (int64_t pl = blockIdx.z; pl < planes; pl += gridDim.z) {
        const T* xp = x + pl * Hs * (int64_t)Ws;
        T* yp = y + (pl * Hd + h_begin) * (int64_t)Wd + col0;
        float ha[V], hb[V];  // blended source rows ya and yb
        int32_t ya = -1, yb = -1;
        auto blend_row = [&](float* hrow, int32_t ys) {
            const T* row = xp + (int64_t)ys * Ws;
            if (pairs) {
                PairBits pr[V];
#pragma unroll
                for (int i = 0; i < V; i++) {
                    __builtin_memcpy(&pr[i], row + xo0[i], sizeof(PairBits));
                }
#pragma unroll
                for (int i = 0; i < V; i++) {
                    T two[2];
                    __builtin_memcpy(two, &pr[i], sizeof(PairBits));
                    const float lo = ElemIO<T>::load(&two[0]), hi = ElemIO<T>::load(&two[1]);
                    const float l = ((left_is_lo >> i) & 1u) ? lo : hi;
                    const float r = ((right_is_lo >> i) & 1u) ? lo : hi;
                    hrow[i] = (1.0f - dx[i]) * l + dx[i] * r;
                }
            } else {
#pragma unroll
                for (int i = 0; i < V; i++) {
                    const float l = ElemIO<T>::load(row + xo0[i]);
                    const float r = ElemIO<T>::load(row + xo1[i]);
                    hrow[i] = (1.0f - dx[i]) * l + dx[i] * r;
                }
            }
        };
        for (int32_t h = h_begin; h < h_end; h++) {
            const AxisTap ty = axis_tap<HALF_PIXEL>(h, scale_h, Hs, raw_lambda);
            const int32_t y0 = __builtin_amdgcn_readfirstlane(ty.i0);
            const int32_t y1 = __builtin_amdgcn_readfirstlane(ty.i1);
            const float dy = ty.lambda;
            // top row -> ha
            if (y0 != ya) {
                if (y0 == yb) {
#pragma unroll
                    for (int i = 0; i < V; i++) {
                        ha[i] = hb[i];
                    }
                } else {
                    blend_row(ha, y0);
                }
                ya = y0;
            }
            // bottom row -> hb (or ha again when both taps are the same source row)
            if (y1 != ya && y1 != yb) {
                blend_row(hb, y1);
                yb = y1;
            }
            T outv[V];
#pragma unroll
            for (int i = 0; i < V; i++) {
                const float bot = (y1 == ya) ? ha[i] : hb[i];
                const float o = (1.0f - dy) * ha[i] + dy * bot;
                ElemIO<T>::store(&outv[i], o);
            }
            if (nvalid == V) {
                typedef uint32_t u32x4_any __attribute__((ext_vector_type(4), aligned(2)));
                u32x4_any packed;
                __builtin_memcpy(&packed, outv, sizeof(packed));
                *reinterpret_cast<u32x4_any*>(yp) = packed;
            } else {
#pragma unroll
                for (int i = 0; i < V; i++) {
                    if (i < nvalid) {
                        yp[i] = outv[i];
                    }
                }
            }
            yp += Wd;
        }
    }
}

// Generic NHWC variant: one lane per (w, c) element of an output row.
template <typename T, bool HALF_PIXEL>
__global__ __launch_bounds__(kThreads) void resize_nhwc_generic_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                        int64_t N, int32_t C, int32_t Hs, int32_t Ws,
                                                                        int32_t Hd, int32_t Wd, float scale_h,
                                                                        float scale_w)
{
    const int64_t row_elems = (int64_t)Wd * C;
    const int64_t e = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= row_elems) {
        return;
    }
    const int32_t w = (int32_t)(e / C);
    const int32_t c = (int32_t)(e - (int64_t)w * C);
    const AxisTap tx = axis_tap<HALF_PIXEL>(w, scale_w, Ws);
    const float dx = tx.lambda;
    const int64_t rows = N * Hd;
    for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
        const int64_t n = r / Hd;
        const int32_t h = (int32_t)(r - n * Hd);
        const AxisTap ty = axis_tap<HALF_PIXEL>(h, scale_h, Hs);
        const float dy = ty.lambda;
        const T* top = x + ((n * Hs + ty.i0) * (int64_t)Ws) * C + c;
        const T* bot = x + ((n * Hs + ty.i1) * (int64_t)Ws) * C + c;
        const float tl = ElemIO<T>::load(top + (int64_t)tx.i0 * C);
        const float tr = ElemIO<T>::load(top + (int64_t)tx.i1 * C);
        const float bl = ElemIO<T>::load(bot + (int64_t)tx.i0 * C);
        const float br = ElemIO<T>::load(bot + (int64_t)tx.i1 * C);
        const float out = (1.0f - dy) * ((1.0f - dx) * tl + dx * tr) + dy * ((1.0f - dx) * bl + dx * br);
        ElemIO<T>::store(y + r * row_elems + e, out);
    }
}

// Vector NHWC variant: one lane per 16-byte run of channels of an output column (V = 16/sizeof(T) channels, needs
// C % V == 0 and 16-byte aligned tensors), walking down a band of BAND output rows.  The reference formula is
// separable as written, so the horizontally blended source row  (1-dx)*x[y,x0,c] + dx*x[y,x1,c]  stays in
// registers and is reused by every output row of the band that touches source row y (two of them for a x2
// upscale): two 16-byte loads per source row instead of four per output row, same operations in the same order.
constexpr int kNhwcBand = 8;

template <typename T, bool HALF_PIXEL, int BAND>
__global__ __launch_bounds__(kThreads) void resize_nhwc_vec_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                    int64_t N, int32_t C, int32_t Hs, int32_t Ws,
                                                                    int32_t Hd, int32_t Wd, float scale_h,
                                                                    float scale_w, int streaming)
{
    constexpr int V = 16 / (int)sizeof(T);
    const int32_t cvecs = C / V;
    const int64_t row_vecs = (int64_t)Wd * cvecs;
    const int64_t e = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= row_vecs) {
        return;
    }
    const int32_t w = (int32_t)(e / cvecs);
    const int32_t c = (int32_t)(e - (int64_t)w * cvecs) * V;
    const AxisTap tx = axis_tap<HALF_PIXEL>(w, scale_w, Ws);
    const float dx = tx.lambda;
    const float omdx = 1.0f - dx;
    const int64_t o0 = (int64_t)tx.i0 * C + c;
    const int64_t o1 = (int64_t)tx.i1 * C + c;
    const int64_t src_row = (int64_t)Ws * C;
    const int32_t h_begin = blockIdx.y * BAND;
    const int32_t h_end = (h_begin + BAND < Hd) ? h_begin + BAND : Hd;
    for (int64_t n = blockIdx.z; n < N; n += gridDim.z) {
        const T* xn = x + n * Hs * src_row;
        float ha[V], hb[V];  // blended source rows ya and yb
        int32_t ya = -1, yb = -1;
        auto blend_row = [&](float* hrow, int32_t ys) {
            const T* row = xn + (int64_t)ys * src_row;
            T l[V], r[V];
            uint4 raw = *reinterpret_cast<const uint4*>(row + o0);
            __builtin_memcpy(l, &raw, 16);
            raw = *reinterpret_cast<const uint4*>(row + o1);
            __builtin_memcpy(r, &raw, 16);
#pragma unroll
            for (int i = 0; i < V; i++) {
                hrow[i] = omdx * ElemIO<T>::load(&l[i]) + dx * ElemIO<T>::load(&r[i]);
            }
        };
        for (int32_t h = h_begin; h < h_end; h++) {
            const AxisTap ty = axis_tap<HALF_PIXEL>(h, scale_h, Hs);
            const int32_t y0 = __builtin_amdgcn_readfirstlane(ty.i0);
            const int32_t y1 = __builtin_amdgcn_readfirstlane(ty.i1);
            const float dy = ty.lambda;
            const float omdy = 1.0f - dy;
            if (y0 != ya) {
                if (y0 == yb) {
#pragma unroll
                    for (int i = 0; i < V; i++) {
                        ha[i] = hb[i];
                    }
                } else {
                    blend_row(ha, y0);
                }
                ya = y0;
            }
            if (y1 != ya && y1 != yb) {
                blend_row(hb, y1);
                yb = y1;
            }
            T outv[V];
#pragma unroll
            for (int i = 0; i < V; i++) {
                const float bot = (y1 == ya) ? ha[i] : hb[i];
                ElemIO<T>::store(&outv[i], omdy * ha[i] + dy * bot);
            }
            uint4 raw;
            __builtin_memcpy(&raw, outv, 16);
            uint4* dst = reinterpret_cast<uint4*>(y + ((n * Hd + h) * row_vecs + e) * V);
            if (streaming) {
                store_streaming(dst, raw);
            } else {
                *dst = raw;
            }
        }
    }
}

// Element-aligned copies of VB bytes (a run of channels of one pixel), built from power-of-two pieces so that each
// piece is one memory instruction: global memory accesses need only element alignment.
template <int VB>
__device__ __forceinline__ void copy_unit(void* dst, const void* src)
{
    char* d = static_cast<char*>(dst);
    const char* s = static_cast<const char*>(src);
    if constexpr (VB == 16) {
        typedef uint32_t u32x4_any __attribute__((ext_vector_type(4), aligned(2)));
        *reinterpret_cast<u32x4_any*>(d) = *reinterpret_cast<const u32x4_any*>(s);
    } else {
        if constexpr (VB >= 8) {
            uint64_t t;
            __builtin_memcpy(&t, s, 8);
            __builtin_memcpy(d, &t, 8);
        }
        if constexpr ((VB & 4) != 0) {
            uint32_t t;
            __builtin_memcpy(&t, s + (VB & 8), 4);
            __builtin_memcpy(d + (VB & 8), &t, 4);
        }
        if constexpr ((VB & 2) != 0) {
            uint16_t t;
            __builtin_memcpy(&t, s + (VB & 12), 2);
            __builtin_memcpy(d + (VB & 12), &t, 2);
        }
    }
}

// NHWC variant for channel counts that are not whole aligned 16-byte vectors (three-channel images, C = 20 ...): the
// band kernel above with a unit of VB bytes -- the widest of 16, 12, 8, 6, 4, 2 that divides a pixel's channels --
// moved by element-aligned loads and stores.  A lane owns UPL units next to each other in the output row and stores
// them as one run of UPL * VB bytes.  Same operations in the same order.
template <typename T, bool HALF_PIXEL, int BAND, int VB, int UPL>
__global__ __launch_bounds__(kThreads) void resize_nhwc_unit_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                     int64_t N, int32_t C, int32_t Hs, int32_t Ws,
                                                                     int32_t Hd, int32_t Wd, float scale_h,
                                                                     float scale_w)
{
    constexpr int V = VB / (int)sizeof(T);
    const int32_t cvecs = C / V;
    const int64_t row_vecs = (int64_t)Wd * cvecs;
    const int64_t e = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * UPL;
    if (e >= row_vecs) {
        return;
    }
    const bool whole = e + UPL <= row_vecs;
    float dx[UPL], omdx[UPL];
    int64_t o0[UPL], o1[UPL];
#pragma unroll
    for (int u = 0; u < UPL; u++) {
        const int64_t eu = (e + u < row_vecs) ? e + u : row_vecs - 1;  // past the row: a repeat that is never stored
        const int32_t w = (int32_t)(eu / cvecs);
        const int32_t c = (int32_t)(eu - (int64_t)w * cvecs) * V;
        const AxisTap tx = axis_tap<HALF_PIXEL>(w, scale_w, Ws);
        dx[u] = tx.lambda;
        omdx[u] = 1.0f - tx.lambda;
        o0[u] = (int64_t)tx.i0 * C + c;
        o1[u] = (int64_t)tx.i1 * C + c;
    }
    const int64_t src_row = (int64_t)Ws * C;
    const int32_t h_begin = blockIdx.y * BAND;
    const int32_t h_end = (h_begin + BAND < Hd) ? h_begin + BAND : Hd;
    for (int64_t n = blockIdx.z; n < N; n += gridDim.z) {
        const T* xn = x + n * Hs * src_row;
        float ha[UPL * V], hb[UPL * V];  // blended source rows ya and yb
        int32_t ya = -1, yb = -1;
        auto blend_row = [&](float* hrow, int32_t ys) {
            const T* row = xn + (int64_t)ys * src_row;
            T l[UPL * V], r[UPL * V];
#pragma unroll
            for (int u = 0; u < UPL; u++) {
                copy_unit<VB>(l + u * V, row + o0[u]);
                copy_unit<VB>(r + u * V, row + o1[u]);
            }
#pragma unroll
            for (int i = 0; i < UPL * V; i++) {
                hrow[i] = omdx[i / V] * ElemIO<T>::load(&l[i]) + dx[i / V] * ElemIO<T>::load(&r[i]);
            }
        };
        for (int32_t h = h_begin; h < h_end; h++) {
            const AxisTap ty = axis_tap<HALF_PIXEL>(h, scale_h, Hs);
            const int32_t y0 = __builtin_amdgcn_readfirstlane(ty.i0);
            const int32_t y1 = __builtin_amdgcn_readfirstlane(ty.i1);
            const float dy = ty.lambda;
            const float omdy = 1.0f - dy;
            if (y0 != ya) {
                if (y0 == yb) {
#pragma unroll
                    for (int i = 0; i < UPL * V; i++) {
                        ha[i] = hb[i];
                    }
                } else {
                    blend_row(ha, y0);
                }
                ya = y0;
            }
            if (y1 != ya && y1 != yb) {
                blend_row(hb, y1);
                yb = y1;
            }
            T outv[UPL * V];
#pragma unroll
            for (int i = 0; i < UPL * V; i++) {
                const float bot = (y1 == ya) ? ha[i] : hb[i];
                ElemIO<T>::store(&outv[i], omdy * ha[i] + dy * bot);
            }
            T* dst = y + ((n * Hd + h) * row_vecs + e) * V;
            if (whole) {
                copy_unit<UPL * VB>(dst, outv);
            } else {
                for (int u = 0; u < UPL && e + u < row_vecs; u++) {
                    copy_unit<VB>(dst + u * V, outv + u * V);
                }
            }
        }
    }
}

// Four-weights NHWC variant (image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_c_parallel.h:122-147,190-232):
// the reference's template for channel runs of 128 bytes and more shrunk to half or less forms the four corner weights
//   (1-dy)(1-dx), (1-dy)dx, dy(1-dx), dy*dx
// first and adds  (NW*w + NE*w) + (SW*w + SE*w),  which rounds differently from the nested blends of the per-element
// template.  Its taps are "floor, then +1 when the fraction is positive"; for the non-negative source positions that a
// scale of two or more produces these are the floor/ceil taps of axis_tap().  One lane per run of UE channels of an
// output pixel; a shrink of two or more touches every source pixel at most once, so there is nothing to reuse.
template <typename T, bool HALF_PIXEL, int UE>
__global__ __launch_bounds__(kThreads) void resize_nhwc_four_weights_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                             int64_t N, int32_t C, int32_t Hs,
                                                                             int32_t Ws, int32_t Hd, int32_t Wd,
                                                                             float scale_h, float scale_w,
                                                                             int streaming)
{
    typedef uint32_t words_t __attribute__((ext_vector_type((UE * sizeof(T) >= 4) ? UE * sizeof(T) / 4 : 1)));
    const int32_t units = C / UE;
    const int64_t row_units = (int64_t)Wd * units;
    const int64_t e = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= row_units) {
        return;
    }
    const int32_t w = (int32_t)(e / units);
    const int32_t c = (int32_t)(e - (int64_t)w * units) * UE;
    const AxisTap tx = axis_tap<HALF_PIXEL>(w, scale_w, Ws);
    const float dx = tx.lambda;
    const int64_t o0 = (int64_t)tx.i0 * C + c;
    const int64_t o1 = (int64_t)tx.i1 * C + c;
    const int64_t src_row = (int64_t)Ws * C;
    const int64_t rows = N * Hd;
    auto fetch = [&](T* dst, const T* src) {
        if (UE * sizeof(T) >= 4) {
            const words_t raw = *reinterpret_cast<const words_t*>(src);
            __builtin_memcpy(dst, &raw, UE * sizeof(T));
        } else {
            dst[0] = src[0];
        }
    };
    for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
        const int64_t n = r / Hd;
        const int32_t h = (int32_t)(r - n * Hd);
        const AxisTap ty = axis_tap<HALF_PIXEL>(h, scale_h, Hs);
        const float dy = ty.lambda;
        const float w_nw = (1.0f - dy) * (1.0f - dx);
        const float w_ne = (1.0f - dy) * dx;
        const float w_sw = dy * (1.0f - dx);
        const float w_se = dy * dx;
        const T* top = x + (n * Hs + ty.i0) * src_row;
        const T* bot = x + (n * Hs + ty.i1) * src_row;
        T nw[UE], ne[UE], sw[UE], se[UE], outv[UE];
        fetch(nw, top + o0);
        fetch(ne, top + o1);
        fetch(sw, bot + o0);
        fetch(se, bot + o1);
#pragma unroll
        for (int i = 0; i < UE; i++) {
            const float sum_top = ElemIO<T>::load(&nw[i]) * w_nw + ElemIO<T>::load(&ne[i]) * w_ne;
            const float sum_bot = ElemIO<T>::load(&sw[i]) * w_sw + ElemIO<T>::load(&se[i]) * w_se;
            ElemIO<T>::store(&outv[i], sum_top + sum_bot);
        }
        T* dst = y + (r * row_units + e) * UE;
        if (UE * sizeof(T) >= 4) {
            words_t raw;
            __builtin_memcpy(&raw, outv, UE * sizeof(T));
            if (streaming) {
                __builtin_nontemporal_store(raw, reinterpret_cast<words_t*>(dst));
            } else {
                *reinterpret_cast<words_t*>(dst) = raw;
            }
        } else {
            dst[0] = outv[0];
        }
    }
}

// Nearest-neighbour resize (align_corners = false, half_pixel_centers = false):
//   src = min(floor(float(dst) * scale), len_src - 1)
// image/resize_nearest_neighbor_v2/op_kernel/arch35/resize_nearest_neighbor_v2_simt.h:103-124.
// With rep > 0: src = dst / rep in integer arithmetic, the rule of the reference's channels-last template that
// replicates every source pixel a whole number of times (resize_nearest_neighbor_v2_data_copy_nhwc.h:205-231; the
// launch plan says when the reference takes it).  The two first differ at a factor of 41.
__device__ __forceinline__ int32_t nearest_src(int32_t d, float scale, int32_t len_src, int32_t rep)
{
    if (rep > 0) {
        return d / rep;
    }
    const float f = __builtin_floorf((float)d * scale);
    // the reference converts to an unsigned index and clamps from above only; dst and scale are non-negative
    const int32_t i = (f >= 2147483648.0f) ? INT32_MAX : (int32_t)f;
    return (i < len_src - 1) ? i : len_src - 1;
}

// scales of the float rule, factors of the replicating rule (0: the float rule)
struct NearestRule {
    float scale_h, scale_w;
    int32_t rep_h, rep_w;
};

constexpr int kNearestBand = 8;

// A pure gather-copy: V = 16/sizeof(T) (VEC) or 1 output elements per lane along the contiguous axis.
// NCHW: the contiguous axis is w, each element has its own source column.  NHWC: the contiguous axis is (w, c);
// a vector never straddles a pixel because VEC requires C % V == 0.
template <typename T, bool NHWC, bool VEC>
__global__ __launch_bounds__(kThreads) void resize_nearest_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                   int64_t outer, int32_t C, int32_t Hs, int32_t Ws,
                                                                   int32_t Hd, int32_t Wd, NearestRule rule, int streaming)
{
    constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
    const int64_t row_elems = NHWC ? (int64_t)Wd * C : (int64_t)Wd;
    const int64_t src_row_elems = NHWC ? (int64_t)Ws * C : (int64_t)Ws;
    const int64_t e0 = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * V;
    if (e0 >= row_elems) {
        return;
    }
    int64_t src_off[NHWC ? 1 : V];
    if (NHWC) {
        const int32_t w = (int32_t)(e0 / C);
        const int32_t c = (int32_t)(e0 - (int64_t)w * C);
        src_off[0] = (int64_t)nearest_src(w, rule.scale_w, Ws, rule.rep_w) * C + c;
    } else {
#pragma unroll
        for (int i = 0; i < V; i++) {
            const int32_t col = ((int32_t)e0 + i < Wd) ? (int32_t)e0 + i : Wd - 1;  // past a ragged row end: unused
            src_off[i] = nearest_src(col, rule.scale_w, Ws, rule.rep_w);
        }
    }
    // NCHW rows of any width: the vector store is element-aligned, the lane at a ragged row end stores singly
    const int nvalid = (row_elems - e0 < V) ? (int)(row_elems - e0) : V;
    const int64_t rows = outer * Hd;  // outer = N*C planes (NCHW) or N images (NHWC)
    // a workgroup copies kNearestBand consecutive output rows per step: the column offsets above are reused and
    // neighbouring output rows of an upscale read the same source row out of L1
    for (int64_t r0 = (int64_t)blockIdx.y * kNearestBand; r0 < rows; r0 += (int64_t)gridDim.y * kNearestBand) {
      const int64_t r_end = (r0 + kNearestBand < rows) ? r0 + kNearestBand : rows;
      for (int64_t r = r0; r < r_end; r++) {
        const int64_t o = r / Hd;
        const int32_t h = (int32_t)(r - o * Hd);
        const T* src = x + (o * Hs + nearest_src(h, rule.scale_h, Hs, rule.rep_h)) * src_row_elems;
        T* dst = y + r * row_elems + e0;
        if (VEC) {
            uint4 packed;
            if (NHWC) {
                packed = *reinterpret_cast<const uint4*>(src + src_off[0]);
            } else {
                T v[V];
#pragma unroll
                for (int i = 0; i < V; i++) {
                    v[i] = src[src_off[i]];
                }
                __builtin_memcpy(&packed, v, sizeof(packed));
            }
            if (NHWC) {
                if (streaming) {
                    store_streaming(reinterpret_cast<uint4*>(dst), packed);
                } else {
                    *reinterpret_cast<uint4*>(dst) = packed;
                }
            } else if (nvalid == V) {
                typedef uint32_t u32x4_any __attribute__((ext_vector_type(4), aligned(2)));
                u32x4_any t;
                __builtin_memcpy(&t, &packed, 16);
                if (streaming) {
                    __builtin_nontemporal_store(t, reinterpret_cast<u32x4_any*>(dst));
                } else {
                    *reinterpret_cast<u32x4_any*>(dst) = t;
                }
            } else {
                T v[V];
                __builtin_memcpy(v, &packed, 16);
#pragma unroll
                for (int i = 0; i < V; i++) {
                    if (i < nvalid) {
                        dst[i] = v[i];
                    }
                }
            }
        } else {
            dst[0] = src[src_off[0]];
        }
      }
    }
}

// Nearest, NCHW, whole 16-byte output vectors, source rows staged in LDS.  Per element the gather-copy above issues a
// two-byte global load, which binds it to the address rate of the memory pipeline rather than to memory.  Here a
// workgroup owns (chunk of 256 output vectors, band of kNearestBand output rows): the source-row segments the chunk
// reads -- one per distinct source row of the band, each a single 16-byte aligned byte range -- are copied into LDS
// with the asynchronous global->LDS loads, and a lane assembles its vector from V two-byte LDS reads, once per
// distinct source row.  Needs source rows that are whole 16-byte vectors (Ws % V == 0, aligned base); the output may
// have any width.
template <typename T>
__global__ __launch_bounds__(kThreads) void resize_nearest_lds_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                       int64_t outer, int32_t Hs, int32_t Ws,
                                                                       int32_t Hd, int32_t Wd, NearestRule rule,
                                                                       uint32_t slot_bytes, int streaming, int32_t ci)
{
    // ci = 1: planes of Hs x Ws.  ci = C: channels-last images, resized as planes whose rows are Ws * C elements
    // (element j of a row is channel j % C of pixel j / C); "columns" below are row elements.
    constexpr int V = 16 / (int)sizeof(T);
    extern __shared__ uint4 nearest_smem[];
    char* lds = reinterpret_cast<char*>(nearest_smem);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)tid >> 6);
    const int32_t Wse = Ws * ci, Wde = Wd * ci;
    const int32_t col_first = blockIdx.x * kThreads * V;
    const int32_t col_last = ((col_first + kThreads * V < Wde) ? col_first + kThreads * V : Wde) - 1;
    const int32_t s_lo = nearest_src(col_first / ci, rule.scale_w, Ws, rule.rep_w) * ci / V * V;
    const int32_t s_hi = nearest_src(col_last / ci, rule.scale_w, Ws, rule.rep_w) * ci + ci - 1;
    const uint32_t seg_bytes = (uint32_t)((s_hi - s_lo) / V + 1) * 16u;
    const bool use_lds = seg_bytes <= slot_bytes;  // uniform; the launch sizes the slots so that this holds
    const int32_t e0 = col_first + tid * V;
    const bool active = e0 < Wde;
    const int nvalid = (Wde - e0 < V) ? Wde - e0 : V;
    int32_t src_col[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        const int32_t c = (e0 + i < Wde) ? e0 + i : Wde - 1;
        const int32_t px = (ci == 1) ? c : c / ci;
        src_col[i] = nearest_src(px, rule.scale_w, Ws, rule.rep_w) * ci + (c - px * ci);
    }
    const int64_t rows = outer * Hd;
    for (int64_t r0 = (int64_t)blockIdx.y * kNearestBand; r0 < rows; r0 += (int64_t)gridDim.y * kNearestBand) {
        int64_t src_row[kNearestBand];
        int slot_of[kNearestBand];
        int nslots = 0;
        int64_t prev = -1;
#pragma unroll
        for (int j = 0; j < kNearestBand; j++) {
            const int64_t r = r0 + j;
            if (r < rows) {
                const int64_t o = r / Hd;
                const int32_t h = (int32_t)(r - o * Hd);
                src_row[j] = o * Hs + nearest_src(h, rule.scale_h, Hs, rule.rep_h);
                if (src_row[j] != prev) {
                    if (use_lds) {
                        const char* src = reinterpret_cast<const char*>(x + src_row[j] * (int64_t)Wse + s_lo);
                        for (uint32_t cb = wave * 1024u; cb < seg_bytes; cb += (kThreads / 64) * 1024u) {
                            const uint32_t lane_off = cb + (uint32_t)lane * 16u;
                            if (lane_off < seg_bytes) {
                                __builtin_amdgcn_global_load_lds((rs_global_cptr_t)(src + lane_off),
                                                                 (rs_lds_ptr_t)(lds + nslots * slot_bytes + cb), 16, 0,
                                                                 0);
                            }
                        }
                    }
                    nslots++;
                    prev = src_row[j];
                }
                slot_of[j] = nslots - 1;
            } else {
                src_row[j] = -1;
                slot_of[j] = -1;
            }
        }
        if (use_lds) {
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
        }
        if (active) {
            int last = -1;
            uint4 packed = make_uint4(0, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < kNearestBand; j++) {
                if (slot_of[j] < 0) {
                    continue;
                }
                if (slot_of[j] != last) {
                    T v[V];
                    if (use_lds) {
                        const T* seg = reinterpret_cast<const T*>(lds + slot_of[j] * slot_bytes);
#pragma unroll
                        for (int i = 0; i < V; i++) {
                            v[i] = seg[src_col[i] - s_lo];
                        }
                    } else {
                        const T* src = x + src_row[j] * (int64_t)Wse;
#pragma unroll
                        for (int i = 0; i < V; i++) {
                            v[i] = src[src_col[i]];
                        }
                    }
                    __builtin_memcpy(&packed, v, sizeof(packed));
                    last = slot_of[j];
                }
                // rows of a width that is not a multiple of V start anywhere: the vector store is element-aligned,
                // and the lane at the ragged end of a row stores its elements singly
                T* dst = y + (r0 + j) * (int64_t)Wde + e0;
                if (nvalid == V) {
                    typedef uint32_t u32x4_any __attribute__((ext_vector_type(4), aligned(2)));
                    u32x4_any t;
                    __builtin_memcpy(&t, &packed, 16);
                    if (streaming) {
                        __builtin_nontemporal_store(t, reinterpret_cast<u32x4_any*>(dst));
                    } else {
                        *reinterpret_cast<u32x4_any*>(dst) = t;
                    }
                } else {
                    T v[V];
                    __builtin_memcpy(v, &packed, 16);
#pragma unroll
                    for (int i = 0; i < V; i++) {
                        if (i < nvalid) {
                            dst[i] = v[i];
                        }
                    }
                }
            }
        }
        if (use_lds) {
            __syncthreads();  // the slots are refilled by the next band
        }
    }
}

// Point copy (channels-last, whole shrink factors whose sampling points are source pixels): every destination pixel
// is the copy of one source pixel.  Source index as in
// image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_point_copy.h:117-124, clamped to the last pixel.
// U is the unit copied per lane: a 16-byte vector when a pixel's channels are whole vectors, else one element.
template <typename U>
__global__ __launch_bounds__(kThreads) void resize_point_copy_kernel(const U* __restrict__ x, U* __restrict__ y,
                                                                      int64_t total, int32_t units, int32_t Hs,
                                                                      int32_t Ws, int32_t Hd, int32_t Wd,
                                                                      int64_t step_h, int64_t step_w, int half_pixel)
{
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
        int64_t r = i;
        const int32_t u = (int32_t)(r % units);
        r /= units;
        const int64_t w = r % Wd;
        r /= Wd;
        const int64_t h = r % Hd;
        const int64_t n = r / Hd;
        int64_t hs = half_pixel ? ((2 * h + 1) * step_h - 1) / 2 : h * step_h;
        int64_t ws = half_pixel ? ((2 * w + 1) * step_w - 1) / 2 : w * step_w;
        hs = (hs < Hs - 1) ? hs : Hs - 1;
        ws = (ws < Ws - 1) ? ws : Ws - 1;
        y[i] = x[((n * Hs + hs) * Ws + ws) * units + u];
    }
}

// Broadcast of one source element per plane (mode Broadcast: 1x1 source; FirstPixel: 1x1 destination).
// For NHWC the "plane" index is (n, c) with element stride C inside a batch.
template <typename T>
__global__ __launch_bounds__(kThreads) void resize_fill_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                int64_t N, int64_t C, int64_t src_hw, int64_t dst_hw,
                                                                int channels_last)
{
    const int64_t total = N * C * dst_hw;
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
        int64_t src;
        if (channels_last) {
            const int64_t n = i / (dst_hw * C);
            const int64_t c = i % C;
            src = n * src_hw * C + c;
        } else {
            src = (i / dst_hw) * src_hw;
        }
        y[i] = x[src];
    }
}

constexpr int kBand = 32;  // output rows a workgroup walks down (vertical reuse of blended source rows)

// The band variant serves every NCHW shape whose band count fits the grid (its vector stores are element-aligned).
template <typename T>
bool band_variant_ok(const ResizeArgs& a)
{
    if (a.channels_last || a.mode != ResizeMode::Bilinear) {
        return false;
    }
    if (reinterpret_cast<uintptr_t>(a.x) % sizeof(T) != 0 || reinterpret_cast<uintptr_t>(a.y) % sizeof(T) != 0) {
        return false;
    }
    if ((a.Hd + kBand - 1) / kBand > 65535) {
        return false;
    }
    return a.force_variant != kResizeGeneric;  // option "resize_variant" = generic forces the generic kernel
}

// The vector NHWC variant moves whole 16-byte runs of channels.
template <typename T>
bool nhwc_vec_ok(const ResizeArgs& a)
{
    constexpr int V = 16 / (int)sizeof(T);
    return a.channels_last && a.mode == ResizeMode::Bilinear && a.C % V == 0 &&
           (a.Hd + kNhwcBand - 1) / kNhwcBand <= 65535 && reinterpret_cast<uintptr_t>(a.x) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(a.y) % 16 == 0;
}

// Bytes per lane of the element-aligned NHWC band variant: the widest of 16, 12, 8, 6, 4, 2 that divides the bytes of
// a pixel's channels; 0 when the variant does not apply (the per-element kernel runs).
template <typename T>
int nhwc_unit_bytes(const ResizeArgs& a)
{
    const int esz = (int)sizeof(T);
    if (!a.channels_last || a.mode != ResizeMode::Bilinear || (a.Hd + kNhwcBand - 1) / kNhwcBand > 65535 ||
        reinterpret_cast<uintptr_t>(a.x) % esz != 0 || reinterpret_cast<uintptr_t>(a.y) % esz != 0) {
        return 0;
    }
    if (a.force_variant == kResizeGeneric) {
        return 0;
    }
    const int64_t pixel_bytes = a.C * esz;
    static const int kUnits[6] = {16, 12, 8, 6, 4, 2};
    for (int u : kUnits) {
        if (u % esz == 0 && pixel_bytes % u == 0) {
            return u;
        }
    }
    return 0;
}

// Channels per lane of the four-weights kernel: the widest of 16 bytes, 8 bytes or one element that divides C and
// that both tensors are aligned to.
template <typename T>
int four_weights_unit(const ResizeArgs& a)
{
    constexpr int V = 16 / (int)sizeof(T);
    const uintptr_t both = reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.y);
    if (a.C % V == 0 && both % 16 == 0) {
        return V;
    }
    if (a.C % (V / 2) == 0 && both % 8 == 0) {
        return V / 2;
    }
    return 1;
}

// LDS bytes per staged source-row segment of the nearest kernel that gathers out of LDS, 0 when that kernel does not
// apply.  It serves NCHW planes and channels-last images whose pixels are not whole 16-byte vectors (rows of Ws * C
// elements), with source rows on the 16-byte grid.  The slot is the longest source segment a chunk of kThreads
// vectors can touch, with slack for the rounding of the per-column products; the kernel checks the real length and
// gathers from global memory otherwise.
template <typename T>
uint64_t nearest_lds_slot(const ResizeArgs& a)
{
    constexpr int V = 16 / (int)sizeof(T);
    const bool nhwc = a.channels_last != 0;
    const int64_t ci = nhwc ? a.C : 1;
    if (a.mode != ResizeMode::Nearest || reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || (a.Ws * ci) % V != 0 ||
        a.Ws * ci > INT32_MAX || a.Wd * ci > INT32_MAX) {
        return 0;
    }
    if (nhwc && (a.C % V == 0 || reinterpret_cast<uintptr_t>(a.y) % sizeof(T) != 0)) {
        return 0;  // whole vectors per pixel: one vector load per lane does it
    }
    if (nhwc && a.Hd * a.Wd < a.Hs * a.Ws) {
        return 0;  // shrinking images: nothing is reused, the gather from memory is as fast (measured)
    }
    if (a.force_nearest == kNearestGather) {
        return 0;
    }
    const double span = (double)(kThreads * V) * (double)a.scale_w * 1.001 + 2.0 + 2.0 * V + 2.0 * (double)ci;
    const uint64_t slot = ((uint64_t)(span * sizeof(T)) + 15u) / 16u * 16u;
    return (slot * kNearestBand <= 64u * 1024u) ? slot : 0;
}

template <typename T>
hipError_t run_resize(const ResizeArgs& a, hipStream_t stream)
{
    const T* x = (const T*)a.x;
    T* y = (T*)a.y;
    const int64_t out_elems = a.N * a.C * a.Hd * a.Wd;
    if (a.mode == ResizeMode::Copy) {
        return hipMemcpyAsync(y, x, (size_t)out_elems * sizeof(T), hipMemcpyDeviceToDevice, stream);
    }
    if (a.mode == ResizeMode::PointCopy) {
        constexpr int V = 16 / (int)sizeof(T);
        const bool vec = a.C % V == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
        const int64_t units = vec ? a.C / V : a.C;
        const int64_t total = a.N * a.Hd * a.Wd * units;
        int64_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 256 * 256) {
            blocks = 256 * 256;
        }
        if (vec) {
            hipLaunchKernelGGL((resize_point_copy_kernel<uint4>), dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                               reinterpret_cast<const uint4*>(x), reinterpret_cast<uint4*>(y), total, (int32_t)units,
                               (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.point_step_h,
                               a.point_step_w, a.half_pixel);
        } else {
            hipLaunchKernelGGL((resize_point_copy_kernel<T>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, x, y,
                               total, (int32_t)units, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd,
                               a.point_step_h, a.point_step_w, a.half_pixel);
        }
        return hipGetLastError();
    }
    if (a.mode == ResizeMode::Broadcast || a.mode == ResizeMode::FirstPixel) {
        int64_t blocks = (out_elems + kThreads - 1) / kThreads;
        if (blocks > 256 * 64) {
            blocks = 256 * 64;
        }
        hipLaunchKernelGGL((resize_fill_kernel<T>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, x, y, a.N, a.C,
                           a.Hs * a.Ws, a.Hd * a.Wd, a.channels_last);
        return hipGetLastError();
    }
    if (a.mode == ResizeMode::Nearest) {
        constexpr int V = 16 / (int)sizeof(T);
        const bool nhwc = a.channels_last != 0;
        const int64_t row_elems = nhwc ? a.Wd * a.C : a.Wd;
        const int64_t outer = nhwc ? a.N : a.N * a.C;
        const int64_t rows = outer * a.Hd;
        const bool aligned = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
        // whole 16-byte vectors: rows start aligned (row_elems % V == 0); for NHWC a vector stays inside one pixel
        // (NCHW takes vectors at any width and alignment: its loads are per element, its stores element-aligned)
        const bool whole = aligned && row_elems % V == 0;
        const bool vec = nhwc ? (whole && a.C % V == 0 && (a.Ws * a.C) % V == 0) : true;
        const int64_t lanes = vec ? (row_elems + V - 1) / V : row_elems;
        const int64_t bands = (rows + kNearestBand - 1) / kNearestBand;
        dim3 grid((unsigned)((lanes + kThreads - 1) / kThreads), (unsigned)(bands < 65535 ? bands : 65535));
#define OPSCV_NEAREST(NHWC_, VEC_)                                                                                  \
    hipLaunchKernelGGL((resize_nearest_kernel<T, NHWC_, VEC_>), grid, dim3(kThreads), 0, stream, x, y, outer,      \
                       (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, rule, streaming)
        const int streaming = (out_elems * (int64_t)sizeof(T) >= kResizeStreamingBytes) ? 1 : 0;
        const NearestRule rule{a.scale_h, a.scale_w, a.rep_h, a.rep_w};
        if (const uint64_t slot = nearest_lds_slot<T>(a)) {
            const int64_t vlanes = (row_elems + V - 1) / V;
            dim3 lgrid((unsigned)((vlanes + kThreads - 1) / kThreads), (unsigned)(bands < 65535 ? bands : 65535));
            hipLaunchKernelGGL((resize_nearest_lds_kernel<T>), lgrid, dim3(kThreads), slot * kNearestBand, stream, x, y,
                               outer, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, rule, (uint32_t)slot,
                               streaming, (int32_t)(nhwc ? a.C : 1));
            return hipGetLastError();
        }
        if (nhwc) {
            if (vec) {
                OPSCV_NEAREST(true, true);
            } else {
                OPSCV_NEAREST(true, false);
            }
        } else {
            if (vec) {
                OPSCV_NEAREST(false, true);
            } else {
                OPSCV_NEAREST(false, false);
            }
        }
#undef OPSCV_NEAREST
        return hipGetLastError();
    }
    if (a.mode == ResizeMode::FourWeights) {
        constexpr int V = 16 / (int)sizeof(T);
        const int ue = four_weights_unit<T>(a);
        const int64_t row_units = a.Wd * (a.C / ue);
        const int64_t rows = a.N * a.Hd;
        const int streaming = (out_elems * (int64_t)sizeof(T) >= kResizeStreamingBytes) ? 1 : 0;
        dim3 grid((unsigned)((row_units + kThreads - 1) / kThreads), (unsigned)(rows < 65535 ? rows : 65535));
#define OPSCV_FOUR(HP, UE)                                                                                           \
    hipLaunchKernelGGL((resize_nhwc_four_weights_kernel<T, HP, UE>), grid, dim3(kThreads), 0, stream, x, y, a.N,      \
                       (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h,           \
                       a.scale_w, streaming)
        if (a.half_pixel) {
            if (ue == V) {
                OPSCV_FOUR(true, V);
            } else if (ue == V / 2) {
                OPSCV_FOUR(true, V / 2);
            } else {
                OPSCV_FOUR(true, 1);
            }
        } else {
            if (ue == V) {
                OPSCV_FOUR(false, V);
            } else if (ue == V / 2) {
                OPSCV_FOUR(false, V / 2);
            } else {
                OPSCV_FOUR(false, 1);
            }
        }
#undef OPSCV_FOUR
        return hipGetLastError();
    }
    if (nhwc_vec_ok<T>(a)) {
        constexpr int V = 16 / (int)sizeof(T);
        const int64_t row_vecs = a.Wd * (a.C / V);
        const int64_t bands = (a.Hd + kNhwcBand - 1) / kNhwcBand;
        const int streaming = (out_elems * (int64_t)sizeof(T) >= kResizeStreamingBytes) ? 1 : 0;
        dim3 grid((unsigned)((row_vecs + kThreads - 1) / kThreads), (unsigned)bands,
                  (unsigned)(a.N < 65535 ? a.N : 65535));
        if (a.half_pixel) {
            hipLaunchKernelGGL((resize_nhwc_vec_kernel<T, true, kNhwcBand>), grid, dim3(kThreads), 0, stream, x, y, a.N,
                               (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h,
                               a.scale_w, streaming);
        } else {
            hipLaunchKernelGGL((resize_nhwc_vec_kernel<T, false, kNhwcBand>), grid, dim3(kThreads), 0, stream, x, y, a.N,
                               (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h,
                               a.scale_w, streaming);
        }
        return hipGetLastError();
    }
    if (a.channels_last) {
        if (!nhwc_vec_ok<T>(a)) {
            // pixels that are not whole vectors: rows of Ws * C elements through the LDS-staged band kernel
            bool handled = false;
            const hipError_t e = run_resize_band_lds(a, stream, &handled);
            if (handled || e != hipSuccess) {
                return e;
            }
        }
        const int vb = nhwc_unit_bytes<T>(a);
        if (vb != 0) {
            // Units per lane.  Several units of 2 or 4 bytes per lane make the stores 16 bytes wide, which pays when
            // rows grow (neighbouring units read neighbouring source pixels); when rows shrink, and for wider units,
            // the lanes' loads coalesce better with one unit each.
            const int upl = (vb > 4 || a.Wd < a.Ws) ? 1 : 16 / vb;
            const int64_t row_lanes = (a.Wd * (a.C * (int64_t)sizeof(T) / vb) + upl - 1) / upl;
            const int64_t bands = (a.Hd + kNhwcBand - 1) / kNhwcBand;
            dim3 grid((unsigned)((row_lanes + kThreads - 1) / kThreads), (unsigned)bands,
                      (unsigned)(a.N < 65535 ? a.N : 65535));
#define OPSCV_NHWC_UNIT(HP, VB, UPL)                                                                                 \
    hipLaunchKernelGGL((resize_nhwc_unit_kernel<T, HP, kNhwcBand, VB, UPL>), grid, dim3(kThreads), 0, stream, x, y,   \
                       a.N, (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h,      \
                       a.scale_w)
#define OPSCV_NHWC_UNITS(HP)                                                                                         \
    switch (vb * 16 + upl) {                                                                                         \
        case 16 * 16 + 1: OPSCV_NHWC_UNIT(HP, 16, 1); break;                                                         \
        case 12 * 16 + 1: OPSCV_NHWC_UNIT(HP, 12, 1); break;                                                         \
        case 8 * 16 + 1: OPSCV_NHWC_UNIT(HP, 8, 1); break;                                                           \
        case 6 * 16 + 1: if constexpr (sizeof(T) == 2) { OPSCV_NHWC_UNIT(HP, 6, 1); } break;                         \
        case 4 * 16 + 1: OPSCV_NHWC_UNIT(HP, 4, 1); break;                                                           \
        case 4 * 16 + 4: OPSCV_NHWC_UNIT(HP, 4, 4); break;                                                           \
        case 2 * 16 + 1: if constexpr (sizeof(T) == 2) { OPSCV_NHWC_UNIT(HP, 2, 1); } break;                         \
        default: if constexpr (sizeof(T) == 2) { OPSCV_NHWC_UNIT(HP, 2, 8); } break;                                 \
    }
            if (a.half_pixel) {
                OPSCV_NHWC_UNITS(true)
            } else {
                OPSCV_NHWC_UNITS(false)
            }
#undef OPSCV_NHWC_UNITS
#undef OPSCV_NHWC_UNIT
            return hipGetLastError();
        }
        const int64_t row_elems = a.Wd * a.C;
        const int64_t rows = a.N * a.Hd;
        dim3 grid((unsigned)((row_elems + kThreads - 1) / kThreads), (unsigned)(rows < 65535 ? rows : 65535));
        if (a.half_pixel) {
            hipLaunchKernelGGL((resize_nhwc_generic_kernel<T, true>), grid, dim3(kThreads), 0, stream, x, y, a.N,
                               (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h,
                               a.scale_w);
        } else {
            hipLaunchKernelGGL((resize_nhwc_generic_kernel<T, false>), grid, dim3(kThreads), 0, stream, x, y, a.N,
                               (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h,
                               a.scale_w);
        }
        return hipGetLastError();
    }
    const int64_t planes = a.N * a.C;
    {
        bool handled = false;
        const hipError_t e = run_resize_band_lds(a, stream, &handled);
        if (handled || e != hipSuccess) {
            return e;
        }
    }
    if (band_variant_ok<T>(a)) {
        constexpr int V = 16 / (int)sizeof(T);
        const int64_t chunks = (a.Wd + V - 1) / V;
        const int64_t bands = (a.Hd + kBand - 1) / kBand;
        dim3 grid((unsigned)((chunks + kThreads - 1) / kThreads), (unsigned)bands,
                  (unsigned)(planes < 65535 ? planes : 65535));
        if (a.half_pixel) {
            hipLaunchKernelGGL((resize_nchw_band_kernel<T, true, kBand>), grid, dim3(kThreads), 0, stream, x, y,
                               planes, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h,
                               a.scale_w, a.raw_lambda);
        } else {
            hipLaunchKernelGGL((resize_nchw_band_kernel<T, false, kBand>), grid, dim3(kThreads), 0, stream, x, y,
                               planes, (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h,
                               a.scale_w, a.raw_lambda);
        }
        return hipGetLastError();
    }
    const int64_t rows = planes * a.Hd;
    dim3 grid((unsigned)((a.Wd + kThreads - 1) / kThreads), (unsigned)(rows < 65535 ? rows : 65535));
    if (a.half_pixel) {
        hipLaunchKernelGGL((resize_nchw_generic_kernel<T, true>), grid, dim3(kThreads), 0, stream, x, y, planes,
                           (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h, a.scale_w,
                           a.raw_lambda);
    } else {
        hipLaunchKernelGGL((resize_nchw_generic_kernel<T, false>), grid, dim3(kThreads), 0, stream, x, y, planes,
                           (int32_t)a.Hs, (int32_t)a.Ws, (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h, a.scale_w,
                           a.raw_lambda);
    }
    return hipGetLastError();
}

}  // namespace

const char* resize_variant(const ResizeArgs& a)
{
    switch (a.mode) {
        case ResizeMode::Copy: return "copy";
        case ResizeMode::Broadcast: return "broadcast";
        case ResizeMode::FirstPixel: return "first_pixel";
        case ResizeMode::PointCopy: return "point_copy";
        case ResizeMode::FourWeights: return "nhwc_four_weights";
        case ResizeMode::Nearest: {
            uint64_t slot = 0;
            switch (a.elem) {
                case Elem::F32: slot = nearest_lds_slot<float>(a); break;
                case Elem::F16: slot = nearest_lds_slot<_Float16>(a); break;
                case Elem::BF16: slot = nearest_lds_slot<__bf16>(a); break;
            }
            if (a.channels_last) {
                return slot != 0 ? "nearest_nhwc_lds" : "nearest_nhwc";
            }
            return slot != 0 ? "nearest_nchw_lds" : "nearest_nchw";
        }
        default: break;
    }
    if (a.channels_last) {
        bool vec = false;
        switch (a.elem) {
            case Elem::F32: vec = nhwc_vec_ok<float>(a); break;
            case Elem::F16: vec = nhwc_vec_ok<_Float16>(a); break;
            case Elem::BF16: vec = nhwc_vec_ok<__bf16>(a); break;
        }
        if (vec) {
            return "nhwc_vec";
        }
        if (const char* lds_variant = resize_lds_variant(a)) {
            return lds_variant;
        }
        int vb = 0;
        switch (a.elem) {
            case Elem::F32: vb = nhwc_unit_bytes<float>(a); break;
            case Elem::F16: vb = nhwc_unit_bytes<_Float16>(a); break;
            case Elem::BF16: vb = nhwc_unit_bytes<__bf16>(a); break;
        }
        return vb != 0 ? "nhwc_unit" : "nhwc_generic";
    }
    if (const char* lds_variant = resize_lds_variant(a)) {
        return lds_variant;
    }
    bool band = false;
    switch (a.elem) {
        case Elem::F32: band = band_variant_ok<float>(a); break;
        case Elem::F16: band = band_variant_ok<_Float16>(a); break;
        case Elem::BF16: band = band_variant_ok<__bf16>(a); break;
    }
    return band ? "nchw_band32" : "nchw_generic";
}

hipError_t launch_resize(const ResizeArgs& a, hipStream_t stream)
{
    const int64_t lim = INT32_MAX;
    if (a.N < 0 || a.C < 0 || a.Hs <= 0 || a.Ws <= 0 || a.Hd < 0 || a.Wd < 0 || a.Hs > lim || a.Ws > lim ||
        a.Hd > lim || a.Wd > lim || a.C > lim || a.N > lim) {
        return hipErrorInvalidValue;
    }
    // one output row (NHWC: Wd*C elements) must be addressable by the x grid axis
    if (a.Wd * (a.channels_last ? a.C : 1) > lim) {
        return hipErrorInvalidValue;
    }
    if (a.N == 0 || a.C == 0 || a.Hd == 0 || a.Wd == 0) {
        return hipSuccess;
    }
    if (a.x == nullptr || a.y == nullptr) {
        return hipErrorInvalidValue;
    }
    switch (a.elem) {
        case Elem::F32: return run_resize<float>(a, stream);
        case Elem::F16: return run_resize<_Float16>(a, stream);
        case Elem::BF16: return run_resize<__bf16>(a, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
