// Bilinear resize, NCHW (and channels-last images of few channels), LDS-staged row-band variant for gfx950: device
// code.
//
// Arithmetic: image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_simt_nchw.h:108-144 (see resize_math.hpp).
//
// A workgroup owns (plane, band of BAND output rows, block of THREADS*V output columns), V = 16/sizeof(T).
//   * The source rows the band touches, cut to the columns the block touches, are copied from HBM into LDS
//     once with the asynchronous global->LDS loads (16 or 4 bytes per lane), so every source element is read
//     from memory once per workgroup and the unaligned two-byte tap reads never leave the CU.
//   * A lane owns V consecutive output columns; its column taps (two LDS byte offsets and lambda per column)
//     are computed once.  The reference formula  out = (1-dy)*((1-dx)*TL + dx*TR) + dy*((1-dx)*BL + dx*BR)  is
//     separable as written: the horizontally blended source row  Hrow(y)[col] = (1-dx)*x[y,x0] + dx*x[y,x1]  is
//     kept in registers and reused by every output row that touches source row y -- same operations in the
//     same order, so the result is bit-identical to the per-pixel evaluation.
//   * Row taps (y0, y1, dy) of the band are computed by the first BAND lanes once and broadcast per row.
//   * Each lane writes one 16-byte vector per output row through a buffer descriptor (lanes past the row end
//     are dropped by its range check; the lane holding the ragged end of a row whose width is not a multiple of V
//     stores its elements singly); a wavefront writes 1 KiB contiguous.
#pragma once

#include <hip/hip_runtime.h>

#include "resize_math.hpp"
#include "sampler_math.hpp"

namespace opscv {

typedef __attribute__((address_space(1))) const void* rs_global_cptr_t;
typedef __attribute__((address_space(3))) void* rs_lds_ptr_t;

constexpr uint32_t kRsBufferFlags = 0x00020000u;  // raw buffer, 32-bit data format

struct BandLdsParams {
    int64_t planes;
    int32_t Hs, Ws, Hd, Wd;
    float scale_h, scale_w;
    int32_t lds_pitch;  // bytes between staged source rows (multiple of 16)
    int32_t lds_rows;   // staged rows the LDS allocation holds
    int32_t gran;       // bytes per lane of the asynchronous copy: 16 or 4; 1: 16 in the shifted layout (kernel)
    int32_t streaming;  // 1: mark the output stores non-temporal (outputs much larger than the caches)
    int32_t raw_lambda;  // fraction from the unclamped source coordinate (see axis_tap)
    int32_t interleave;  // 1: planes of Hs x Ws; C: channels-last images, a row is Ws pixels of C elements each
    float neg_zero;     // -0.0f, passed in so that fma(v, w, -0) is not folded back into a multiply
};

template <typename T, bool HALF_PIXEL, int THREADS, int BAND>
__global__ __launch_bounds__(THREADS) void resize_band_lds_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                   BandLdsParams p)
{
    static_assert(BAND <= 64, "row taps are held one per lane of a wavefront");
    constexpr int V = 16 / (int)sizeof(T);
    constexpr int NWAVES = THREADS / 64;
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    const int tid = threadIdx.x;
    const int lane = tid & 63;

    // ---- block geometry (uniform) ----
    // Channels-last images are resized as planes whose rows are Ws * C elements: output element j of a row is channel
    // j % C of pixel j / C, and its taps sit C elements apart.  Everything below counts row elements ("columns").
    const int32_t ci = p.interleave;
    const int32_t Wse = p.Ws * ci, Wde = p.Wd * ci;
    const int32_t c_begin = blockIdx.x * (THREADS * V);
    const int32_t c_last = ((c_begin + THREADS * V < Wde) ? c_begin + THREADS * V : Wde) - 1;
    const int32_t h_begin = blockIdx.y * BAND;
    const int32_t h_end = (h_begin + BAND < p.Hd) ? h_begin + BAND : p.Hd;
    // gran 16 or 4: source rows on that grid, copied as they are.  gran 1: rows anywhere (an odd width of 16-bit
    // elements, a view that starts anywhere) -- a row's segment is then copied in 16-byte units from the boundary
    // before its first byte to the boundary after its last (the bytes outside share an aligned unit with bytes inside,
    // so they are readable), and lands `shift` bytes into its LDS row; the shift goes into the row's base address.
    const bool shifted = p.gran == 1;
    const int32_t ge = shifted ? 1 : p.gran / (int)sizeof(T);  // elements per copy granule
    const uint32_t copy_unit = shifted ? 16u : (uint32_t)p.gran;
    const int32_t xs_lo = axis_tap<HALF_PIXEL>(c_begin / ci, p.scale_w, p.Ws).i0 * ci;
    const int32_t xs_hi = axis_tap<HALF_PIXEL>(c_last / ci, p.scale_w, p.Ws).i1 * ci + ci - 1;
    const int32_t seg_col0 = xs_lo / ge * ge;
    const int32_t seg_elems = (xs_hi + 1 - seg_col0 + ge - 1) / ge * ge;  // stays inside the row: Wse % ge == 0
    const uint32_t seg_bytes = (uint32_t)seg_elems * (uint32_t)sizeof(T);
    const int32_t ys_lo = axis_tap<HALF_PIXEL>(h_begin, p.scale_h, p.Hs).i0;
    const int32_t ys_hi = axis_tap<HALF_PIXEL>(h_end - 1, p.scale_h, p.Hs).i1;
    int32_t rows = ys_hi - ys_lo + 1;
    rows = (rows < p.lds_rows) ? rows : p.lds_rows;  // the host sized the allocation for the exact maximum

    // ---- per-lane column taps ----
    const int32_t col0 = c_begin + tid * V;
    uint32_t to0[V], to1[V];
    float dx[V], omdx[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        int32_t c = col0 + i;
        c = (c < Wde) ? c : Wde - 1;
        const int32_t px = (ci == 1) ? c : c / ci;
        const int32_t ch = c - px * ci;
        const AxisTap t = axis_tap<HALF_PIXEL>(px, p.scale_w, p.Ws, p.raw_lambda);
        to0[i] = (uint32_t)(t.i0 * ci + ch - seg_col0) * (uint32_t)sizeof(T);
        to1[i] = (uint32_t)(t.i1 * ci + ch - seg_col0) * (uint32_t)sizeof(T);
        dx[i] = t.lambda;
        omdx[i] = 1.0f - t.lambda;
    }
    // ---- row taps of the band: lane l holds output row h_begin + l ----
    int32_t my_y0, my_y1;
    float my_dy;
    {
        int32_t h = h_begin + lane;
        h = (h < p.Hd) ? h : p.Hd - 1;
        const AxisTap t = axis_tap<HALF_PIXEL>(h, p.scale_h, p.Hs, p.raw_lambda);
        my_y0 = t.i0 - ys_lo;
        my_y1 = t.i1 - ys_lo;
        my_dy = t.lambda;
    }
    const uint32_t out_row_bytes = (uint32_t)Wde * (uint32_t)sizeof(T);
    const uint32_t out_off = (col0 < Wde) ? (uint32_t)col0 * (uint32_t)sizeof(T) : 0x80000000u;
    const int32_t nvalid = (Wde - col0 < V) ? Wde - col0 : V;  // output columns of this lane inside the row
    const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)tid >> 6);
    const float neg_zero = p.neg_zero;

    for (int64_t pl = blockIdx.z; pl < p.planes; pl += gridDim.z) {
        // ---- stage the source rows of this band ----
        const char* src0 = reinterpret_cast<const char*>(x + (pl * p.Hs + ys_lo) * (int64_t)Wse + seg_col0);
        const uint32_t chunk = 64u * copy_unit;
        const uint32_t chunks_per_row = (seg_bytes + (shifted ? 15u : 0u) + chunk - 1) / chunk;
        const uint32_t total_chunks = chunks_per_row * (uint32_t)rows;
        const uint32_t src0_low = (uint32_t)(reinterpret_cast<uintptr_t>(src0) & 15u);
        const uint32_t row_low = (uint32_t)(((uint32_t)Wse * (uint32_t)sizeof(T)) & 15u);
        // bytes by which the copy of staged row r starts before the row's segment
        auto row_shift = [&](uint32_t r) -> uint32_t { return shifted ? ((src0_low + r * row_low) & 15u) : 0u; };
        for (uint32_t q = wave; q < total_chunks; q += NWAVES) {
            const uint32_t r = q / chunks_per_row;
            const uint32_t cb = (q - r * chunks_per_row) * chunk;
            const uint32_t lane_off = cb + (uint32_t)lane * copy_unit;
            const uint32_t shift = row_shift(r);
            const uint32_t limit = shifted ? ((seg_bytes + shift + 15u) & ~15u) : seg_bytes;
            if (lane_off < limit) {
                const rs_global_cptr_t g =
                    (rs_global_cptr_t)(src0 + (size_t)r * Wse * sizeof(T) - shift + lane_off);
                const rs_lds_ptr_t l = (rs_lds_ptr_t)(lds + r * p.lds_pitch + cb);
                if (copy_unit == 16u) {
                    __builtin_amdgcn_global_load_lds(g, l, 16, 0, 0);
                } else {
                    __builtin_amdgcn_global_load_lds(g, l, 4, 0, 0);
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();

        T* yp = y + (pl * p.Hd + h_begin) * (int64_t)Wde;
        float ha[V], hb[V];  // blended source rows ya and yb (row indices relative to ys_lo)
        int32_t ya = -1, yb = -1;
        auto blend_row = [&](float* hrow, int32_t ys) {
            const char* row = lds + ys * p.lds_pitch + row_shift((uint32_t)ys);
            T l[V], r[V];
#pragma unroll
            for (int i = 0; i < V; i++) {
                l[i] = *reinterpret_cast<const T*>(row + to0[i]);
                r[i] = *reinterpret_cast<const T*>(row + to1[i]);
            }
#pragma unroll
            for (int i = 0; i < V; i++) {
                // fma(v, w, -0) is v * w bit for bit (also for zero products of either sign); written as an
                // fma with an addend the compiler cannot see through so that, for 16-bit floats, the conversion
                // rides on the multiply (mixed-precision fma) instead of costing an instruction of its own
                hrow[i] = __builtin_fmaf(ElemIO<T>::load(&l[i]), omdx[i], neg_zero) +
                          __builtin_fmaf(ElemIO<T>::load(&r[i]), dx[i], neg_zero);
            }
        };
        for (int32_t h = h_begin; h < h_end; h++) {
            const int32_t y0 = __builtin_amdgcn_readlane(my_y0, h - h_begin);
            const int32_t y1 = __builtin_amdgcn_readlane(my_y1, h - h_begin);
            const float dy = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int32_t, my_dy),
                                                                                  h - h_begin));
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
            const float omdy = 1.0f - dy;
            T outv[V];
            if (y1 == ya) {
#pragma unroll
                for (int i = 0; i < V; i++) {
                    ElemIO<T>::store(&outv[i], omdy * ha[i] + dy * ha[i]);
                }
            } else {
#pragma unroll
                for (int i = 0; i < V; i++) {
                    ElemIO<T>::store(&outv[i], omdy * ha[i] + dy * hb[i]);
                }
            }
            const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(yp, 0, out_row_bytes, kRsBufferFlags);
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            u32x4 packed;
            __builtin_memcpy(&packed, outv, sizeof(packed));
            if (nvalid == V) {
                // rows of a width that is not a multiple of V start anywhere: the store is element-aligned
                if (p.streaming) {
                    __builtin_amdgcn_raw_buffer_store_b128(packed, rsrc, (int)out_off, 0, 2);
                } else {
                    __builtin_amdgcn_raw_buffer_store_b128(packed, rsrc, (int)out_off, 0, 0);
                }
            } else {
                // the lane that holds the ragged end of the row stores its elements singly (lanes past the end
                // have nvalid <= 0 and an offset outside the descriptor's range)
#pragma unroll
                for (int i = 0; i < V; i++) {
                    if (i < nvalid) {
                        if constexpr (sizeof(T) == 4) {
                            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, outv[i]), rsrc,
                                                                  (int)(out_off + i * 4), 0, 0);
                        } else {
                            __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(uint16_t, outv[i]), rsrc,
                                                                  (int)(out_off + i * 2), 0, 0);
                        }
                    }
                }
            }
            yp += Wde;
        }
        __syncthreads();  // everybody is done with the staged rows before the next plane overwrites them
    }
}

}  // namespace opscv
