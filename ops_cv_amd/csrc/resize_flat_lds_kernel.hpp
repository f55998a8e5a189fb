// Bilinear resize, NCHW, LDS-staged variant for narrow images on gfx950: device code.
//
// Arithmetic: image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_simt_nchw.h:108-144 (see resize_math.hpp).
//
// The row-band variant gives a lane one 16-byte output vector of a row, so an output row narrower than the
// workgroup leaves most lanes idle.  Here the lanes of a workgroup form a 2-D arrangement instead:
// `cl` column lanes (one 16-byte output vector each, together a whole output row) times `rg` row groups.
//   * A workgroup owns (plane, band of output rows).  The source rows the band touches are whole rows and
//     therefore one contiguous byte range; they are copied from HBM into LDS once with the asynchronous
//     global->LDS loads.
//   * A lane computes its column taps once; it then walks the band rows  hb + group, hb + group + rg, ...  and
//     evaluates the reference formula per output element from eight (fp32: four-byte, else two-byte) LDS reads
//     per column pair -- same operations in the same order as the per-pixel reference.
//   * One 16-byte store per lane and row through a buffer descriptor over the output plane, non-temporal (the lines
//     are written through instead of staying dirty in L2 for the end of the kernel to write back: fp32 8x64x56x56 ->
//     112x112 8.7 -> 6.7 us).
#pragma once

#include <hip/hip_runtime.h>

#include "resize_band_lds_kernel.hpp"

namespace opscv {

struct FlatLdsParams {
    int64_t planes;
    int32_t Hs, Ws, Hd, Wd;
    float scale_h, scale_w;
    int32_t band_rows;  // output rows per workgroup
    int32_t cl;         // column lanes = ceil(Wd / V)
    int32_t rg;         // row groups at work: at most THREADS / cl
    int32_t gran;       // bytes per lane of the asynchronous copy: 16 or 4; 1: 16 in the shifted layout (kernel)
    int32_t raw_lambda;  // fraction from the unclamped source coordinate (see axis_tap)
    float neg_zero;     // -0.0f, passed in so that fma(v, w, -0) is not folded back into a multiply
};

template <typename T, bool HALF_PIXEL, int THREADS>
__global__ __launch_bounds__(THREADS) void resize_flat_lds_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                   FlatLdsParams p)
{
    constexpr int V = 16 / (int)sizeof(T);
    constexpr int NWAVES = THREADS / 64;
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)tid >> 6);

    const int32_t group = tid / p.cl;
    const int32_t cvec = tid - group * p.cl;
    const bool active = group < p.rg;

    const int32_t h_begin = blockIdx.x * p.band_rows;
    const int32_t h_end = (h_begin + p.band_rows < p.Hd) ? h_begin + p.band_rows : p.Hd;
    const int32_t ys_lo = axis_tap<HALF_PIXEL>(h_begin, p.scale_h, p.Hs).i0;
    const int32_t ys_hi = axis_tap<HALF_PIXEL>(h_end - 1, p.scale_h, p.Hs).i1;
    const uint32_t src_row_bytes = (uint32_t)p.Ws * (uint32_t)sizeof(T);
    const uint32_t stage_bytes = (uint32_t)(ys_hi - ys_lo + 1) * src_row_bytes;

    // The staging copy of a plane's band: gran 1 = source rows anywhere (an odd width of 16-bit elements, a view
    // that starts anywhere).  The band's rows are one contiguous byte range; it is copied in 16-byte units from the
    // boundary before its first byte to the boundary after its last (the bytes outside share an aligned unit with
    // bytes inside, so they are readable) and lands `shift` bytes into LDS.
    const uint32_t copy_unit = (p.gran == 1) ? 16u : (uint32_t)p.gran;
    const uint32_t chunk = 64u * copy_unit;
    auto stage = [&](int64_t pl) -> uint32_t {
        const char* src0 = reinterpret_cast<const char*>(x + (pl * p.Hs + ys_lo) * (int64_t)p.Ws);
        const uint32_t shift = (p.gran == 1) ? (uint32_t)(reinterpret_cast<uintptr_t>(src0) & 15u) : 0u;
        const uint32_t copy_bytes = (p.gran == 1) ? ((stage_bytes + shift + 15u) & ~15u) : stage_bytes;
        src0 -= shift;
        for (uint32_t cb = wave * chunk; cb < copy_bytes; cb += NWAVES * chunk) {
            const uint32_t lane_off = cb + (uint32_t)lane * copy_unit;
            if (lane_off < copy_bytes) {
                const rs_global_cptr_t g = (rs_global_cptr_t)(src0 + lane_off);
                const rs_lds_ptr_t l = (rs_lds_ptr_t)(lds + cb);
                if (copy_unit == 16u) {
                    __builtin_amdgcn_global_load_lds(g, l, 16, 0, 0);
                } else {
                    __builtin_amdgcn_global_load_lds(g, l, 4, 0, 0);
                }
            }
        }
        return shift;
    };
    // the first plane's copy is on its way while the lanes work out their column taps
    uint32_t shift = (blockIdx.y < p.planes) ? stage(blockIdx.y) : 0u;

    // ---- per-lane column taps ----
    const int32_t col0 = cvec * V;
    const int32_t nvalid = (p.Wd - col0 < V) ? p.Wd - col0 : V;  // output columns of this lane inside the row
    uint32_t to0[V], to1[V];
    float dx[V], omdx[V];
#pragma unroll
    for (int i = 0; i < V; i++) {
        int32_t c = col0 + i;
        c = (c < p.Wd) ? c : p.Wd - 1;
        const AxisTap t = axis_tap<HALF_PIXEL>(c, p.scale_w, p.Ws, p.raw_lambda);
        to0[i] = (uint32_t)t.i0 * (uint32_t)sizeof(T);
        to1[i] = (uint32_t)t.i1 * (uint32_t)sizeof(T);
        dx[i] = t.lambda;
        omdx[i] = 1.0f - t.lambda;
    }
    const uint32_t out_row_bytes = (uint32_t)p.Wd * (uint32_t)sizeof(T);
    const uint32_t out_plane_bytes = (uint32_t)p.Hd * out_row_bytes;
    const uint32_t col_off = (uint32_t)col0 * (uint32_t)sizeof(T);
    const float neg_zero = p.neg_zero;

    for (int64_t pl = blockIdx.y; pl < p.planes; pl += gridDim.y) {
        if (pl != (int64_t)blockIdx.y) {
            shift = stage(pl);
        }
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();

        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(y + pl * (int64_t)p.Hd * p.Wd, 0, out_plane_bytes, kRsBufferFlags);
        for (int32_t h = active ? h_begin + group : h_end; h < h_end; h += p.rg) {
            const AxisTap t = axis_tap<HALF_PIXEL>(h, p.scale_h, p.Hs, p.raw_lambda);
            const char* r0 = lds + shift + (uint32_t)(t.i0 - ys_lo) * src_row_bytes;
            const char* r1 = lds + shift + (uint32_t)(t.i1 - ys_lo) * src_row_bytes;
            T tl[V], tr[V], bl[V], br[V];
#pragma unroll
            for (int i = 0; i < V; i++) {
                tl[i] = *reinterpret_cast<const T*>(r0 + to0[i]);
                tr[i] = *reinterpret_cast<const T*>(r0 + to1[i]);
                bl[i] = *reinterpret_cast<const T*>(r1 + to0[i]);
                br[i] = *reinterpret_cast<const T*>(r1 + to1[i]);
            }
            const float dy = t.lambda;
            const float omdy = 1.0f - dy;
            T outv[V];
#pragma unroll
            for (int i = 0; i < V; i++) {
                // fma(v, w, -0) is v * w bit for bit; see resize_band_lds_kernel.hpp
                const float top = __builtin_fmaf(ElemIO<T>::load(&tl[i]), omdx[i], neg_zero) +
                                  __builtin_fmaf(ElemIO<T>::load(&tr[i]), dx[i], neg_zero);
                const float bot = __builtin_fmaf(ElemIO<T>::load(&bl[i]), omdx[i], neg_zero) +
                                  __builtin_fmaf(ElemIO<T>::load(&br[i]), dx[i], neg_zero);
                ElemIO<T>::store(&outv[i], omdy * top + dy * bot);
            }
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            u32x4 packed;
            __builtin_memcpy(&packed, outv, sizeof(packed));
            const uint32_t out_off = (uint32_t)h * out_row_bytes + col_off;
            if (nvalid == V) {
                // rows of a width that is not a multiple of V start anywhere: the store is element-aligned
                __builtin_amdgcn_raw_buffer_store_b128(packed, rsrc, (int)out_off, 0, 2);
            } else {
                // the lane that holds the ragged end of the row stores its elements singly
#pragma unroll
                for (int i = 0; i < V; i++) {
                    if (i < nvalid) {
                        if constexpr (sizeof(T) == 4) {
                            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, outv[i]), rsrc,
                                                                  (int)(out_off + i * 4), 0, 2);
                        } else {
                            __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(uint16_t, outv[i]), rsrc,
                                                                  (int)(out_off + i * 2), 0, 2);
                        }
                    }
                }
            }
        }
        __syncthreads();  // everybody is done with the staged rows before the next plane overwrites them
    }
}

}  // namespace opscv
