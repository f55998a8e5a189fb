// Grid sampler 2-D forward, bicubic, 16-bit elements, zeros or border padding: LDS-staged variant with a pair layout,
// for gfx950.
//
// Same arithmetic as the other variants (sampler_math.hpp, decide_bicubic_rt; reference kernel
// image/grid_sampler2_d/op_kernel/arch35/grid_sampler2_d_simt.h:362-458 and :499-503).  A bicubic sample reads sixteen
// taps; taken one by one from a staged plane they are sixteen two-byte LDS reads, and the LDS is what bounds the ring
// kernel in this mode (it is busy for 60 % of the kernel's time, half of that in bank-conflict replays).  Here a staged
// plane holds, for every column position k, the pair (v[k-1], v[k]) as one dword (the layout of gs2d_pair_kernel.hpp),
// with the padding already applied in a margin of four entries on either side of each row:
//   zeros  : v[c] = 0 for c outside the row
//   border : v[c] = v[0] or v[W-1] for c outside the row
// so the four taps x0-1 .. x0+2 of a row are entry x0 and entry x0+2, whatever x0 is: eight four-byte reads per sample,
// two per row at a fixed distance, no per-tap bounds handling.  x0 is limited to [-3, W+1] first, which changes no
// tap value (further out every tap is padding).  Rows outside the image (zeros padding) read one staged row of zeros;
// under border padding the row coordinates are clamped like the reference clamps them.
//
// LDS layout of one staged plane, PITCH dwords per row (compile-time, >= W + 8):
//   row r, dword 4 + k    (v[r][k-1], v[r][k]) for k = -4 .. W + 3, padded as above
//   row H                 zeros
// The two ring slots are interleaved row by row (row q of slot s at byte q * row_step + s * PITCH * 4), so that the slot
// is an immediate offset of the read.  `row_step` is a kernel argument: it must be an odd number of 16-byte units, which
// spreads the sixteen rows that the lanes of a loader's 16-byte write cover over all banks, and by how many banks it
// shifts consecutive rows against each other decides how often the lanes of a sampler wavefront, which follow a
// slanted line through the plane, meet on a bank (fp16 N16 C256 64x64, rotations up to 30 degrees: 35.5 us with a
// shift of 12 banks, 38.4 with 20, 55.8 with 28, 60.7 with 4; even numbers of 16-byte units: 44 with 16, 67 with none).
//
// Workgroup roles, loader scheme and the samplers' rotating-register pipeline are those of gs2d_pair_kernel.hpp.  One
// output pixel per lane and store: the lanes of a wavefront then read neighbouring entries (with two neighbouring
// pixels per lane they are two entries apart and use every other bank: 38 us).
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "gs2d_pair_kernel.hpp"
#include "sampler_math.hpp"

namespace opscv {

// grid_sampler2_d_simt.h:418-455: each row is c0*v0 followed by three fused multiply-adds, and so is the column of
// the four row results (blend() in gs2d_lds_kernel.hpp, INTERP == 2, from pairs: raw[2 * r] = taps 0, 1 of row r,
// raw[2 * r + 1] = taps 2, 3)
template <typename T>
__device__ __forceinline__ float blend_bicubic_pairs(const uint32_t* raw, const float* tw, float neg_zero)
{
    float r[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t a = raw[2 * j], b = raw[2 * j + 1];
        float acc = __builtin_fmaf(pair_lo<T>(a), tw[0], neg_zero);
        acc = __builtin_fmaf(tw[1], pair_hi<T>(a), acc);
        acc = __builtin_fmaf(tw[2], pair_lo<T>(b), acc);
        acc = __builtin_fmaf(tw[3], pair_hi<T>(b), acc);
        r[j] = acc;
    }
    float out = tw[4] * r[0];
    out = __builtin_fmaf(tw[5], r[1], out);
    out = __builtin_fmaf(tw[6], r[2], out);
    out = __builtin_fmaf(tw[7], r[3], out);
    return as_fp32_value(out);
}

// W must be a multiple of 32, the tensor 16-byte aligned, PITCH >= W + 8 and a multiple of 4; `pad` is 0 (zeros) or 1
// (border).  RMAX is the most 32-element runs one loader lane takes per plane.
template <typename T, int SWAVES, int LWAVES, int PPT, int PITCH, int RMAX, int ADJ>
__global__ __launch_bounds__((SWAVES + LWAVES) * 64) void gs2d_bicubic_pair_kernel(
    const T* __restrict__ x, const T* __restrict__ grid, T* __restrict__ y, FastDiv N, int32_t C, int32_t H, int32_t W,
    int32_t out_plane, FastDiv tiles_per_n, int32_t chans_per_block, uint32_t wide_blocks, int32_t chans_wide,
    int32_t chan_stride, int32_t pair_aligned, int32_t xcd_swizzle,
    uint32_t row_step, int32_t pad, int32_t align, int32_t bw_shift, int32_t blocks_per_row, float neg_zero)
{
    static_assert(sizeof(T) == 2, "pairs of 16-bit elements");
    static_assert(PPT % ADJ == 0, "whole groups of neighbouring pixels per store");
    static_assert(LWAVES % 2 == 0, "two groups of loader wavefronts");
    static_assert(PITCH % 4 == 0, "rows start on 16-byte boundaries");
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    constexpr int STHREADS = SWAVES * 64;
    constexpr int GTHREADS = LWAVES * 32;       // lanes of one loader group
    constexpr uint32_t ROW_BYTES = PITCH * 4u;  // one row of one slot; the rows of the two slots alternate
    // distance between consecutive rows of one slot (a kernel argument: the launch plan picks the padding behind the
    // rows of the slots)
    const uint32_t ROW_STEP = row_step;
    constexpr uint32_t MARGIN = 4u;  // entries in front of column 0
    const int tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)tid >> 6);
    const bool border = pad == 1;

    // groups (channel block, n) numbered with the batch item fastest, as in the ring kernel (gs2d_lds_kernel.hpp)
    uint32_t group, tile;
    if (xcd_swizzle) {
        const uint32_t xcd = blockIdx.x & 7u;
        const uint32_t i = blockIdx.x >> 3;
        const uint32_t k = fast_div(i, tiles_per_n);
        group = k * 8u + xcd;
        tile = i - k * tiles_per_n.div;
    } else {
        group = fast_div(blockIdx.x, tiles_per_n);
        tile = blockIdx.x - group * tiles_per_n.div;
    }
    const uint32_t cb = fast_div(group, N);
    const uint32_t n = group - cb * N.div;
    const int32_t plane_elems = H * W;
    // Which channels, as in the ring kernel (gs2d_lds_kernel.hpp): a contiguous range, or -- `chan_stride` != 0,
    // every block's count exact -- channels dealt out in turn, the first `wide_blocks` blocks taking `chans_wide`
    // each and the others `chans_per_block`.  The block's j-th channel is  first + j * step1  up to j = switch_at and
    // step2 apart from there on.
    const bool wide = cb < wide_blocks;
    int32_t first, step1, step2, nchan;
    if (chan_stride != 0) {
        first = (int32_t)cb;
        step1 = chan_stride;
        step2 = (int32_t)wide_blocks;
        nchan = wide ? chans_wide : chans_per_block;
    } else {
        const int32_t c_begin = (int32_t)cb * chans_per_block;
        const int32_t c_end = (c_begin + chans_per_block < C) ? c_begin + chans_per_block : C;
        first = c_begin;
        step1 = 1;
        step2 = 1;
        nchan = c_end - c_begin;
    }
    const int32_t switch_at = chans_per_block;
    auto chan_of = [&](int32_t j) -> int32_t {
        return first + (j < switch_at ? j * step1 : switch_at * step1 + (j - switch_at) * step2);
    };

    if (wave >= (uint32_t)SWAVES) {
        // ------------------------------------------------ loader wavefronts ------------------------------------
        // Group g stages the planes of parity g: it asks for plane p right after the barrier of plane p - 2, sits
        // through the barrier of plane p - 1 (the samplers are done with plane p - 2, the previous tenant of its slot)
        // and writes plane p while the samplers work on plane p - 1.
        __builtin_amdgcn_s_setprio(3);
        const uint32_t lwave = wave - SWAVES;
        const uint32_t g = lwave / (LWAVES / 2);
        const uint32_t lg = (lwave % (LWAVES / 2)) * 64u + ((uint32_t)tid & 63u);
        const char* xn = reinterpret_cast<const char*>(x + (int64_t)n * C * plane_elems);  // the batch item's planes
        const size_t plane_bytes = (size_t)plane_elems * 2u;
        const uint32_t rpr = (uint32_t)W / 32u;  // runs per row
        typedef uint32_t dwordx4_t __attribute__((ext_vector_type(4)));
        typedef dwordx4_t __attribute__((address_space(3))) * lds_vec_ptr_t;
        // a lane's runs are the same for every plane
        uint32_t src[RMAX], dst[RMAX];  // byte offset in the plane; byte offset in slot 0 (bit 0: row start, bit 1: row end)
#pragma unroll
        for (int i = 0; i < RMAX; i++) {
            // sixteen consecutive lanes take the same run of sixteen consecutive rows (the LDS serves a 16-byte write
            // sixteen lanes at a time; lanes on one row would be 128 bytes apart, on the same banks)
            const uint32_t run = (uint32_t)i * GTHREADS + lg;
            const uint32_t blk = run / (16u * rpr), j = run - blk * (16u * rpr);
            const uint32_t r = blk * 16u + (j & 15u), q = j >> 4;
            src[i] = (r * (uint32_t)W + 32u * q) * 2u;
            dst[i] = (r * ROW_STEP + MARGIN * 4u + 128u * q) | (q == 0u ? 1u : 0u) | (q + 1u == rpr ? 2u : 0u);
            if (r >= (uint32_t)H) {
                dst[i] = 0xFFFFFFFFu;
            }
        }
        dwordx4_t va[RMAX][4];
        uint32_t vb[RMAX];
        const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
        int32_t done = 0;  // barriers this wavefront has been through
        for (int32_t p = (int32_t)g; p < nchan; p += 2) {
            const char* sp = xn + (size_t)chan_of(p) * plane_bytes;
#pragma unroll
            for (int i = 0; i < RMAX; i++) {
                if (dst[i] != 0xFFFFFFFFu) {
                    const char* a = sp + src[i];
#pragma unroll
                    for (int m = 0; m < 4; m++) {
                        va[i][m] = *reinterpret_cast<const dwordx4_t*>(a + 16 * m);
                    }
                    // the two elements in front of the run; at a row start they are not this row's (or lie in front
                    // of the tensor), so the run itself is read again and the value dropped
                    vb[i] = *reinterpret_cast<const uint32_t*>((dst[i] & 1u) ? a : a - 4);
                }
            }
            while (done < p) {
                lds_barrier();
                done++;
            }
            const uint32_t slot_base = lds_base + ((uint32_t)p & 1u) * ROW_BYTES;
#pragma unroll
            for (int i = 0; i < RMAX; i++) {
                if (dst[i] != 0xFFFFFFFFu) {
                    const uint32_t d = slot_base + (dst[i] & ~3u);
                    uint32_t prev = vb[i];
                    if (dst[i] & 1u) {
                        // row start: the element in front of the row (the high half of `prev`) is padding, and so
                        // are entries -4 .. -1
                        const uint32_t first = va[i][0].x << 16;  // v[0] in the high half
                        prev = border ? first : 0u;
                        const uint32_t e = border ? (first | (first >> 16)) : 0u;
                        const dwordx4_t edge = {e, e, e, e};
                        *reinterpret_cast<lds_vec_ptr_t>((uintptr_t)(d - MARGIN * 4u)) = edge;
                    }
#pragma unroll
                    for (int m = 0; m < 4; m++) {
                        // entry k = (v[k-1], v[k]): odd entries are the loaded dwords, even ones straddle two of them
                        const dwordx4_t a = va[i][m];
                        const dwordx4_t e0 = {__builtin_amdgcn_alignbit(a.x, prev, 16), a.x,
                                              __builtin_amdgcn_alignbit(a.y, a.x, 16), a.y};
                        const dwordx4_t e1 = {__builtin_amdgcn_alignbit(a.z, a.y, 16), a.z,
                                              __builtin_amdgcn_alignbit(a.w, a.z, 16), a.w};
                        *reinterpret_cast<lds_vec_ptr_t>((uintptr_t)(d + 32u * m)) = e0;
                        *reinterpret_cast<lds_vec_ptr_t>((uintptr_t)(d + 32u * m + 16u)) = e1;
                        prev = a.w;
                    }
                    if (dst[i] & 2u) {
                        // row end: entry W = (v[W-1], padding), entries W + 1 .. W + 3 padding
                        const uint32_t last = prev >> 16;  // v[W-1] in the low half
                        const uint32_t e = border ? (last | (last << 16)) : 0u;
                        const dwordx4_t edge = {border ? e : last, e, e, e};
                        *reinterpret_cast<lds_vec_ptr_t>((uintptr_t)(d + 128u)) = edge;
                    }
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);  // the LDS writes, before the barrier publishes them
            lds_barrier();                       // plane p is staged
            done++;
        }
        while (done < nchan) {
            lds_barrier();
            done++;
        }
        return;
    }

    // ---------------------------------------------------- sampler wavefronts -----------------------------------
    // the row of zeros of both slots
    for (uint32_t i = (uint32_t)tid; i < 2u * PITCH; i += STHREADS) {
        const uint32_t s = i / PITCH, col = i - s * PITCH;
        *reinterpret_cast<uint32_t*>(lds + (uint32_t)H * ROW_STEP + s * ROW_BYTES + col * 4u) = 0u;
    }

    constexpr int NGRP = PPT / ADJ;
    uint32_t taddr[PPT][4];  // LDS address of entry x0 of each tap row in slot 0; entry x0 + 2 lies 8 bytes behind it
    float tw[PPT][8];
    uint32_t pixoff[NGRP];
    float gxs[PPT], gys[PPT];
    const T* gridn = grid + (int64_t)n * out_plane * 2;
    const T* gptr[PPT];
#pragma unroll
    for (int q = 0; q < NGRP; q++) {
        int32_t pix0 = (int32_t)tile * (STHREADS * PPT) + q * (STHREADS * ADJ) + tid * ADJ;
        bool valid = pix0 < out_plane;  // the output plane holds whole groups (launch plan)
        if (ADJ == 1 && bw_shift != 0) {
            // a wavefront's 64 pixels as a block of 2^bw_shift columns by 64 >> bw_shift rows
            const int32_t unit = pix0 >> 6;
            const int32_t lane = tid & 63;
            const int32_t bx = lane & ((1 << bw_shift) - 1), by = lane >> bw_shift;
            const int32_t brow = unit / blocks_per_row, bcol = unit - brow * blocks_per_row;
            pix0 = (brow * (64 >> bw_shift) + by) * (blocks_per_row << bw_shift) + (bcol << bw_shift) + bx;
            valid = unit < (out_plane >> 6);
        }
        const int32_t pc = valid ? pix0 : out_plane - ADJ;
        pixoff[q] = valid ? (uint32_t)pc * 2u : 0x80000000u;
#pragma unroll
        for (int a = 0; a < ADJ; a++) {
            gptr[ADJ * q + a] = gridn + (int64_t)(pc + a) * 2;
        }
    }
    load_grid_points<T, PPT, true>(gptr, pair_aligned != 0, gxs, gys);
    uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
    asm volatile("" : "+s"(lds_base));  // kept as a value: seen as the allocation's symbol it is re-added per use
#pragma unroll
    for (int j = 0; j < PPT; j++) {
        const BicubicTap b = decide_bicubic_rt(gxs[j], gys[j], H, W, border ? 1 : 0, align != 0);
        // the column of the second tap before padding, limited to [-3, W + 1] (NaN, flagged below, becomes -3)
        const float ixf = __builtin_floorf(unnormalize_rt(gxs[j], W, align != 0));
        const float xl = __builtin_fminf(__builtin_fmaxf(ixf, -3.0f), (float)(W + 1));
        const uint32_t col_off = (uint32_t)((int32_t)xl + (int32_t)MARGIN) * 4u;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const bool row_in = (uint32_t)b.by[r] < (uint32_t)H && !b.flag;
            const uint32_t row = row_in ? (uint32_t)b.by[r] : (uint32_t)H;
            taddr[j][r] = lds_base + row * ROW_STEP + col_off;
            tw[j][r] = b.cx[r];
            tw[j][4 + r] = b.cy[r];
        }
        if (b.flag) {
            tw[j][0] = __builtin_nanf("");  // 0 * NaN: every channel becomes NaN, as the reference writes
        }
    }

    T* yn = y + (int64_t)n * C * out_plane;  // the batch item's output planes
    const uint32_t out_plane_bytes = (uint32_t)out_plane * 2u;
    typedef const uint32_t __attribute__((address_space(3))) * lds_dw_ptr_t;
    uint32_t raw[PPT][8];
    auto read_pixel = [&](int j, uint32_t slot_off) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            raw[j][2 * r] = *reinterpret_cast<lds_dw_ptr_t>((uintptr_t)(taddr[j][r] + slot_off));
            raw[j][2 * r + 1] = *reinterpret_cast<lds_dw_ptr_t>((uintptr_t)(taddr[j][r] + slot_off + 8u));
        }
    };

    // The rotating-register pipeline of the ring kernel: a pixel's registers are reloaded with the next plane's pairs
    // right after the pixel has been blended; the barrier of plane p + 1 sits behind the first pixel of plane p.  A
    // wavefront enters it with all its reads returned: behind it the loaders overwrite the slot of plane p - 1, and
    // plane p + 1's pairs are read.  (A third slot, which lets the barrier go without that wait, measured the same.)
    __builtin_amdgcn_s_waitcnt(0xC07F);  // the zero rows, before the first barrier publishes them
    lds_barrier();                        // plane 0 is staged
#pragma unroll
    for (int j = 0; j < PPT; j++) {
        read_pixel(j, 0u);
    }
    for (int32_t b = 0; b < nchan; b += 2) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int32_t p = b + u;
            if (p >= nchan) {
                break;
            }
            const uint32_t next_off = (u == 0) ? ROW_BYTES : 0u;  // slot of plane p + 1
            const __amdgpu_buffer_rsrc_t rsrc =
                __builtin_amdgcn_make_buffer_rsrc(yn + (int64_t)chan_of(p) * out_plane, 0, out_plane_bytes, kBufferFlags);
#pragma unroll
            for (int q = 0; q < NGRP; q++) {
                float v[ADJ];
#pragma unroll
                for (int a = 0; a < ADJ; a++) {
                    const int j = ADJ * q + a;
                    v[a] = blend_bicubic_pairs<T>(raw[j], tw[j], neg_zero);
                    if (j == 0 && p + 1 < nchan) {
                        __builtin_amdgcn_s_waitcnt(0xC07F);  // every read of plane p has returned
                        lds_barrier();                       // plane p + 1 is staged
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    read_pixel(j, next_off);
                    __builtin_amdgcn_sched_barrier(0);
                }
                buffer_store_group<T, ADJ, true>(v, rsrc, pixoff[q]);
            }
        }
    }
}

}  // namespace opscv
