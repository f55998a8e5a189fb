// Grid sampler 2-D forward, bilinear, 16-bit elements: LDS-staged variant with a pair layout, for gfx950.
//
// Same arithmetic as the other variants (sampler_math.hpp; reference kernel
// image/grid_sampler2_d/op_kernel/arch35/grid_sampler2_d_simt.h:303-339,461-514).  It exists for shapes whose time
// goes into the LDS reads themselves: many output pixels per staged input plane at scattered positions.  A two-byte
// LDS read at a random address costs a wavefront as many LDS cycles as a four-byte one (the lanes collide on banks
// either way), and a bilinear sample needs four of them.  Here a staged plane holds, for every column position, the
// pair (v[x-1], v[x]) as one dword, so the west and east tap of a row come with one four-byte read and a sample takes
// two reads instead of four; the two reads share one address register (the south pair lies a fixed distance behind
// the north pair).
//
// LDS layout of one staged plane, PITCH dwords per row (compile-time):
//   row 0                 zeros               (the row above the image: y0 = -1)
//   row 1 + r             image row r:  entry k = (v[r][k-1], v[r][k]) for k = 0 .. W, with v[r][-1] = v[r][W] = 0
//   row H + 1, H + 2      zeros               (below the image; a sample that lies outside altogether reads here)
// The two ring slots are interleaved row by row (row q of slot s at byte q * ROW_STEP + s * PITCH * 4), so that the
// slot, like the south row, is an immediate offset of the read.
//
// A workgroup owns (batch n, a tile of SWAVES*64*PPT output pixels, a range of channels).  LWAVES loader wavefronts
// bring each plane in through registers -- 16-byte global loads, four funnel shifts per eight entries, 16-byte LDS
// writes -- two planes ahead of the samplers; SWAVES sampler wavefronts run the same rotating-register pipeline as
// the ring kernel (gs2d_lds_kernel.hpp).
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "gs2d_lds_kernel.hpp"
#include "sampler_math.hpp"

namespace opscv {

// west / east value of a pair dword
template <typename T>
__device__ __forceinline__ float pair_lo(uint32_t d)
{
    if constexpr (std::is_same<T, _Float16>::value) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)d);
    } else {
        return __builtin_bit_cast(float, d << 16);
    }
}

template <typename T>
__device__ __forceinline__ float pair_hi(uint32_t d)
{
    if constexpr (std::is_same<T, _Float16>::value) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)(d >> 16));
    } else {
        return __builtin_bit_cast(float, d & 0xFFFF0000u);
    }
}

// grid_sampler2_d_simt.h:321-338: 0 + nw + ne + sw + se, products and sums rounded separately (see blend() in
// gs2d_lds_kernel.hpp for the fma spelling)
template <typename T>
__device__ __forceinline__ float blend_pairs(uint32_t north, uint32_t south, const float* tw, float neg_zero)
{
    float out = __builtin_fmaf(pair_lo<T>(north), tw[0], 0.0f);
    out += __builtin_fmaf(pair_hi<T>(north), tw[1], neg_zero);
    out += __builtin_fmaf(pair_lo<T>(south), tw[2], neg_zero);
    out += __builtin_fmaf(pair_hi<T>(south), tw[3], neg_zero);
    return out;
}

// LWAVES loader wavefronts in two groups: the group of a plane's parity stages it.  A loader lane brings in runs of 32
// consecutive elements of an image row (four 16-byte loads and the dword in front of them) and writes the 32 entries
// they give as eight 16-byte LDS writes; RMAX is the most runs one lane takes per plane.  W must be a multiple of 32,
// the tensor 16-byte aligned and PITCH >= W + 4.  The lanes of a write instruction are 128 bytes apart along a row,
// i.e. on the same banks; the distance between staged rows is therefore an odd multiple of 16 bytes modulo 128, which
// spreads the sixteen rows a wavefront covers over all banks (a 16-way conflict otherwise).
template <typename T, int SWAVES, int LWAVES, int PPT, int PITCH, int RMAX>
__global__ __launch_bounds__((SWAVES + LWAVES) * 64) void gs2d_pair_kernel(
    const T* __restrict__ x, const T* __restrict__ grid, T* __restrict__ y, FastDiv N, int32_t C, int32_t H, int32_t W,
    int32_t out_plane, FastDiv tiles_per_n, int32_t chans_per_block, int32_t pair_aligned, int32_t xcd_swizzle,
    int32_t pad, int32_t align, float neg_zero)
{
    static_assert(sizeof(T) == 2, "pairs of 16-bit elements");
    static_assert(PPT % 2 == 0, "two neighbouring pixels per store");
    static_assert(LWAVES % 2 == 0, "two groups of loader wavefronts");
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    constexpr int STHREADS = SWAVES * 64;
    constexpr int GTHREADS = LWAVES * 32;       // lanes of one loader group
    constexpr uint32_t ROW_BYTES = PITCH * 4u;  // one row of one slot; rows of the two slots alternate
    // distance between consecutive rows of one slot: two rows plus, if needed, 16 bytes to make it an odd number of
    // 16-byte units
    constexpr uint32_t ROW_STEP = 2u * ROW_BYTES + (((2u * ROW_BYTES / 16u) & 1u) ? 0u : 16u);
    static_assert(ROW_BYTES % 16u == 0u, "rows start on 16-byte boundaries");
    const int tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)tid >> 6);

    // groups (channel block, n) are numbered with the batch item fastest, as in the ring kernel (gs2d_lds_kernel.hpp):
    // the workgroups in flight together cover every batch item (bf16 N8 C128 128x128 -> 256x256: 51.5 -> 49.0 us)
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
    const int32_t c_begin = (int32_t)cb * chans_per_block;
    const int32_t c_end = (c_begin + chans_per_block < C) ? c_begin + chans_per_block : C;
    const int32_t nchan = c_end - c_begin;

    if (wave >= (uint32_t)SWAVES) {
        // ------------------------------------------------ loader wavefronts ------------------------------------
        // Group g stages the planes of parity g.  It asks for plane p right after the barrier of plane p - 2, sits
        // through the barrier of plane p - 1 (which tells it that the samplers are done with plane p - 2, the previous
        // tenant of its slot) and then has the time the samplers spend on plane p - 1 to write plane p.  The loads
        // thus have a whole plane's sampling time to arrive, with one set of registers per lane.
        // the loaders' few instructions go first: a plane that is late stalls all samplers at the next barrier
        __builtin_amdgcn_s_setprio(3);
        const uint32_t lwave = wave - SWAVES;
        const uint32_t g = lwave / (LWAVES / 2);
        const uint32_t lg = (lwave % (LWAVES / 2)) * 64u + ((uint32_t)tid & 63u);
        const char* xb = reinterpret_cast<const char*>(x + ((int64_t)n * C + c_begin) * plane_elems);
        const size_t plane_bytes = (size_t)plane_elems * 2u;
        const uint32_t rpr = (uint32_t)W / 32u;  // runs per row
        typedef uint32_t dwordx4_t __attribute__((ext_vector_type(4)));
        typedef dwordx4_t __attribute__((address_space(3))) * lds_vec_ptr_t;
        typedef uint32_t __attribute__((address_space(3))) * lds_dword_ptr_t;
        // a lane's runs are the same for every plane
        uint32_t src[RMAX], dst[RMAX];  // byte offset in the plane; byte offset in slot 0 (bit 0: row start, bit 1: row end)
#pragma unroll
        for (int i = 0; i < RMAX; i++) {
            // Runs are numbered so that sixteen consecutive lanes take the same run of sixteen consecutive rows: the
            // LDS serves a 16-byte write sixteen lanes at a time, and lanes on one row would be 128 bytes apart, on
            // the same banks
            const uint32_t run = (uint32_t)i * GTHREADS + lg;
            const uint32_t blk = run / (16u * rpr), j = run - blk * (16u * rpr);
            const uint32_t r = blk * 16u + (j & 15u), q = j >> 4;
            src[i] = (r * (uint32_t)W + 32u * q) * 2u;
            dst[i] = ((r + 1u) * ROW_STEP + 128u * q) | (q == 0u ? 1u : 0u) | (q + 1u == rpr ? 2u : 0u);
            if (r >= (uint32_t)H) {
                dst[i] = 0xFFFFFFFFu;
            }
        }
        dwordx4_t va[RMAX][4];
        uint32_t vb[RMAX];
        const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
        int32_t done = 0;  // barriers this wavefront has been through
        for (int32_t p = (int32_t)g; p < nchan; p += 2) {
            const char* sp = xb + (size_t)p * plane_bytes;
#pragma unroll
            for (int i = 0; i < RMAX; i++) {
                if (dst[i] != 0xFFFFFFFFu) {
                    const char* a = sp + src[i];
#pragma unroll
                    for (int m = 0; m < 4; m++) {
                        va[i][m] = *reinterpret_cast<const dwordx4_t*>(a + 16 * m);
                    }
                    // the two elements in front of the run; at a row start they belong to the previous row (or lie in
                    // front of the tensor), so the run itself is read again and the value dropped
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
                    uint32_t prev = (dst[i] & 1u) ? 0u : vb[i];
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
                        *reinterpret_cast<lds_dword_ptr_t>((uintptr_t)(d + 128u)) = prev >> 16;  // entry W = (v[W-1], 0)
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
    // the zero rows of both slots: row 0, row H + 1 and row H + 2
    {
        for (uint32_t i = (uint32_t)tid; i < 6u * PITCH; i += STHREADS) {
            const uint32_t q = i / PITCH, col = i - q * PITCH;  // q = 2 * k + slot for the k-th zero row
            const uint32_t row = (q < 2u) ? 0u : (uint32_t)H + (q >> 1);
            *reinterpret_cast<uint32_t*>(lds + row * ROW_STEP + (q & 1u) * ROW_BYTES + col * 4u) = 0u;
        }
    }

    constexpr int NGRP = PPT / 2;
    uint32_t taddr[PPT];  // LDS address of the north pair in slot 0; the south pair lies ROW_STEP behind it
    float tw[PPT][4];
    uint32_t pixoff[NGRP];
    float gxs[PPT], gys[PPT];
    const T* gridn = grid + (int64_t)n * out_plane * 2;
    const T* gptr[PPT];
#pragma unroll
    for (int q = 0; q < NGRP; q++) {
        const int32_t pix0 = (int32_t)tile * (STHREADS * PPT) + q * (STHREADS * 2) + tid * 2;
        const bool valid = pix0 < out_plane;  // the output plane holds whole pairs (launch plan)
        const int32_t pc = valid ? pix0 : out_plane - 2;
        pixoff[q] = valid ? (uint32_t)pc * 2u : 0x80000000u;
        gptr[2 * q] = gridn + (int64_t)pc * 2;
        gptr[2 * q + 1] = gridn + (int64_t)(pc + 1) * 2;
    }
    // grid points and results stream (non-temporal hint), the plane loads of the loaders do not: see
    // load_grid_points in gs2d_lds_kernel.hpp (bf16 N8 C128 128x128 -> 256x256: 69.3 -> 51.0 us; with streaming plane
    // loads as well 102 us)
    load_grid_points<T, PPT, true>(gptr, pair_aligned != 0, gxs, gys);
    uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
    asm volatile("" : "+s"(lds_base));  // kept as a value: seen as the allocation's symbol it is re-added per use
    const uint32_t outside = ((uint32_t)H + 1u) * ROW_STEP;  // rows H + 1 and H + 2: zeros for both pairs
    // padding mode and align_corners are kernel arguments: one wave-uniform switch around the source coordinates of all
    // the lane's pixels (they act once per pixel, outside the channel loop)
    float ixs[PPT], iys[PPT];
    source_indices_rt<PPT>(gxs, gys, H, W, pad, align != 0, false, ixs, iys);
#pragma unroll
    for (int j = 0; j < PPT; j++) {
        // the decisions of decide_pixel() (sampler_math.hpp; grid_sampler2_d_simt.h:479-498, 307-316) without branches
        float ix = ixs[j];
        float iy = iys[j];
        const bool finite = __builtin_fabsf(ix) < __builtin_inff() && __builtin_fabsf(iy) < __builtin_inff();
        const bool x_far = ix > 2147483646.0f || ix < -2147483648.0f;  // safe_downgrade: -> -100, always outside
        const bool y_far = iy > 2147483646.0f || iy < -2147483648.0f;
        ix = x_far ? -100.0f : ix;
        iy = y_far ? -100.0f : iy;
        const float ixf = __builtin_floorf(ix), iyf = __builtin_floorf(iy);
        // column entry x0 + 1 and row y0 + 1 of the staged plane; a tap pair exists for x0 in [-1, W-1], y0 in
        // [-1, H-1] (single unsigned compares: anything else, INT32_MAX + 1 included, is a huge unsigned number)
        const uint32_t xk = (uint32_t)float_to_i32(ixf) + 1u, yk = (uint32_t)float_to_i32(iyf) + 1u;
        const bool in = finite && xk <= (uint32_t)W && yk <= (uint32_t)H;
        taddr[j] = lds_base + (in ? yk * ROW_STEP + xk * 4u : outside);
        const float wx1 = ix - ixf, wx0 = ixf + 1.0f - ix;
        const float wy1 = iy - iyf, wy0 = iyf + 1.0f - iy;
        // non-finite source coordinate: zeros are read and 0 * NaN makes every channel NaN, as the reference writes
        // (grid_sampler2_d_simt.h:485-487)
        tw[j][0] = finite ? wx0 * wy0 : __builtin_nanf("");
        tw[j][1] = wx1 * wy0;
        tw[j][2] = wx0 * wy1;
        tw[j][3] = wx1 * wy1;
    }

    T* yb = y + ((int64_t)n * C + c_begin) * out_plane;
    const uint32_t out_plane_bytes = (uint32_t)out_plane * 2u;
    typedef const uint32_t __attribute__((address_space(3))) * lds_dw_ptr_t;
    uint32_t north[PPT], south[PPT];
    auto read_pixel = [&](int j, uint32_t slot_off) {
        north[j] = *reinterpret_cast<lds_dw_ptr_t>((uintptr_t)(taddr[j] + slot_off));
        south[j] = *reinterpret_cast<lds_dw_ptr_t>((uintptr_t)(taddr[j] + slot_off + ROW_STEP));
    };

    // the rotating-register pipeline of the ring kernel: a pixel's registers are reloaded with the next plane's pairs
    // right after the pixel has been blended; the barrier of plane p + 1 sits behind the first pixel of plane p
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
                __builtin_amdgcn_make_buffer_rsrc(yb + (int64_t)p * out_plane, 0, out_plane_bytes, kBufferFlags);
#pragma unroll
            for (int q = 0; q < NGRP; q++) {
                float v[2];
#pragma unroll
                for (int a = 0; a < 2; a++) {
                    const int j = 2 * q + a;
                    v[a] = blend_pairs<T>(north[j], south[j], tw[j], neg_zero);
                    if (j == 0 && p + 1 < nchan) {
                        __builtin_amdgcn_s_waitcnt(0xC07F);  // every read of plane p has returned
                        lds_barrier();                       // plane p + 1 is staged
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    read_pixel(j, next_off);
                    __builtin_amdgcn_sched_barrier(0);
                }
                buffer_store_group<T, 2, true>(v, rsrc, pixoff[q]);
            }
        }
    }
}

}  // namespace opscv
