// Grid sampler 2-D forward, LDS-staged variant for gfx950: device code.
//
// Same arithmetic as the direct variant (see sampler_math.hpp; reference kernel
// image/grid_sampler2_d/op_kernel/arch35/grid_sampler2_d_simt.h:461-514), different data movement:
//
//   * a workgroup owns (batch n, a tile of THREADS*PPT output pixels, a range of channels);
//   * every lane decides its PPT pixels once -- four LDS byte offsets and four weights per pixel stay in
//     registers for the whole channel range;
//   * the channel range is walked in stages of CGS whole input planes.  The planes go from HBM straight into
//     LDS with the asynchronous global->LDS loads of gfx950 (no registers, 16 bytes per lane, 1 KiB per
//     wavefront instruction), double-buffered: stage s+1 is in flight while stage s is sampled;
//   * every tap is a 2- or 4-byte LDS read, so the scattered part of the gather never leaves the CU;
//   * a tap outside the image points at a 16-byte slot of zeros behind each staged plane, which reproduces the
//     reference's "skip the tap" exactly (0 * w adds nothing) without per-channel selects;
//   * every output channel plane is written once, 64 consecutive pixels per wavefront store, through a buffer
//     descriptor whose range check drops the lanes of a partial last tile.
#pragma once

#include <hip/hip_runtime.h>

#include "sampler_math.hpp"

namespace opscv {

constexpr int kLdsLimit = 160 * 1024;  // LDS bytes per CU on gfx950

__host__ __device__ constexpr uint32_t round_up16(uint32_t v) { return (v + 15u) & ~15u; }

typedef __attribute__((address_space(1))) const void* global_cptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

constexpr uint32_t kBufferFlags = 0x00020000u;  // raw buffer, 32-bit data format

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

// Raw tap values of one pixel from a staged plane (LDS reads only, no arithmetic, so that the reads of
// many pixels can be in flight together).
template <typename T, int NT>
__device__ __forceinline__ void load_taps(const char* plane, const uint32_t* toff, T* raw)
{
#pragma unroll
    for (int t = 0; t < NT; t++) {
        raw[t] = *reinterpret_cast<const T*>(plane + toff[t]);
    }
}

// One output sample from its tap values: grid_sampler2_d_simt.h:321-338 (0 + nw + ne + sw + se, products and
// sums rounded separately) for bilinear, :341-360 (the value passes through fp32) for nearest.
template <typename T, int INTERP>
__device__ __forceinline__ float blend(const T* raw, const float* tw)
{
    if (INTERP == 0) {
        float out = 0.0f;
        out += ElemIO<T>::load(&raw[0]) * tw[0];
        out += ElemIO<T>::load(&raw[1]) * tw[1];
        out += ElemIO<T>::load(&raw[2]) * tw[2];
        out += ElemIO<T>::load(&raw[3]) * tw[3];
        return out;
    }
    return ElemIO<T>::load(&raw[0]);
}

template <typename T>
__device__ __forceinline__ void buffer_store_elem(float v, __amdgpu_buffer_rsrc_t rsrc, uint32_t byte_off)
{
    if constexpr (sizeof(T) == 4) {
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), rsrc, (int)byte_off, 0, 0);
    } else {
        T h;
        ElemIO<T>::store(&h, v);
        __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(uint16_t, h), rsrc, (int)byte_off, 0, 0);
    }
}

// Starts the asynchronous copy of `nch` consecutive input planes (plane_bytes each, contiguous in global memory
// from `src`) to LDS at `dst` with PITCH bytes between planes.  G = bytes per lane (16 or 4): the largest
// granule that divides the plane size and the source alignment.  Each wavefront instruction moves 64*G
// contiguous bytes; lanes past the end of a plane are masked off.
template <int G, int THREADS, int CGS, int PITCH>
__device__ __forceinline__ void issue_stage_copy(const char* src, char* dst, uint32_t plane_bytes, int nch)
{
    constexpr int NWAVES = THREADS / 64;
    constexpr uint32_t CHUNK = 64u * G;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane_off = (threadIdx.x & 63u) * G;
#pragma unroll
    for (int k = 0; k < CGS; k++) {
        if (k < nch) {
            const char* sp = src + (size_t)k * plane_bytes;
            char* dp = dst + k * PITCH;
            for (uint32_t base = wave * CHUNK; base < plane_bytes; base += NWAVES * CHUNK) {
                if (base + lane_off < plane_bytes) {
                    const global_cptr_t gsrc = (global_cptr_t)(sp + base + lane_off);
                    const lds_ptr_t ldst = (lds_ptr_t)(dp + base);
                    // the size operand must be a literal
                    if constexpr (G == 16) {
                        __builtin_amdgcn_global_load_lds(gsrc, ldst, 16, 0, 0);
                    } else {
                        __builtin_amdgcn_global_load_lds(gsrc, ldst, 4, 0, 0);
                    }
                }
            }
        }
    }
}

// PITCH: compile-time byte distance between staged planes in LDS (>= padded plane size + 16).  The LDS holds two
// buffers of CGS planes each.  Compile-time so that a tap address is "register + immediate".
template <typename T, int INTERP, int PAD, bool ALIGN, int THREADS, int PPT, int CGS, int PITCH>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(1, 4))) void gs2d_lds_kernel(const T* __restrict__ x, const T* __restrict__ grid,
                                                           T* __restrict__ y, int32_t C, int32_t H, int32_t W,
                                                           int32_t out_plane, uint32_t tiles_per_n,
                                                           uint32_t cblocks, int32_t chans_per_block,
                                                           int32_t copy_gran, int32_t pair_aligned)
{
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    constexpr int NT = (INTERP == 0) ? 4 : 1;
    constexpr int BUF_BYTES = CGS * PITCH;
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
    const int32_t nstages = (c_end - c_begin + CGS - 1) / CGS;
    const char* xb = reinterpret_cast<const char*>(x + ((int64_t)n * C + c_begin) * plane_elems);
    const size_t stage_bytes = (size_t)CGS * plane_bytes;

    auto start_stage = [&](int32_t s, int buf) {
        const int32_t left = c_end - c_begin - s * CGS;
        const int nch = left < CGS ? left : CGS;
        const char* src = xb + (size_t)s * stage_bytes;
        char* dst = lds + buf * BUF_BYTES;
        if (copy_gran == 16) {
            issue_stage_copy<16, THREADS, CGS, PITCH>(src, dst, plane_bytes, nch);
        } else if (copy_gran == 4) {
            issue_stage_copy<4, THREADS, CGS, PITCH>(src, dst, plane_bytes, nch);
        } else {
            // planes whose size or address is not a multiple of 4 bytes: element-wise copy through registers
            const T* se = reinterpret_cast<const T*>(src);
            for (int k = 0; k < nch; k++) {
                T* de = reinterpret_cast<T*>(dst + k * PITCH);
                for (int32_t i = tid; i < plane_elems; i += THREADS) {
                    de[i] = se[(int64_t)k * plane_elems + i];
                }
            }
        }
    };

    // the zero slots behind each staged plane (both buffers); stage copies never touch them
    if (tid < 2 * CGS * 4) {
        reinterpret_cast<uint32_t*>(lds + (tid >> 2) * PITCH + zero_off)[tid & 3] = 0u;
    }
    start_stage(0, 0);

    // ---- per-pixel decisions, once for the whole channel range (overlaps the first stage copy) ----
    uint32_t toff[PPT][NT];
    float tw[PPT][4];
    uint32_t pixoff[PPT];  // byte offset of the pixel inside an output plane; out of range for lanes past the end
#pragma unroll
    for (int j = 0; j < PPT; j++) {
        const int32_t pix = (int32_t)tile * (THREADS * PPT) + j * THREADS + tid;
        const bool valid = pix < out_plane;
        const int32_t pc = valid ? pix : out_plane - 1;
        pixoff[j] = valid ? (uint32_t)pc * (uint32_t)sizeof(T) : 0x80000000u;
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

    T* yb = y + ((int64_t)n * C + c_begin) * out_plane;
    const uint32_t out_plane_bytes = (uint32_t)out_plane * (uint32_t)sizeof(T);

    auto sample_stage = [&](int32_t s, const char* buf) {
        const int32_t left = c_end - c_begin - s * CGS;
        T* ys = yb + (int64_t)s * CGS * out_plane;
        if (left >= CGS) {
            // software pipeline over the channels of the stage: the taps of channel k+1 are read from LDS
            // while channel k is blended and stored
            T raw[2][PPT][NT];
#pragma unroll
            for (int j = 0; j < PPT; j++) {
                load_taps<T, NT>(buf, toff[j], raw[0][j]);
            }
#pragma unroll
            for (int k = 0; k < CGS; k++) {
                if (k + 1 < CGS) {
#pragma unroll
                    for (int j = 0; j < PPT; j++) {
                        load_taps<T, NT>(buf + (k + 1) * PITCH, toff[j], raw[(k + 1) & 1][j]);
                    }
                }
                const __amdgpu_buffer_rsrc_t rsrc =
                    __builtin_amdgcn_make_buffer_rsrc(ys + (int64_t)k * out_plane, 0, out_plane_bytes, kBufferFlags);
#pragma unroll
                for (int j = 0; j < PPT; j++) {
                    buffer_store_elem<T>(blend<T, INTERP>(raw[k & 1][j], tw[j]), rsrc, pixoff[j]);
                }
            }
        } else {
            for (int k = 0; k < left; k++) {
                const __amdgpu_buffer_rsrc_t rsrc =
                    __builtin_amdgcn_make_buffer_rsrc(ys + (int64_t)k * out_plane, 0, out_plane_bytes, kBufferFlags);
                T raw[PPT][NT];
#pragma unroll
                for (int j = 0; j < PPT; j++) {
                    load_taps<T, NT>(buf + k * PITCH, toff[j], raw[j]);
                }
#pragma unroll
                for (int j = 0; j < PPT; j++) {
                    buffer_store_elem<T>(blend<T, INTERP>(raw[j], tw[j]), rsrc, pixoff[j]);
                }
            }
        }
    };

    // Stage s lives in buffer s & 1.  Per stage: wait for its copy (issued one stage earlier), barrier (which
    // also tells that everybody left the other buffer), start the next copy into the other buffer, sample.
    for (int32_t s = 0; s < nstages; s += 2) {
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (s + 1 < nstages) {
            start_stage(s + 1, 1);
        }
        sample_stage(s, lds);
        if (s + 1 < nstages) {
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            if (s + 2 < nstages) {
                start_stage(s + 2, 0);
            }
            sample_stage(s + 1, lds + BUF_BYTES);
        }
    }
}

}  // namespace opscv
