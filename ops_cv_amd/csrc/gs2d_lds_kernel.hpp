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

#include <type_traits>

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

// s_waitcnt that waits only for the vector-memory counter to drop to `n` (gfx9 encoding: vmcnt is split over
// bits 3:0 and 15:14; the other counters are left at their "do not wait" maximum).
template <int N>
__device__ __forceinline__ void wait_vmcnt_imm()
{
    static_assert(N >= 0 && N <= 63, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

// Waits until at most  per_copy_stage * mine + per_sampled_stage * sampled  vector-memory operations of this
// wavefront are outstanding; `mine` (copy instructions per plane of this wavefront, 0..4) and `sampled`
// (0..MAX_SAMPLED) are wave-uniform run-time values, the products are turned into immediates here.
// Anything outside the table waits for everything.
template <int PER_COPY, int PER_SAMPLED, int MAX_SAMPLED>
__device__ __forceinline__ void wait_vmcnt_table(uint32_t mine, uint32_t sampled)
{
    static_assert(MAX_SAMPLED <= 3, "table covers up to three sampled stages");
    constexpr int kMaxMine = 4;
    if (mine > (uint32_t)kMaxMine || sampled > (uint32_t)MAX_SAMPLED ||
        PER_COPY * kMaxMine + PER_SAMPLED * MAX_SAMPLED > 63) {
        wait_vmcnt_imm<0>();
        return;
    }
    const uint32_t key = __builtin_amdgcn_readfirstlane(mine * 4u + sampled);
    switch (key) {
#define OPSCV_W(M, S)                                                             \
    case (M) * 4 + (S):                                                           \
        wait_vmcnt_imm<(PER_COPY * (M) + PER_SAMPLED * (S)) <= 63 ? (PER_COPY * (M) + PER_SAMPLED * (S)) : 0>(); \
        break;
#define OPSCV_WM(M) OPSCV_W(M, 0) OPSCV_W(M, 1) OPSCV_W(M, 2) OPSCV_W(M, 3)
        OPSCV_WM(0) OPSCV_WM(1) OPSCV_WM(2) OPSCV_WM(3) OPSCV_WM(4)
#undef OPSCV_WM
#undef OPSCV_W
        default: wait_vmcnt_imm<0>(); break;
    }
}

// Workgroup barrier without the memory fences of __syncthreads(): a fence would make the compiler drain the
// vector-memory counter (the global->LDS copies count there), which is exactly what the ring must not do.
// The caller has already waited for the operations it depends on; the empty asm statements keep the compiler
// from moving LDS accesses across the barrier.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Starts the asynchronous copy of `nch` consecutive input planes (plane_bytes each, contiguous in global memory
// from `src`) to LDS at `dst` with PITCH bytes between planes.  G = bytes per lane (16 or 4): the largest
// granule that divides the plane size and the source alignment.  Each wavefront instruction moves 64*G
// contiguous bytes; lanes past the end of a plane are masked off.  Wavefront w takes chunks w, w+NWAVES, ...
// of every plane, so it issues the same number of instructions for every full stage.
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

// LDS layout: a ring of NBUF stage slots, each CGS planes at PITCH bytes (PITCH >= padded plane size + 16,
// compile-time so that a tap address is "register + immediate").  Stage s lives in slot s % NBUF and up to
// NBUF-1 later stages are in flight while it is sampled.
//
// Completion of a stage copy is tracked with the wavefront's own vector-memory counter, which retires in issue
// order: when stage s is needed, the operations this wavefront issued after the copy of stage s are the copies
// of the NBUF-2 following stages and the output stores of the stages sampled since, so waiting until at most
// that many operations are outstanding guarantees the copy has landed without draining the newer ones.  The
// count is exact only while every stage involved is a full one; otherwise the wait is for everything.
template <typename T, int INTERP, int PAD, bool ALIGN, int THREADS, int PPT, int CGS, int NBUF, int PITCH>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(1, 4))) void gs2d_lds_kernel(
    const T* __restrict__ x, const T* __restrict__ grid, T* __restrict__ y, int32_t C, int32_t H, int32_t W,
    int32_t out_plane, uint32_t tiles_per_n, uint32_t cblocks, int32_t chans_per_block, int32_t copy_gran,
    int32_t pair_aligned, int32_t xcd_swizzle)
{
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    constexpr int NT = (INTERP == 0) ? 4 : 1;
    constexpr int SLOT_BYTES = CGS * PITCH;
    constexpr int DEPTH = NBUF - 1;          // stages in flight ahead of the one being sampled
    constexpr int NWAVES = THREADS / 64;
    constexpr uint32_t STORES_PER_STAGE = PPT * CGS;
    const int tid = threadIdx.x;

    // Block -> (group = (n, channel block), tile).  Workgroups are handed to the 8 XCDs round-robin by index;
    // with the swizzle all tiles of one group (they read the same input planes) land on the same XCD next to
    // each other in time, so the planes are fetched into one L2 once.
    uint32_t group, tile;
    if (xcd_swizzle) {
        const uint32_t xcd = blockIdx.x & 7u;
        const uint32_t i = blockIdx.x >> 3;
        group = (i / tiles_per_n) * 8u + xcd;
        tile = i % tiles_per_n;
    } else {
        group = blockIdx.x / tiles_per_n;
        tile = blockIdx.x % tiles_per_n;
    }
    const uint32_t cb = group % cblocks;
    const uint32_t n = group / cblocks;

    const int32_t plane_elems = H * W;
    const uint32_t plane_bytes = (uint32_t)plane_elems * (uint32_t)sizeof(T);
    const uint32_t zero_off = round_up16(plane_bytes);
    const int32_t c_begin = (int32_t)cb * chans_per_block;
    const int32_t c_end = (c_begin + chans_per_block < C) ? c_begin + chans_per_block : C;
    const int32_t nchan = c_end - c_begin;
    const int32_t nstages = (nchan + CGS - 1) / CGS;
    const int32_t nfull = nchan / CGS;  // stages 0 .. nfull-1 hold CGS planes
    const char* xb = reinterpret_cast<const char*>(x + ((int64_t)n * C + c_begin) * plane_elems);
    const size_t stage_bytes = (size_t)CGS * plane_bytes;

    // copy instructions this wavefront issues per plane (copy_gran is 16 or 4 bytes per lane)
    uint32_t copies_per_plane;
    {
        const uint32_t chunk = 64u * (uint32_t)copy_gran;
        const uint32_t chunks = (plane_bytes + chunk - 1) / chunk;
        const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)tid >> 6);
        copies_per_plane = (chunks > wave) ? (chunks - wave + NWAVES - 1) / NWAVES : 0;
    }

    auto start_stage = [&](int32_t s, int slot) {
        const int32_t left = nchan - s * CGS;
        const int nch = left < CGS ? left : CGS;
        const char* src = xb + (size_t)s * stage_bytes;
        char* dst = lds + slot * SLOT_BYTES;
        if (copy_gran == 16) {
            issue_stage_copy<16, THREADS, CGS, PITCH>(src, dst, plane_bytes, nch);
        } else {
            issue_stage_copy<4, THREADS, CGS, PITCH>(src, dst, plane_bytes, nch);
        }
    };

    // the zero slots behind each staged plane (all ring slots); stage copies never touch them
    if (tid < NBUF * CGS * 4) {
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

    // the rest of the prologue: stages 1 .. DEPTH-1 (stage 0 went out before the grid loads so that the wait
    // for the grid values does not also wait for these)
#pragma unroll
    for (int s = 1; s < DEPTH; s++) {
        if (s < nstages) {
            start_stage(s, s);
        }
    }

    T* yb = y + ((int64_t)n * C + c_begin) * out_plane;
    const uint32_t out_plane_bytes = (uint32_t)out_plane * (uint32_t)sizeof(T);

    auto sample_stage = [&](int32_t s, const char* buf) {
        const int32_t left = nchan - s * CGS;
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

    // One step of the ring: wait for the copy of stage s, barrier (it also tells that every wavefront has left
    // the slot that is refilled next), start the copy of stage s + DEPTH, sample stage s.
    auto step = [&](int32_t s, auto slot_tag) {
        constexpr int SLOT = decltype(slot_tag)::value;
        // Operations issued after the copy of stage s: copies of stages s+1 .. s+DEPTH-1 and the stores of the
        // min(s, DEPTH) stages sampled since.  Exact only when those later stages exist and are full.
        if (s + DEPTH - 1 < nfull) {
            const uint32_t sampled = (s < DEPTH) ? (uint32_t)s : (uint32_t)DEPTH;
            wait_vmcnt_table<(DEPTH - 1) * CGS, STORES_PER_STAGE, (DEPTH < 3 ? DEPTH : 3)>(copies_per_plane, sampled);
        } else {
            wait_vmcnt_imm<0>();
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the zero-slot writes before the first barrier
        lds_barrier();
        if (s + DEPTH < nstages) {
            start_stage(s + DEPTH, (SLOT + DEPTH) % NBUF);
        }
        sample_stage(s, lds + SLOT * SLOT_BYTES);
    };

    for (int32_t s = 0; s < nstages; s += NBUF) {
        step(s, std::integral_constant<int, 0>{});
        if constexpr (NBUF > 1) {
            if (s + 1 < nstages) {
                step(s + 1, std::integral_constant<int, 1 % NBUF>{});
            }
        }
        if constexpr (NBUF > 2) {
            if (s + 2 < nstages) {
                step(s + 2, std::integral_constant<int, 2 % NBUF>{});
            }
        }
        if constexpr (NBUF > 3) {
            if (s + 3 < nstages) {
                step(s + 3, std::integral_constant<int, 3 % NBUF>{});
            }
        }
    }
}

}  // namespace opscv
