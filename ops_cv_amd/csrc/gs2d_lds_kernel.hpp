// Grid sampler 2-D forward, LDS-staged variant for gfx950: device code.
//
// Same arithmetic as the direct variant (see sampler_math.hpp; reference kernel
// image/grid_sampler2_d/op_kernel/arch35/grid_sampler2_d_simt.h:461-514), different data movement:
//
//   * a workgroup owns (batch n, a tile of THREADS*PPT output pixels, a range of channels);
//   * every lane decides its PPT pixels once -- four LDS byte offsets and four weights per pixel (bicubic:
//     sixteen offsets, eight coefficients) stay in registers for the whole channel range;
//   * the channel range is walked in stages of CGS whole input planes.  The planes go from HBM straight into
//     LDS with the asynchronous global->LDS loads of gfx950 (no registers, 16 bytes per lane, 1 KiB per
//     wavefront instruction), double-buffered: stage s+1 is in flight while stage s is sampled;
//   * every tap is a 2- or 4-byte LDS read, so the scattered part of the gather never leaves the CU;
//   * a tap outside the image points at a 16-byte slot of zeros behind each staged plane, which reproduces the
//     reference's "skip the tap" exactly (0 * w adds nothing) without per-channel selects;
//   * every output channel plane is written once, 64 consecutive pixels per wavefront store, through a buffer
//     descriptor whose range check drops the lanes of a partial last tile.  The stores (and the loads of the grid
//     points) carry the non-temporal hint; the plane copies do not.
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

// The grid points (x, y interleaved, element type T) of COUNT pixels starting at `gp`, `stride` pixels apart, as raw
// bits.  The loads carry no condition and no use between them, so they are in flight together: one memory latency
// for all pixels of a lane (written per pixel with the alignment test inside, every load was followed by a wait).
//
// STREAM: the loads carry the non-temporal hint.  A kernel whose results leave through non-temporal stores must load
// its grid points the same way: on this part ordinary loads issued by the same kernel take the advantage of the
// streaming stores away again (fp16 N16 C256 64x64: 16.0 us with ordinary loads and stores, 17.3 us with ordinary
// loads and streaming stores, 14.3 us with both streaming).
template <typename V, bool STREAM>
__device__ __forceinline__ V load_maybe_streaming(const V* p)
{
    if constexpr (STREAM) {
        return __builtin_nontemporal_load(p);
    } else {
        return *p;
    }
}

template <typename T, int COUNT, bool STREAM = false>
__device__ __forceinline__ void load_grid_points(const T* const* gp, bool pair_aligned, float* gx, float* gy)
{
    if constexpr (sizeof(T) == 2) {
        if (pair_aligned) {
            uint32_t raw[COUNT];
#pragma unroll
            for (int j = 0; j < COUNT; j++) {
                raw[j] = load_maybe_streaming<uint32_t, STREAM>(reinterpret_cast<const uint32_t*>(gp[j]));
            }
#pragma unroll
            for (int j = 0; j < COUNT; j++) {
                T lo = __builtin_bit_cast(T, (uint16_t)(raw[j] & 0xFFFFu));
                T hi = __builtin_bit_cast(T, (uint16_t)(raw[j] >> 16));
                gx[j] = ElemIO<T>::load(&lo);
                gy[j] = ElemIO<T>::load(&hi);
            }
            return;
        }
    } else {
        if (pair_aligned) {
            typedef float float_pair_t __attribute__((ext_vector_type(2)));
            float_pair_t raw[COUNT];
#pragma unroll
            for (int j = 0; j < COUNT; j++) {
                raw[j] = load_maybe_streaming<float_pair_t, STREAM>(reinterpret_cast<const float_pair_t*>(gp[j]));
            }
#pragma unroll
            for (int j = 0; j < COUNT; j++) {
                gx[j] = raw[j].x;
                gy[j] = raw[j].y;
            }
            return;
        }
    }
    typedef typename std::conditional<sizeof(T) == 2, uint16_t, uint32_t>::type bits_t;
    bits_t ex[COUNT], ey[COUNT];
#pragma unroll
    for (int j = 0; j < COUNT; j++) {
        ex[j] = load_maybe_streaming<bits_t, STREAM>(reinterpret_cast<const bits_t*>(gp[j]));
        ey[j] = load_maybe_streaming<bits_t, STREAM>(reinterpret_cast<const bits_t*>(gp[j]) + 1);
    }
#pragma unroll
    for (int j = 0; j < COUNT; j++) {
        const T tx = __builtin_bit_cast(T, ex[j]), ty = __builtin_bit_cast(T, ey[j]);
        gx[j] = ElemIO<T>::load(&tx);
        gy[j] = ElemIO<T>::load(&ty);
    }
}

// Raw tap values of one pixel from a staged plane (LDS reads only, no arithmetic, so that the reads of
// many pixels can be in flight together).
// `taddr` holds absolute LDS addresses of the taps in the first plane of the ring (base of the LDS allocation
// already added, once, in the prologue); `plane_off` is the compile-time distance of the plane being sampled, which
// ends up in the instruction's immediate offset.
// A tap value stays in a 32-bit register of its own (16-bit elements zero-extended, as the LDS read delivers them):
// left as 16-bit objects the compiler packs two of them into one register, and the packing instruction waits for
// the reads right behind their issue, which undoes the overlap of the reads with the previous plane's arithmetic.
template <typename T, int NT>
__device__ __forceinline__ void load_taps(uint32_t plane_off, const uint32_t* taddr, uint32_t* raw)
{
    typedef typename std::conditional<sizeof(T) == 2, uint16_t, uint32_t>::type bits_t;
    typedef const bits_t __attribute__((address_space(3))) * lds_bits_ptr_t;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        raw[t] = (uint32_t)*reinterpret_cast<lds_bits_ptr_t>((uintptr_t)(taddr[t] + plane_off));
    }
}

template <typename T>
__device__ __forceinline__ float tap_value(uint32_t raw)
{
    if constexpr (std::is_same<T, float>::value) {
        return __builtin_bit_cast(float, raw);
    } else if constexpr (std::is_same<T, _Float16>::value) {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
    } else {
        return __builtin_bit_cast(float, raw << 16);
    }
}

// ... and of a tap held as an element (the channels-last kernel loads vectors of elements)
template <typename T, typename R>
__device__ __forceinline__ float tap_value_of(const R& raw)
{
    if constexpr (std::is_same<R, uint32_t>::value && !std::is_same<T, uint32_t>::value) {
        return tap_value<T>(raw);
    } else {
        return ElemIO<T>::load(&raw);
    }
}

// One output sample from its tap values: grid_sampler2_d_simt.h:321-338 (0 + nw + ne + sw + se, products and
// sums rounded separately) for bilinear, :341-360 (the value passes through fp32) for nearest.
// fma(v, w, +0) is "0 + v*w" with one rounding of the exact product, i.e. the reference's first step bit for
// bit; fma(v, w, -0) is "v*w" bit for bit (also for zero products of either sign).  Writing the products as
// fmas lets the 16-bit -> fp32 conversion ride on the multiply (mixed-precision fma) for fp16; `neg_zero` is
// -0.0f handed in at run time so that the compiler cannot fold the fma back into a multiply.
//
// Bicubic (grid_sampler2_d_simt.h:362-371 and :418-455): raw[4*j + k] is the tap of row j, column k; tw[0..3] are
// the column coefficients, tw[4..7] the row coefficients.  Each row is  c0*v0  followed by three fused
// multiply-adds, and so is the column of the four row results.  A tap outside the image reads the zero slot; a
// row outside the image therefore evaluates to +0 like the reference's literal 0 (the products are zeros and at
// least one of the two middle coefficients is positive, so the sum cannot be -0).
//
// `first` is the addend of the first bilinear product: +0 for "0 + nw" as above; -0 gives the bare product "nw" with
// which the reference's second bilinear kernel starts its sum (grid_sampler_2d_bilinear_smit.h:78-82), which differs
// in the sign of a zero result only.
template <typename T, int INTERP, typename R>
__device__ __forceinline__ float blend(const R* raw, const float* tw, float neg_zero, float first = 0.0f)
{
    if (INTERP == 2) {
        float r[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float acc = __builtin_fmaf(tap_value_of<T>(raw[4 * j]), tw[0], neg_zero);
            acc = __builtin_fmaf(tw[1], tap_value_of<T>(raw[4 * j + 1]), acc);
            acc = __builtin_fmaf(tw[2], tap_value_of<T>(raw[4 * j + 2]), acc);
            acc = __builtin_fmaf(tw[3], tap_value_of<T>(raw[4 * j + 3]), acc);
            r[j] = acc;
        }
        float out = tw[4] * r[0];
        out = __builtin_fmaf(tw[5], r[1], out);
        out = __builtin_fmaf(tw[6], r[2], out);
        out = __builtin_fmaf(tw[7], r[3], out);
        return as_fp32_value(out);
    }
    if (INTERP == 0) {
        float out = __builtin_fmaf(tap_value_of<T>(raw[0]), tw[0], first);
        out += __builtin_fmaf(tap_value_of<T>(raw[1]), tw[1], neg_zero);
        out += __builtin_fmaf(tap_value_of<T>(raw[2]), tw[2], neg_zero);
        out += __builtin_fmaf(tap_value_of<T>(raw[3]), tw[3], neg_zero);
        return out;
    }
    return tap_value_of<T>(raw[0]);
}

// cache-policy operand of the buffer stores: 0 = ordinary, 2 = non-temporal (streaming: the line is written through
// and not kept, so the end of the kernel has no dirty lines to write back)
constexpr int kStoreOrdinary = 0;
constexpr int kStoreStreaming = 2;

template <typename T, bool STREAM = false>
__device__ __forceinline__ void buffer_store_elem(float v, __amdgpu_buffer_rsrc_t rsrc, uint32_t byte_off)
{
    constexpr int AUX = STREAM ? kStoreStreaming : kStoreOrdinary;
    if constexpr (sizeof(T) == 4) {
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), rsrc, (int)byte_off, 0, AUX);
    } else {
        T h;
        ElemIO<T>::store(&h, v);
        __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(uint16_t, h), rsrc, (int)byte_off, 0, AUX);
    }
}

// The results of ADJ neighbouring output pixels of one channel leave as one store: two 16-bit results as one dword
// (each rounded to T on its own, exactly as the single store does), so a wavefront writes 256 contiguous bytes per
// instruction instead of 128.  The caller guarantees a 4-byte aligned address (even pixel index, even plane size).
template <typename T, int ADJ, bool STREAM = false>
__device__ __forceinline__ void buffer_store_group(const float* v, __amdgpu_buffer_rsrc_t rsrc, uint32_t byte_off)
{
    if constexpr (ADJ == 1) {
        buffer_store_elem<T, STREAM>(v[0], rsrc, byte_off);
    } else {
        static_assert(ADJ == 2 && sizeof(T) == 2, "pairs of 16-bit results only");
        // one packed conversion instruction, each half rounded to nearest even like the single conversion
        typedef float float_pair_t __attribute__((ext_vector_type(2)));
        typedef T elem_pair_t __attribute__((ext_vector_type(2)));
        const float_pair_t f = {v[0], v[1]};
        const elem_pair_t e = __builtin_convertvector(f, elem_pair_t);
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, e), rsrc, (int)byte_off, 0,
                                              STREAM ? kStoreStreaming : kStoreOrdinary);
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

// Run-time `n` (wave-uniform, 0..63) -> the matching immediate form; larger values cannot be expressed and wait
// for everything.  The instruction only takes a literal, so the value is found by bisection: six scalar compares.
// (Written as a switch over the 64 values it compiled into a chain of compare-and-branch blocks walked from 63
// downwards, several hundred cycles per wait for the small counts a ring uses.)
template <int LO, int HI>
__device__ __forceinline__ void wait_vmcnt_between(uint32_t n)
{
    if constexpr (LO == HI) {
        wait_vmcnt_imm<LO>();
    } else {
        constexpr int MID = (LO + HI) / 2;
        if (n <= (uint32_t)MID) {
            wait_vmcnt_between<LO, MID>(n);
        } else {
            wait_vmcnt_between<MID + 1, HI>(n);
        }
    }
}

__device__ __forceinline__ void wait_vmcnt(uint32_t n)
{
    n = __builtin_amdgcn_readfirstlane(n);
    if (n > 63u) {
        wait_vmcnt_imm<0>();
    } else {
        wait_vmcnt_between<0, 63>(n);
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

// The last stages of a ring whose stages are PP copy instructions each: stage by stage, wait until at most the K,
// K - 1, ... 0 stages after it are outstanding, and hand it over.
template <int K, int PP>
__device__ __forceinline__ void ring_rundown()
{
    wait_vmcnt_imm<K * PP>();
    lds_barrier();
    if constexpr (K > 0) {
        ring_rundown<K - 1, PP>();
    }
}

// Bank-spreading layout of a staged plane whose rows are exactly 128 bytes (row_shift = 7 | turn << 8; 0 = plain
// layout).  LDS has 32 four-byte banks, i.e. 128 bytes per "line"; with that row pitch column x of every row falls into
// the same bank, and coordinates clamped to the first or last column (border padding) make a wavefront read one bank
// 64 times.  The eight 16-byte chunks of each line are therefore rotated by `turn` chunks per row: byte offset o of the
// plane lives in chunk (chunk(o) + turn * row) mod 8 of its line, which shifts consecutive rows by 4 * turn banks
// (fp16 N16 C256 64x64, border: plain layout 21.2 us; chunks permuted by row & 7 instead 16.1 us; turn 2: 14.9, 4: 15.1,
// 6: 15.0, 7: 19.2).  The rotation stays inside the line, so it maps the plane onto itself.  The copy applies its
// inverse to the source address (the LDS side of the asynchronous copy is fixed per lane); a copy instruction covers
// eight whole rows starting at a multiple of 1 KiB, so the source offset of a lane inside that block is a per-lane
// constant.  The samplers apply it once per tap when they compute offsets.  Where the lanes of a wavefront already
// read different columns (zeros and reflection padding with two neighbouring pixels per lane) any shift between rows
// makes them meet more often: 13.1 us plain, 20 to 24 us rotated.
// Division of a block index by a launch constant without the hardware's reciprocal sequence (a dependent chain of
// conversions and a reciprocal that every wavefront of the kernel would walk before it knows its work): the host hands
// over m = ceil(2^s / d), s = 31 + ceil(log2 d), and floor(x / d) = (x * m) >> s for every x < 2^31.
struct FastDiv {
    uint32_t mul = 0x80000000u;
    uint32_t shift = 31;
    uint32_t div = 1;
};

inline FastDiv make_fast_div(uint32_t d)
{
    FastDiv f;
    uint32_t l = 0;
    while ((1ull << l) < d) {
        l++;
    }
    f.shift = 31 + l;
    f.mul = (uint32_t)(((1ull << f.shift) + d - 1) / d);
    f.div = d;
    return f;
}

__device__ __forceinline__ uint32_t fast_div(uint32_t x, const FastDiv& f)
{
    return (uint32_t)(((uint64_t)x * f.mul) >> f.shift);
}

__device__ __forceinline__ uint32_t lds_swizzle(uint32_t byte_off, uint32_t row_shift)
{
    if (row_shift == 0u) {
        return byte_off;
    }
    const uint32_t turn = row_shift >> 8, row = byte_off >> 7;
    return (byte_off & ~0x70u) | ((((byte_off >> 4) + turn * row) & 7u) << 4);
}

// The chunk of a 1 KiB block (eight rows starting at a multiple of eight) that belongs at LDS position `byte_off` of
// the block: the inverse of lds_swizzle.
__device__ __forceinline__ uint32_t lds_unswizzle(uint32_t byte_off, uint32_t row_shift)
{
    if (row_shift == 0u) {
        return byte_off;
    }
    const uint32_t turn = row_shift >> 8, row = byte_off >> 7;
    return (byte_off & ~0x70u) | ((((byte_off >> 4) - turn * row) & 7u) << 4);
}

// Starts the asynchronous copy of `nch` consecutive input planes (plane_bytes each, contiguous in global memory
// from `src`) to LDS at `dst` with PITCH bytes between planes.  G = bytes per lane (16 or 4): the largest
// granule that divides the plane size and the source alignment.  Each wavefront instruction moves 64*G
// contiguous bytes; lanes past the end of a plane are masked off.  The LWAVES loader wavefronts share the
// chunks of every plane round-robin (`lwave` = index of the calling one).  Returns nothing; the number of
// instructions issued per plane by this wavefront is copies_of() in the kernel.
//
// SHIFTED (G = 16): planes that do not start on a 16-byte boundary or are not whole 16-byte units -- an odd number of
// elements per plane, a tensor view that starts anywhere.  The copy of such a plane starts up to 14 bytes early, on
// the boundary, and ends on the boundary after the plane's last byte, so the plane's first element lands `shift`
// bytes into its LDS slot; the samplers add the same shift (plane_shift() in the kernel).  The bytes read outside the
// plane share an aligned 16-byte unit with bytes inside it, so they are readable wherever the plane is; they land
// in the slot's padding.  The number of copy instructions then depends on the plane: stage_copy_count() below.
template <int G, int LWAVES, int CGS, int PITCH, bool SHIFTED = false>
__device__ __forceinline__ void issue_stage_copy(const char* src, char* dst, uint32_t plane_bytes, int nch,
                                                 uint32_t lwave, uint32_t lane, uint32_t lane_src_off)
{
    constexpr uint32_t CHUNK = 64u * G;
    const uint32_t lane_off = lane * G;
#pragma unroll
    for (int k = 0; k < CGS; k++) {
        if (k < nch) {
            const char* sp = src + (size_t)k * plane_bytes;
            char* dp = dst + k * PITCH;
            uint32_t copy_bytes = plane_bytes;
            if constexpr (SHIFTED) {
                const uint32_t shift = (uint32_t)(reinterpret_cast<uintptr_t>(sp) & 15u);
                sp -= shift;
                copy_bytes = (shift + plane_bytes + 15u) & ~15u;
            }
            // whole chunks first, without a per-lane test (no exec-mask bookkeeping between the copy instructions:
            // 13.2 -> 12.9 us on fp16 N16 C256 64x64), then the one partial chunk if this wavefront is its owner
            const uint32_t whole_bytes = copy_bytes - copy_bytes % CHUNK;
            uint32_t base = lwave * CHUNK;
            for (; base < whole_bytes; base += LWAVES * CHUNK) {
                // lane_src_off: the chunk of this 1 KiB block that belongs at the lane's LDS position
                const global_cptr_t gsrc = (global_cptr_t)(sp + base + lane_src_off);
                const lds_ptr_t ldst = (lds_ptr_t)(dp + base);
                // the size operand must be a literal
                if constexpr (G == 16) {
                    __builtin_amdgcn_global_load_lds(gsrc, ldst, 16, 0, 0);
                } else {
                    __builtin_amdgcn_global_load_lds(gsrc, ldst, 4, 0, 0);
                }
            }
            if (base < copy_bytes && base + lane_off < copy_bytes) {
                const global_cptr_t gsrc = (global_cptr_t)(sp + base + lane_src_off);
                const lds_ptr_t ldst = (lds_ptr_t)(dp + base);
                if constexpr (G == 16) {
                    __builtin_amdgcn_global_load_lds(gsrc, ldst, 16, 0, 0);
                } else {
                    __builtin_amdgcn_global_load_lds(gsrc, ldst, 4, 0, 0);
                }
            }
        }
    }
}

// The per-pixel decisions of one lane: tap offsets (LDS byte offsets inside a staged plane, `zero_off` for a tap outside
// the image) and weights for its PPT pixels.  Padding mode and align_corners are run-time, wave-uniform values
// (kernel arguments; scalar branches around the clip and reflect steps): the decisions run once per workgroup,
// outside the channel loop, so one kernel serves all six combinations at no cost to the loop.
// SWIZZLED: the staged planes use the bank-spreading layout (`rs` = its row shift); without it `rs` is not looked at,
// so the plain layout pays nothing per tap.
// Source coordinates of COUNT grid points for one (padding mode, align_corners) pair, and the one wave-uniform switch
// that picks the pair.  All coordinates of a lane are computed inside one branch, so the chains of the lane's pixels
// interleave as they do with the modes fixed at compile time (a branch per coordinate cost 0.3 us on fp16 N16 C256
// 64x64: each chain then waited out its own latencies).
template <int PAD, bool ALIGN, int COUNT>
__device__ __forceinline__ void source_indices(const float* gxs, const float* gys, int32_t H, int32_t W, float* ixs,
                                               float* iys)
{
#pragma unroll
    for (int j = 0; j < COUNT; j++) {
        ixs[j] = compute_source_index<PAD, ALIGN>(gxs[j], W);
        iys[j] = compute_source_index<PAD, ALIGN>(gys[j], H);
    }
}

// ... by the second coordinate rule (sampler_math.hpp: unnormalize3, clip3): always finite, -100 for what was not
template <int PAD, bool ALIGN, int COUNT>
__device__ __forceinline__ void source_indices_arch35(const float* gxs, const float* gys, int32_t H, int32_t W,
                                                      float* ixs, float* iys)
{
#pragma unroll
    for (int j = 0; j < COUNT; j++) {
        ixs[j] = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gxs[j], W), W);
        iys[j] = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gys[j], H), H);
    }
}

template <int COUNT>
__device__ __forceinline__ void source_indices_rt(const float* gxs, const float* gys, int32_t H, int32_t W, int32_t pad,
                                                  bool align, bool arch35, float* ixs, float* iys)
{
    if (arch35) {
        switch (pad * 2 + (align ? 1 : 0)) {
            case 0: source_indices_arch35<0, false, COUNT>(gxs, gys, H, W, ixs, iys); break;
            case 1: source_indices_arch35<0, true, COUNT>(gxs, gys, H, W, ixs, iys); break;
            case 2: source_indices_arch35<1, false, COUNT>(gxs, gys, H, W, ixs, iys); break;
            case 3: source_indices_arch35<1, true, COUNT>(gxs, gys, H, W, ixs, iys); break;
            case 4: source_indices_arch35<2, false, COUNT>(gxs, gys, H, W, ixs, iys); break;
            default: source_indices_arch35<2, true, COUNT>(gxs, gys, H, W, ixs, iys); break;
        }
        return;
    }
    switch (pad * 2 + (align ? 1 : 0)) {
        case 0: source_indices<0, false, COUNT>(gxs, gys, H, W, ixs, iys); break;
        case 1: source_indices<0, true, COUNT>(gxs, gys, H, W, ixs, iys); break;
        case 2: source_indices<1, false, COUNT>(gxs, gys, H, W, ixs, iys); break;
        case 3: source_indices<1, true, COUNT>(gxs, gys, H, W, ixs, iys); break;
        case 4: source_indices<2, false, COUNT>(gxs, gys, H, W, ixs, iys); break;
        default: source_indices<2, true, COUNT>(gxs, gys, H, W, ixs, iys); break;
    }
}

template <typename T, int INTERP, int PPT, int NT, int NW, bool SWIZZLED>
__device__ __forceinline__ void decide_lane_pixels(const float* gxs, const float* gys, int32_t H, int32_t W,
                                                   uint32_t ldsw, uint32_t row_shift, uint32_t zero_off, int32_t pad,
                                                   bool align, bool arch35, uint32_t (*toff)[NT], float (*tw)[NW])
{
    // ldsw: elements per staged row (W, or more where the loaders pad the rows -- see the kernel)
    const uint32_t rs = SWIZZLED ? row_shift : 0u;
    float ixs[PPT], iys[PPT];
    if constexpr (INTERP != 2) {
        source_indices_rt<PPT>(gxs, gys, H, W, pad, align, arch35 && INTERP == 0, ixs, iys);
    }
#pragma unroll
    for (int j = 0; j < PPT; j++) {
        if constexpr (INTERP == 2) {
            const BicubicTap b = decide_bicubic_rt(gxs[j], gys[j], H, W, pad, align);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const bool row_in = b.by[r] >= 0 && b.by[r] < H && !b.flag;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const bool in = row_in && b.bx[k] >= 0 && b.bx[k] < W;
                    toff[j][4 * r + k] =
                        in ? lds_swizzle(((uint32_t)b.by[r] * ldsw + (uint32_t)b.bx[k]) * (uint32_t)sizeof(T), rs)
                           : zero_off;
                }
                tw[j][r] = b.cx[r];
                tw[j][4 + r] = b.cy[r];
            }
            if (b.flag) {
                tw[j][0] = __builtin_nanf("");  // 0 * NaN: every channel becomes NaN, as the reference writes
            }
            continue;
        }
        // Bilinear and nearest: the decisions of decide_pixel() (sampler_math.hpp; grid_sampler2_d_simt.h:479-498,
        // 307-316, 341-349) written without branches -- this prologue runs once per workgroup for every one of its
        // pixels and is on the critical path to the first sampled stage, so its instruction count matters.
        // Bounds tests are single unsigned compares (a negative index is a huge unsigned one), tap offsets follow
        // from the north-west one by modular arithmetic, and the "+1" of an index saturated at INT32_MAX wraps to
        // 0x80000000, which is out of bounds like the saturated value itself.
        float ix = ixs[j];
        float iy = iys[j];
        const bool finite = __builtin_fabsf(ix) < __builtin_inff() && __builtin_fabsf(iy) < __builtin_inff();
        const bool x_far = ix > 2147483646.0f || ix < -2147483648.0f;  // safe_downgrade: -> -100, always outside
        const bool y_far = iy > 2147483646.0f || iy < -2147483648.0f;
        const uint32_t uw = (uint32_t)W, uh = (uint32_t)H, es = (uint32_t)sizeof(T);
        if (INTERP == 0) {
            ix = x_far ? -100.0f : ix;
            iy = y_far ? -100.0f : iy;
            const float ixf = __builtin_floorf(ix), iyf = __builtin_floorf(iy);
            const uint32_t x0 = (uint32_t)float_to_i32(ixf), y0 = (uint32_t)float_to_i32(iyf);
            // the second rule takes the east / south index from the float "floor + 1"
            // (grid_sampler_2d_bilinear_smit.h:84-99), which is the integer "+ 1" for every index a staged plane has
            const uint32_t x1 = x0 + 1u, y1 = y0 + 1u;
            const bool in_x0 = x0 < uw && finite, in_x1 = x1 < uw && finite;
            const bool in_y0 = y0 < uh, in_y1 = y1 < uh;
            const uint32_t o_nw = (y0 * ldsw + x0) * es;
            const uint32_t o_sw = o_nw + ldsw * es;
            toff[j][0] = (in_y0 && in_x0) ? lds_swizzle(o_nw, rs) : zero_off;
            toff[j][1] = (in_y0 && in_x1) ? lds_swizzle(o_nw + es, rs) : zero_off;
            toff[j][2] = (in_y1 && in_x0) ? lds_swizzle(o_sw, rs) : zero_off;
            toff[j][3] = (in_y1 && in_x1) ? lds_swizzle(o_sw + es, rs) : zero_off;
            // weights: (x0 + 1 - ix), (ix - x0) by the first rule; (1 - d), d with d = ix - floor(ix) by the second
            // (grid_sampler_2d_bilinear_smit.h:72-76)
            const float wx1 = ix - ixf, wx0 = arch35 ? 1.0f - wx1 : ixf + 1.0f - ix;
            const float wy1 = iy - iyf, wy0 = arch35 ? 1.0f - wy1 : iyf + 1.0f - iy;
            // non-finite source coordinate: every tap reads the zero slot and 0 * NaN makes every channel NaN,
            // as the reference writes (grid_sampler2_d_simt.h:485-487); under the second rule the coordinate has
            // become -100 by now and the sample is zero
            tw[j][0] = finite ? wx0 * wy0 : __builtin_nanf("");
            tw[j][1] = wx1 * wy0;
            tw[j][2] = wx0 * wy1;
            tw[j][3] = wx1 * wy1;
        } else {
            ix = (x_far || !finite) ? -100.0f : ix;
            iy = (y_far || !finite) ? -100.0f : iy;
            // round half to even from floor, fraction and parity (grid_sampler2_d_simt.h:219-234)
            const float xf = __builtin_floorf(ix), yf = __builtin_floorf(iy);
            const float fx = ix - xf, fy = iy - yf;
            const uint32_t xi = (uint32_t)float_to_i32(xf), yi = (uint32_t)float_to_i32(yf);
            const uint32_t xr = xi + ((fx > 0.5f || (fx == 0.5f && (xi & 1u))) ? 1u : 0u);
            const uint32_t yr = yi + ((fy > 0.5f || (fy == 0.5f && (yi & 1u))) ? 1u : 0u);
            const bool in = xr < uw && yr < uh;
            toff[j][0] = in ? lds_swizzle((yr * ldsw + xr) * es, rs) : zero_off;
            tw[j][0] = tw[j][1] = tw[j][2] = tw[j][3] = 0.0f;
        }
    }
}

// LDS layout: a ring of NBUF stage slots, each CGS planes at PITCH bytes (PITCH >= padded plane size + 16,
// compile-time so that a tap address is "register + immediate").  Stage s lives in slot s % NBUF and up to
// NBUF-1 later stages are in flight while it is sampled.
//
// The workgroup is split by role.  SWAVES sampler wavefronts own the output pixels (one lane = PPT pixels); they
// only read LDS and store results, and they never wait for their stores.  LWAVES loader wavefronts only issue
// the global->LDS copies.  On this architecture one counter per wavefront tracks loads and stores together and
// retires in issue order, so a wavefront that both copied and stored would have every copy wait behind its
// older stores; with the roles split the loader's counter sees copies only, and "stage s has landed" is "at most
// the copies of the later stages are outstanding".  One workgroup barrier per stage hands the stage over and
// tells the loaders that the slot sampled before is free again.
//
// SHIFTED_PLANES selects the layout for planes off the 16-byte grid (issue_stage_copy); it is a template parameter so
// that the kernels for whole, aligned planes carry no trace of it.
//
// CHANNEL_PAIRS (16-bit elements, bilinear, whole aligned planes of up to (PITCH - 16) / 2 bytes): a stage is two
// neighbouring channels interleaved -- the dword of an input element holds channel c in its low half and c + 1 in its
// high half -- so that one 4-byte LDS read serves a tap of both channels: half the tap reads per result (with the reads
// of two of the four taps left out of a copy of the kernel, fp16 N16 C256 64x64 went from 12.4 to 11.5 us).  The copy
// engine writes consecutive bytes only, so here the loaders go through registers: 16 bytes of either plane, the
// halves interleaved, two 16-byte LDS writes; two slots.  The host hands over channel counts in pairs.
template <typename T, int INTERP, int SWAVES, int LWAVES, int PPT, int ADJ, int CGS, int NBUF, int PITCH,
          bool SHIFTED_PLANES = false, bool CHANNEL_PAIRS = false>
__global__ __launch_bounds__((SWAVES + LWAVES) * 64) __attribute__((amdgpu_waves_per_eu(1, 5))) void gs2d_lds_kernel(
    const T* __restrict__ x, const T* __restrict__ grid, T* __restrict__ y, FastDiv N, int32_t C, int32_t H, int32_t W,
    int32_t out_plane, FastDiv tiles_per_n, int32_t chans_per_block, uint32_t wide_blocks,
    int32_t chans_wide, int32_t chan_stride, int32_t copy_gran, int32_t pair_aligned, int32_t xcd_swizzle, int32_t row_shift, int32_t pad,
    int32_t align, int32_t rule, int32_t ldsw, float neg_zero)
{
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    constexpr int NT = (INTERP == 0) ? 4 : (INTERP == 1 ? 1 : 16);  // taps per pixel
    constexpr int NW = (INTERP == 2) ? 8 : 4;                        // weights per pixel
    constexpr int SLOT_BYTES = CGS * PITCH;
    constexpr int DEPTH = NBUF - 1;  // stages in flight ahead of the one being sampled
    constexpr int STHREADS = SWAVES * 64;
    const int tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)tid >> 6);

    // Block -> (group = (channel block, n), tile).  Workgroups are handed to the 8 XCDs round-robin by index;
    // with the swizzle all tiles of one group (they read the same input planes) land on the same XCD next to
    // each other in time, so the planes are fetched into one L2 once.  Groups are numbered with the batch item
    // fastest: the workgroups that run at the same time then cover every batch item (with the channel block
    // fastest, the first half of the launch worked on the first half of both tensors, the second half on the rest:
    // 14.5 against 13.0 us on fp16 N16 C256 64x64), and an XCD sees the grids of N / 8 batch items only.
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

    static_assert(!CHANNEL_PAIRS || (sizeof(T) == 2 && INTERP != 1 && CGS == 1 && NBUF == 2 && !SHIFTED_PLANES),
                  "channel pairs: 16-bit bilinear or bicubic, one pair per stage, two slots");
    constexpr int PLANES = CHANNEL_PAIRS ? 2 : 1;  // planes that a "channel" of the block's channel loop stands for
    const int32_t plane_elems = H * W;
    const uint32_t plane_bytes = (uint32_t)plane_elems * (uint32_t)sizeof(T);
    // behind the plane, which in the shifted layout (copy_gran == 2) may sit up to 14 bytes into its slot
    // the slot of zeros sits in the last 16 bytes of a plane's pitch: behind any plane, wherever it ends, and behind
    // whatever a plane's last, partial copy writes past the plane's end (see the loaders' loop)
    constexpr uint32_t zero_off = (uint32_t)PITCH - 16u;
    // The first `wide_blocks` channel blocks take `chans_wide` channels each, the others `chans_per_block` (see
    // make_lds_plan: the workgroup that reaches a CU first runs ahead of the one that shares the CU with it).
    const bool wide = cb < wide_blocks;
    const int32_t my_chans = wide ? chans_wide : chans_per_block;
    // Which channels: a contiguous range [c_begin, c_end), or -- `chan_stride` != 0, single-plane stages, every block's
    // count exact -- channels dealt out in turn: block cb takes cb, cb + chan_stride, ... while all blocks draw
    // (`chans_per_block` turns), and the wide blocks then share out the rest among themselves, wide_blocks apart.
    // Both are  first + j * step1  for the block's j-th channel up to j = switch_at, and step2 apart from there on.
    int32_t first, step1, step2, nchan;
    if (chan_stride != 0) {
        first = (int32_t)cb;
        step1 = chan_stride;
        step2 = (int32_t)wide_blocks;
        nchan = my_chans;
    } else {
        const int32_t c_begin = wide ? (int32_t)cb * chans_wide
                                     : (int32_t)wide_blocks * chans_wide + (int32_t)(cb - wide_blocks) * chans_per_block;
        const int32_t c_end = (c_begin + my_chans < C) ? c_begin + my_chans : C;
        first = c_begin;
        step1 = 1;
        step2 = 1;
        nchan = c_end - c_begin;
    }
    const int32_t switch_at = chans_per_block;
    // the block's j-th channel
    auto chan_of = [&](int32_t j) -> int32_t {
        return first + (j < switch_at ? j * step1 : switch_at * step1 + (j - switch_at) * step2);
    };
    const int32_t nstages = (nchan + CGS - 1) / CGS;

    if (wave >= (uint32_t)SWAVES) {
        // ------------------------------------------------ loader wavefronts ------------------------------------
        const uint32_t lwave = wave - SWAVES;
        const uint32_t lane = (uint32_t)tid & 63u;
        const char* xn =
            reinterpret_cast<const char*>(x + (int64_t)n * C * PLANES * plane_elems);  // the batch item's planes
        if constexpr (CHANNEL_PAIRS) {
            // Every lane takes UPL 16-byte units (eight elements) of both planes of a stage.  The loads of RDEPTH
            // stages are on their way at any time, issued on every path alike (those past the last stage from one
            // address that all lanes share) so that the compiler's count of outstanding loads at every use is the
            // same on all paths and exact.  Slot s % 2 is written between the barriers of stages s - 1 and s, while
            // the samplers read the other one.
            constexpr int UPL = ((PITCH - 16) / 2 / 16 + LWAVES * 64 - 1) / (LWAVES * 64);
            constexpr int RDEPTH = UPL <= 2 ? 3 : 2;  // 48 or 64 registers of loads
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            typedef u32x4 __attribute__((address_space(3))) * lds_u32x4_ptr_t;
            const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
            const uint32_t lid = lwave * 64u + lane;
            const uint32_t units = plane_bytes >> 4;
            uint32_t unit[UPL], place[UPL];
            bool mine[UPL];
#pragma unroll
            for (int u = 0; u < UPL; u++) {
                unit[u] = lid + (uint32_t)u * (64u * LWAVES);
                mine[u] = unit[u] < units;
                unit[u] = mine[u] ? unit[u] : units - 1u;  // a lane without a unit reads the last one again
                // Where the unit's 32 bytes go in a slot: twice its offset in the single-channel layout, which is
                // the unit's offset in the plane, or -- `ldsw` > W, rows padded to a multiple of 128 bytes (a row is
                // whole units) -- row by row; the bank-spreading layout moves whole 16-byte chunks of that layout.
                uint32_t staged = unit[u] * 16u;
                if (ldsw != W) {
                    const uint32_t elem = unit[u] * 8u, row = elem / (uint32_t)W;
                    staged = (row * (uint32_t)ldsw + (elem - row * (uint32_t)W)) * 2u;
                }
                place[u] = 2u * lds_swizzle(staged, (uint32_t)row_shift);
            }
            u32x4 regs[RDEPTH][UPL][2];
            auto issue = [&](u32x4 (*r)[2], int32_t st) {
                const bool real = st < nstages;
                const char* base = xn + (real ? (size_t)chan_of(st) * (2 * (size_t)plane_bytes) : (size_t)0);
#pragma unroll
                for (int u = 0; u < UPL; u++) {
                    const uint32_t off = real ? unit[u] * 16u : 0u;
                    r[u][0] = *reinterpret_cast<const u32x4*>(base + off);
                    // (past the last stage: another address than the first load's, or the compiler makes the second
                    // a copy of the first, and a copy waits for its load)
                    r[u][1] = *reinterpret_cast<const u32x4*>(base + (real ? plane_bytes : 16u) + off);
                }
            };
            auto lows = [](uint32_t a, uint32_t b) -> uint32_t { return (a & 0xFFFFu) | (b << 16); };
            auto highs = [](uint32_t a, uint32_t b) -> uint32_t { return (a >> 16) | (b & 0xFFFF0000u); };
#pragma unroll
            for (int k = 0; k < RDEPTH; k++) {
                issue(regs[k], k);
            }
            for (int32_t s0 = 0; s0 < nstages; s0 += RDEPTH) {
#pragma unroll
                for (int k = 0; k < RDEPTH; k++) {
                    const int32_t st = s0 + k;
                    if (st < nstages) {
                        const uint32_t slot = lds_base + ((uint32_t)st & 1u) * (uint32_t)PITCH;
#pragma unroll
                        for (int u = 0; u < UPL; u++) {
                            if (mine[u]) {
                                const u32x4 a = regs[k][u][0], b = regs[k][u][1];
                                const u32x4 lo = {lows(a.x, b.x), highs(a.x, b.x), lows(a.y, b.y), highs(a.y, b.y)};
                                const u32x4 hi = {lows(a.z, b.z), highs(a.z, b.z), lows(a.w, b.w), highs(a.w, b.w)};
                                const uint32_t at = slot + place[u];
                                *reinterpret_cast<lds_u32x4_ptr_t>((uintptr_t)at) = lo;
                                *reinterpret_cast<lds_u32x4_ptr_t>((uintptr_t)(at + 16u)) = hi;
                            }
                        }
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        lds_barrier();  // stage st is in its slot, and the other slot has been read for the last time
                    }
                    issue(regs[k], st + RDEPTH);
                }
            }
            lds_barrier();  // the samplers' barrier behind the last stage
            return;
        }
        const char* xb = xn + (size_t)first * plane_bytes;                                  // the block's first plane
        // copy instructions this wavefront issues per plane
        constexpr bool shifted = SHIFTED_PLANES;  // 16-byte granule, planes off the 16-byte grid (see issue_stage_copy)
        const uint32_t chunk = 64u * (uint32_t)(shifted ? 16 : copy_gran);
        auto planes_of = [&](int32_t s) {
            const int32_t left = nchan - s * CGS;
            return left < CGS ? left : CGS;
        };
        // copy instructions this wavefront issues per plane (whole planes: the same for every plane)
        const uint32_t chunks = (plane_bytes + chunk - 1) / chunk;
        const uint32_t per_plane = (chunks > lwave) ? (chunks - lwave + LWAVES - 1) / LWAVES : 0;
        // ... and for the planes of stage s in the shifted layout, where a plane's copy starts `shift` bytes early and
        // is rounded out to 16-byte units, so that the count depends on the plane
        const uint32_t xb_low = (uint32_t)(reinterpret_cast<uintptr_t>(xb) & 15u);
        auto shifted_copy_count = [&](int32_t s) -> uint32_t {
            uint32_t total = 0;
            for (int32_t k = 0; k < planes_of(s); k++) {
                const uint32_t shift = (xb_low + (uint32_t)(s * CGS + k) * (plane_bytes & 15u)) & 15u;
                const uint32_t units = (((shift + plane_bytes + 15u) & ~15u) + chunk - 1) / chunk;
                total += (units > lwave) ? (units - lwave + LWAVES - 1) / LWAVES : 0;
            }
            return total;
        };
        const uint32_t lane_src16 = lds_unswizzle(lane * 16u, (uint32_t)row_shift);
        auto start_stage = [&](int32_t s, int slot) {
            const char* src = xn + (size_t)chan_of(s * CGS) * plane_bytes;
            char* dst = lds + slot * SLOT_BYTES;
            if constexpr (shifted) {
                issue_stage_copy<16, LWAVES, CGS, PITCH, true>(src, dst, plane_bytes, planes_of(s), lwave, lane,
                                                               lane * 16u);
            } else if (copy_gran == 16) {
                issue_stage_copy<16, LWAVES, CGS, PITCH>(src, dst, plane_bytes, planes_of(s), lwave, lane, lane_src16);
            } else {
                issue_stage_copy<4, LWAVES, CGS, PITCH>(src, dst, plane_bytes, planes_of(s), lwave, lane, lane * 4u);
            }
        };
        // The usual case has a loop of its own: single-plane stages of planes of whole 16-byte units on the 16-byte
        // grid (each loader has a fixed number of copies per plane, PP, a compile-time number in the loop) and at
        // least as many stages as the ring runs ahead.  A loader's step per stage -- wait, barrier, issue -- is in the chain of barriers that every
        // stage goes through, and at the start of the kernel the loaders' first DEPTH stages are what the samplers
        // wait for.  The general loop below finds the wait count of every stage at run time (a sum over the stages in
        // flight, then six compares and branches to reach the matching literal) and tests bounds around every copy:
        // about a hundred scalar instructions and two dozen taken branches per stage, 0.3 us of a wavefront's time.
        // Here the counts are literals and the copies unconditional: steady state while the ring is full, then an
        // unrolled run-down.
        if constexpr (!shifted && CGS == 1) {
            // 1 KiB chunks of a plane, shared out round-robin: this wavefront's copies per plane.  The last chunk may be
            // partial: its lanes past the plane's end copy the plane's last 16 bytes again (no masked copy, no read
            // past the tensor), which land behind the plane and in front of the slot of zeros.
            // A staged row is the plane's row, or -- `ldsw` > W, set by the launch plan for rows that are not a multiple
            // of 128 bytes -- the row padded to one: the copy then goes row by row through per-lane source offsets.
            // With rows of 112 bytes, say, consecutive rows are 28 banks apart, and along a line of slope 1 : 8 (a
            // rotation by 7 degrees) the lanes of a wavefront all read the same bank; rows of 128 bytes put a
            // column on the same bank in every row, so that lanes with different columns never collide (fp16 N16 C256
            // 56x56 under rotations of up to 30 degrees: 21.8 us with rows as they are).
            const uint32_t row_b = (uint32_t)W * (uint32_t)sizeof(T), lrow_b = (uint32_t)ldsw * (uint32_t)sizeof(T);
            const uint32_t staged_bytes = (uint32_t)H * lrow_b;
            const uint32_t chunks1k = (staged_bytes + 1023u) / 1024u;
            const uint32_t my_copies = (chunks1k > lwave) ? (chunks1k - lwave + LWAVES - 1) / LWAVES : 0u;
            if (copy_gran == 16 && chunks1k * 1024u <= (uint32_t)PITCH - 16u && nstages >= DEPTH) {
                auto ring_loop = [&](auto pp_tag) {
                    constexpr int PP = decltype(pp_tag)::value;
                    if constexpr ((DEPTH - 1) * PP <= 63 && PP * LWAVES * 1024 <= PITCH - 16 + (LWAVES - 1) * 1024) {
                        // this lane's 16 bytes of the wavefront's j-th chunk, as an offset into the plane
                        uint32_t lane_off[PP > 0 ? PP : 1];
#pragma unroll
                        for (int j = 0; j < PP; j++) {
                            uint32_t o = ((uint32_t)j * LWAVES + lwave) * 1024u + lane_src16;  // in the staged plane
                            if (lrow_b != row_b) {
                                const uint32_t row = o / lrow_b, col = o - row * lrow_b;
                                o = (col < row_b) ? row * row_b + col : plane_bytes;  // padding: any bytes will do
                            }
                            lane_off[j] = o < plane_bytes ? o : plane_bytes - 16u;
                        }
                        const char* src = xn + (size_t)first * plane_bytes;  // the plane being asked for
                        uint32_t slot_off = lwave * 1024u;                  // the first chunk's place in the slot being filled
                        int fill = 0;
                        int32_t turn = 0;  // the block's channel being asked for
                        auto issue = [&]() {
#pragma unroll
                            for (int j = 0; j < PP; j++) {
                                __builtin_amdgcn_global_load_lds((global_cptr_t)(src + lane_off[j]),
                                                                 (lds_ptr_t)(lds + slot_off + j * (LWAVES * 1024)), 16,
                                                                 0, 0);
                            }
                            src += (size_t)(turn < switch_at ? step1 : step2) * plane_bytes;
                            turn++;
                            fill = (fill + 1 == NBUF) ? 0 : fill + 1;
                            slot_off = (uint32_t)fill * SLOT_BYTES + lwave * 1024u;
                        };
#pragma unroll
                        for (int i = 0; i < DEPTH; i++) {
                            issue();
                        }
                        for (int32_t s = 0; s < nstages - DEPTH; s++) {
                            wait_vmcnt_imm<(DEPTH - 1) * PP>();  // stage s has landed: the DEPTH - 1 after it may be out
                            lds_barrier();                       // ... and the slot of stage s - 1 is free
                            issue();
                        }
                        ring_rundown<DEPTH - 1, PP>();
                        lds_barrier();  // the samplers' barrier behind the last plane (see their loop)
                        return true;
                    } else {
                        return false;
                    }
                };
                bool done = false;
                switch (my_copies) {
                    case 0: done = ring_loop(std::integral_constant<int, 0>{}); break;
                    case 1: done = ring_loop(std::integral_constant<int, 1>{}); break;
                    case 2: done = ring_loop(std::integral_constant<int, 2>{}); break;
                    case 3: done = ring_loop(std::integral_constant<int, 3>{}); break;
                    case 4: done = ring_loop(std::integral_constant<int, 4>{}); break;
                    case 5: done = ring_loop(std::integral_constant<int, 5>{}); break;
                    case 6: done = ring_loop(std::integral_constant<int, 6>{}); break;
                    case 7: done = ring_loop(std::integral_constant<int, 7>{}); break;
                    case 8: done = ring_loop(std::integral_constant<int, 8>{}); break;
                    case 9: done = ring_loop(std::integral_constant<int, 9>{}); break;
                    case 10: done = ring_loop(std::integral_constant<int, 10>{}); break;
                    case 11: done = ring_loop(std::integral_constant<int, 11>{}); break;
                    case 12: done = ring_loop(std::integral_constant<int, 12>{}); break;
                    case 13: done = ring_loop(std::integral_constant<int, 13>{}); break;
                    case 14: done = ring_loop(std::integral_constant<int, 14>{}); break;
                    case 15: done = ring_loop(std::integral_constant<int, 15>{}); break;
                    case 16: done = ring_loop(std::integral_constant<int, 16>{}); break;
                    default: break;
                }
                if (done) {
                    return;
                }
            }
        }
        // `issued` stages have been started; stage q goes to slot q % NBUF, which is free once the samplers are through
        // the barrier of stage q - DEPTH (their reads of stage q - NBUF have returned by then)
        int32_t issued = 0;
        int fill = 0;  // slot of stage `issued`
        auto issue_next = [&]() {
            start_stage(issued, fill);
            issued++;
            fill = (fill + 1 == NBUF) ? 0 : fill + 1;
        };
        while (issued < DEPTH && issued < nstages) {
            issue_next();
        }
        for (int32_t s = 0; s < nstages; s++) {
            // outstanding once stage s has landed: the copies of stages s + 1 .. issued - 1
            if constexpr (shifted) {
                uint32_t later_copies = 0;
                for (int32_t q = s + 1; q < issued; q++) {
                    later_copies += shifted_copy_count(q);
                }
                wait_vmcnt(later_copies);
            } else {
                int32_t later_planes = 0;
                for (int32_t q = s + 1; q < issued; q++) {
                    later_planes += planes_of(q);
                }
                wait_vmcnt((uint32_t)later_planes * per_plane);
            }
            lds_barrier();
            if (issued < nstages) {
                issue_next();
            }
        }
        // the samplers' barrier behind the last plane of a full last stage (see their loop)
        if (nchan % CGS == 0) {
            lds_barrier();
        }
        return;
    }

    // ---------------------------------------------------- sampler wavefronts -----------------------------------
    // the zero slots behind each staged plane (all ring slots); stage copies never touch them
    if (tid < NBUF * CGS * 4) {
        reinterpret_cast<uint32_t*>(lds + (tid >> 2) * PITCH + zero_off)[tid & 3] = 0u;
    }

    // per-pixel decisions, once for the whole channel range
    // A lane owns PPT / ADJ groups of ADJ neighbouring pixels; the groups of a lane are STHREADS * ADJ pixels apart.
    // With ADJ = 2 (16-bit elements) the two results of a channel leave as one 4-byte store, and the lanes of a
    // wavefront read taps two source columns apart, i.e. from different LDS banks for an undistorted grid.
    static_assert(PPT % ADJ == 0, "whole groups per lane");
    constexpr int NGRP = PPT / ADJ;
    uint32_t toff[PPT][NT];
    float tw[PPT][NW];
    uint32_t pixoff[NGRP];  // byte offset of the group inside an output plane; out of range for lanes past the end
    float gxs[PPT], gys[PPT];
    const T* gridn = grid + (int64_t)n * out_plane * 2;
    const T* gptr[PPT];
#pragma unroll
    for (int q = 0; q < NGRP; q++) {
        const int32_t pix0 = (int32_t)tile * (STHREADS * PPT) + q * (STHREADS * ADJ) + tid * ADJ;
        // the output plane holds a whole number of groups (the launch plan picks ADJ accordingly)
        const bool valid = pix0 < out_plane;
        const int32_t pc = valid ? pix0 : out_plane - ADJ;
        pixoff[q] = valid ? (uint32_t)pc * (uint32_t)sizeof(T) : 0x80000000u;
#pragma unroll
        for (int a = 0; a < ADJ; a++) {
            gptr[q * ADJ + a] = gridn + (int64_t)(pc + a) * 2;
        }
    }
    load_grid_points<T, PPT, true>(gptr, pair_aligned != 0, gxs, gys);
    // the bank-spreading layout exists for border padding only (see make_lds_plan: row_shift is 0 otherwise)
    const uint32_t rs = (uint32_t)row_shift;
    // `rule` != 0: the coordinate rule of the reference's second bilinear kernel (bilinear only)
    const bool arch35 = rule != 0;
    if (rs != 0u) {
        decide_lane_pixels<T, INTERP, PPT, NT, NW, true>(gxs, gys, H, W, (uint32_t)ldsw, rs, zero_off, pad, align != 0, arch35, toff,
                                                         tw);
    } else {
        decide_lane_pixels<T, INTERP, PPT, NT, NW, false>(gxs, gys, H, W, (uint32_t)ldsw, rs, zero_off, pad, align != 0, arch35, toff,
                                                          tw);
    }
    const float first_zero = arch35 ? neg_zero : 0.0f;
    if constexpr (CHANNEL_PAIRS) {
        // an element is four bytes of its slot; the zeros stay where they are
#pragma unroll
        for (int j = 0; j < PPT; j++) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                toff[j][t] = (toff[j][t] == zero_off) ? zero_off : toff[j][t] * 2u;
            }
        }
    }

    // tap offsets become absolute LDS addresses (left as offsets, the compiler re-adds the allocation's base to
    // every tap in every stage)
    {
        uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
        // opaque to the compiler from here on: seen as the allocation's symbol, the base would be split off the sum
        // again and re-added at every use
        asm volatile("" : "+s"(lds_base));
#pragma unroll
        for (int j = 0; j < PPT; j++) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                toff[j][t] += lds_base;
                asm volatile("" : "+v"(toff[j][t]));  // the sum itself is what stays in the register
            }
        }
    }

    T* yplane = y + ((int64_t)n * C + first) * PLANES * out_plane;  // the output plane of the channel being blended
    const uint32_t out_plane_bytes = (uint32_t)out_plane * (uint32_t)sizeof(T);

    // the bytes by which a plane's copy started early (SHIFTED_PLANES, see issue_stage_copy): the low four bits of the
    // plane's first byte address, from those of the tensor's address and of the plane size.  The shift makes the
    // plane distance a run-time value where it is a literal otherwise (one more add per tap).
    const uint32_t addr_low = (uint32_t)(reinterpret_cast<uintptr_t>(x) & 15u);
    const uint32_t size_low = plane_bytes & 15u;
    const uint32_t first_plane = (uint32_t)n * (uint32_t)C + (uint32_t)first;
    auto plane_shift = [&](int32_t p) -> uint32_t {
        if constexpr (SHIFTED_PLANES) {
            return (addr_low + (first_plane + (uint32_t)p) * size_low) & 15u;
        } else {
            (void)p;
            return 0u;
        }
    };
    // One software pipeline over all planes of the block, across stage boundaries.  A lane keeps one set of tap
    // registers per pixel; as soon as a pixel of plane p has been blended, its registers are reloaded with the taps
    // of plane p + 1, so the LDS reads of a pixel are in flight while the lane's other pixels are blended and
    // stored (the per-wavefront counter of outstanding LDS operations is exact in straight-line code, which is why
    // nothing in the steady state is conditional: past the last plane the reload reads whatever the ring holds and
    // the values are dropped).  The barrier that hands over a stage sits in front of the first read of the stage's
    // first plane, inside the previous stage's last plane.  A wavefront's LDS reads have all returned when it
    // enters the barrier (lgkmcnt(0)), so the loaders, which refill the previous stage's slot once they are through
    // the same barrier, never overwrite a plane that is still being read.  The loop is unrolled over one turn of
    // the ring (NBUF stages of CGS planes) so that a plane's offset in the ring is an immediate.
    constexpr int UNR = NBUF * CGS;
    uint32_t raw[PPT][NT];
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the zero-slot writes, before the first barrier publishes them
    lds_barrier();                        // stage 0 has landed
    // (channel pairs: whole dwords, both channels of a tap)
    typedef typename std::conditional<CHANNEL_PAIRS, uint32_t, T>::type tap_read_t;
#pragma unroll
    for (int j = 0; j < PPT; j++) {
        load_taps<tap_read_t, NT>(plane_shift(0), toff[j], raw[j]);
    }
    // Every plane runs the same straight-line body, barrier included (behind the block's last plane the loaders add
    // one more barrier to meet it).  With the barrier under a condition of its own ("is there a next plane") two
    // paths met in front of the next blend, and the compiler, merging their counts of outstanding LDS reads, made
    // every plane wait for all sixteen of its reads before the first product (14.0 against 12.9 us on fp16 N16 C256
    // 64x64).
    for (int32_t b = 0; b < nchan; b += UNR) {
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            const int32_t p = b + u;
            if (p >= nchan) {
                break;
            }
            const int un = (u + 1) % UNR;  // a literal once the loop is unrolled
            const uint32_t next_off = (uint32_t)((un / CGS) * SLOT_BYTES + (un % CGS) * PITCH) + plane_shift(p + 1);
            const __amdgpu_buffer_rsrc_t rsrc =
                __builtin_amdgcn_make_buffer_rsrc(yplane, 0, out_plane_bytes, kBufferFlags);
            const __amdgpu_buffer_rsrc_t rsrc_hi =
                __builtin_amdgcn_make_buffer_rsrc(yplane + (PLANES - 1) * out_plane, 0, out_plane_bytes, kBufferFlags);
            yplane += (int64_t)(p < switch_at ? step1 : step2) * PLANES * out_plane;
#pragma unroll
            for (int q = 0; q < NGRP; q++) {
                float v[ADJ], v_hi[ADJ];
#pragma unroll
                for (int a = 0; a < ADJ; a++) {
                    const int j = q * ADJ + a;
                    v[a] = blend<T, INTERP>(raw[j], tw[j], neg_zero, first_zero);
                    if constexpr (CHANNEL_PAIRS) {
                        uint32_t upper[NT];
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            upper[t] = raw[j][t] >> 16;
                        }
                        v_hi[a] = blend<T, INTERP>(upper, tw[j], neg_zero, first_zero);
                    }
                    if (j == 0 && un % CGS == 0) {
                        __builtin_amdgcn_s_waitcnt(0xC07F);
                        lds_barrier();  // stage (p + 1) / CGS has landed (or, behind the last plane, nothing)
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    load_taps<tap_read_t, NT>(next_off, toff[j], raw[j]);
                    __builtin_amdgcn_sched_barrier(0);
                }
                buffer_store_group<T, ADJ, true>(v, rsrc, pixoff[q]);
                if constexpr (CHANNEL_PAIRS) {
                    buffer_store_group<T, ADJ, true>(v_hi, rsrc_hi, pixoff[q]);
                }
            }
        }
    }
}

}  // namespace opscv
