// Volumetric grid sampler (5-D), forward, NCDHW: device code and launcher.
//
// Arithmetic of the bilinear mode follows, operation for operation, the reference SIMT kernel
//   image/grid_sample/op_kernel/arch35/grid_sampler_3d_bilinear_smit.h:66-135  (eight-corner blend)
//   image/grid_sample/op_kernel/arch35/grid_sampler_3d_bilinear_smit.h:168-183 (unnormalize, clip order d, w, h)
//   image/grid_sample/op_kernel/arch35/grid_sampler_bilinear_smit_common.h:37-94 (ClipCoordinates,
//   reflectCoordinates, safeDowngradeToIntRange, Clip)
// with every product and sum rounded separately (the translation unit is compiled with -ffp-contract=off).
// The nearest mode uses the same coordinate pipeline and rounds each coordinate half to even, as the reference's
// vector kernel does (image/grid_sample/op_kernel/grid_sampler_3d_nearest.h:569-571, CAST_RINT).
//
// Work split: the reference gives one thread to every (n, c, d, h, w) output element and repeats the coordinate
// arithmetic per channel.  Here a lane owns one output point (n, d, h, w): it computes the eight corner offsets and
// weights once and then walks a chunk of channels, so the grid is read once per channel chunk and the stores of a
// wavefront are 64 consecutive elements of one output row.  The weights do not depend on the channel, so hoisting
// them changes no bit of the result.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "kernels.hpp"
#include "sampler_math.hpp"

namespace opscv {

namespace {

constexpr int kThreads = 256;

struct Gs3dParams {
    int32_t C, Din, Hin, Win;
    int64_t out_vol;     // Dout * Hout * Wout
    int64_t points;      // N * out_vol
    int32_t chan_chunk;  // channels per blockIdx.y
};

template <typename T, int INTERP, int PAD, bool ALIGN>
__global__ __launch_bounds__(kThreads) void gs3d_kernel(const T* __restrict__ x, const T* __restrict__ grid,
                                                         T* __restrict__ y, Gs3dParams p)
{
    const int64_t pt = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (pt >= p.points) {
        return;
    }
    const int64_t n = pt / p.out_vol;
    const int64_t sp = pt - n * p.out_vol;
    const T* g = grid + pt * 3;
    const float gw = ElemIO<T>::load(g);
    const float gh = ElemIO<T>::load(g + 1);
    const float gd = ElemIO<T>::load(g + 2);
    const float pd = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gd, p.Din), p.Din);
    const float pw = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gw, p.Win), p.Win);
    const float ph = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gh, p.Hin), p.Hin);

    const int32_t in_plane = p.Hin * p.Win;
    const int64_t in_vol = (int64_t)p.Din * in_plane;
    const int32_t c_begin = blockIdx.y * p.chan_chunk;
    const int32_t c_end = (c_begin + p.chan_chunk < p.C) ? c_begin + p.chan_chunk : p.C;
    const T* xc = x + (n * p.C + c_begin) * in_vol;
    T* yc = y + (n * p.C + c_begin) * p.out_vol + sp;

    if (INTERP == 1) {
        const int32_t id = float_to_i32(__builtin_rintf(pd));
        const int32_t ih = float_to_i32(__builtin_rintf(ph));
        const int32_t iw = float_to_i32(__builtin_rintf(pw));
        const bool in = id >= 0 && id < p.Din && ih >= 0 && ih < p.Hin && iw >= 0 && iw < p.Win;
        const int64_t off = in ? (int64_t)id * in_plane + ih * p.Win + iw : 0;
        T zero;
        ElemIO<T>::store(&zero, 0.0f);
        for (int32_t c = c_begin; c < c_end; c++) {
            *yc = in ? xc[off] : zero;
            xc += in_vol;
            yc += p.out_vol;
        }
        return;
    }

    const float fd = __builtin_floorf(pd), fh = __builtin_floorf(ph), fw = __builtin_floorf(pw);
    const float dd = pd - fd, dh = ph - fh, dw = pw - fw;
    const int32_t d0 = float_to_i32(fd), d1 = float_to_i32(fd + 1.0f);
    const int32_t h0 = float_to_i32(fh), h1 = float_to_i32(fh + 1.0f);
    const int32_t w0 = float_to_i32(fw), w1 = float_to_i32(fw + 1.0f);
    const bool vd0 = d0 >= 0 && d0 < p.Din, vd1 = d1 >= 0 && d1 < p.Din;
    const bool vh0 = h0 >= 0 && h0 < p.Hin, vh1 = h1 >= 0 && h1 < p.Hin;
    const bool vw0 = w0 >= 0 && w0 < p.Win, vw1 = w1 >= 0 && w1 < p.Win;
    // corner order of the reference: (d0,h0,w0) (d0,h0,w1) (d0,h1,w0) (d0,h1,w1) (d1,h0,w0) (d1,h0,w1) (d1,h1,w0) (d1,h1,w1)
    float wt[8];
    wt[0] = (1.0f - dw) * (1.0f - dh) * (1.0f - dd);
    wt[1] = dw * (1.0f - dh) * (1.0f - dd);
    wt[2] = (1.0f - dw) * dh * (1.0f - dd);
    wt[3] = dw * dh * (1.0f - dd);
    wt[4] = (1.0f - dw) * (1.0f - dh) * dd;
    wt[5] = dw * (1.0f - dh) * dd;
    wt[6] = (1.0f - dw) * dh * dd;
    wt[7] = dw * dh * dd;
    bool ok[8];
    int64_t off[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const bool vd = (k & 4) ? vd1 : vd0;
        const bool vh = (k & 2) ? vh1 : vh0;
        const bool vw = (k & 1) ? vw1 : vw0;
        ok[k] = vd && vh && vw;
        const int32_t d = (k & 4) ? d1 : d0, h = (k & 2) ? h1 : h0, w = (k & 1) ? w1 : w0;
        off[k] = ok[k] ? (int64_t)d * in_plane + h * p.Win + w : 0;
    }
    if (p.Win >= 2) {
        // The two corners of a row, w0 and w0 + 1, are neighbours in memory: one load of two elements (aligned to one
        // element only, which global memory accesses allow) instead of two loads halves the number of addresses the
        // gather puts through the memory pipeline, which is what bounds it.  The pair is taken at column
        // pb = clamp(w0, 0, Win - 2) so that it never leaves the row; which half is which corner follows from pb.
        const int32_t pb = (w0 < 0) ? 0 : ((w0 > p.Win - 2) ? p.Win - 2 : w0);
        const bool lo_is_w0 = (w0 == pb), lo_is_w1 = (w1 == pb);  // else the high half (or the corner is outside)
        int64_t poff[4];
        bool pok[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const bool vd = (r & 2) ? vd1 : vd0;
            const bool vh = (r & 1) ? vh1 : vh0;
            const int32_t d = (r & 2) ? d1 : d0, h = (r & 1) ? h1 : h0;
            pok[r] = vd && vh && (vw0 || vw1);
            poff[r] = pok[r] ? (int64_t)d * in_plane + h * p.Win + pb : 0;
        }
        // the pair as one integer of twice the element size, so that it is fetched by a single load instruction
        using PairBits = typename std::conditional<sizeof(T) == 2, uint32_t, uint64_t>::type;
        for (int32_t c = c_begin; c < c_end; c++) {
            PairBits pr[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                pr[r] = 0;
                if (pok[r]) {
                    __builtin_memcpy(&pr[r], xc + poff[r], sizeof(PairBits));
                }
            }
            float v[8];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                T halves[2];
                __builtin_memcpy(halves, &pr[r], sizeof(PairBits));
                const float lo = ElemIO<T>::load(&halves[0]), hi = ElemIO<T>::load(&halves[1]);
                v[2 * r] = ok[2 * r] ? (lo_is_w0 ? lo : hi) : 0.0f;
                v[2 * r + 1] = ok[2 * r + 1] ? (lo_is_w1 ? lo : hi) : 0.0f;
            }
            float acc = v[0] * wt[0];
#pragma unroll
            for (int k = 1; k < 8; k++) {
                acc += v[k] * wt[k];
            }
            store_streaming<T>(yc, acc);
            xc += in_vol;
            yc += p.out_vol;
        }
        return;
    }
    for (int32_t c = c_begin; c < c_end; c++) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            v[k] = ok[k] ? ElemIO<T>::load(xc + off[k]) : 0.0f;
        }
        float acc = v[0] * wt[0];
#pragma unroll
        for (int k = 1; k < 8; k++) {
            acc += v[k] * wt[k];
        }
        store_streaming<T>(yc, acc);
        xc += in_vol;
        yc += p.out_vol;
    }
}

// The bilinear kernel for two-byte elements, rows of two columns and more and volumes below 2^31 elements: the same
// results as gs3d_kernel from fewer instructions, which is what bounds either (their wavefronts keep the SIMDs'
// instruction issue busy for most of the kernel's time; memory is far from its limits).  Per channel a lane makes four
// loads of a pair of neighbouring columns, as gs3d_kernel does, but
//  * one byte-permute instruction per pair puts the value of column w0 into the low half and that of w1 into the high
//    half and zeroes the half whose corner lies outside the volume (selector bytes 0x0c give zero bytes), in place of
//    two conversions and four selects: the selector of a row is made once per point;
//  * the loads are unconditional (a row without a valid corner reads the volume's first pair and its selector zeroes
//    both halves), so no branches around them;
//  * offsets inside a volume are 32-bit.
// Products and sums per element exactly as in gs3d_kernel.
typedef uint32_t UnalignedWord __attribute__((aligned(2)));  // a pair of two-byte elements, aligned to one of them
constexpr uint32_t kSelLow = 0x0100u, kSelHigh = 0x0302u, kSelZero = 0x0c0cu;

template <typename T>
__device__ __forceinline__ float half_value(uint32_t word, bool high)
{
    if constexpr (std::is_same<T, __bf16>::value) {
        return __builtin_bit_cast(float, high ? (word & 0xffff0000u) : (word << 16));
    } else {
        return (float)__builtin_bit_cast(_Float16, (uint16_t)(high ? (word >> 16) : (word & 0xffffu)));
    }
}

template <typename T, int PAD, bool ALIGN>
__global__ __launch_bounds__(kThreads) void gs3d_pair16_kernel(const T* __restrict__ x, const T* __restrict__ grid,
                                                                T* __restrict__ y, Gs3dParams p)
{
    static_assert(sizeof(T) == 2, "pairs of two-byte elements");
    const int64_t pt = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (pt >= p.points) {
        return;
    }
    const int64_t n = pt / p.out_vol;
    const int64_t sp = pt - n * p.out_vol;
    const T* g = grid + pt * 3;
    const float gw = ElemIO<T>::load(g);
    const float gh = ElemIO<T>::load(g + 1);
    const float gd = ElemIO<T>::load(g + 2);
    const float pd = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gd, p.Din), p.Din);
    const float pw = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gw, p.Win), p.Win);
    const float ph = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gh, p.Hin), p.Hin);

    const uint32_t in_plane = (uint32_t)p.Hin * (uint32_t)p.Win;
    const uint32_t in_vol = (uint32_t)p.Din * in_plane;
    const int32_t c_begin = blockIdx.y * p.chan_chunk;
    const int32_t c_end = (c_begin + p.chan_chunk < p.C) ? c_begin + p.chan_chunk : p.C;
    const T* xc = x + (n * p.C + c_begin) * (int64_t)in_vol;
    T* yc = y + (n * p.C + c_begin) * p.out_vol + sp;

    const float fd = __builtin_floorf(pd), fh = __builtin_floorf(ph), fw = __builtin_floorf(pw);
    const float dd = pd - fd, dh = ph - fh, dw = pw - fw;
    const int32_t d0 = float_to_i32(fd), d1 = float_to_i32(fd + 1.0f);
    const int32_t h0 = float_to_i32(fh), h1 = float_to_i32(fh + 1.0f);
    const int32_t w0 = float_to_i32(fw), w1 = float_to_i32(fw + 1.0f);
    const bool vd0 = d0 >= 0 && d0 < p.Din, vd1 = d1 >= 0 && d1 < p.Din;
    const bool vh0 = h0 >= 0 && h0 < p.Hin, vh1 = h1 >= 0 && h1 < p.Hin;
    const bool vw0 = w0 >= 0 && w0 < p.Win, vw1 = w1 >= 0 && w1 < p.Win;
    float wt[8];
    wt[0] = (1.0f - dw) * (1.0f - dh) * (1.0f - dd);
    wt[1] = dw * (1.0f - dh) * (1.0f - dd);
    wt[2] = (1.0f - dw) * dh * (1.0f - dd);
    wt[3] = dw * dh * (1.0f - dd);
    wt[4] = (1.0f - dw) * (1.0f - dh) * dd;
    wt[5] = dw * (1.0f - dh) * dd;
    wt[6] = (1.0f - dw) * dh * dd;
    wt[7] = dw * dh * dd;
    // the pair of a row starts at column pb = clamp(w0, 0, Win - 2); a valid corner sits in its low half if its column
    // is pb and in its high half otherwise
    const int32_t pb = (w0 < 0) ? 0 : ((w0 > p.Win - 2) ? p.Win - 2 : w0);
    const uint32_t at_w0 = (w0 == pb) ? kSelLow : kSelHigh, at_w1 = (w1 == pb) ? kSelLow : kSelHigh;
    typedef const __attribute__((address_space(1))) T* GlobalRow;  // keeps the loads below global ones, not flat
    GlobalRow row[4];
    uint32_t sel[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const bool vdh = ((r & 2) ? vd1 : vd0) && ((r & 1) ? vh1 : vh0);
        const bool k0 = vdh && vw0, k1 = vdh && vw1;
        const uint32_t d = (uint32_t)((r & 2) ? d1 : d0), h = (uint32_t)((r & 1) ? h1 : h0);
        sel[r] = (k0 ? at_w0 : kSelZero) | ((k1 ? at_w1 : kSelZero) << 16);
        row[r] = (GlobalRow)(xc + ((k0 || k1) ? d * in_plane + h * (uint32_t)p.Win + (uint32_t)pb : 0u));
    }
    auto fetch = [&](uint32_t (&pairs)[4]) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            pairs[r] = *(const __attribute__((address_space(1), aligned(2))) UnalignedWord*)row[r];
            row[r] += in_vol;
        }
    };
    auto blend_and_store = [&](const uint32_t (&pairs)[4]) {
        float v[8];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint32_t m = __builtin_amdgcn_perm(pairs[r], pairs[r], sel[r]);
            v[2 * r] = half_value<T>(m, false);
            v[2 * r + 1] = half_value<T>(m, true);
        }
        float acc = v[0] * wt[0];
#pragma unroll
        for (int k = 1; k < 8; k++) {
            acc += v[k] * wt[k];
        }
        store_streaming<T>(yc, acc);
        yc += p.out_vol;
    };
    for (int32_t c = c_begin; c < c_end; c++) {
        uint32_t pairs[4];
        fetch(pairs);
        blend_and_store(pairs);
    }
}

// Channels-last (NDHWC) variant: the C values of a voxel are contiguous, so a corner is one load of up to 16 bytes
// instead of C scattered two- or four-byte loads.  A lane owns one unit of UE consecutive channels of one output
// point (consecutive lanes own consecutive units, so loads and stores of neighbouring lanes are contiguous); the
// lanes of a point compute its coordinates redundantly.  Arithmetic per element as in gs3d_kernel.
template <typename T, int INTERP, int PAD, bool ALIGN, int UE>
__global__ __launch_bounds__(kThreads) void gs3d_ndhwc_kernel(const T* __restrict__ x, const T* __restrict__ grid,
                                                               T* __restrict__ y, Gs3dParams p, int32_t units)
{
    typedef T Unit __attribute__((ext_vector_type(UE)));
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= p.points * units) {
        return;
    }
    const int64_t pt = idx / units;
    const int32_t u = (int32_t)(idx - pt * units);
    const int64_t n = pt / p.out_vol;
    const T* g = grid + pt * 3;
    const float gw = ElemIO<T>::load(g);
    const float gh = ElemIO<T>::load(g + 1);
    const float gd = ElemIO<T>::load(g + 2);
    const float pd = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gd, p.Din), p.Din);
    const float pw = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gw, p.Win), p.Win);
    const float ph = clip3<PAD, ALIGN>(unnormalize3<ALIGN>(gh, p.Hin), p.Hin);
    const int64_t in_vol = (int64_t)p.Din * p.Hin * p.Win;
    const Unit* xu = reinterpret_cast<const Unit*>(x + n * in_vol * p.C) + u;  // voxel v, unit u: xu[v * units]
    Unit* yu = reinterpret_cast<Unit*>(y) + idx;
    Unit zero;
#pragma unroll
    for (int e = 0; e < UE; e++) {
        T z;
        ElemIO<T>::store(&z, 0.0f);
        zero[e] = z;
    }
    if (INTERP == 1) {
        const int32_t id = float_to_i32(__builtin_rintf(pd));
        const int32_t ih = float_to_i32(__builtin_rintf(ph));
        const int32_t iw = float_to_i32(__builtin_rintf(pw));
        const bool in = id >= 0 && id < p.Din && ih >= 0 && ih < p.Hin && iw >= 0 && iw < p.Win;
        *yu = in ? xu[(((int64_t)id * p.Hin + ih) * p.Win + iw) * units] : zero;
        return;
    }
    const float fd = __builtin_floorf(pd), fh = __builtin_floorf(ph), fw = __builtin_floorf(pw);
    const float dd = pd - fd, dh = ph - fh, dw = pw - fw;
    const int32_t d0 = float_to_i32(fd), d1 = float_to_i32(fd + 1.0f);
    const int32_t h0 = float_to_i32(fh), h1 = float_to_i32(fh + 1.0f);
    const int32_t w0 = float_to_i32(fw), w1 = float_to_i32(fw + 1.0f);
    const bool vd0 = d0 >= 0 && d0 < p.Din, vd1 = d1 >= 0 && d1 < p.Din;
    const bool vh0 = h0 >= 0 && h0 < p.Hin, vh1 = h1 >= 0 && h1 < p.Hin;
    const bool vw0 = w0 >= 0 && w0 < p.Win, vw1 = w1 >= 0 && w1 < p.Win;
    float wt[8];
    wt[0] = (1.0f - dw) * (1.0f - dh) * (1.0f - dd);
    wt[1] = dw * (1.0f - dh) * (1.0f - dd);
    wt[2] = (1.0f - dw) * dh * (1.0f - dd);
    wt[3] = dw * dh * (1.0f - dd);
    wt[4] = (1.0f - dw) * (1.0f - dh) * dd;
    wt[5] = dw * (1.0f - dh) * dd;
    wt[6] = (1.0f - dw) * dh * dd;
    wt[7] = dw * dh * dd;
    Unit v[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const bool ok = ((k & 4) ? vd1 : vd0) && ((k & 2) ? vh1 : vh0) && ((k & 1) ? vw1 : vw0);
        const int32_t d = (k & 4) ? d1 : d0, h = (k & 2) ? h1 : h0, w = (k & 1) ? w1 : w0;
        // an always valid address for the corners outside the volume, their values replaced by zeros
        const int64_t vox = ok ? ((int64_t)d * p.Hin + h) * p.Win + w : 0;
        const Unit raw = xu[vox * units];
        v[k] = ok ? raw : zero;
    }
    Unit out;
#pragma unroll
    for (int e = 0; e < UE; e++) {
        T t0 = v[0][e];
        float acc = ElemIO<T>::load(&t0) * wt[0];
#pragma unroll
        for (int k = 1; k < 8; k++) {
            T tk = v[k][e];
            acc += ElemIO<T>::load(&tk) * wt[k];
        }
        T o;
        ElemIO<T>::store(&o, acc);
        out[e] = o;
    }
    *yu = out;
}

template <typename T, int INTERP, int PAD, bool ALIGN>
hipError_t launch_ndhwc(const GridSampler3DArgs& a, hipStream_t stream)
{
    Gs3dParams p;
    p.C = (int32_t)a.C;
    p.Din = (int32_t)a.Din;
    p.Hin = (int32_t)a.Hin;
    p.Win = (int32_t)a.Win;
    p.out_vol = a.Dout * a.Hout * a.Wout;
    p.points = a.N * p.out_vol;
    p.chan_chunk = 0;
    // the widest unit (16, 8, 4 bytes or one element) that divides a voxel's channels and keeps every access aligned
    const int64_t vox_bytes = a.C * (int64_t)sizeof(T);
    const uintptr_t both = reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.y);
    int ub = (int)sizeof(T);
    for (int cand = 16; cand > (int)sizeof(T); cand /= 2) {
        if (vox_bytes % cand == 0 && both % cand == 0) {
            ub = cand;
            break;
        }
    }
    const int64_t units = vox_bytes / ub;
    const int64_t blocks = (p.points * units + kThreads - 1) / kThreads;
    if (blocks > INT32_MAX || units > INT32_MAX) {
        return hipErrorInvalidValue;
    }
#define OPSCV_GS3D_CL(UE_)                                                                                          \
    hipLaunchKernelGGL((gs3d_ndhwc_kernel<T, INTERP, PAD, ALIGN, UE_>), dim3((unsigned)blocks), dim3(kThreads), 0,  \
                       stream, (const T*)a.x, (const T*)a.grid, (T*)a.y, p, (int32_t)units)
    switch (ub / (int)sizeof(T)) {
        case 1: OPSCV_GS3D_CL(1); break;
        case 2: OPSCV_GS3D_CL(2); break;
        case 4: OPSCV_GS3D_CL(4); break;
        case 8:
            if constexpr (sizeof(T) == 2) {
                OPSCV_GS3D_CL(8);
            }
            break;
        default: return hipErrorInvalidValue;
    }
#undef OPSCV_GS3D_CL
    return hipGetLastError();
}

template <typename T, int INTERP, int PAD, bool ALIGN>
hipError_t launch_one(const GridSampler3DArgs& a, hipStream_t stream)
{
    if (a.channels_last) {
        return launch_ndhwc<T, INTERP, PAD, ALIGN>(a, stream);
    }
    Gs3dParams p;
    p.C = (int32_t)a.C;
    p.Din = (int32_t)a.Din;
    p.Hin = (int32_t)a.Hin;
    p.Win = (int32_t)a.Win;
    p.out_vol = a.Dout * a.Hout * a.Wout;
    p.points = a.N * p.out_vol;
    const int64_t pblocks = (p.points + kThreads - 1) / kThreads;
    // enough workgroups to fill 256 compute units several times over, else whole channel ranges per lane
    int64_t chunks = 1;
    while (pblocks * chunks < 4096 && chunks * 2 <= a.C) {
        chunks *= 2;
    }
    p.chan_chunk = (int32_t)((a.C + chunks - 1) / chunks);
    const int64_t ychunks = (a.C + p.chan_chunk - 1) / p.chan_chunk;
    if (pblocks > INT32_MAX || ychunks > 65535) {
        return hipErrorInvalidValue;
    }
    if constexpr (sizeof(T) == 2 && INTERP == 0) {
        if (a.Win >= 2 && a.Din * a.Hin * a.Win <= INT32_MAX) {
            hipLaunchKernelGGL((gs3d_pair16_kernel<T, PAD, ALIGN>), dim3((unsigned)pblocks, (unsigned)ychunks),
                               dim3(kThreads), 0, stream, (const T*)a.x, (const T*)a.grid, (T*)a.y, p);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((gs3d_kernel<T, INTERP, PAD, ALIGN>), dim3((unsigned)pblocks, (unsigned)ychunks),
                       dim3(kThreads), 0, stream, (const T*)a.x, (const T*)a.grid, (T*)a.y, p);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_typed(const GridSampler3DArgs& a, hipStream_t stream)
{
    const int key = a.interp * 6 + a.pad * 2 + a.align;
    switch (key) {
#define OPSCV_GS3D_CASE(I, P, A) \
    case (I) * 6 + (P) * 2 + (A): return launch_one<T, I, P, (A) != 0>(a, stream);
        OPSCV_GS3D_CASE(0, 0, 0)
        OPSCV_GS3D_CASE(0, 0, 1)
        OPSCV_GS3D_CASE(0, 1, 0)
        OPSCV_GS3D_CASE(0, 1, 1)
        OPSCV_GS3D_CASE(0, 2, 0)
        OPSCV_GS3D_CASE(0, 2, 1)
        OPSCV_GS3D_CASE(1, 0, 0)
        OPSCV_GS3D_CASE(1, 0, 1)
        OPSCV_GS3D_CASE(1, 1, 0)
        OPSCV_GS3D_CASE(1, 1, 1)
        OPSCV_GS3D_CASE(1, 2, 0)
        OPSCV_GS3D_CASE(1, 2, 1)
#undef OPSCV_GS3D_CASE
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t launch_grid_sampler3d(const GridSampler3DArgs& a, hipStream_t stream)
{
    if (a.x == nullptr || a.grid == nullptr || a.y == nullptr) {
        return hipErrorInvalidValue;
    }
    if (a.interp < 0 || a.interp > 1 || a.pad < 0 || a.pad > 2) {
        return hipErrorInvalidValue;
    }
    if (a.N <= 0 || a.C <= 0 || a.Din <= 0 || a.Hin <= 0 || a.Win <= 0 || a.Dout < 0 || a.Hout < 0 || a.Wout < 0) {
        return hipErrorInvalidValue;
    }
    if (a.C > INT32_MAX || a.Din > INT32_MAX || a.Hin > INT32_MAX || a.Win > INT32_MAX ||
        a.Hin * a.Win > INT32_MAX) {
        return hipErrorInvalidValue;
    }
    if (a.N * a.Dout * a.Hout * a.Wout == 0) {
        return hipSuccess;
    }
    switch (a.elem) {
        case Elem::F32: return launch_typed<float>(a, stream);
        case Elem::F16: return launch_typed<_Float16>(a, stream);
        case Elem::BF16: return launch_typed<__bf16>(a, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
