// Grid sampler 2-D forward, 16-bit elements, input planes too large for the LDS variants: box variant.
//
// Same arithmetic as the other variants (sampler_math.hpp, blend() in gs2d_lds_kernel.hpp; reference kernel
// image/grid_sampler2_d/op_kernel/arch35/grid_sampler2_d_simt.h:303-339,461-514).  The direct kernel reads every tap
// pair from global memory, a scattered four bytes a lane, and on image-sized planes under a rotation the 64 lanes of
// such a load touch dozens of input lines of which each uses a few bytes: the CUs' first-level caches refill at a few
// GB/s each and that is the kernel's time.  Here a workgroup owns a tile of kTileW x kTileH output pixels, two
// neighbouring pixels a lane.  It finds the box of input pixels its taps lie in (minimum and maximum column and row
// over the tile), copies the box -- rows of whole 16-byte units, kBoxChans channels at a time, with 16-byte loads,
// eight lanes a row -- into LDS and takes the taps from there with two-byte LDS reads.  The box of a tile under a
// smooth warp is little larger than the tile turned and scaled.  Two channel groups are on their way in registers
// while one is sampled (two LDS buffers, a barrier per group).  A tile whose box does not fit (scattered points,
// strong minification) falls back, the whole workgroup together, to loads from global memory as the direct
// kernel makes them (bilinear: the west and east tap of a row as one load).
// fp16 2x32x1080x1920, warps of up to 30 degrees: 318 us direct, 202 us here.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "gs2d_common.hpp"
#include "gs2d_lds_kernel.hpp"
#include "kernels.hpp"
#include "sampler_math.hpp"

namespace opscv {

namespace {

constexpr int kBoxThreads = 256;
constexpr int kBoxPpl = 2;  // output pixels a lane, neighbours in a row: their results leave as one four-byte store
constexpr int kTileW = 32, kTileH = kBoxPpl * kBoxThreads / kTileW;
constexpr int kRowLanes = kTileW / kBoxPpl;  // lanes along a row of the tile
constexpr int kBoxChans = 4;                          // channels copied and sampled together
constexpr uint32_t kBoxChanBytes = 4096;              // LDS of one channel's box: the box, then sixteen bytes of zeros
constexpr uint32_t kBoxZero = kBoxChanBytes - 16u;    // ... which a tap outside the image reads
constexpr uint32_t kBoxRowUnits = 8;                  // most 16-byte units a box row may have (eight lanes copy a row)
constexpr uint32_t kBoxRows = kBoxThreads / kBoxRowUnits;  // most rows of a box: one copy a lane and channel
constexpr uint32_t kBoxBuf = kBoxChans * kBoxChanBytes;

typedef uint32_t UnalignedWord __attribute__((aligned(2)));  // a pair of two-byte elements, aligned to one of them
constexpr uint32_t kSelLow = 0x0100u, kSelHigh = 0x0302u, kSelZero = 0x0c0cu;  // byte selectors of v_perm_b32

// Minimum (MAX false) or maximum of `v` over the wavefront, the same in every lane: four steps inside each row of
// sixteen lanes as data-parallel-primitive moves, then the four rows' values.
template <bool MAX>
__device__ __forceinline__ int32_t wave_extreme(int32_t v)
{
    auto pick = [](int32_t a, int32_t b) { return MAX ? (a > b ? a : b) : (a < b ? a : b); };
    v = pick(v, __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
    v = pick(v, __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
    v = pick(v, __builtin_amdgcn_update_dpp(v, v, 0x141, 0xF, 0xF, false));  // row_half_mirror
    v = pick(v, __builtin_amdgcn_update_dpp(v, v, 0x140, 0xF, 0xF, false));  // row_mirror
    const int32_t r0 = __builtin_amdgcn_readlane(v, 0), r1 = __builtin_amdgcn_readlane(v, 16);
    const int32_t r2 = __builtin_amdgcn_readlane(v, 32), r3 = __builtin_amdgcn_readlane(v, 48);
    return pick(pick(r0, r1), pick(r2, r3));
}

struct BoxParams {
    int32_t C, H, W, Hout, Wout;
    uint32_t tiles_x, tiles_y;
    int32_t chan_chunk;
    float neg_zero;
};

template <typename T, int INTERP, int PAD, bool ALIGN>
__global__ __launch_bounds__(kBoxThreads) void gs2d_box_kernel(const T* __restrict__ x, const T* __restrict__ grid,
                                                                T* __restrict__ y, BoxParams p)
{
    static_assert(sizeof(T) == 2, "two-byte elements");
    // taps per axis: bilinear 2 x 2, nearest 1, bicubic 4 x 4; tap (r, k) is row by[r], column bx[k]
    constexpr int NA = (INTERP == 0) ? 2 : (INTERP == 1 ? 1 : 4);
    constexpr int NT = NA * NA;
    constexpr int NW = (INTERP == 2) ? 8 : 4;
    __shared__ __attribute__((aligned(16))) char lds[2 * kBoxBuf];
    __shared__ int32_t s_box[4];  // lowest column and row, highest column and row a tap of the tile lies in
    const uint32_t tid = threadIdx.x;
    // The eight XCDs (workgroups go to them in turn, each has an L2 of its own) take one contiguous eighth of the tiles
    // each: neighbouring tiles share the input lines at their edges in one L2.
    const uint32_t per_xcd = gridDim.x >> 3;
    const uint32_t xcd = blockIdx.x & 7u, turn = blockIdx.x >> 3;
    uint32_t t = (turn < per_xcd) ? xcd * per_xcd + turn : blockIdx.x;
    const uint32_t tx = t % p.tiles_x;
    t /= p.tiles_x;
    const uint32_t ty = t % p.tiles_y;
    const int64_t n = t / p.tiles_y;
    const int64_t out_plane = (int64_t)p.Hout * p.Wout;
    const int64_t in_plane = (int64_t)p.H * p.W;
    const int32_t c_begin = blockIdx.y * p.chan_chunk;
    const int32_t c_end = (c_begin + p.chan_chunk < p.C) ? c_begin + p.chan_chunk : p.C;
    const T* xc = x + (n * p.C + c_begin) * in_plane;
    T* ybase = y + (n * p.C + c_begin) * out_plane;

    // the decisions of decide_pixel() / decide_bicubic() (sampler_math.hpp; grid_sampler2_d_simt.h:479-503, 307-316,
    // 341-349, 379-412), bilinear and nearest without branches as in the LDS kernels, for the lane's kBoxPpl pixels
    const int32_t ox0 = (int32_t)(tx * kTileW + kBoxPpl * (tid % kRowLanes));
    const int32_t oy = (int32_t)(ty * kTileH + tid / kRowLanes);
    bool live[kBoxPpl];
    uint32_t out_off[kBoxPpl];  // byte offset in an output plane; out of the plane's range for lanes off the image
    uint32_t bx[kBoxPpl][NA], by[kBoxPpl][NA];  // tap columns and rows
    bool okx[kBoxPpl][NA], oky[kBoxPpl][NA];    // ... inside the image (none for a non-finite source coordinate)
    float tw[kBoxPpl][NW];
    const uint32_t uw = (uint32_t)p.W, uh = (uint32_t)p.H;
    float gxs[kBoxPpl], gys[kBoxPpl];
#pragma unroll
    for (int j = 0; j < kBoxPpl; j++) {
        // rows of even length (launch condition): a lane's pixels are both on the image or both off it
        live[j] = ox0 + j < p.Wout && oy < p.Hout;
        const int64_t pix = live[j] ? (int64_t)oy * p.Wout + ox0 + j : 0;  // lanes off the image: a valid pixel, unused
        out_off[j] = live[j] ? (uint32_t)pix * 2u : 0x80000000u;
        const T* g = grid + (n * out_plane + pix) * 2;
        gxs[j] = ElemIO<T>::load(g);
        gys[j] = ElemIO<T>::load(g + 1);
    }
#pragma unroll
    for (int j = 0; j < kBoxPpl; j++) {
        if constexpr (INTERP == 2) {
            const BicubicTap b = decide_bicubic<PAD, ALIGN>(gxs[j], gys[j], p.H, p.W);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                bx[j][k] = (uint32_t)b.bx[k];
                by[j][k] = (uint32_t)b.by[k];
                okx[j][k] = b.bx[k] >= 0 && b.bx[k] < p.W && !b.flag;
                oky[j][k] = b.by[k] >= 0 && b.by[k] < p.H;
                tw[j][k] = b.cx[k];
                tw[j][4 + k] = b.cy[k];
            }
            if (b.flag) {
                tw[j][0] = __builtin_nanf("");  // 0 * NaN: every channel becomes NaN, as the reference writes
            }
        } else {
            float ix = compute_source_index<PAD, ALIGN>(gxs[j], p.W);
            float iy = compute_source_index<PAD, ALIGN>(gys[j], p.H);
            const bool finite = __builtin_fabsf(ix) < __builtin_inff() && __builtin_fabsf(iy) < __builtin_inff();
            const bool x_far = ix > 2147483646.0f || ix < -2147483648.0f;  // safe_downgrade: -> -100, always outside
            const bool y_far = iy > 2147483646.0f || iy < -2147483648.0f;
            if constexpr (INTERP == 0) {
                ix = x_far ? -100.0f : ix;
                iy = y_far ? -100.0f : iy;
                const float ixf = __builtin_floorf(ix), iyf = __builtin_floorf(iy);
                bx[j][0] = (uint32_t)float_to_i32(ixf);
                by[j][0] = (uint32_t)float_to_i32(iyf);
                bx[j][1] = bx[j][0] + 1u;  // wraps at INT32_MAX: out of bounds either way
                by[j][1] = by[j][0] + 1u;
                okx[j][0] = bx[j][0] < uw && finite;
                okx[j][1] = bx[j][1] < uw && finite;
                oky[j][0] = by[j][0] < uh;
                oky[j][1] = by[j][1] < uh;
                const float wx1 = ix - ixf, wx0 = ixf + 1.0f - ix;
                const float wy1 = iy - iyf, wy0 = iyf + 1.0f - iy;
                // non-finite source coordinate: every tap reads zeros and 0 * NaN makes every channel NaN, as the
                // reference writes (grid_sampler2_d_simt.h:485-487)
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
                bx[j][0] = xi + ((fx > 0.5f || (fx == 0.5f && (xi & 1u))) ? 1u : 0u);
                by[j][0] = yi + ((fy > 0.5f || (fy == 0.5f && (yi & 1u))) ? 1u : 0u);
                okx[j][0] = bx[j][0] < uw;
                oky[j][0] = by[j][0] < uh;
                tw[j][0] = tw[j][1] = tw[j][2] = tw[j][3] = 0.0f;
            }
        }
    }

    if (tid < 4) {
        s_box[tid] = (tid < 2) ? INT32_MAX : -1;
    }
    if (tid < 2 * kBoxChans * 4) {
        reinterpret_cast<uint32_t*>(lds + (tid >> 2) * kBoxChanBytes + kBoxZero)[tid & 3u] = 0u;
    }
    __syncthreads();
    {
        // the columns and rows inside the image among a pixel's taps; a pixel with none on an axis reads nothing
        int32_t lo_x = INT32_MAX, lo_y = INT32_MAX, hi_x = -1, hi_y = -1;
#pragma unroll
        for (int j = 0; j < kBoxPpl; j++) {
            int32_t lx = INT32_MAX, ly = INT32_MAX, hx = -1, hy = -1;
#pragma unroll
            for (int k = 0; k < NA; k++) {
                const int32_t cx = (int32_t)bx[j][k], cy = (int32_t)by[j][k];
                lx = (okx[j][k] && cx < lx) ? cx : lx;
                hx = (okx[j][k] && cx > hx) ? cx : hx;
                ly = (oky[j][k] && cy < ly) ? cy : ly;
                hy = (oky[j][k] && cy > hy) ? cy : hy;
            }
            if (live[j] && hx >= 0 && hy >= 0) {
                lo_x = lx < lo_x ? lx : lo_x;
                hi_x = hx > hi_x ? hx : hi_x;
                lo_y = ly < lo_y ? ly : lo_y;
                hi_y = hy > hi_y ? hy : hi_y;
            }
        }
        lo_x = wave_extreme<false>(lo_x);
        hi_x = wave_extreme<true>(hi_x);
        lo_y = wave_extreme<false>(lo_y);
        hi_y = wave_extreme<true>(hi_y);
        if ((tid & 63u) == 0u) {
            atomicMin(&s_box[0], lo_x);
            atomicMin(&s_box[1], lo_y);
            atomicMax(&s_box[2], hi_x);
            atomicMax(&s_box[3], hi_y);
        }
    }
    __syncthreads();
    const int32_t x_lo = s_box[0], y_lo = s_box[1], x_hi = s_box[2], y_hi = s_box[3];
    // box geometry: `rows` rows of `upr` 16-byte units from byte `byte_lo` of an input row on (nothing to copy for a tile
    // none of whose pixels reads the image)
    const bool any = x_hi >= 0;
    const uint32_t rows = any ? (uint32_t)(y_hi - y_lo + 1) : 0u;
    const uint32_t byte_lo = any ? ((uint32_t)x_lo * 2u) & ~15u : 0u;
    const uint32_t upr = any ? (((uint32_t)x_hi + 1u) * 2u - byte_lo + 15u) >> 4 : 0u;
    const uint32_t pitch = upr * 16u;

    if (rows * pitch > kBoxZero || upr > kBoxRowUnits || rows > kBoxRows) {
        // ------------------------------------------------ the box does not fit: loads from global memory ---------
#pragma unroll
        for (int j = 0; j < kBoxPpl; j++) {
            if (!live[j]) {
                continue;
            }
            T* yc = reinterpret_cast<T*>(reinterpret_cast<char*>(ybase) + out_off[j]);
            if constexpr (INTERP == 0) {
                // The west and east tap of a row as one load of two elements from column pb = clamp(x0, 0, W - 2); one
                // byte-permute puts the west value in the low half, the east value in the high half and zeroes the
                // half whose tap is outside the image; a row without a valid tap reads the plane's first pair, zeroed
                // the same way.
                const int32_t sx0 = (int32_t)bx[j][0];
                const int32_t pb = (sx0 < 0) ? 0 : ((sx0 > p.W - 2) ? p.W - 2 : sx0);
                const uint32_t at_w = (sx0 == pb) ? kSelLow : kSelHigh, at_e = ((int32_t)bx[j][1] == pb) ? kSelLow : kSelHigh;
                const uint32_t sel_n = ((oky[j][0] && okx[j][0]) ? at_w : kSelZero) | (((oky[j][0] && okx[j][1]) ? at_e : kSelZero) << 16);
                const uint32_t sel_s = ((oky[j][1] && okx[j][0]) ? at_w : kSelZero) | (((oky[j][1] && okx[j][1]) ? at_e : kSelZero) << 16);
                typedef const __attribute__((address_space(1))) T* GlobalRow;
                const bool any_x = okx[j][0] || okx[j][1];
                GlobalRow pn = (GlobalRow)(xc + ((oky[j][0] && any_x) ? (int64_t)by[j][0] * p.W + pb : 0));
                GlobalRow ps = (GlobalRow)(xc + ((oky[j][1] && any_x) ? (int64_t)by[j][1] * p.W + pb : 0));
#pragma unroll 4
                for (int32_t c = c_begin; c < c_end; c++) {
                    const uint32_t north = *(const __attribute__((address_space(1), aligned(2))) UnalignedWord*)pn;
                    const uint32_t south = *(const __attribute__((address_space(1), aligned(2))) UnalignedWord*)ps;
                    const uint32_t mn = __builtin_amdgcn_perm(north, north, sel_n);
                    const uint32_t ms = __builtin_amdgcn_perm(south, south, sel_s);
                    const uint32_t raw[4] = {mn & 0xffffu, mn >> 16, ms & 0xffffu, ms >> 16};
                    ElemIO<T>::store(yc, blend<T, 0>(raw, tw[j], p.neg_zero));
                    pn += in_plane;
                    ps += in_plane;
                    yc += out_plane;
                }
            } else {
                // one load per tap, none with a branch around it: a tap outside the image reads the plane's first
                // element and is replaced by zero
                uint32_t at[NT];  // element offsets in a plane (planes hold fewer than 2^31 elements)
                bool ok[NT];
#pragma unroll
                for (int r = 0; r < NA; r++) {
#pragma unroll
                    for (int k = 0; k < NA; k++) {
                        ok[r * NA + k] = oky[j][r] && okx[j][k];
                        at[r * NA + k] = ok[r * NA + k] ? by[j][r] * uw + bx[j][k] : 0u;
                    }
                }
                const __attribute__((address_space(1))) uint16_t* xp =
                    (const __attribute__((address_space(1))) uint16_t*)xc;
                for (int32_t c = c_begin; c < c_end; c++) {
                    uint32_t raw[NT];
#pragma unroll
                    for (int i = 0; i < NT; i++) {
                        raw[i] = xp[at[i]];
                    }
#pragma unroll
                    for (int i = 0; i < NT; i++) {
                        raw[i] = ok[i] ? raw[i] : 0u;
                    }
                    ElemIO<T>::store(yc, blend<T, INTERP>(raw, tw[j], p.neg_zero));
                    xp += in_plane;
                    yc += out_plane;
                }
            }
        }
        return;
    }

    // LDS byte offsets of the taps in a channel's box
    uint32_t toff[kBoxPpl][NT];
#pragma unroll
    for (int j = 0; j < kBoxPpl; j++) {
        // a lane off the image decided a pixel of some other tile: its taps are not in this box, it reads the zeros
#pragma unroll
        for (int r = 0; r < NA; r++) {
            const uint32_t row = (by[j][r] - (uint32_t)y_lo) * pitch - byte_lo;
#pragma unroll
            for (int k = 0; k < NA; k++) {
                toff[j][r * NA + k] = (live[j] && oky[j][r] && okx[j][k]) ? row + bx[j][k] * 2u : kBoxZero;
            }
        }
    }
    // copying: eight lanes a box row, lane k of them its k-th unit; the same unit of every channel of a group
    const uint32_t my_unit = tid % kBoxRowUnits, my_row = tid / kBoxRowUnits;
    const bool copies = my_unit < upr && my_row < rows;
    const int32_t groups = (c_end - c_begin + kBoxChans - 1) / kBoxChans;
    // a lane that copies nothing reads the first unit of the tile's first channel again and again (no branch around the
    // loads: the wait before a group is stored then counts the loads of the groups after it, which stay on their way)
    const char* mine = reinterpret_cast<const char*>(xc) +
                       (copies ? ((int64_t)(y_lo + (int32_t)my_row) * p.W * 2 + byte_lo + my_unit * 16u) : 0);
    const uint32_t lds_at = (my_row * upr + my_unit) * 16u;
    const int64_t plane_bytes = in_plane * 2;
    // past the last group the last one again, past the last channel the last one (valid addresses, never read)
#define OPSCV_BOX_FETCH(GRP, SET)                                                                  \
    do {                                                                                           \
        const int32_t g_ = (GRP) < groups ? (GRP) : groups - 1;                                    \
        const int32_t left_ = c_end - c_begin - g_ * kBoxChans;                                    \
        const char* at_ = mine + (int64_t)g_ * kBoxChans * plane_bytes;                            \
        SET##0 = *reinterpret_cast<const uint4*>(at_);                                             \
        SET##1 = *reinterpret_cast<const uint4*>(at_ + ((1 < left_) ? 1 : left_ - 1) * plane_bytes); \
        SET##2 = *reinterpret_cast<const uint4*>(at_ + ((2 < left_) ? 2 : left_ - 1) * plane_bytes); \
        SET##3 = *reinterpret_cast<const uint4*>(at_ + ((3 < left_) ? 3 : left_ - 1) * plane_bytes); \
    } while (0)
#define OPSCV_BOX_STASH(BUF, SET)                                                                  \
    do {                                                                                           \
        if (copies) {                                                                              \
            char* to_ = lds + (BUF) * kBoxBuf + lds_at;                                            \
            *reinterpret_cast<uint4*>(to_) = SET##0;                                               \
            *reinterpret_cast<uint4*>(to_ + kBoxChanBytes) = SET##1;                               \
            *reinterpret_cast<uint4*>(to_ + 2 * kBoxChanBytes) = SET##2;                           \
            *reinterpret_cast<uint4*>(to_ + 3 * kBoxChanBytes) = SET##3;                           \
        }                                                                                          \
    } while (0)
    static_assert(kBoxChans == 4, "the two macros above spell four channels out");
    // Sampling a group is straight-line code, so that the wait in front of the LDS stores of the next group can count
    // the loads and stores issued since: the stores go through a buffer descriptor whose range check drops the lanes
    // off the image (offset out of range) and the channels past the last (a range of zero bytes).
    const uint32_t out_plane_bytes = (uint32_t)out_plane * 2u;
    auto sample = [&](uint32_t buf, int32_t grp) {
        const int32_t left = c_end - c_begin - grp * kBoxChans;
#pragma unroll
        for (int cc = 0; cc < kBoxChans; cc++) {
            const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
                ybase + ((int64_t)grp * kBoxChans + cc) * out_plane, 0, (cc < left) ? out_plane_bytes : 0u, kBufferFlags);
            float v[kBoxPpl];
#pragma unroll
            for (int j = 0; j < kBoxPpl; j++) {
                uint32_t raw[NT];
#pragma unroll
                for (int k = 0; k < NT; k++) {
                    raw[k] = *reinterpret_cast<const uint16_t*>(lds + buf * kBoxBuf + cc * kBoxChanBytes + toff[j][k]);
                }
                v[j] = blend<T, INTERP>(raw, tw[j], p.neg_zero);
            }
            buffer_store_group<T, kBoxPpl>(v, rsrc, out_off[0]);
        }
    };
    // Two groups on their way while one is sampled: register sets A and B take turns, LDS buffers 0 and 1 take turns.
    // Step g: ask for group g + 2 (into the set group g came through), sample group g, store group g + 1 to the other
    // buffer -- last read a step ago, before that step's barrier --, barrier.
    uint4 a0, a1, a2, a3, b0, b1, b2, b3;
    OPSCV_BOX_FETCH(0, a);
    OPSCV_BOX_FETCH(1, b);
    OPSCV_BOX_STASH(0u, a);
    __syncthreads();
    for (int32_t grp = 0; grp < groups; grp += 2) {
        OPSCV_BOX_FETCH(grp + 2, a);
        sample(0u, grp);
        OPSCV_BOX_STASH(1u, b);
        __syncthreads();
        OPSCV_BOX_FETCH(grp + 3, b);
        sample(1u, grp + 1);
        OPSCV_BOX_STASH(0u, a);
        __syncthreads();
    }
#undef OPSCV_BOX_FETCH
#undef OPSCV_BOX_STASH
}

template <typename T, int INTERP, int PAD, bool ALIGN>
hipError_t launch_box(const GridSamplerArgs& a, hipStream_t stream)
{
    BoxParams p;
    p.C = (int32_t)a.C;
    p.H = (int32_t)a.Hin;
    p.W = (int32_t)a.Win;
    p.Hout = (int32_t)a.Hout;
    p.Wout = (int32_t)a.Wout;
    const int64_t tx = (a.Wout + kTileW - 1) / kTileW, ty = (a.Hout + kTileH - 1) / kTileH;
    p.tiles_x = (uint32_t)tx;
    p.tiles_y = (uint32_t)ty;
    const int64_t tiles = a.N * tx * ty;
    // whole groups of kBoxChans channels per workgroup; runs of channels to different workgroups where the tiles alone
    // are too few to fill the machine
    int64_t chunks = 1;
    while (tiles * chunks < 4096 && chunks * 2 * kBoxChans <= a.C) {
        chunks *= 2;
    }
    int64_t per = (a.C + chunks - 1) / chunks;
    per = (per + kBoxChans - 1) / kBoxChans * kBoxChans;
    p.chan_chunk = (int32_t)per;
    const int64_t by = (a.C + per - 1) / per;
    p.neg_zero = -0.0f;
    hipLaunchKernelGGL((gs2d_box_kernel<T, INTERP, PAD, ALIGN>), dim3((unsigned)tiles, (unsigned)by), dim3(kBoxThreads), 0,
                       stream, (const T*)a.x, (const T*)a.grid, (T*)a.y, p);
    return hipGetLastError();
}

template <typename T, int INTERP>
hipError_t launch_box_interp(const GridSamplerArgs& a, hipStream_t stream)
{
    switch (a.pad * 2 + a.align) {
        case 0: return launch_box<T, INTERP, 0, false>(a, stream);
        case 1: return launch_box<T, INTERP, 0, true>(a, stream);
        case 2: return launch_box<T, INTERP, 1, false>(a, stream);
        case 3: return launch_box<T, INTERP, 1, true>(a, stream);
        case 4: return launch_box<T, INTERP, 2, false>(a, stream);
        case 5: return launch_box<T, INTERP, 2, true>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

template <typename T>
hipError_t launch_box_typed(const GridSamplerArgs& a, hipStream_t stream)
{
    switch (a.interp) {
        case 0: return launch_box_interp<T, 0>(a, stream);
        case 1: return launch_box_interp<T, 1>(a, stream);
        case 2: return launch_box_interp<T, 2>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

// What the kernel assumes: two-byte elements; input rows of whole 16-byte units on 16-byte
// boundaries, two columns or more; output planes that fill the tiles; counts that fit the launch.
bool box_applies(const GridSamplerArgs& a)
{
    if (a.elem == Elem::F32 || a.interp < 0 || a.interp > 2 || a.channels_last) {
        return false;
    }
    if (a.Win < 2 || (a.Win * 2) % 16 != 0 || reinterpret_cast<uintptr_t>(a.x) % 16 != 0) {
        return false;
    }
    // pairs of neighbouring results as one store: rows of even length, output words on word boundaries
    if (a.Wout % 2 != 0 || reinterpret_cast<uintptr_t>(a.y) % 4 != 0) {
        return false;
    }
    if (a.Wout < 2 * kTileW || a.Hout < 2 * kTileH || a.Hout * a.Wout * 2 >= ((int64_t)1 << 31)) {
        return false;
    }
    const int64_t tx = (a.Wout + kTileW - 1) / kTileW, ty = (a.Hout + kTileH - 1) / kTileH;
    if (a.N * tx * ty > INT32_MAX || a.C > INT32_MAX || (a.C + kBoxChans - 1) / kBoxChans > 65535) {
        return false;
    }
    return true;
}

}  // namespace

const char* gs2d_box_variant_name(const GridSamplerArgs& a) { return box_applies(a) ? "box_lds" : nullptr; }

hipError_t run_gs2d_box(const GridSamplerArgs& a, hipStream_t stream, bool* handled)
{
    *handled = false;
    if (!box_applies(a)) {
        return hipSuccess;
    }
    *handled = true;
    return (a.elem == Elem::F16) ? launch_box_typed<_Float16>(a, stream) : launch_box_typed<__bf16>(a, stream);
}

}  // namespace opscv
