// Backward of the 3-D grid sampler for gfx950: gradient of the input volume as a gather over the contributions of
// every voxel (bilinear, up to 65536 grid points per batch item).
//
// The sum that reaches a voxel is a fixed sequence (grid_sampler3_d_grad_simt_det.h:63-96, see gs3d_grad.hip): its
// contributions ordered by (chunk of 256 grid points, corner tnw .. bse, point), every add rounded to the element
// type.  gs3d_grad.hip walks the chunks in order and elects, round after round, who may add to a voxel: chains of
// dependent LDS round trips and barriers, a few hundred microseconds on volumes where the operands would move in ten.
// Which points reach which voxel, through which corner and with what weight, depends on the grid alone, so here the
// scatter becomes a gather, as for the 2-D sampler (gs2d_grad_csr.hip):
//
//   slots (one lane per grid point, workgroups along the reference's chunks): the eight corner weights of the point go
//     to scratch memory, and the point takes one of the eight slots of the cell (z0, y0, x0) of its low corner (an
//     atomic count per cell: which slot a point gets depends on timing, which points a cell holds does not).  A point
//     that finds its cell full goes to a short overflow list of the item, where the voxels of a crowded cell look for
//     it; an item with more than 1024 such points is flagged.  The workgroup also notes the span of voxels its chunk
//     touches, which the ordered kernel wants should the item be flagged.
//   gather (one lane per voxel): voxel (z, y, x) is corner (xs, ys, zs) of the points of cell (z - zs, y - ys, x - xs).
//     The lane collects the points of its eight cells, keyed (chunk, corner, point), into a list of its own in LDS,
//     sorts the list through a bitonic network in registers (eight entries on average) and then walks it once per
//     group of four channels:
//     gradOutput[channel][point] times weight[point][corner], folded into the sum with the reference's roundings.
//     A voxel with more contributions than its list holds flags the item.
//   A flagged item is left to the ordered kernel of gs3d_grad.hip, which runs afterwards, skips the items that are not
//     flagged and writes the whole gradient of those that are.
//
// fp16 22x4x16x64x64 with a registration-style warp: 297 us (ordered kernel) -> see the profile of that workload.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "gs3d_grad_math.hpp"
#include "kernels.hpp"
#include "options.hpp"

namespace opscv {

namespace {

constexpr int kLThreads = kChunkPoints3;
constexpr int kCellSlots = 8;   // points a cell can hold in its slot record
constexpr int kOverflowMax = 1024;  // points of an item that found their cell's record full and wait in a list
constexpr int kListMax = 32;    // contributions a voxel's list can hold
constexpr int kChanBlock = 4;   // channels per walk of a list
constexpr uint32_t kPtBits = 16;

// 32-bit words of scratch per batch item
struct Lists3Layout {
    uint32_t flag;    // 4 words; [0] != 0: the item is left to the ordered kernel; [1]: points in the overflow list
    uint32_t counts;  // one per cell of the (D + 1) x (H + 1) x (W + 1) lattice of low corners.  Dense, apart from the
                      // slots: the atomics of neighbouring points then meet in few cache lines (a count inside the
                      // cell's 16-byte slot record made the slots kernel 17 us slower on fp16 22x4x16x64x64)
    uint32_t slots;   // kCellSlots 16-bit point numbers per cell: one 16-byte load per cell
    uint32_t overflow;  // kOverflowMax (cell, point) pairs: the points beyond the eighth of a cell
    uint32_t wts;     // eight weights of the element type per point
    uint32_t go4;     // gradOutput with the channels of a group of four side by side: [group][point][4]
    uint32_t item_words;
};

inline uint32_t align4(uint64_t v) { return (uint32_t)((v + 3u) & ~(uint64_t)3u); }

Lists3Layout make_layout(int64_t cells, int64_t points, int64_t esz, int64_t channels)
{
    Lists3Layout l;
    l.flag = 0;
    l.counts = 4;
    l.slots = align4((uint64_t)l.counts + (uint64_t)cells);
    l.overflow = align4((uint64_t)l.slots + (uint64_t)cells * 4);
    l.wts = align4((uint64_t)l.overflow + 2u * kOverflowMax);
    l.go4 = align4((uint64_t)l.wts + (uint64_t)points * 8 * (uint64_t)esz / 4);
    const uint64_t groups = ((uint64_t)channels + kChanBlock - 1) / kChanBlock;
    l.item_words = align4((uint64_t)l.go4 + groups * (uint64_t)points * kChanBlock * (uint64_t)esz / 4);
    return l;
}

// All workgroups of a batch item on one XCD (workgroups go to the eight XCDs in turn): the item's slots, weights and
// gradOutput then pass through one L2 instead of eight.  Item n lives on XCD n % 8; the grid has
// 8 * ceil(N / 8) * per_item workgroups, and those of an item beyond the last return at once (-1).
__device__ __forceinline__ int64_t item_of_block(uint32_t per_item, int32_t N, uint32_t* local)
{
    const uint32_t xcd = blockIdx.x & 7u, i = blockIdx.x >> 3;
    *local = i % per_item;
    const int64_t n = (int64_t)(i / per_item) * 8 + xcd;
    return n < N ? n : -1;
}

// zeroes the flag and the cell counts of every item
__global__ __launch_bounds__(256) void gs3d_lists_clear_kernel(uint32_t* __restrict__ ws, uint32_t words,
                                                               uint32_t item_words)
{
    uint32_t* wsn = ws + (size_t)blockIdx.y * item_words;
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < words) {
        wsn[i] = 0u;  // the flag words and the counts lie at the start of an item's scratch
    }
}

// GRID: the lane goes on to the gradient of its grid point -- the corner decisions are the same, and the atomics
// and stores above are on their way while the corners of the input are read.
template <typename T, int GRID>
__global__ __launch_bounds__(kLThreads) void gs3d_lists_slots_kernel(const T* __restrict__ grid,
                                                                      const T* __restrict__ gout,
                                                                      uint32_t* __restrict__ ws,
                                                                      int32_t* __restrict__ ranges, Grad3Params p,
                                                                      Lists3Layout lay, int32_t N,
                                                                      const T* __restrict__ x, T* __restrict__ dgrid)
{
    using Taps = GradTaps3<T, 0>;
    __shared__ int32_t s_lo[kLThreads / 64], s_hi[kLThreads / 64];
    const int t = threadIdx.x;
    uint32_t chunk;
    const int64_t n = item_of_block((uint32_t)p.chunks, N, &chunk);
    if (n < 0) {
        return;
    }
    uint32_t* wsn = ws + (size_t)n * lay.item_words;
    const int32_t pt = -chunk_phase(n, p) + (int32_t)chunk * kLThreads + t;
    int32_t lo = INT32_MAX, hi = -1;
    if (pt >= 0 && pt < p.points) {
        const T* g = grid + (n * (int64_t)p.points + pt) * 3;
        Taps tp;
        decide_grad_taps3<T, 0>(tp, ElemIO<T>::load(g), ElemIO<T>::load(g + 1), ElemIO<T>::load(g + 2), p.D, p.H, p.W,
                                p.pad, p.align);
        T w8[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            ElemIO<T>::store(&w8[k], tp.w[k]);  // exact: the weight is a value of the element type
            if (tp.off[k] >= 0) {
                lo = tp.off[k] < lo ? tp.off[k] : lo;
                hi = tp.off[k] > hi ? tp.off[k] : hi;
            }
        }
        T* wts = reinterpret_cast<T*>(wsn + lay.wts) + (size_t)pt * 8;
        if constexpr (sizeof(T) == 2) {
            *reinterpret_cast<uint4*>(wts) = *reinterpret_cast<const uint4*>(w8);
        } else {
            reinterpret_cast<uint4*>(wts)[0] = reinterpret_cast<const uint4*>(w8)[0];
            reinterpret_cast<uint4*>(wts)[1] = reinterpret_cast<const uint4*>(w8)[1];
        }
        // gradOutput of the point, four channels side by side: the gather then takes them with one load (past the
        // last channel the last one again, never used)
        {
            const T* go_n = gout + n * p.C * (int64_t)p.points + pt;
            T* go4 = reinterpret_cast<T*>(wsn + lay.go4);
            for (int32_t c0 = 0; c0 < p.C; c0 += kChanBlock) {
                T four[kChanBlock];
#pragma unroll
                for (int j = 0; j < kChanBlock; j++) {
                    const int32_t c = (c0 + j < p.C) ? c0 + j : p.C - 1;
                    four[j] = go_n[(int64_t)c * p.points];
                }
                T* dst = go4 + ((size_t)(c0 / kChanBlock) * p.points + pt) * kChanBlock;
                if constexpr (sizeof(T) == 2) {
                    *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(four);
                } else {
                    *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(four);
                }
            }
        }
        // the cell of the low corner; a point none of whose corners is inside the volume has no cell
        if (tp.x0 >= -1 && tp.x0 < p.W && tp.y0 >= -1 && tp.y0 < p.H && tp.z0 >= -1 && tp.z0 < p.D) {
            const uint32_t cell = ((uint32_t)(tp.z0 + 1) * (uint32_t)(p.H + 1) + (uint32_t)(tp.y0 + 1)) *
                                      (uint32_t)(p.W + 1) +
                                  (uint32_t)(tp.x0 + 1);
            const uint32_t r = atomicAdd(&wsn[lay.counts + cell], 1u);
            if (r < (uint32_t)kCellSlots) {
                reinterpret_cast<uint16_t*>(wsn + lay.slots + (size_t)cell * 4)[r] = (uint16_t)pt;
            } else {
                // the record is full: the point waits in the item's overflow list, where the voxels of a crowded cell
                // look for it; an item with more of those than the list holds is left to the ordered kernel
                const uint32_t o = atomicAdd(&wsn[lay.flag + 1], 1u);
                if (o < (uint32_t)kOverflowMax) {
                    reinterpret_cast<uint2*>(wsn + lay.overflow)[o] = make_uint2(cell, (uint32_t)pt);
                } else {
                    wsn[lay.flag] = 1u;
                }
            }
        }
        if constexpr (GRID > 0) {  // GRID: channels in flight together (gs3d_point_grid_gradient)
            gs3d_point_grid_gradient<T, GRID>(tp, gout, x, dgrid, n * (int64_t)p.points + pt, n, pt, p);
        }
    }
    if (ranges == nullptr) {
        return;
    }
    // the span of voxels this chunk touches (lowest > highest for a chunk that touches none)
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const int32_t olo = __shfl_xor(lo, d), ohi = __shfl_xor(hi, d);
        lo = olo < lo ? olo : lo;
        hi = ohi > hi ? ohi : hi;
    }
    if ((t & 63) == 0) {
        s_lo[t >> 6] = lo;
        s_hi[t >> 6] = hi;
    }
    __syncthreads();
    if (t == 0) {
#pragma unroll
        for (int w = 1; w < kLThreads / 64; w++) {
            lo = s_lo[w] < lo ? s_lo[w] : lo;
            hi = s_hi[w] > hi ? s_hi[w] : hi;
        }
        int32_t* r = ranges + (n * (int64_t)p.chunks + chunk) * 2;
        r[0] = lo;
        r[1] = hi;
    }
}

// One more contribution: weight times gradOutput rounded to the element type, added to the sum with a rounding to the
// element type (contribution3 and the ordered kernel's read-modify-write).  For fp16 both steps are the native
// instructions: the exact product of two fp16 values fits fp32, so rounding it to fp16 is the fp16 product, and the
// fp32 sum of two fp16 values rounded to fp16 is the fp16 sum (24 >= 2 x 11 + 2 bits).
template <typename T>
struct Fold3 {
    typedef float acc_t;
    static __device__ __forceinline__ acc_t zero() { return 0.0f; }
    static __device__ __forceinline__ acc_t add(acc_t acc, T go, T w)
    {
        return rt<T>(acc + contribution3<T, 0>(ElemIO<T>::load(&go), ElemIO<T>::load(&w)));
    }
    static __device__ __forceinline__ void store(T* p, acc_t acc) { store_streaming<T>(p, acc); }
};
template <>
struct Fold3<_Float16> {
    typedef _Float16 acc_t;
    static __device__ __forceinline__ acc_t zero() { return (_Float16)0.0f; }
    static __device__ __forceinline__ acc_t add(acc_t acc, _Float16 go, _Float16 w)
    {
        const _Float16 val = w * go;
        return acc + val;
    }
    static __device__ __forceinline__ void store(_Float16* p, acc_t acc) { __builtin_nontemporal_store(acc, p); }
};

// The first NK entries of a lane's list (every kLThreads-th word from `mine`), sorted ascending through registers.
template <int NK>
__device__ __forceinline__ void sort_list(uint32_t* mine, uint32_t len)
{
    uint32_t key[NK];
#pragma unroll
    for (int i = 0; i < NK; i++) {
        const uint32_t v = mine[i * kLThreads];
        key[i] = ((uint32_t)i < len) ? v : 0xFFFFFFFFu;
    }
#pragma unroll
    for (int size = 2; size <= NK; size *= 2) {
#pragma unroll
        for (int stride = size / 2; stride > 0; stride /= 2) {
#pragma unroll
            for (int i = 0; i < NK; i++) {
                const int l = i ^ stride;
                if (l > i) {
                    const uint32_t lo = key[i] < key[l] ? key[i] : key[l];
                    const uint32_t hi = key[i] < key[l] ? key[l] : key[i];
                    const bool ascending = (i & size) == 0;
                    key[i] = ascending ? lo : hi;
                    key[l] = ascending ? hi : lo;
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < NK; i++) {
        mine[i * kLThreads] = key[i];
    }
}

template <typename T>
__global__ __launch_bounds__(kLThreads) void gs3d_lists_gather_kernel(T* __restrict__ dx,
                                                                       uint32_t* __restrict__ ws, Grad3Params p,
                                                                       Lists3Layout lay, uint32_t tiles,
                                                                       uint32_t cblocks, int32_t chans_per_block,
                                                                       int32_t N)
{
    typedef Fold3<T> F;
    typedef typename F::acc_t acc_t;
    __shared__ uint32_t list[kListMax * kLThreads];  // entry i of lane t at [i * kLThreads + t]: a bank of its own
    const int t = threadIdx.x;
    uint32_t local;
    const int64_t n = item_of_block(tiles * cblocks, N, &local);
    if (n < 0) {
        return;
    }
    uint32_t* wsn = ws + (size_t)n * lay.item_words;
    if (wsn[lay.flag] != 0u) {
        return;  // the item is the ordered kernel's
    }
    const int32_t vol = p.D * p.H * p.W;
    const int32_t v = (int32_t)(local % tiles) * kLThreads + t;
    if (v >= vol) {
        return;
    }
    const int32_t c_begin = (int32_t)(local / tiles) * chans_per_block;
    const int32_t c_end = (c_begin + chans_per_block < p.C) ? c_begin + chans_per_block : p.C;
    const int32_t x = v % p.W, yz = v / p.W;
    const int32_t y = yz % p.H, z = yz / p.H;
    const uint32_t w1 = (uint32_t)(p.W + 1), h1 = (uint32_t)(p.H + 1);
    const uint32_t phase = (uint32_t)chunk_phase(n, p);
    const uint32_t* counts = wsn + lay.counts;
    const uint4* slots = reinterpret_cast<const uint4*>(wsn + lay.slots);
    uint32_t* mine = list + t;

    // collect: corner k = xs + 2 ys + 4 zs of the points whose low corner is (z - zs, y - ys, x - xs)
    uint32_t cnt[8];
    uint4 rec[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const uint32_t xs = k & 1, ys = (k >> 1) & 1, zs = k >> 2;
        const uint32_t cell = (((uint32_t)z + 1u - zs) * h1 + ((uint32_t)y + 1u - ys)) * w1 + ((uint32_t)x + 1u - xs);
        cnt[k] = counts[cell];
        rec[k] = slots[cell];
    }
    uint32_t len = 0;
    bool crowded = false;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        len += cnt[k];
        crowded = crowded || cnt[k] > (uint32_t)kCellSlots;
    }
    if (len > (uint32_t)kListMax) {
        wsn[lay.flag] = 1u;  // the ordered kernel redoes the item
        return;
    }
    auto key_of = [&](uint32_t pt, uint32_t k) {
        return (((pt + phase) >> 8) << (kPtBits + 3)) | (k << kPtBits) | pt;
    };
    uint32_t at = 0;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        // a cell holds a point or two as a rule: those without a loop
        const uint32_t have = cnt[k] < (uint32_t)kCellSlots ? cnt[k] : (uint32_t)kCellSlots;
        if (have > 0u) {
            mine[at * kLThreads] = key_of(rec[k].x & 0xFFFFu, (uint32_t)k);
        }
        if (have > 1u) {
            mine[(at + 1u) * kLThreads] = key_of(rec[k].x >> 16, (uint32_t)k);
        }
        for (uint32_t i = 2; i < have; i++) {
            const uint32_t word = (i < 4u) ? rec[k].y : ((i < 6u) ? rec[k].z : rec[k].w);
            mine[(at + i) * kLThreads] = key_of((word >> ((i & 1u) * 16u)) & 0xFFFFu, (uint32_t)k);
        }
        at += have;
    }
    if (crowded) {
        // the points of a crowded cell beyond its record: the item's overflow list holds them, with their cell
        const uint32_t listed = wsn[lay.flag + 1] < (uint32_t)kOverflowMax ? wsn[lay.flag + 1] : (uint32_t)kOverflowMax;
        const uint2* waiting = reinterpret_cast<const uint2*>(wsn + lay.overflow);
        const uint32_t xb = (uint32_t)x + 1u, yb = (uint32_t)y + 1u, zb = (uint32_t)z + 1u;
        for (uint32_t i = 0; i < listed; i++) {
            const uint2 e = waiting[i];
            // which corner of this voxel the waiting point's cell is, if any
            const uint32_t cx = e.x % w1, cyz = e.x / w1;
            const uint32_t cy = cyz % h1, cz = cyz / h1;
            const uint32_t xs = xb - cx, ys = yb - cy, zs = zb - cz;
            if (xs <= 1u && ys <= 1u && zs <= 1u) {
                mine[at * kLThreads] = key_of(e.y, xs + 2u * ys + 4u * zs);
                at++;
            }
        }
    }
    // Sort, ascending keys = the reference's order: the list goes through registers and a bitonic network of 16 keys,
    // or of 32 where a lane of the wavefront has more (past its end a list is padded with the largest key).  An
    // insertion sort in LDS, chains of dependent reads and writes, took three times as long as everything else here.
    if (__builtin_amdgcn_ballot_w64(len > 16u) == 0) {
        sort_list<16>(mine, len);
    } else {
        sort_list<32>(mine, len);
    }
    // Walk the list once per group of channels, two entries in flight: the operands of the entry after this one are
    // asked for before this one is folded in.  No branches in the loop -- past the end of the list or of the channels
    // the last entry or channel is loaded again and not used.
    const char* wts = reinterpret_cast<const char*>(wsn + lay.wts);
    const uint32_t last = len > 0 ? len - 1u : 0u;
    for (int32_t c0 = c_begin; c0 < c_end; c0 += kChanBlock) {
        const int32_t nc = (c_end - c0 < kChanBlock) ? c_end - c0 : kChanBlock;
        // the group's gradOutput, four channels per point (byte offsets in 32 bits: launch plan)
        const char* go4 = reinterpret_cast<const char*>(wsn + lay.go4) +
                          (size_t)(c0 / kChanBlock) * p.points * (kChanBlock * sizeof(T));
        acc_t acc[kChanBlock];
#pragma unroll
        for (int j = 0; j < kChanBlock; j++) {
            acc[j] = F::zero();
        }
        T wa, wb, ga[kChanBlock], gb[kChanBlock];
        auto fetch = [&](uint32_t i, T& w, T (&g)[kChanBlock]) {
            const uint32_t key = mine[(i < last ? i : last) * kLThreads];
            const uint32_t pt = key & 0xFFFFu, k = (key >> kPtBits) & 7u;
            w = *reinterpret_cast<const T*>(wts + (pt * 8u + k) * (uint32_t)sizeof(T));
            typedef typename std::conditional<sizeof(T) == 2, uint2, uint4>::type four_t;
            const four_t four = *reinterpret_cast<const four_t*>(go4 + pt * (uint32_t)(kChanBlock * sizeof(T)));
            __builtin_memcpy(g, &four, sizeof(four));
        };
        if (len > 0) {
            fetch(0, wa, ga);
        }
        for (uint32_t i = 0; i < len; i += 2) {
            fetch(i + 1, wb, gb);
#pragma unroll
            for (int j = 0; j < kChanBlock; j++) {
                acc[j] = F::add(acc[j], ga[j], wa);
            }
            fetch(i + 2, wa, ga);
            if (i + 1 < len) {
#pragma unroll
                for (int j = 0; j < kChanBlock; j++) {
                    acc[j] = F::add(acc[j], gb[j], wb);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < kChanBlock; j++) {
            if (j < nc) {
                F::store(dx + (n * p.C + c0 + j) * (int64_t)vol + v, acc[j]);
            }
        }
    }
}

// profitability limits of the gather variant (see make_plan).  Measured on fp16 volumes, four channels, input gradient
// and grid gradient together, ordered kernel / gather: 1 voxel per grid point 313 / 97 us (22 x 16x64x64), 4 voxels 83 /
// 41 us, 16 voxels 35 / 38 us, 32 voxels 35 / 50 us, 128 voxels 56 / 262 us (2 x 128^3), 4096 voxels 80 / 2049 us
// (256^3 with 4096 points).
constexpr int64_t kSparseVoxelsPerPoint = 8;
constexpr int64_t kMaxScratchBytes = (int64_t)1 << 30;

struct Lists3Plan {
    bool ok = false;
    Lists3Layout lay;
    int64_t cells = 0;
    uint32_t tiles = 0, cblocks = 0;
    int32_t chans_per_block = 0;
};

Lists3Plan make_plan(const GridSampler3DGradArgs& a)
{
    Lists3Plan pl;
    const int64_t points = a.Dout * a.Hout * a.Wout, vol = a.Din * a.Hin * a.Win;
    const int64_t cells = (a.Din + 1) * (a.Hin + 1) * (a.Win + 1);
    const int64_t esz = elem_size(a.elem);
    // 16-bit point numbers in the slots; the item's scratch is indexed in 32 bits; items along a grid axis
    if (a.interp != 0 || points > 65536 || vol > INT32_MAX || cells > (int64_t)1 << 27 || a.N > 65535 ||
        a.C * points * esz > (int64_t)UINT32_MAX) {
        return pl;
    }
    const int64_t groups = (a.C + kChanBlock - 1) / kChanBlock;
    const int64_t item_words_estimate =
        4 + cells * 5 + 2 * kOverflowMax + points * 8 * esz / 4 + groups * points * kChanBlock * esz / 4 + 16;
    if (item_words_estimate > (int64_t)1 << 31) {
        return pl;  // an item's scratch is indexed in 32 bits
    }
    if (a.force_variant == kGs3dGradOrdered) {
        return pl;
    }
    if (a.force_variant != kGs3dGradGather) {
        // The gather spends a lane, eight cell look-ups and five words of scratch on every voxel whether grid points
        // fall near it or not, the ordered kernel works per grid point: a volume sampled at few points (below one
        // point per kSparseVoxelsPerPoint voxels) stays with the ordered kernel, and so does a call whose scratch
        // would pass kMaxScratchBytes.
        if (points * kSparseVoxelsPerPoint < vol || item_words_estimate * 4 * a.N > kMaxScratchBytes) {
            return pl;
        }
    }
    pl.cells = cells;
    pl.lay = make_layout(cells, points, esz, a.C);
    pl.tiles = (uint32_t)((vol + kLThreads - 1) / kLThreads);
    // channel blocks: lanes enough for the chip (a lane walks its list once per four channels)
    const int64_t base = a.N * pl.tiles;
    const int64_t max_cblocks = (a.C + kChanBlock - 1) / kChanBlock;
    int64_t cblocks = (2048 + base - 1) / base;
    cblocks = cblocks > max_cblocks ? max_cblocks : cblocks;
    int64_t cpb = (a.C + cblocks - 1) / cblocks;
    cpb = (cpb + kChanBlock - 1) / kChanBlock * kChanBlock;
    cblocks = (a.C + cpb - 1) / cpb;
    const int64_t item_slots = 8 * ((a.N + 7) / 8);
    if (item_slots * pl.tiles * cblocks > INT32_MAX || item_slots * chunk_count(points, 2) > INT32_MAX) {
        return pl;
    }
    pl.cblocks = (uint32_t)cblocks;
    pl.chans_per_block = (int32_t)cpb;
    pl.ok = true;
    return pl;
}

template <typename T>
hipError_t run_typed(const GridSampler3DGradArgs& a, const Lists3Plan& pl, const Grad3Params& p, int32_t* ranges,
                     hipStream_t stream)
{
    uint32_t* ws = (uint32_t*)a.lists;
    const uint32_t clear_words = pl.lay.counts + (uint32_t)pl.cells;
    hipLaunchKernelGGL(gs3d_lists_clear_kernel, dim3((clear_words + 255u) / 256u, (unsigned)a.N), dim3(256), 0, stream, ws,
                       clear_words, pl.lay.item_words);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        return e;
    }
    const uint32_t item_slots = 8u * (uint32_t)((a.N + 7) / 8);  // items, rounded up to whole turns of the XCDs
    const dim3 slots_grid(item_slots * (uint32_t)p.chunks);
    if (a.dgrid != nullptr && a.N * (int64_t)p.points < kGridGradFewPoints) {
        hipLaunchKernelGGL((gs3d_lists_slots_kernel<T, 4>), slots_grid, dim3(kLThreads), 0, stream, (const T*)a.grid,
                           (const T*)a.gout, ws, ranges, p, pl.lay, (int32_t)a.N, (const T*)a.x, (T*)a.dgrid);
    } else if (a.dgrid != nullptr) {
        hipLaunchKernelGGL((gs3d_lists_slots_kernel<T, 1>), slots_grid, dim3(kLThreads), 0, stream, (const T*)a.grid,
                           (const T*)a.gout, ws, ranges, p, pl.lay, (int32_t)a.N, (const T*)a.x, (T*)a.dgrid);
    } else {
        hipLaunchKernelGGL((gs3d_lists_slots_kernel<T, 0>), slots_grid, dim3(kLThreads), 0, stream, (const T*)a.grid,
                           (const T*)a.gout, ws, ranges, p, pl.lay, (int32_t)a.N, (const T*)nullptr, (T*)nullptr);
    }
    e = hipGetLastError();
    if (e != hipSuccess) {
        return e;
    }
    hipLaunchKernelGGL((gs3d_lists_gather_kernel<T>), dim3(item_slots * pl.tiles * pl.cblocks), dim3(kLThreads), 0,
                       stream, (T*)a.dx, ws, p, pl.lay, pl.tiles, pl.cblocks, pl.chans_per_block,
                       (int32_t)a.N);
    return hipGetLastError();
}

}  // namespace

int64_t gs3d_grad_list_words(const GridSampler3DGradArgs& a)
{
    const Lists3Plan pl = make_plan(a);
    return pl.ok ? (int64_t)pl.lay.item_words * a.N : 0;
}

hipError_t run_gs3d_grad_input_lists(const GridSampler3DGradArgs& a, const Grad3Params& p, int32_t* ranges,
                                     hipStream_t stream, const uint32_t** item_flags, uint32_t* flag_stride,
                                     bool* dgrid_done)
{
    *item_flags = nullptr;
    *flag_stride = 0;
    *dgrid_done = false;
    if (a.dx == nullptr || a.lists == nullptr) {
        return hipSuccess;
    }
    const Lists3Plan pl = make_plan(a);
    if (!pl.ok) {
        return hipSuccess;
    }
    *item_flags = (const uint32_t*)a.lists + pl.lay.flag;
    *flag_stride = pl.lay.item_words;
    *dgrid_done = a.dgrid != nullptr;
    switch (a.elem) {
        case Elem::F32: return run_typed<float>(a, pl, p, ranges, stream);
        case Elem::F16: return run_typed<_Float16>(a, pl, p, ranges, stream);
        case Elem::BF16: return run_typed<__bf16>(a, pl, p, ranges, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
