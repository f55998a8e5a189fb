// Backward of grid_sampler2d for gfx950: gradient of the input (bilinear) as a gather over precomputed lists.
//
// The reference's deterministic mode (image/grid_sampler2_d_grad/op_kernel/arch35/grid_sampler2_d_grad_simt_det.h:
// 75-101) fixes the order in which contributions reach an element of the gradient: the grid points of a batch item
// in chunks of 256, per chunk corner after corner (nw, ne, sw, se), per corner point after point, every add rounded
// to the element type.  Which points reach which element, through which corner and with what weight, depends on
// the grid alone -- it is the same for every channel.  So instead of scattering per channel (gs2d_grad.hip elects, per
// corner and round, who may add to an element: about 250 workgroup barriers per group of four planes), a few kernels:
//
//   slots (one lane per grid point, all CUs): the four corner weights of every point go to scratch memory, and the
//     point takes one of the eight slots of the cell (y0, x0) of its north-west corner (an atomic count per cell: which
//     slot a point gets depends on timing, which points a cell holds does not).  A cell with more than eight points
//     flags its batch item.
//   sort (one workgroup per flagged batch item, else it returns at once): the item's points are sorted by cell -- a
//     stable block radix sort of (cell, point) keys, so the points of a cell come out in ascending order -- and the
//     start of every cell's run is noted.
//   lists (one lane per element, all CUs): element (y, x) is the nw corner of the points of cell (y, x), the ne corner
//     of cell (y, x-1), the sw corner of cell (y-1, x) and the se corner of cell (y-1, x-1).  The up to eight points of
//     each of the four cells are read at once (from the slots, or from the sorted runs of a flagged item), keyed
//     (chunk, corner, point) and sorted in registers by a bitonic network: the element's contributions in exactly the
//     reference's order, whatever order the slots were filled in.  A corner outside the image never comes
//     up: no element asks for it.  The first eight (point, weight) pairs of an element go to a fixed slot, the rest to
//     an overflow area.  A cell with more than eight points (points piled up on one spot) takes a walk with cursors
//     instead of the network.
//   apply (per batch item, tile of 512 elements, block of channels): a lane owns one element and holds its first
//     eight contributions in registers (more: in LDS); the gradOutput planes of the channels stream through LDS
//     (asynchronous global->LDS copies by loader wavefronts into a ring of slots; 16-bit planes of up to 16 KiB
//     instead go through the loaders' registers and lie in LDS interleaved, all channels of a point side by side, so
//     that one read serves them all), and per channel the lane folds gradOutput[point] * weight into its sum in list
//     order with the reference's roundings.  No atomics, no elections; one barrier per group of planes.
//
// The result is the same sequence of rounded operations per element as the scatter in gs2d_grad.hip, bit for bit.
#include <hip/hip_runtime.h>

#include <type_traits>

#include <rocprim/block/block_radix_sort.hpp>

#include "gs2d_grad_math.hpp"
#include "gs2d_lds_kernel.hpp"
#include "kernels.hpp"

namespace opscv {

namespace {

constexpr int kSortThreads = 1024;
constexpr int kMaxIpt = 16;                       // points per sorting thread: up to 16384 grid points per batch item
constexpr int kPointBits = 14;                    // 16384 points
constexpr uint32_t kPointMask = (1u << kPointBits) - 1u;
constexpr int kMaxCells = 32768;                  // (H + 1) * (W + 1): the keys keep 32 bits
constexpr uint32_t kNoCell = 0xFFFFFFFFu;         // key of a point none of whose corners can be inside, and of padding
constexpr int kChunkShift = 8;                    // 256 points per chunk of the accumulation order
constexpr int kListThreads = 256;
constexpr int kRun = 8;                           // points of a cell the sorting network takes
constexpr int kApplyLanes = 512;                  // elements per workgroup of the apply kernel
constexpr int kApplyLoaders = 2;                  // loader wavefronts
constexpr int kApplyThreads = kApplyLanes + 64 * kApplyLoaders;
// The interleaved layout of 16-bit planes (apply kernel): loader wavefronts that interleave through registers, the
// 16-byte loads each of their lanes has per step (units of a plane times planes), the steps whose loads they keep on
// their way, the slots of LDS
constexpr int kPairLoaders = 4;
constexpr int kPairThreads = kApplyLanes + 64 * kPairLoaders;
constexpr int kPairLoads = 8;
constexpr int kPairDepth = 2;
constexpr int kPairNbuf = 2;
constexpr int kHeld = 8;                          // contributions of an element kept in registers
constexpr int kApplyBufBytes = 64 * 1024;         // the ring of gradOutput planes (twice that for planes over 16 KiB)
constexpr int kApplyNbuf = 4;                     // its slots: three groups of planes on their way while one is read
constexpr int kApplySpill = 1024;                 // contributions beyond the held ones that a workgroup keeps in LDS

struct GradParams {
    int32_t C, H, W, Ho, Wo;
    int32_t pad, align;
};

// scratch of one batch item, offsets in 32-bit words
struct CsrLayout {
    uint32_t wts;         // 4 floats per point: the corner weights nw, ne, sw, se
    uint32_t sorted;      // kSortThreads * ipt keys (cell << kPointBits | point), sorted
    uint32_t cell_start;  // cells + 1 positions in `sorted`
    uint32_t count;       // H * W list lengths
    uint32_t held;        // H * W slots of kHeld (point, weight) pairs
    uint32_t more_start;  // H * W positions in `more` (elements with more than kHeld contributions)
    uint32_t more_used;   // 1 word: pairs handed out in `more`
    uint32_t more;        // up to 4 * points (point, weight) pairs
    uint32_t slot_count;  // cells counts of points per cell; behind them 2 words: the item's flag "a cell overflowed"
                          // and the count of workgroups that have handed out their slots
    uint32_t slots;       // cells * kRun points
    uint32_t item_words;
};

CsrLayout make_layout(int64_t points, int64_t plane_px, int64_t cells, int ipt)
{
    auto align4 = [](uint32_t v) { return (v + 3u) & ~3u; };
    CsrLayout l;
    l.wts = 0;
    l.sorted = (uint32_t)(4 * points);
    l.cell_start = l.sorted + (uint32_t)(kSortThreads * ipt);
    l.count = align4(l.cell_start + (uint32_t)cells + 1u);
    l.held = align4(l.count + (uint32_t)plane_px);
    l.more_start = l.held + (uint32_t)(2 * kHeld * plane_px);
    l.more_used = align4(l.more_start + (uint32_t)plane_px);
    l.more = l.more_used + 4u;
    l.slot_count = align4(l.more + (uint32_t)(8 * points));
    l.slots = align4(l.slot_count + (uint32_t)cells + 2u);
    l.item_words = align4(l.slots + (uint32_t)(kRun * cells));
    return l;
}

// zeroes the cell counts of every item, the two words behind them and the overflow counter (a kernel rather than a
// memset: a caller may capture the launch sequence in a graph).  The backward's other kernel does the same on its way
// when it runs first (GradClear).
__global__ __launch_bounds__(256) void gs2d_grad_csr_clear_kernel(GradClear c)
{
    uint32_t* wsn = c.base + (size_t)blockIdx.y * c.item_words;
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < c.count) {
        wsn[c.first + i] = 0u;
    }
    if (i == 0) {
        wsn[c.single] = 0u;
    }
}

// The points of one item sorted by cell, and where every cell's run starts: all threads of a workgroup of
// kSortThreads.
template <typename T, int IPT>
__device__ __forceinline__ void sort_item(const T* __restrict__ grid, uint32_t* __restrict__ wsn, const GradParams& p,
                                          const CsrLayout& lay, int64_t n,
                                          typename rocprim::block_radix_sort<uint32_t, kSortThreads, IPT>::storage_type&
                                              sort_storage,
                                          uint32_t* sorted_lds)
{
    using sort_t = rocprim::block_radix_sort<uint32_t, kSortThreads, IPT>;
    const int32_t points = p.Ho * p.Wo;
    const int32_t cells = (p.H + 1) * (p.W + 1);
    const uint32_t cell_bits = 32u - (uint32_t)__builtin_clz((uint32_t)cells);  // `cells` itself fits: the sentinel
    const int t = threadIdx.x;
    uint32_t* sorted = wsn + lay.sorted;
    uint32_t* cell_start = wsn + lay.cell_start;

    // keys (cell << kPointBits | point)
    uint32_t keys[IPT];
#pragma unroll
    for (int i = 0; i < IPT; i++) {
        const int32_t pt = t * IPT + i;
        keys[i] = kNoCell;
        if (pt < points) {
            GradTaps<T, 0> tp;
            const int64_t idx = n * points + pt;
            decide_grad_taps<T, 0>(tp, ElemIO<T>::load(grid + 2 * idx), ElemIO<T>::load(grid + 2 * idx + 1), p.H, p.W,
                                   p.pad, p.align);
            if (tp.x0 >= -1 && tp.x0 < p.W && tp.y0 >= -1 && tp.y0 < p.H) {
                const uint32_t cell = (uint32_t)(tp.y0 + 1) * (uint32_t)(p.W + 1) + (uint32_t)(tp.x0 + 1);
                keys[i] = (cell << kPointBits) | (uint32_t)pt;
            }
        }
    }
    // The keys enter in ascending point order (a thread's points, and thread after thread) and the radix sort is
    // stable, so sorting by the cell field alone leaves the points of a cell ascending; kNoCell (all ones in the sorted
    // bits, more than any cell) comes last.
    sort_t().sort(keys, sort_storage, kPointBits, kPointBits + cell_bits);
#pragma unroll
    for (int i = 0; i < IPT; i++) {
        sorted_lds[t * IPT + i] = keys[i];
        sorted[t * IPT + i] = keys[i];
    }
    __syncthreads();

    // where every cell's run starts: the first position whose key is not below the cell's (a binary search per cell,
    // cells shared out among the threads; a thread that walked from its key's predecessor to its key would cross
    // thousands of empty cells alone where the grid leaves part of the image untouched)
    constexpr uint32_t total = kSortThreads * IPT;
    for (int32_t c = t; c <= cells; c += kSortThreads) {
        const uint32_t want = (uint32_t)c << kPointBits;
        uint32_t lo = 0, hi = total;
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (sorted_lds[mid] < want) {
                lo = mid + 1;
            } else {
                hi = mid;
            }
        }
        cell_start[c] = lo;
    }
}

// One lane per grid point (workgroups of kSortThreads points, `blocks_per_item` of them per batch item): weights to
// scratch, a slot in the point's cell.  The workgroup of an item that finishes last sorts the item when one of its
// cells overflowed -- it knows that it is the last from a count of finished workgroups, it waits for nobody, and it
// reads nothing that the others wrote.
template <typename T, int IPT>
__global__ __launch_bounds__(kSortThreads) void gs2d_grad_csr_slots_kernel(const T* __restrict__ grid,
                                                                            uint32_t* __restrict__ ws, GradParams p,
                                                                            CsrLayout lay, uint32_t blocks_per_item)
{
    using sort_t = rocprim::block_radix_sort<uint32_t, kSortThreads, IPT>;
    __shared__ typename sort_t::storage_type sort_storage;
    __shared__ uint32_t sort_it;
    extern __shared__ uint32_t sorted_lds[];  // kSortThreads * IPT keys
    const int32_t points = p.Ho * p.Wo;
    const uint32_t cells = (uint32_t)(p.H + 1) * (uint32_t)(p.W + 1);
    const int t = threadIdx.x;
    const int64_t n = blockIdx.x / blocks_per_item;
    const int32_t pt = (int32_t)(blockIdx.x % blocks_per_item) * kSortThreads + t;
    uint32_t* wsn = ws + (size_t)n * lay.item_words;
    uint32_t* flag = wsn + lay.slot_count + cells;
    uint32_t* finished = flag + 1;  // low half: workgroups of the item that are through; high half: those that flagged
    bool crowded = false;
    if (pt < points) {
        float* wts = reinterpret_cast<float*>(wsn + lay.wts);
        GradTaps<T, 0> tp;
        const int64_t idx = n * points + pt;
        decide_grad_taps<T, 0>(tp, ElemIO<T>::load(grid + 2 * idx), ElemIO<T>::load(grid + 2 * idx + 1), p.H, p.W,
                               p.pad, p.align);
        *reinterpret_cast<float4*>(wts + 4 * pt) = make_float4(tp.w[0], tp.w[1], tp.w[2], tp.w[3]);
        if (tp.x0 >= -1 && tp.x0 < p.W && tp.y0 >= -1 && tp.y0 < p.H) {
            const uint32_t cell = (uint32_t)(tp.y0 + 1) * (uint32_t)(p.W + 1) + (uint32_t)(tp.x0 + 1);
            const uint32_t r = atomicAdd(&wsn[lay.slot_count + cell], 1u);
            if (r < (uint32_t)kRun) {
                wsn[lay.slots + cell * (uint32_t)kRun + r] = (uint32_t)pt;
            } else {
                crowded = true;  // the item is to be sorted
            }
        }
    }
    // The workgroup counts itself as finished, and in the same atomic says whether one of its points found its cell
    // full: the workgroup that counts last has the flags of all the others in what the atomic returns.
    const int any = __syncthreads_or(crowded ? 1 : 0);
    if (t == 0) {
        const uint32_t before = atomicAdd(finished, 1u + ((uint32_t)any << 16));
        const bool last = (before & 0xFFFFu) == blocks_per_item - 1u;
        const bool sort = last && ((before >> 16) != 0u || any != 0);
        if (sort) {
            *flag = 1u;  // for the kernel that makes the lists
        }
        sort_it = sort ? 1u : 0u;
    }
    __syncthreads();
    if (sort_it != 0u) {
        sort_item<T, IPT>(grid, wsn, p, lay, n, sort_storage, sorted_lds);
    }
}

__device__ __forceinline__ uint2 pair_of(uint32_t pt, uint32_t corner, const float* wts)
{
    return make_uint2(pt, __builtin_bit_cast(uint32_t, wts[4u * pt + corner]));
}

__global__ __launch_bounds__(kListThreads) void gs2d_grad_csr_lists_kernel(uint32_t* __restrict__ ws, int32_t H,
                                                                            int32_t W, uint32_t tiles, CsrLayout lay)
{
    const int64_t n = blockIdx.x / tiles;
    const int32_t e = (int32_t)(blockIdx.x % tiles) * kListThreads + (int32_t)threadIdx.x;
    if (e >= H * W) {
        return;
    }
    uint32_t* wsn = ws + (size_t)n * lay.item_words;
    const float* wts = reinterpret_cast<const float*>(wsn + lay.wts);
    const uint32_t* sorted = wsn + lay.sorted;
    const uint32_t* cell_start = wsn + lay.cell_start;
    uint2* held = reinterpret_cast<uint2*>(wsn + lay.held) + (size_t)e * kHeld;
    uint2* more = reinterpret_cast<uint2*>(wsn + lay.more);

    const uint32_t y = (uint32_t)(e / W), x = (uint32_t)(e - (int32_t)y * W);
    const uint32_t w1 = (uint32_t)(W + 1);
    uint32_t cid[4], cur[4], end[4];
    cid[0] = (y + 1u) * w1 + (x + 1u);  // nw corner of the points of cell (y, x)
    cid[1] = (y + 1u) * w1 + x;         // ne corner of cell (y, x - 1)
    cid[2] = y * w1 + (x + 1u);         // sw corner of cell (y - 1, x)
    cid[3] = y * w1 + x;                // se corner of cell (y - 1, x - 1)
    // the points of a cell: its slots, or, in an item where some cell overflowed its slots, its run in the sorted keys
    const uint32_t cells = (uint32_t)(H + 1) * w1;
    // One round of loads for the usual case: the item's flag, the four cells' counts and, unasked, the first two slots
    // of every cell (a cell of a smooth grid holds a point or two) -- not flag, then counts, then slots, each waiting
    // for the one before.
    const uint32_t flag = wsn[lay.slot_count + cells];
    uint32_t slot_cnt[4];
    uint2 first_two[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        slot_cnt[k] = wsn[lay.slot_count + cid[k]];
        first_two[k] = *reinterpret_cast<const uint2*>(wsn + lay.slots + cid[k] * (uint32_t)kRun);
    }
    const bool from_runs = flag != 0u;
    const uint32_t* source = from_runs ? sorted : wsn + lay.slots;
    uint32_t cnt = 0;
    bool crowded = false;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        if (from_runs) {
            cur[k] = cell_start[cid[k]];
            end[k] = cell_start[cid[k] + 1];
        } else {
            cur[k] = cid[k] * (uint32_t)kRun;
            end[k] = cur[k] + slot_cnt[k];
        }
        cnt += end[k] - cur[k];
        crowded = crowded || end[k] - cur[k] > (uint32_t)kRun;
    }
    wsn[lay.count + (uint32_t)e] = cnt;
    uint32_t more_at = 0;
    if (cnt > (uint32_t)kHeld) {
        // the order in which elements get their place does not matter: nothing depends on where a list lies
        more_at = atomicAdd(&wsn[lay.more_used], cnt - (uint32_t)kHeld);
        wsn[lay.more_start + (uint32_t)e] = more_at;
    }
    auto put = [&](uint32_t i, uint32_t pt, uint32_t corner) {
        const uint2 v = pair_of(pt, corner, wts);
        if (i < (uint32_t)kHeld) {
            held[i] = v;
        } else {
            more[more_at + i - (uint32_t)kHeld] = v;
        }
    };
    if (!crowded) {
        // all candidates at once (independent loads), keyed (chunk, corner, point), sorted by a bitonic network.  The
        // network takes R candidates from each of the four cells; R is the smallest of 2, 4 and 8 that covers the
        // fullest cell of any lane of the wavefront (a cell of a smooth grid holds a point or two: 8 loads and a
        // network of 8 keys instead of 32 and 32).
        auto sort_and_put = [&](auto r_tag) {
            constexpr int R = decltype(r_tag)::value;
            uint32_t key[4 * R];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t len = end[k] - cur[k];
#pragma unroll
                for (int i = 0; i < R; i++) {
                    const bool valid = (uint32_t)i < len;
                    uint32_t pt;
                    if (R == 2 && !from_runs) {
                        pt = (i == 0 ? first_two[k].x : first_two[k].y) & kPointMask;  // already here
                    } else {
                        pt = source[valid ? cur[k] + (uint32_t)i : 0u] & kPointMask;
                    }
                    key[k * R + i] = valid ? (((pt >> kChunkShift) << (kPointBits + 2)) | ((uint32_t)k << kPointBits) | pt)
                                           : 0xFFFFFFFFu;
                }
            }
#pragma unroll
            for (int size = 2; size <= 4 * R; size *= 2) {
#pragma unroll
                for (int stride = size / 2; stride > 0; stride /= 2) {
#pragma unroll
                    for (int i = 0; i < 4 * R; i++) {
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
            for (int i = 0; i < 4 * R; i++) {
                if ((uint32_t)i < cnt) {
                    put((uint32_t)i, key[i] & kPointMask, (key[i] >> kPointBits) & 3u);
                }
            }
        };
        uint32_t fullest = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            fullest = (end[k] - cur[k] > fullest) ? end[k] - cur[k] : fullest;
        }
        static_assert(kRun == 8, "the three sizes below end at a cell's eight slots");
        if (__builtin_amdgcn_ballot_w64(fullest > 4u) != 0) {
            sort_and_put(std::integral_constant<int, 8>{});
        } else if (__builtin_amdgcn_ballot_w64(fullest > 2u) != 0) {
            sort_and_put(std::integral_constant<int, 4>{});
        } else {
            sort_and_put(std::integral_constant<int, 2>{});
        }
        return;
    }
    // a run longer than the network takes (only in an item that went through the sort): chunk by chunk, corner by
    // corner, with a cursor into every run
    uint32_t i = 0;
    for (;;) {
        uint32_t chunk = 0xFFFFFFFFu;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            if (cur[k] < end[k]) {
                const uint32_t c = (sorted[cur[k]] & kPointMask) >> kChunkShift;
                chunk = c < chunk ? c : chunk;
            }
        }
        if (chunk == 0xFFFFFFFFu) {
            break;
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            while (cur[k] < end[k]) {
                const uint32_t pt = sorted[cur[k]] & kPointMask;
                if ((pt >> kChunkShift) != chunk) {
                    break;
                }
                put(i++, pt, (uint32_t)k);
                cur[k]++;
            }
        }
    }
}

// One more contribution: gradOutput times weight rounded to fp32 and then to the element type, added to the sum with
// a rounding to the element type (grid_sampler2_d_grad_simt_det.h:75-101).
//   fp16: weight and gradOutput are fp16 values, their exact product has 22 significant bits and so is exact in fp32;
//     rounding it to fp16 is the fp16 product.  The fp32 sum of two fp16 values rounded to fp16 is the fp16 sum (24
//     bits are 2 x 11 + 2: the double rounding cannot differ).  So the sum lives in an fp16 register and a
//     contribution is one fp16 multiply and one fp16 add, with the same results bit for bit.
//   bf16 has no such instructions, fp32 needs no rounding steps: the generic form, the fp32 product pinned so that the
//     compiler cannot merge product and conversion into one instruction that rounds once.
template <typename T>
struct Fold {
    typedef float acc_t;
    static __device__ __forceinline__ acc_t zero() { return 0.0f; }
    static __device__ __forceinline__ acc_t weight(float w) { return w; }
    static __device__ __forceinline__ acc_t add(acc_t acc, uint32_t go_bits, acc_t w)
    {
        return rt<T>(acc + rt<T>(as_fp32_value(w * tap_value<T>(go_bits))));
    }
    static __device__ __forceinline__ void store(T* p, acc_t acc)
    {
        T v;
        ElemIO<T>::store(&v, acc);
        __builtin_nontemporal_store(v, p);  // the gradient streams out: written once, not read again by this kernel
    }
};
template <>
struct Fold<_Float16> {
    typedef _Float16 acc_t;
    static __device__ __forceinline__ acc_t zero() { return (_Float16)0.0f; }
    static __device__ __forceinline__ acc_t weight(float w) { return (_Float16)w; }  // exact: the weight is an fp16 value
    static __device__ __forceinline__ acc_t add(acc_t acc, uint32_t go_bits, acc_t w)
    {
        const _Float16 val = w * __builtin_bit_cast(_Float16, (uint16_t)go_bits);
        return acc + val;
    }
    static __device__ __forceinline__ void store(_Float16* p, acc_t acc) { __builtin_nontemporal_store(acc, p); }
    // two channels at once: the same two operations as packed fp16 instructions (each half rounds on its own)
    typedef _Float16 pair_t __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ pair_t add2(pair_t acc, uint32_t go_lo, uint32_t go_hi, acc_t w)
    {
        const pair_t go = {__builtin_bit_cast(_Float16, (uint16_t)go_lo), __builtin_bit_cast(_Float16, (uint16_t)go_hi)};
        const pair_t ww = {w, w};
        const pair_t val = ww * go;
        return acc + val;
    }
};

template <typename T, int CB, int EPL, bool PAIRS>
__global__ __launch_bounds__(PAIRS ? kPairThreads : kApplyThreads, PAIRS ? 6 : 1) void gs2d_grad_csr_apply_kernel(
    const T* __restrict__ gout, T* __restrict__ dx, const uint32_t* __restrict__ ws, GradParams p, CsrLayout lay,
    uint32_t tiles, uint32_t cblocks, int32_t chans_per_block, int32_t xcd_swizzle, uint32_t items_fastest,
    uint32_t wide_blocks, int32_t chans_wide, int32_t unit_stride)
{
    typedef Fold<T> F;
    typedef typename F::acc_t acc_t;
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    __shared__ uint32_t spill_used;
    const int tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)tid >> 6);
    const int32_t points = p.Ho * p.Wo;
    const int32_t plane_px = p.H * p.W;
    const uint32_t row_bytes = (uint32_t)points * (uint32_t)sizeof(T);  // one gradOutput plane
    const uint32_t buf_bytes = (uint32_t)CB * row_bytes;
    // Interleaved layout (PAIRS: 16-bit elements, two or four channels per step): a slot of LDS holds the planes of a
    // step interleaved -- point p is CB neighbouring 16-bit values, one per channel -- and 16 bytes of zeros behind
    // them.  One 4- or 8-byte LDS read then serves all channels of a contribution, and a contribution that a lane
    // does not have reads the zeros with weight 0: adding +0 changes no sum (a sum that starts at +0 is never -0), so
    // the rounds need no selects.  The copy engine cannot interleave, so the loaders go through registers.
    // fp16 N16 C256 64x64, this kernel: 29.7 us with the planes side by side (two per step), 25.4 with two interleaved.
    static_assert(!PAIRS || ((CB == 2 || CB == 4) && sizeof(T) == 2), "the interleaved layout is 16-bit planes");
    const uint32_t pair_pitch = buf_bytes + 16u;
    const uint32_t pair_zero = buf_bytes;  // offset of the zeros inside a slot
    uint2* spill = reinterpret_cast<uint2*>(lds + (PAIRS ? (uint32_t)kPairNbuf * pair_pitch
                                                         : (uint32_t)kApplyNbuf * buf_bytes));  // behind the ring

    // all element tiles of one (batch item, channel block) on one XCD: they stream the same gradOutput planes
    uint32_t group, tile;
    if (xcd_swizzle) {
        const uint32_t xcd = blockIdx.x & 7u, i = blockIdx.x >> 3;
        group = (i / tiles) * 8u + xcd;
        tile = i % tiles;
    } else {
        group = blockIdx.x / tiles;
        tile = blockIdx.x % tiles;
    }
    // groups numbered with the batch item fastest (`items_fastest` = N, else 0): an XCD then sees the lists of N / 8
    // items only, and the channel blocks with the low numbers are the workgroups handed out first
    const uint32_t cb = items_fastest ? group / items_fastest : group % cblocks;
    const int64_t n = items_fastest ? group % items_fastest : group / cblocks;
    // A step works on a unit of CB neighbouring channels.  Which units: a contiguous range, or -- `unit_stride` != 0,
    // every block's count exact -- units dealt out in turn, the first `wide_blocks` blocks taking `chans_wide`
    // channels each and the others `chans_per_block` (see gs2d_lds.hip for the why of both).  The block's s-th unit
    // is  first + s * step1  up to s = switch_at and step2 apart from there on.
    const bool wide = cb < wide_blocks;
    int32_t first, step1, step2, nchan;
    if (unit_stride != 0) {
        first = (int32_t)cb;
        step1 = unit_stride;
        step2 = (int32_t)wide_blocks;
        nchan = wide ? chans_wide : chans_per_block;
    } else {
        const int32_t c_begin = (int32_t)cb * chans_per_block;
        const int32_t c_end = (c_begin + chans_per_block < p.C) ? c_begin + chans_per_block : p.C;
        first = c_begin / CB;
        step1 = 1;
        step2 = 1;
        nchan = c_end - c_begin;
    }
    const int32_t switch_at = chans_per_block / CB;
    auto unit_of = [&](int32_t s) -> int32_t {
        return first + (s < switch_at ? s * step1 : switch_at * step1 + (s - switch_at) * step2);
    };
    const int32_t steps = (nchan + CB - 1) / CB;
    const T* go_n = gout + n * p.C * (int64_t)points;  // the batch item's gradOutput planes
    if (tid == 0) {
        spill_used = 0u;
    }

    if (wave >= (uint32_t)(kApplyLanes / 64)) {
        // ------------------------------------------------ loader wavefronts ------------------------------------
        // A ring of kApplyNbuf slots: with two, a group of planes was asked for when the one before it had landed, and
        // every step waited out a memory latency.  The copy loop is kept to a few instructions per KiB (a pointer that
        // advances, no bounds test except for a last partial KiB): one wavefront issuing a general copy routine
        // moved 16 KiB per microsecond, and the steps waited for that (43 us on fp16 N16 C256 64x64, where the
        // arithmetic needs a quarter).
        const uint32_t lwave = wave - (uint32_t)(kApplyLanes / 64);
        const uint32_t lane = (uint32_t)tid & 63u;
        if constexpr (PAIRS) {
            // Every lane takes UPL 16-byte units (eight points) of every plane of a step: CB loads per unit, the
            // halves interleaved, CB 16-byte LDS writes.  The loads of kPairDepth steps are on their way at any time;
            // they are issued on every path alike, those past the last step from one address all lanes share (one
            // cache line), so that the compiler's count of outstanding loads at every use is the same on all paths
            // and exact.  Slot s % 2 is written between the barriers of steps s - 1 and s, while the element lanes
            // read the other one.
            constexpr int UPL = kPairLoads / CB;
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            typedef u32x4 __attribute__((address_space(3))) * lds_u32x4_ptr_t;
            const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
            const uint32_t lid = lwave * 64u + lane;
            const uint32_t units = row_bytes >> 4;
            if (lid < (uint32_t)kPairNbuf) {
                *reinterpret_cast<lds_u32x4_ptr_t>((uintptr_t)(lds_base + lid * pair_pitch + pair_zero)) =
                    u32x4{0u, 0u, 0u, 0u};
            }
            uint32_t unit[UPL];
            bool mine[UPL];
#pragma unroll
            for (int u = 0; u < UPL; u++) {
                unit[u] = lid + (uint32_t)u * (64u * kPairLoaders);
                mine[u] = unit[u] < units;
                unit[u] = mine[u] ? unit[u] : units - 1u;  // a lane without a unit reads the last one again
            }
            const char* go_bytes = reinterpret_cast<const char*>(go_n);
            u32x4 regs[kPairDepth][UPL][CB];
            // A load that has nothing to fetch -- past the last step, or a plane that a last, partial step does not
            // have -- reads an address of its own near the start of the planes: were two of a lane's loads to ask for
            // the same address, the compiler would make the second a register copy of the first, and a copy waits
            // for its load (`s_waitcnt vmcnt(0)` behind the loads of every step, which is the end of the prefetch).
            auto issue = [&](u32x4 (*r)[CB], int32_t s) {
                const bool real = s < steps;
                const char* base = go_bytes + (real ? (size_t)unit_of(s) * buf_bytes : (size_t)0);
                const int32_t left = real ? nchan - s * CB : 0;
#pragma unroll
                for (int u = 0; u < UPL; u++) {
#pragma unroll
                    for (int j = 0; j < CB; j++) {
                        const uint32_t spare = (uint32_t)(u * CB + j) * 16u;
                        const uint32_t idle = spare < row_bytes ? spare : row_bytes - 16u;
                        const uint32_t off = (j < left) ? (uint32_t)j * row_bytes + unit[u] * 16u : idle;
                        r[u][j] = *reinterpret_cast<const u32x4*>(base + off);
                    }
                }
            };
            // the low halves of two dwords in one, and the high halves
            auto lows = [](uint32_t a, uint32_t b) -> uint32_t { return (a & 0xFFFFu) | (b << 16); };
            auto highs = [](uint32_t a, uint32_t b) -> uint32_t { return (a >> 16) | (b & 0xFFFF0000u); };
#pragma unroll
            for (int k = 0; k < kPairDepth; k++) {
                issue(regs[k], k);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the zeros are written
            lds_barrier();                                       // the element lanes' set-up barrier
            for (int32_t s0 = 0; s0 < steps; s0 += kPairDepth) {
#pragma unroll
                for (int k = 0; k < kPairDepth; k++) {
                    const int32_t s = s0 + k;
                    if (s < steps) {
                        const uint32_t slot = lds_base + ((uint32_t)s & 1u) * pair_pitch;
#pragma unroll
                        for (int u = 0; u < UPL; u++) {
                            if (mine[u]) {
                                const uint32_t at = slot + unit[u] * (16u * CB);
                                if constexpr (CB == 2) {
                                    const u32x4 a = regs[k][u][0], b = regs[k][u][1];
                                    const u32x4 lo = {lows(a.x, b.x), highs(a.x, b.x), lows(a.y, b.y), highs(a.y, b.y)};
                                    const u32x4 hi = {lows(a.z, b.z), highs(a.z, b.z), lows(a.w, b.w), highs(a.w, b.w)};
                                    *reinterpret_cast<lds_u32x4_ptr_t>((uintptr_t)at) = lo;
                                    *reinterpret_cast<lds_u32x4_ptr_t>((uintptr_t)(at + 16u)) = hi;
                                } else {
                                    const u32x4 a = regs[k][u][0], b = regs[k][u][1], c = regs[k][u][2],
                                                d = regs[k][u][3];
#pragma unroll
                                    for (int q = 0; q < 4; q++) {  // dword q of a plane: points 2q and 2q + 1
                                        const u32x4 two = {lows(a[q], b[q]), lows(c[q], d[q]), highs(a[q], b[q]),
                                                           highs(c[q], d[q])};
                                        *reinterpret_cast<lds_u32x4_ptr_t>((uintptr_t)(at + 16u * (uint32_t)q)) = two;
                                    }
                                }
                            }
                        }
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        lds_barrier();  // step s is in its slot, and the other slot has been read for the last time
                    }
                    issue(regs[k], s + kPairDepth);
                }
            }
            return;
        }
        auto bytes_of = [&](int32_t s) -> uint32_t {
            const int32_t left = nchan - s * CB;
            return (uint32_t)(left < CB ? left : CB) * row_bytes;  // the planes are neighbours in memory
        };
        // copy instructions this wavefront issues for a group of `bytes`: every kApplyLoaders-th KiB, the last one partial
        auto copies_of = [&](uint32_t bytes) -> uint32_t {
            const uint32_t kib = (bytes + 1023u) >> 10;
            return (kib > lwave) ? (kib - lwave + kApplyLoaders - 1) / kApplyLoaders : 0u;
        };
        const uint32_t copies_full = copies_of(buf_bytes);
        const char* src_lane = reinterpret_cast<const char*>(go_n) + lwave * 1024u + lane * 16u;
        int32_t issued = 0;
        auto issue_next = [&]() {
            const uint32_t bytes = bytes_of(issued);
            const char* src = src_lane + (size_t)unit_of(issued) * buf_bytes;
            char* dst = lds + (uint32_t)(issued % kApplyNbuf) * buf_bytes + lwave * 1024u;
            const uint32_t whole = bytes >> 10;
            uint32_t j = lwave;
            for (; j < whole; j += kApplyLoaders) {
                __builtin_amdgcn_global_load_lds((global_cptr_t)src, (lds_ptr_t)dst, 16, 0, 0);
                src += kApplyLoaders * 1024;
                dst += kApplyLoaders * 1024;
            }
            if ((bytes & 1023u) != 0u && j == whole) {
                if (lane * 16u < (bytes & 1023u)) {
                    __builtin_amdgcn_global_load_lds((global_cptr_t)src, (lds_ptr_t)dst, 16, 0, 0);
                }
            }
            issued++;
        };
        while (issued < kApplyNbuf - 1 && issued < steps) {
            issue_next();
        }
        lds_barrier();  // the element lanes' set-up barrier
        for (int32_t s = 0; s < steps; s++) {
            // the planes of step s have landed when at most the copies of the groups after it are out
            uint32_t later = 0;
            for (int32_t q = s + 1; q < issued; q++) {
                later += (q == steps - 1) ? copies_of(bytes_of(q)) : copies_full;
            }
            wait_vmcnt(later);
            lds_barrier();  // ... and the slot of step s - 1 has been read for the last time
            if (issued < steps) {
                issue_next();
            }
        }
        return;
    }

    // ---------------------------------------------------- element lanes ----------------------------------------
    // A lane owns EPL elements, kApplyLanes apart (a workgroup's tile is EPL * kApplyLanes elements): with two, every
    // gradOutput plane is staged by half as many workgroups, and the copies into LDS run at the rate the L2s deliver
    // (268 MB in all for fp16 N16 C256 64x64 with one element per lane, 12 of the kernel's 34 us).
    const uint32_t* wsn = ws + (size_t)n * lay.item_words;
    int32_t e[EPL];
    bool live[EPL];
    uint32_t cnt[EPL];
    uint32_t hoff[EPL][kHeld];  // byte offset of the point inside a gradOutput plane
    acc_t hw[EPL][kHeld];
#pragma unroll
    for (int i = 0; i < EPL; i++) {
        e[i] = ((int32_t)tile * EPL + i) * kApplyLanes + tid;
        live[i] = e[i] < plane_px;
        cnt[i] = live[i] ? wsn[lay.count + (uint32_t)e[i]] : 0u;
    }
#pragma unroll
    for (int i = 0; i < EPL; i++) {
        const uint4* slot = reinterpret_cast<const uint4*>(wsn + lay.held) + (size_t)(live[i] ? e[i] : 0) * (kHeld / 2);
        uint4 raw[kHeld / 2];
#pragma unroll
        for (int k = 0; k < kHeld / 2; k++) {
            raw[k] = slot[k];
        }
#pragma unroll
        for (int k = 0; k < kHeld / 2; k++) {
            const bool a = (uint32_t)(2 * k) < cnt[i], b = (uint32_t)(2 * k + 1) < cnt[i];
            constexpr uint32_t point_bytes = PAIRS ? (uint32_t)(2 * CB) : (uint32_t)sizeof(T);
            const uint32_t none = PAIRS ? pair_zero : 0u;
            hoff[i][2 * k] = a ? raw[k].x * point_bytes : none;
            hw[i][2 * k] = F::weight(a ? __builtin_bit_cast(float, raw[k].y) : 0.0f);
            hoff[i][2 * k + 1] = b ? raw[k].z * point_bytes : none;
            hw[i][2 * k + 1] = F::weight(b ? __builtin_bit_cast(float, raw[k].w) : 0.0f);
        }
    }
    __syncthreads();  // spill_used is zero
    // contributions beyond the held ones: a place in LDS while there is room, else they stay in scratch memory
    const uint2* rest[EPL];  // where the lane reads them in every step
    bool rest_in_lds[EPL];
    uint32_t rest_at[EPL];
    uint32_t kmax[EPL];
    bool any_rest[EPL];
#pragma unroll
    for (int i = 0; i < EPL; i++) {
        rest[i] = nullptr;
        rest_in_lds[i] = false;
        rest_at[i] = 0;
        if (cnt[i] > (uint32_t)kHeld) {
            const uint32_t extra = cnt[i] - (uint32_t)kHeld;
            const uint2* src = reinterpret_cast<const uint2*>(wsn + lay.more) + wsn[lay.more_start + (uint32_t)e[i]];
            rest[i] = src;
            rest_at[i] = atomicAdd(&spill_used, extra);
            if (rest_at[i] + extra <= (uint32_t)kApplySpill) {
                rest_in_lds[i] = true;
                for (uint32_t k = 0; k < extra; k++) {
                    spill[rest_at[i] + k] = src[k];
                }
            }
        }
        // the longest held list of the wavefront decides how many rounds its lanes run
        uint32_t km = cnt[i] < (uint32_t)kHeld ? cnt[i] : (uint32_t)kHeld;
        uint32_t cm = cnt[i];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const uint32_t other = (uint32_t)__shfl_xor((int)km, o);
            km = other > km ? other : km;
            const uint32_t other2 = (uint32_t)__shfl_xor((int)cm, o);
            cm = other2 > cm ? other2 : cm;
        }
        kmax[i] = __builtin_amdgcn_readfirstlane(km);
        any_rest[i] = (uint32_t)__builtin_amdgcn_readfirstlane(cm) > (uint32_t)kHeld;
    }
    T* dx_n = dx + n * p.C * (int64_t)plane_px;  // the batch item's gradient planes
    // the lists are in registers or LDS from here on: nothing below waits for memory except an overfull spill area
    __builtin_amdgcn_s_waitcnt(0);

    typedef typename std::conditional<sizeof(T) == 2, uint16_t, uint32_t>::type bits_t;
    typedef const bits_t __attribute__((address_space(3))) * lds_bits_ptr_t;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
    auto go_at = [&](uint32_t off) -> uint32_t {
        return (uint32_t)*reinterpret_cast<lds_bits_ptr_t>((uintptr_t)(lds_base + off));
    };
    // all channels of a point in the interleaved layout: CB / 2 dwords
    typedef uint32_t group_t __attribute__((ext_vector_type(CB >= 2 ? CB / 2 : 1)));
    typedef const group_t __attribute__((address_space(3))) * lds_group_ptr_t;
    auto group_at = [&](uint32_t off) -> group_t {
        return *reinterpret_cast<lds_group_ptr_t>((uintptr_t)(lds_base + off));
    };
    auto dword_of = [](const group_t& g, int j) -> uint32_t { return g[CB >= 4 ? j : 0]; };
    // R rounds of one step for one of the lane's elements, straight-line: all gradOutput values first (raw bits, so
    // that nothing waits between the reads), then the sums in list order; a lane whose list is shorter keeps its sum
    // (a select, not arithmetic: a value read for a contribution that does not exist may be anything)
    auto rounds = [&](auto r_tag, uint32_t buf_off, const uint32_t* ho, const acc_t* w, uint32_t count, acc_t* acc) {
        constexpr int R = decltype(r_tag)::value;
        if constexpr (PAIRS) {
            // one read per contribution; a contribution the lane does not have is zeros times weight 0
            (void)count;
            group_t got[R];
#pragma unroll
            for (int k = 0; k < R; k++) {
                got[k] = group_at(buf_off + ho[k]);
            }
            if constexpr (std::is_same<T, _Float16>::value) {
                typename F::pair_t acc2[CB / 2];
#pragma unroll
                for (int j = 0; j < CB / 2; j++) {
                    acc2[j] = typename F::pair_t{acc[2 * j], acc[2 * j + 1]};
                }
#pragma unroll
                for (int k = 0; k < R; k++) {
                    const typename F::pair_t ww = {w[k], w[k]};
#pragma unroll
                    for (int j = 0; j < CB / 2; j++) {
                        const typename F::pair_t val = ww * __builtin_bit_cast(typename F::pair_t, dword_of(got[k], j));
                        acc2[j] = acc2[j] + val;
                    }
                }
#pragma unroll
                for (int j = 0; j < CB / 2; j++) {
                    acc[2 * j] = acc2[j].x;
                    acc[2 * j + 1] = acc2[j].y;
                }
            } else {
#pragma unroll
                for (int k = 0; k < R; k++) {
#pragma unroll
                    for (int j = 0; j < CB / 2; j++) {
                        const uint32_t two = dword_of(got[k], j);
                        acc[2 * j] = F::add(acc[2 * j], two & 0xFFFFu, w[k]);
                        acc[2 * j + 1] = F::add(acc[2 * j + 1], two >> 16, w[k]);
                    }
                }
            }
            return;
        }
        uint32_t raw[R][CB];
#pragma unroll
        for (int k = 0; k < R; k++) {
#pragma unroll
            for (int j = 0; j < CB; j++) {
                raw[k][j] = go_at(buf_off + (uint32_t)j * row_bytes + ho[k]);
            }
        }
        if constexpr (std::is_same<T, _Float16>::value && CB % 2 == 0) {
            typename F::pair_t acc2[CB / 2];
#pragma unroll
            for (int j = 0; j < CB / 2; j++) {
                acc2[j] = typename F::pair_t{acc[2 * j], acc[2 * j + 1]};
            }
#pragma unroll
            for (int k = 0; k < R; k++) {
                const bool mine = (uint32_t)k < count;
#pragma unroll
                for (int j = 0; j < CB / 2; j++) {
                    const typename F::pair_t next = F::add2(acc2[j], raw[k][2 * j], raw[k][2 * j + 1], w[k]);
                    acc2[j] = mine ? next : acc2[j];
                }
            }
#pragma unroll
            for (int j = 0; j < CB / 2; j++) {
                acc[2 * j] = acc2[j].x;
                acc[2 * j + 1] = acc2[j].y;
            }
        } else {
#pragma unroll
            for (int k = 0; k < R; k++) {
                const bool mine = (uint32_t)k < count;
#pragma unroll
                for (int j = 0; j < CB; j++) {
                    const acc_t next = F::add(acc[j], raw[k][j], w[k]);
                    acc[j] = mine ? next : acc[j];
                }
            }
        }
    };

    for (int32_t s = 0; s < steps; s++) {
        lds_barrier();  // the planes of step s have landed
        const uint32_t buf_off = PAIRS ? ((uint32_t)s & 1u) * pair_pitch : (uint32_t)(s % kApplyNbuf) * buf_bytes;
#pragma unroll
        for (int i = 0; i < EPL; i++) {
            acc_t acc[CB];
#pragma unroll
            for (int j = 0; j < CB; j++) {
                acc[j] = F::zero();
            }
            switch (kmax[i]) {
                case 0: break;
                case 1: rounds(std::integral_constant<int, 1>{}, buf_off, hoff[i], hw[i], cnt[i], acc); break;
                case 2: rounds(std::integral_constant<int, 2>{}, buf_off, hoff[i], hw[i], cnt[i], acc); break;
                case 3: rounds(std::integral_constant<int, 3>{}, buf_off, hoff[i], hw[i], cnt[i], acc); break;
                case 4: rounds(std::integral_constant<int, 4>{}, buf_off, hoff[i], hw[i], cnt[i], acc); break;
                case 5: rounds(std::integral_constant<int, 5>{}, buf_off, hoff[i], hw[i], cnt[i], acc); break;
                case 6: rounds(std::integral_constant<int, 6>{}, buf_off, hoff[i], hw[i], cnt[i], acc); break;
                case 7: rounds(std::integral_constant<int, 7>{}, buf_off, hoff[i], hw[i], cnt[i], acc); break;
                default: rounds(std::integral_constant<int, 8>{}, buf_off, hoff[i], hw[i], cnt[i], acc); break;
            }
            if (any_rest[i] && cnt[i] > (uint32_t)kHeld) {
                for (uint32_t k = 0; k < cnt[i] - (uint32_t)kHeld; k++) {
                    const uint2 v = rest_in_lds[i] ? spill[rest_at[i] + k] : rest[i][k];
                    const acc_t w = F::weight(__builtin_bit_cast(float, v.y));
                    if constexpr (PAIRS) {
                        const group_t got = group_at(buf_off + v.x * (uint32_t)(2 * CB));
#pragma unroll
                        for (int j = 0; j < CB / 2; j++) {
                            const uint32_t two = dword_of(got, j);
                            acc[2 * j] = F::add(acc[2 * j], two & 0xFFFFu, w);
                            acc[2 * j + 1] = F::add(acc[2 * j + 1], two >> 16, w);
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < CB; j++) {
                            acc[j] = F::add(acc[j],
                                            go_at(buf_off + (uint32_t)j * row_bytes + v.x * (uint32_t)sizeof(T)), w);
                        }
                    }
                }
            }
            if (live[i]) {
#pragma unroll
                for (int j = 0; j < CB; j++) {
                    if (s * CB + j < nchan) {
                        F::store(dx_n + (int64_t)(unit_of(s) * CB + j) * plane_px + e[i], acc[j]);
                    }
                }
            }
        }
    }
}

struct CsrPlan {
    bool ok = false;
    int ipt = 1;
    int cb = 1;
    int epl = 1;  // elements per lane of the apply kernel
    bool pairs = false;  // the apply kernel's paired layout
    uint32_t tiles = 0, cblocks = 0;
    int32_t chans_per_block = 0;
    int xcd_swizzle = 0;
    uint32_t items_fastest = 0;  // N when the apply kernel numbers its groups with the batch item fastest
    uint32_t wide_blocks = 0;    // the first channel blocks take chans_wide channels each ...
    int32_t chans_wide = 0;
    int32_t unit_stride = 0;     // ... and units of cb channels are dealt out in turn, this many apart
    CsrLayout lay;
};

CsrPlan make_plan(const GridSamplerGradArgs& a)
{
    CsrPlan pl;
    const int64_t esz = elem_size(a.elem);
    const int64_t points = a.Hout * a.Wout, plane_px = a.Hin * a.Win;
    const int64_t cells = (a.Hin + 1) * (a.Win + 1);
    // what the kernels assume: the sort holds an item's points in one workgroup, a gradOutput plane is whole 16-byte
    // units on 16-byte boundaries and fits a slot of the ring
    if (a.interp != 0 || points > (int64_t)kSortThreads * kMaxIpt || cells > kMaxCells || (points * esz) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(a.gout) % 16 != 0 || points * esz > 2 * kApplyBufBytes / kApplyNbuf) {
        return pl;
    }
    // worth three extra kernels only with channels to share the lists among
    if (a.C < 8 || a.N * a.C > INT32_MAX || a.N > 65535) {  // the clear kernel indexes items by blockIdx.y
        return pl;
    }
    pl.ipt = 1;
    while ((int64_t)kSortThreads * pl.ipt < points) {
        pl.ipt *= 2;
    }
    pl.cb = 4;
    while (pl.cb > 1 && (int64_t)kApplyNbuf * pl.cb * points * esz > kApplyBufBytes) {
        pl.cb /= 2;
    }
    // the interleaved layout: 16-bit elements, four channels per step for planes of up to 8 KiB and two for planes of
    // up to 16 KiB (what the loaders' lanes cover with kPairLoads loads each; two slots of LDS either way)
    if (esz == 2 && points * esz <= 16 * 64 * kPairLoaders * (kPairLoads / 2)) {
        pl.pairs = true;
        pl.cb = (points * esz <= 16 * 64 * kPairLoaders * (kPairLoads / 4)) ? 4 : 2;
    }
    // two elements per lane where that still leaves workgroups for every CU
    pl.epl = (plane_px >= 2 * kApplyLanes && a.N * ((plane_px + 2 * kApplyLanes - 1) / (2 * kApplyLanes)) *
                                                      ((a.C + pl.cb - 1) / pl.cb) >= 512)
                 ? 2
                 : 1;
    pl.tiles = (uint32_t)((plane_px + kApplyLanes * pl.epl - 1) / (kApplyLanes * pl.epl));
    // channel blocks: about two workgroups per CU, whole groups of planes each
    const int64_t base = a.N * pl.tiles;
    int64_t cblocks = (512 + base - 1) / base;
    const int64_t max_cblocks = (a.C + pl.cb - 1) / pl.cb;
    cblocks = cblocks > max_cblocks ? max_cblocks : cblocks;
    int64_t cpb = (a.C + cblocks - 1) / cblocks;
    cpb = (cpb + pl.cb - 1) / pl.cb * pl.cb;
    cblocks = (a.C + cpb - 1) / cpb;
    const int64_t list_tiles = (plane_px + kListThreads - 1) / kListThreads;
    if (base * cblocks > INT32_MAX || a.N * list_tiles > INT32_MAX ||
        a.N * ((points + kSortThreads - 1) / kSortThreads) > INT32_MAX) {
        return pl;
    }
    pl.chans_per_block = (int32_t)cpb;
    pl.cblocks = (uint32_t)cblocks;
    pl.xcd_swizzle = ((a.N * cblocks) % 8 == 0) ? 1 : 0;
    // The apply kernel numbers its groups with the batch item fastest where the items fill the XCDs evenly: an XCD then
    // reads the lists of N / 8 items only (with the channel block fastest every XCD read every item's lists), and the
    // channel blocks with the low numbers are the workgroups that are handed out first.
    if (a.N % 8 == 0) {
        pl.items_fastest = (uint32_t)a.N;
    }
    // Units of cb channels dealt out to the channel blocks in turn where every block's count is exact, and, with
    // exactly two workgroups per CU, 5 channels for the first of a CU for every 3 of the second (gs2d_lds.hip has the
    // why; backward of fp16 N16 C256 64x64, both gradients: 77.0 us with 32 + 32, 75.6 with 36 + 28, 74.9 with 38 + 26
    // and 40 + 24, 75.7 with 42 + 22, 76.7 with 44 + 20).
    if (a.C == cblocks * cpb && cblocks > 1) {
        const int64_t wide = (cpb * 5 / 4) / pl.cb * pl.cb;
        if (pl.items_fastest != 0 && cblocks % 2 == 0 && base * cblocks == 2 * (int64_t)compute_unit_count() &&
            (a.N * cblocks / 2) % 8 == 0 && wide > cpb && wide < 2 * cpb) {
            pl.wide_blocks = (uint32_t)(cblocks / 2);
            pl.chans_wide = (int32_t)wide;
            pl.chans_per_block = (int32_t)(2 * cpb - wide);
        }
        pl.unit_stride = (int32_t)cblocks;
    }
    pl.lay = make_layout(points, plane_px, cells, pl.ipt);
    pl.ok = true;
    return pl;
}

template <typename T, int IPT>
hipError_t launch_slots(const GridSamplerGradArgs& a, const CsrPlan& pl, const GradParams& p, hipStream_t stream)
{
    static std::atomic<uint32_t> lds_allowed{0};  // sixteen keys per thread take 64 KB beside the sort's own storage
    const hipError_t ea = allow_dynamic_lds(reinterpret_cast<const void*>(gs2d_grad_csr_slots_kernel<T, IPT>),
                                            kSortThreads * IPT * 4, lds_allowed);
    if (ea != hipSuccess) {
        return ea;
    }
    const int64_t blocks_per_item = (a.Hout * a.Wout + kSortThreads - 1) / kSortThreads;
    hipLaunchKernelGGL((gs2d_grad_csr_slots_kernel<T, IPT>), dim3((unsigned)(a.N * blocks_per_item)),
                       dim3(kSortThreads), kSortThreads * IPT * 4, stream, (const T*)a.grid, (uint32_t*)a.scratch, p,
                       pl.lay, (uint32_t)blocks_per_item);
    return hipGetLastError();
}

GradClear clear_of(const GridSamplerGradArgs& a, const CsrPlan& pl)
{
    GradClear c{};
    c.base = (uint32_t*)a.scratch;
    c.item_words = pl.lay.item_words;
    c.first = pl.lay.slot_count;
    c.count = (uint32_t)((a.Hin + 1) * (a.Win + 1)) + 2u;  // the counts, the flag, the count of finished workgroups
    c.single = pl.lay.more_used;
    return c;
}

template <typename T, int CB, int EPL, bool PAIRS = false>
hipError_t launch_apply(const GridSamplerGradArgs& a, const CsrPlan& pl, const GradParams& p, hipStream_t stream)
{
    auto kernel = gs2d_grad_csr_apply_kernel<T, CB, EPL, PAIRS>;
    constexpr int kLdsMax = 2 * kApplyBufBytes + kApplySpill * 8;
    static std::atomic<uint32_t> lds_allowed{0};
    const hipError_t ea = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLdsMax, lds_allowed);
    if (ea != hipSuccess) {
        return ea;
    }
    const uint32_t blocks = (uint32_t)(a.N * pl.tiles * pl.cblocks);
    const int plane_bytes = (int)(a.Hout * a.Wout) * (int)sizeof(T);
    const int lds_bytes = (PAIRS ? kPairNbuf * (CB * plane_bytes + 16) : kApplyNbuf * CB * plane_bytes) + kApplySpill * 8;
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(PAIRS ? kPairThreads : kApplyThreads), lds_bytes, stream, (const T*)a.gout, (T*)a.dx,
                       (const uint32_t*)a.scratch, p, pl.lay, pl.tiles, pl.cblocks, pl.chans_per_block, pl.xcd_swizzle,
                       pl.items_fastest, pl.wide_blocks, pl.chans_wide, pl.unit_stride);
    return hipGetLastError();
}

template <typename T>
hipError_t run_typed(const GridSamplerGradArgs& a, const CsrPlan& pl, bool cleared, hipStream_t stream)
{
    GradParams p{};
    p.C = (int32_t)a.C;
    p.H = (int32_t)a.Hin;
    p.W = (int32_t)a.Win;
    p.Ho = (int32_t)a.Hout;
    p.Wo = (int32_t)a.Wout;
    p.pad = a.pad;
    p.align = a.align;
    hipError_t e = hipSuccess;
    if (!cleared) {
        const GradClear c = clear_of(a, pl);
        hipLaunchKernelGGL(gs2d_grad_csr_clear_kernel, dim3((c.count + 255u) / 256u, (unsigned)a.N), dim3(256), 0, stream,
                           c);
        e = hipGetLastError();
        if (e != hipSuccess) {
            return e;
        }
    }
    e = hipErrorInvalidValue;
    switch (pl.ipt) {
        case 1: e = launch_slots<T, 1>(a, pl, p, stream); break;
        case 2: e = launch_slots<T, 2>(a, pl, p, stream); break;
        case 4: e = launch_slots<T, 4>(a, pl, p, stream); break;
        case 8: e = launch_slots<T, 8>(a, pl, p, stream); break;
        case 16: e = launch_slots<T, 16>(a, pl, p, stream); break;
        default: break;
    }
    if (e != hipSuccess) {
        return e;
    }
    const uint32_t list_tiles = (uint32_t)((a.Hin * a.Win + kListThreads - 1) / kListThreads);
    hipLaunchKernelGGL(gs2d_grad_csr_lists_kernel, dim3((unsigned)(a.N * list_tiles)), dim3(kListThreads), 0, stream,
                       (uint32_t*)a.scratch, (int32_t)a.Hin, (int32_t)a.Win, list_tiles, pl.lay);
    e = hipGetLastError();
    if (e != hipSuccess) {
        return e;
    }
    if constexpr (sizeof(T) == 2) {
        if (pl.pairs) {
            switch (pl.cb * 4 + pl.epl) {
                case 4 * 4 + 1: return launch_apply<T, 4, 1, true>(a, pl, p, stream);
                case 4 * 4 + 2: return launch_apply<T, 4, 2, true>(a, pl, p, stream);
                case 2 * 4 + 1: return launch_apply<T, 2, 1, true>(a, pl, p, stream);
                case 2 * 4 + 2: return launch_apply<T, 2, 2, true>(a, pl, p, stream);
                default: return hipErrorInvalidValue;
            }
        }
    }
    switch (pl.cb * 4 + pl.epl) {
        case 4 * 4 + 1: return launch_apply<T, 4, 1>(a, pl, p, stream);
        case 4 * 4 + 2: return launch_apply<T, 4, 2>(a, pl, p, stream);
        case 2 * 4 + 1: return launch_apply<T, 2, 1>(a, pl, p, stream);
        case 2 * 4 + 2: return launch_apply<T, 2, 2>(a, pl, p, stream);
        case 1 * 4 + 1: return launch_apply<T, 1, 1>(a, pl, p, stream);
        case 1 * 4 + 2: return launch_apply<T, 1, 2>(a, pl, p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

int64_t gs2d_grad_csr_words(const GridSamplerGradArgs& a)
{
    const CsrPlan pl = make_plan(a);
    return pl.ok ? (int64_t)pl.lay.item_words * a.N : 0;
}

bool gs2d_grad_csr_clear(const GridSamplerGradArgs& a, GradClear* clear)
{
    if (a.dx == nullptr || a.scratch == nullptr) {
        return false;
    }
    const CsrPlan pl = make_plan(a);
    if (pl.ok) {
        *clear = clear_of(a, pl);
    }
    return pl.ok;
}

hipError_t run_gs2d_grad_input_csr(const GridSamplerGradArgs& a, hipStream_t stream, bool* handled, bool cleared)
{
    *handled = false;
    if (a.dx == nullptr || a.scratch == nullptr) {
        return hipSuccess;
    }
    const CsrPlan pl = make_plan(a);
    if (!pl.ok) {
        return hipSuccess;
    }
    *handled = true;
    switch (a.elem) {
        case Elem::F32: return run_typed<float>(a, pl, cleared, stream);
        case Elem::F16: return run_typed<_Float16>(a, pl, cleared, stream);
        case Elem::BF16: return run_typed<__bf16>(a, pl, cleared, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
