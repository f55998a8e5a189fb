// Backward of grid_sampler2d for gfx950: gradient of the grid (bilinear), input planes staged through LDS.
// Two kernels: one lane per grid point with whole planes staged (described first), and, further down, two lanes per
// point with only the box of each plane staged that a block of points reaches, for the shapes that allow it.
//
// Same arithmetic, in the same order, as the one-lane-per-point kernel in gs2d_grad.hip (reference:
// image/grid_sampler2_d_grad/op_kernel/arch35/grid_sampler2_d_grad_simt_det.h:103-196): a lane owns one grid point
// and walks the channels in order, adding eight terms  v * distance * gradOutput  per channel to two running sums.
// What differs is where the operands come from.  Read from global memory, the corners of the 64 points of a
// wavefront lie in up to 128 different cache lines per channel, and the gather -- not the bytes -- sets the pace
// (fp16 N16 C256 64x64: 47 us for 67 MB of operands).  Here a workgroup of 256 points streams every input plane of
// its batch item, and its own 256 gradOutput values of every channel, through rings of LDS slots with the
// asynchronous global->LDS copies (loader wavefronts, see gs2d_lds_kernel.hpp); the corners and the gradOutput value
// are 2- or 4-byte LDS reads.
//
// The point wavefronts are one per SIMD, so every instruction they issue is time nothing else covers: their loop is
// the 29 arithmetic instructions of a plane, five LDS reads, one wait and one barrier, and nothing else (no address
// arithmetic, no global loads).
//
// All workgroups of a batch item want the same plane at about the same time, so few distinct bytes are on their way
// from HBM at any moment -- a ring's depth times the number of items.  One more wavefront per workgroup therefore
// runs ahead of the rings and touches one byte per 128-byte line of the planes to come (shared out among the item's
// workgroups) and of the workgroup's own gradOutput rows: the lines are in L2 when the copies ask for them, and what
// is in flight from HBM no longer depends on the rings.  It never waits for what it touched.
//
// A corner outside the image reads a slot of zeros behind the staged plane and its gradOutput factor is replaced by
// zero, so its terms are (0 * d) * 0 = +-0: the running sums start at +0 and can never become -0, so adding or
// subtracting a zero of either sign leaves them as the reference's "skip this corner" does.  (The distances d are
// finite: a non-finite source coordinate has been replaced by -100 before, source_index_set_grad.)
#include <hip/hip_runtime.h>

#include <type_traits>

#include "gs2d_grad_math.hpp"
#include "gs2d_lds_kernel.hpp"
#include "kernels.hpp"

namespace opscv {

namespace {

constexpr int kPointWaves = 4;   // 256 grid points per workgroup, one per lane
constexpr int kCopyWaves = 4;    // loader wavefronts
constexpr int kPoints = kPointWaves * 64;
constexpr int kUnroll = 16;      // channels per turn of the unrolled loop
constexpr int kAheadGout = 48;   // channels the L2 prefetch of gradOutput runs ahead
constexpr int kThreadsLds = (kPointWaves + kCopyWaves + 1) * 64;  // + the prefetch wavefront

// Brings the line of the byte at `p` into L2 (and L1): an asynchronous global->LDS copy of that byte into a dump area
// of LDS that nobody reads (`dump`, 256 bytes: a dword per lane).  A copy to LDS rather than a load into a register
// on purpose: the wavefront never waits for these, and data that arrives late in a register the compiler has
// meanwhile given to another value (it cannot know about a load hidden in an asm statement) would corrupt it.
__device__ __forceinline__ void touch_line(const char* p, char* dump)
{
    __builtin_amdgcn_global_load_lds((global_cptr_t)p, (lds_ptr_t)dump, 1, 0, 0);
}
constexpr int kDumpBytes = 256;

template <typename T, int NBUF, int PITCH>
__global__ __launch_bounds__(kThreadsLds) void gs2d_grad_grid_lds_kernel(
    const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ grid, T* __restrict__ dgrid, int32_t C,
    int32_t H, int32_t W, int32_t points, uint32_t tiles_per_n, int32_t pad, int32_t align, int32_t xcd_swizzle,
    int32_t ahead_x, float neg_zero, GradClear clear)
{
    static_assert(kUnroll % NBUF == 0, "a turn of the loop is whole turns of the ring");
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    // planes in flight ahead of the one whose values are being used: the point wavefronts hold on to two slots, the
    // plane whose reads may still be out and the one before it
    constexpr int DEPTH = NBUF - 2;
    // LDS: NBUF plane slots, then NBUF gradOutput rows (256 elements each), then the prefetch wavefront's dump area
    constexpr uint32_t GOUT_PITCH = kPoints * sizeof(T);
    constexpr uint32_t GOUT_RING = NBUF * PITCH;
    constexpr uint32_t DUMP = GOUT_RING + NBUF * GOUT_PITCH;
    const int tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)tid >> 6);

    // all tiles of one batch item on one XCD, next to each other in time: its planes come into one L2 once
    uint32_t n, tile;
    if (xcd_swizzle) {
        const uint32_t xcd = blockIdx.x & 7u, i = blockIdx.x >> 3;
        n = (i / tiles_per_n) * 8u + xcd;
        tile = i % tiles_per_n;
    } else {
        n = blockIdx.x / tiles_per_n;
        tile = blockIdx.x % tiles_per_n;
    }
    const int32_t plane_elems = H * W;
    const uint32_t plane_bytes = (uint32_t)plane_elems * (uint32_t)sizeof(T);
    const uint32_t zero_off = round_up16(plane_bytes);
    const int32_t c_turns = (C + kUnroll - 1) / kUnroll * kUnroll;  // planes the workgroup steps through

    if (wave == (uint32_t)(kPointWaves + kCopyWaves)) {
        // ------------------------------------------------ prefetch wavefront -----------------------------------
        // This wavefront is in the chain of barriers, so its steady-state step is kept to a few instructions:
        // pointers that advance, a countdown instead of a modulo.
        const uint32_t lane = (uint32_t)tid & 63u;
        char* dump = lds + DUMP;  // behind the rings
        const char* xb = reinterpret_cast<const char*>(x + (int64_t)n * C * plane_elems);
        // A plane of the item, when it is this workgroup's turn (planes tile, tile + tiles_per_n, ...): a byte every
        // 128 from the plane's start, and the plane's last byte unless the planes are whole, aligned lines.
        const bool whole_lines = (reinterpret_cast<uintptr_t>(xb) % 128u == 0) && (plane_bytes % 128u == 0);
        const uint32_t touches = plane_bytes / 128u + (whole_lines ? 0u : 1u);
        int32_t mine = (int32_t)tile;  // the next plane that is this workgroup's to touch
        auto touch_plane = [&](int32_t c) {
            if (c == mine) {
                mine += (int32_t)tiles_per_n;
                if (c < C) {
                    const char* pl = xb + (size_t)c * plane_bytes;
                    for (uint32_t j = lane; j < touches; j += 64u) {
                        const uint32_t off = j * 128u;
                        touch_line(pl + (off < plane_bytes ? off : plane_bytes - 1u), dump);
                    }
                }
            }
        };
        // the workgroup's own gradOutput rows, four channels per call: sixteen lanes per channel, a byte every 128 from
        // the row's start and its last byte
        const int32_t first = (int32_t)tile * kPoints;
        const uint32_t row_bytes = (uint32_t)((points - first < kPoints) ? points - first : kPoints) * (uint32_t)sizeof(T);
        const uint32_t goff = (lane & 15u) * 128u;
        const bool glane = goff < row_bytes + 128u;
        const size_t gstep = (size_t)4 * points * sizeof(T);
        const char* gp = reinterpret_cast<const char*>(gout + ((int64_t)n * C + (lane >> 4)) * points + first) +
                         (goff < row_bytes ? goff : row_bytes - 1u);
        int32_t gc = (int32_t)(lane >> 4);  // channel `gp` points at
        auto touch_gout = [&]() {
            if (glane && gc < C) {
                touch_line(gp, dump);
            }
            gp += gstep;
            gc += 4;
        };
        for (int32_t c = 0; c < ahead_x; c++) {
            touch_plane(c);
        }
        for (int32_t c0 = 0; c0 < kAheadGout; c0 += 4) {
            touch_gout();
        }
        for (int32_t s = 0; s <= c_turns + 1; s++) {
            touch_plane(s + ahead_x);
            if ((s & 3) == 0) {
                touch_gout();
            }
            lds_barrier();  // keeps pace with the ring
        }
        wait_vmcnt_imm<0>();  // everything touched has arrived: nothing outstanding at the end
        return;
    }
    if (wave >= (uint32_t)kPointWaves) {
        // ------------------------------------------------ loader wavefronts ------------------------------------
        // A loader's step per plane -- wait, barrier, issue -- is in the chain of barriers too.  The s_waitcnt count
        // must be a literal, and finding the literal for a run-time count costs a few dozen scalar instructions, as
        // does a general copy routine with bounds tests; at 8 KiB per plane that was most of the kernel's time
        // (101 us against 43).  The launch plan therefore only admits planes whose KiB-chunks divide evenly among
        // the loaders (PP copies each, a compile-time number) and at least as many channels as the ring is deep: the
        // loop has literal counts and unconditional copies, steady state while the ring is full, then an unrolled
        // run-down.  Loader 0 also copies the workgroup's gradOutput row of every channel (GO = 1 more copy a plane).
        const uint32_t lwave = wave - kPointWaves;
        const uint32_t lane = (uint32_t)tid & 63u;
        const char* xb = reinterpret_cast<const char*>(x + (int64_t)n * C * plane_elems);
        auto ring_loop = [&](auto pp_tag, auto go_tag) {
            constexpr int PP = decltype(pp_tag)::value;
            constexpr int GO = decltype(go_tag)::value;
            const char* src = xb + lwave * 1024u + lane * 16u;  // this lane's 16 bytes of the wavefront's first chunk
            uint32_t slot_off = lwave * 1024u;                  // the chunk's place in the slot being filled
            // gradOutput row of this workgroup: row_bytes (a multiple of 16) from `gsrc`, `points` elements on per plane
            const int32_t first = (int32_t)tile * kPoints;
            const uint32_t row_bytes =
                (uint32_t)((points - first < kPoints) ? points - first : kPoints) * (uint32_t)sizeof(T);
            const char* gsrc = reinterpret_cast<const char*>(gout + (int64_t)n * C * points + first) + lane * 16u;
            const bool glane = lane * 16u < row_bytes;
            const size_t gstep = (size_t)points * sizeof(T);
            uint32_t gslot_off = GOUT_RING;
            int fill = 0;
            auto issue = [&]() {
#pragma unroll
                for (int j = 0; j < PP; j++) {
                    __builtin_amdgcn_global_load_lds((global_cptr_t)(src + j * (kCopyWaves * 1024)),
                                                     (lds_ptr_t)(lds + slot_off + j * (kCopyWaves * 1024)), 16, 0, 0);
                }
                if constexpr (GO) {
                    if (glane) {
                        __builtin_amdgcn_global_load_lds((global_cptr_t)gsrc, (lds_ptr_t)(lds + gslot_off), 16, 0, 0);
                    }
                    gsrc += gstep;
                }
                src += plane_bytes;
                fill = (fill + 1 == NBUF) ? 0 : fill + 1;
                slot_off = (uint32_t)fill * PITCH + lwave * 1024u;
                gslot_off = GOUT_RING + (uint32_t)fill * GOUT_PITCH;
            };
            for (int i = 0; i < DEPTH; i++) {
                issue();
            }
            for (int32_t s = 0; s < C - DEPTH; s++) {
                wait_vmcnt_imm<(DEPTH - 1) * (PP + GO)>();  // plane s has landed: the DEPTH - 1 after it may be out
                lds_barrier();                              // ... and the slot of plane s - 2 is free
                issue();
            }
            ring_rundown<DEPTH - 1, PP + GO>();
            for (int32_t s = C; s <= c_turns + 1; s++) {
                lds_barrier();
            }
        };
        auto with_pp = [&](auto pp_tag) {
            constexpr int PP = decltype(pp_tag)::value;
            // the copy counts this ring class can see: outstanding ones fit the counter, the chunks fit the slot
            if constexpr ((NBUF - 2) * (PP + 1) <= 63 && PP * kCopyWaves * 1024 + 16 <= PITCH) {
                if (lwave == 0) {
                    ring_loop(pp_tag, std::integral_constant<int, 1>{});
                } else {
                    ring_loop(pp_tag, std::integral_constant<int, 0>{});
                }
            } else {
                // not reachable from the launch plan; keeps the workgroup's barrier count whole if it ever were
                for (int32_t s = 0; s <= c_turns + 1; s++) {
                    lds_barrier();
                }
            }
        };
        switch (plane_bytes / (kCopyWaves * 1024u)) {  // a whole number between 1 and 8 (launch plan)
            case 1: with_pp(std::integral_constant<int, 1>{}); break;
            case 2: with_pp(std::integral_constant<int, 2>{}); break;
            case 3: with_pp(std::integral_constant<int, 3>{}); break;
            case 4: with_pp(std::integral_constant<int, 4>{}); break;
            case 5: with_pp(std::integral_constant<int, 5>{}); break;
            case 6: with_pp(std::integral_constant<int, 6>{}); break;
            case 7: with_pp(std::integral_constant<int, 7>{}); break;
            default: with_pp(std::integral_constant<int, 8>{}); break;
        }
        return;
    }

    // ---------------------------------------------------- point wavefronts -------------------------------------
    if (tid < NBUF * 4) {
        reinterpret_cast<uint32_t*>(lds + (tid >> 2) * PITCH + zero_off)[tid & 3] = 0u;
    }
    // words of scratch memory that a later kernel wants zeroed (none when clear.count is 0): the item's tiles share
    // them out
    if (clear.count != 0u) {
        uint32_t* words = clear.base + (size_t)n * clear.item_words;
        const uint32_t share = (clear.count + tiles_per_n - 1u) / tiles_per_n;
        const uint32_t from = tile * share;
        const uint32_t to = (from + share < clear.count) ? from + share : clear.count;
        for (uint32_t i = from + (uint32_t)tid; i < to; i += (uint32_t)kPoints) {
            words[clear.first + i] = 0u;
        }
        if (tile == 0u && tid == 0) {
            words[clear.single] = 0u;
        }
    }
    const int32_t pix = (int32_t)tile * kPoints + tid;
    const bool live = pix < points;
    const int32_t pc = live ? pix : points - 1;  // lanes past the end work on a valid point and write nothing
    const int64_t idx = (int64_t)n * points + pc;
    GradTaps<T, 0> tp;
    decide_grad_taps<T, 0>(tp, ElemIO<T>::load(grid + 2 * idx), ElemIO<T>::load(grid + 2 * idx + 1), H, W, pad, align);
    const float dxe = (float)(tp.x0 == INT32_MAX ? tp.x0 : tp.x0 + 1) - tp.fx, dxw = tp.fx - (float)tp.x0;
    const float dys = (float)(tp.y0 == INT32_MAX ? tp.y0 : tp.y0 + 1) - tp.fy, dyn = tp.fy - (float)tp.y0;
    uint32_t taddr[4], taddr_hi[4];  // in the first slot, and in slot NBUF / 2 (an LDS read's literal offset has 16 bits)
    uint32_t keep[4];  // all ones for a corner inside the image: mask of its gradOutput bits
    {
        uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
        asm volatile("" : "+s"(lds_base));  // see gs2d_lds_kernel.hpp: keeps base + offset as one register per tap
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const bool in = tp.off[k] >= 0;
            taddr[k] = lds_base + (in ? (uint32_t)tp.off[k] * (uint32_t)sizeof(T) : zero_off);
            asm volatile("" : "+v"(taddr[k]));
            taddr_hi[k] = taddr[k] + (NBUF / 2) * PITCH;
            asm volatile("" : "+v"(taddr_hi[k]));
            keep[k] = in ? 0xFFFFFFFFu : 0u;
        }
    }
    // fifth "tap": the point's gradOutput value in the row that loader 0 copies next to each plane
    uint32_t gaddr;
    {
        uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
        asm volatile("" : "+s"(lds_base));
        gaddr = lds_base + GOUT_RING + (uint32_t)tid * (uint32_t)sizeof(T);
        asm volatile("" : "+v"(gaddr));
    }
    float gix = 0.0f, giy = 0.0f;
    // (v * d) * go as two fused multiply-adds onto -0: bit for bit the two rounded products (see blend() in
    // gs2d_lds_kernel.hpp), and the conversions of 16-bit operands ride on the instruction
    auto term = [&](uint32_t vraw, float d, uint32_t gobits) -> float {
        const float t = __builtin_fmaf(tap_value<T>(vraw), d, neg_zero);
        return __builtin_fmaf(tap_value<T>(gobits), t, neg_zero);
    };

    // One software pipeline over the planes, two deep: while plane p is in the arithmetic, the reads of plane p + 1 are
    // on their way and those of plane p + 2 are issued.  The four point wavefronts issue their reads together, right
    // behind a barrier, and the 20 scattered read instructions keep the LDS busy for most of a plane's time; a
    // wavefront that had to see its reads back before the next barrier (one deep: 37.7 us on fp16 N16 C256 64x64)
    // would add that time to its arithmetic instead of hiding it.  Barrier s says: plane s has landed, and the slot of
    // plane s - 2 is free -- a wavefront enters it with the reads of plane s - 2 returned (those of plane s - 1 may
    // be out: at most five, LDS reads return in order).  The loop body is straight-line code for kUnroll planes (slot
    // offsets are literals, no conditions).  The channel count is therefore rounded up to whole turns: all
    // wavefronts of the workgroup go through one barrier per plane of the rounded count, and two more; in the last,
    // partial turn the planes past the last channel read whatever the ring holds and have their corner values and
    // their gradOutput masked to zero, so they add +-0.
    uint32_t r0[5], r1[5];  // four corners and the gradOutput value of plane p and of plane p + 1
    // read k of a plane: corner k (0..3) or the gradOutput value (4)
    auto read_one = [&](int slot, int k, uint32_t* r) {
        if (k == 4) {
            load_taps<T, 1>((uint32_t)(slot * GOUT_PITCH), &gaddr, r + 4);
        } else if (slot < NBUF / 2) {
            load_taps<T, 1>((uint32_t)(slot * PITCH), taddr + k, r + k);
        } else {
            load_taps<T, 1>((uint32_t)((slot - NBUF / 2) * PITCH), taddr_hi + k, r + k);
        }
    };
    auto read_plane = [&](int slot, uint32_t* r) {
#pragma unroll
        for (int k = 0; k < 5; k++) {
            read_one(slot, k, r);
        }
    };
    __builtin_amdgcn_s_waitcnt(0xC07F);  // the zero-slot writes, before the first barrier publishes them
    lds_barrier();                        // plane 0 has landed
    read_plane(0, r0);
    lds_barrier();                        // plane 1 has landed
    read_plane(1 % NBUF, r1);
    auto turn = [&](auto masked, int32_t b) {
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const int32_t p = b + u;
            uint32_t v0 = r0[0], v1 = r0[1], v2 = r0[2], v3 = r0[3], g = r0[4];
            uint32_t r2[5];
            __builtin_amdgcn_sched_barrier(0);   // the arithmetic of the plane before stays in front of the wait
            __builtin_amdgcn_s_waitcnt(0xC57F);  // lgkmcnt(5): the reads of plane p are back
            lds_barrier();                       // plane p + 2 has landed (or there is none)
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (decltype(masked)::value) {
                const uint32_t m = (p < C) ? 0xFFFFFFFFu : 0u;
                v0 &= m;
                v1 &= m;
                v2 &= m;
                v3 &= m;
                g &= m;
            }
            const uint32_t g0 = g & keep[0], g1 = g & keep[1], g2 = g & keep[2], g3 = g & keep[3];
            // The five reads of plane p + 2 go out one at a time between the terms of plane p.  Issued in one go they
            // meet the other three wavefronts' reads at the LDS, and a wavefront whose read is not accepted yet
            // issues nothing behind it: the scattered reads' time would add to the arithmetic's instead of hiding
            // under it.
            const int slot = (u + 2) % NBUF;  // a literal once the loop is unrolled
            // grid_sampler2_d_grad_simt_det.h:150-185
            read_one(slot, 0, r2);
            __builtin_amdgcn_sched_barrier(0);
            gix -= term(v0, dys, g0);
            giy -= term(v0, dxe, g0);
            __builtin_amdgcn_sched_barrier(0);
            read_one(slot, 1, r2);
            __builtin_amdgcn_sched_barrier(0);
            gix += term(v1, dys, g1);
            giy -= term(v1, dxw, g1);
            __builtin_amdgcn_sched_barrier(0);
            read_one(slot, 2, r2);
            __builtin_amdgcn_sched_barrier(0);
            gix -= term(v2, dyn, g2);
            giy += term(v2, dxe, g2);
            __builtin_amdgcn_sched_barrier(0);
            read_one(slot, 3, r2);
            read_one(slot, 4, r2);
            __builtin_amdgcn_sched_barrier(0);
            gix += term(v3, dyn, g3);
            giy += term(v3, dxw, g3);
#pragma unroll
            for (int k = 0; k < 5; k++) {
                r0[k] = r1[k];
                r1[k] = r2[k];
            }
        }
    };
    int32_t b = 0;
    for (; b + kUnroll <= C; b += kUnroll) {
        turn(std::false_type{}, b);
    }
    if (b < C) {
        turn(std::true_type{}, b);
    }
    if (live) {
        // products in fp32 first, then the conversion
        ElemIO<T>::store(dgrid + 2 * idx, as_fp32_value(tp.mx * gix));
        ElemIO<T>::store(dgrid + 2 * idx + 1, as_fp32_value(tp.my * giy));
    }
}


// ---------------------------------------------------------------------------------------------------------------------
// Two lanes per grid point.  The kernel above has one point wavefront per SIMD, and whatever that wavefront waits for
// (a barrier, an LDS read) the SIMD waits for.  Here the lanes 2i and 2i + 1 of a wavefront own one grid point and one
// component of its gradient each: both read the four corners and the gradOutput value of every plane, the even lane
// multiplies by the row distances and keeps the x sum, the odd lane by the column distances and keeps the y sum.  The
// two sums are independent chains in the reference too, so nothing is exchanged and each sum sees its terms in the
// reference's order.  A step is two planes (half as many barriers); per step a lane issues 32 arithmetic instructions
// where a lane of the kernel above issues 58, and a workgroup of 256 points has eight point wavefronts, two per SIMD.
// Needs an even channel count.
//
// Only the box of each plane is staged that the workgroup's points reach: the 256 points are a block of 16 x 16 of the
// output, whose corners under a smooth grid lie in a small part of the plane.  The point wavefronts find the box first
// (rows and columns of the corners inside the image, reduced over the wavefronts through LDS), the loaders copy it
// as consecutive 16-byte units, the corners' LDS offsets are taken inside the box.
constexpr int kPointWaves2 = 8;
constexpr int kThreadsLds2 = (kPointWaves2 + kCopyWaves + 1) * 64;
constexpr int kUnrollSteps = 8;  // steps per turn of the unrolled loop

template <typename T, int NBUF, int PITCH>
__global__ __launch_bounds__(kThreadsLds2) void gs2d_grad_grid_lds2_kernel(
    const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ grid, T* __restrict__ dgrid, int32_t C,
    int32_t H, int32_t W, int32_t points, uint32_t tiles_per_n, int32_t pad, int32_t align, int32_t xcd_swizzle,
    int32_t ahead_x, float neg_zero, GradClear clear, int32_t Wo)
{
    constexpr int SBUF = NBUF / 2;  // steps the ring holds
    static_assert(NBUF % 2 == 0 && kUnrollSteps % SBUF == 0, "a turn of the loop is whole turns of the ring");
    static_assert(SBUF >= 4, "two steps held by the point wavefronts, two or more on their way");
    extern __shared__ uint4 smem_raw[];
    char* lds = reinterpret_cast<char*>(smem_raw);
    constexpr int DEPTH = SBUF - 2;  // steps in flight ahead of the one whose values are being used
    constexpr uint32_t GOUT_PITCH = kPoints * sizeof(T);
    constexpr uint32_t GOUT_RING = NBUF * PITCH;
    constexpr uint32_t DUMP = GOUT_RING + NBUF * GOUT_PITCH;
    constexpr uint32_t BOX = DUMP + kDumpBytes;  // 4 words per point wavefront: the corners' row and column ranges
    const int tid = threadIdx.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane((uint32_t)tid >> 6);

    uint32_t n, tile;
    if (xcd_swizzle) {
        const uint32_t xcd = blockIdx.x & 7u, i = blockIdx.x >> 3;
        n = (i / tiles_per_n) * 8u + xcd;
        tile = i % tiles_per_n;
    } else {
        n = blockIdx.x / tiles_per_n;
        tile = blockIdx.x % tiles_per_n;
    }
    const int32_t plane_elems = H * W;
    const uint32_t plane_bytes = (uint32_t)plane_elems * (uint32_t)sizeof(T);
    const uint32_t zero_off = round_up16(plane_bytes);
    // the workgroup's 256 points are a block of 16 x 16 of the output (launch plan: both extents multiples of 16)
    const uint32_t tiles_per_row = (uint32_t)Wo / 16u;
    const uint32_t trow = tile / tiles_per_row, tcol = tile - trow * tiles_per_row;
    // The box of the plane that the block's corners lie in, after the point wavefronts have published it (barrier):
    // rows [ylo, yhi], columns [xa, xa + wb) on 16-byte boundaries.  Only the box is staged, as consecutive 16-byte
    // units: unit u holds columns 8 / sizeof(T) * 2 ... of row ylo + u / row_units.
    struct Box {
        int32_t ylo, rows, xa, wb;
    };
    auto read_box = [&]() -> Box {
        const int32_t* bw = reinterpret_cast<const int32_t*>(lds + BOX);
        int32_t ylo = INT32_MAX, yhi = -1, xlo = INT32_MAX, xhi = -1;
        for (int w8 = 0; w8 < kPointWaves2; w8++) {
            const int32_t a = bw[w8 * 4 + 0], b2 = bw[w8 * 4 + 1], c2 = bw[w8 * 4 + 2], d2 = bw[w8 * 4 + 3];
            ylo = a < ylo ? a : ylo;
            yhi = b2 > yhi ? b2 : yhi;
            xlo = c2 < xlo ? c2 : xlo;
            xhi = d2 > xhi ? d2 : xhi;
        }
        constexpr int32_t EPU = 16 / (int32_t)sizeof(T);  // elements per 16-byte unit
        Box bx;
        if (yhi < 0) {  // no corner inside the image: a box of one unit that nobody reads
            bx.ylo = 0;
            bx.rows = 1;
            bx.xa = 0;
            bx.wb = EPU;
        } else {
            bx.ylo = ylo;
            bx.rows = yhi - ylo + 1;
            bx.xa = xlo / EPU * EPU;
            const int32_t xe = (xhi + EPU) / EPU * EPU;  // one past the last column, rounded up
            bx.wb = (xe < W ? xe : W) - bx.xa;
        }
        bx.ylo = __builtin_amdgcn_readfirstlane(bx.ylo);
        bx.rows = __builtin_amdgcn_readfirstlane(bx.rows);
        bx.xa = __builtin_amdgcn_readfirstlane(bx.xa);
        bx.wb = __builtin_amdgcn_readfirstlane(bx.wb);
        return bx;
    };
    const int32_t steps_real = C / 2;                                                  // C is even (launch plan)
    const int32_t steps = (steps_real + kUnrollSteps - 1) / kUnrollSteps * kUnrollSteps;  // steps the workgroup walks

    if (wave == (uint32_t)(kPointWaves2 + kCopyWaves)) {
        // ------------------------------------------------ prefetch wavefront -----------------------------------
        const uint32_t lane = (uint32_t)tid & 63u;
        char* dump = lds + DUMP;
        const char* xb = reinterpret_cast<const char*>(x + (int64_t)n * C * plane_elems);
        const bool whole_lines = (reinterpret_cast<uintptr_t>(xb) % 128u == 0) && (plane_bytes % 128u == 0);
        const uint32_t touches = plane_bytes / 128u + (whole_lines ? 0u : 1u);
        int32_t mine = (int32_t)tile;
        auto touch_plane = [&](int32_t c) {
            if (c == mine) {
                mine += (int32_t)tiles_per_n;
                if (c < C) {
                    const char* pl = xb + (size_t)c * plane_bytes;
                    for (uint32_t j = lane; j < touches; j += 64u) {
                        const uint32_t off = j * 128u;
                        touch_line(pl + (off < plane_bytes ? off : plane_bytes - 1u), dump);
                    }
                }
            }
        };
        // the block's sixteen gradOutput segments of a channel (32 or 64 bytes each): sixteen lanes per channel
        const size_t gstep = (size_t)4 * points * sizeof(T);
        const char* gp = reinterpret_cast<const char*>(gout + ((int64_t)n * C + (lane >> 4)) * points +
                                                       (int64_t)(trow * 16u + (lane & 15u)) * Wo + tcol * 16u);
        int32_t gc = (int32_t)(lane >> 4);
        auto touch_gout = [&]() {
            if (gc < C) {
                touch_line(gp, dump);
            }
            gp += gstep;
            gc += 4;
        };
        for (int32_t c = 0; c < ahead_x; c++) {
            touch_plane(c);
        }
        for (int32_t c0 = 0; c0 < kAheadGout; c0 += 4) {
            touch_gout();
        }
        lds_barrier();  // the box is published (nothing to do with it here)
        for (int32_t s = 0; s <= steps + 1; s++) {
            touch_plane(2 * s + ahead_x);
            touch_plane(2 * s + 1 + ahead_x);
            if ((s & 1) == 0) {
                touch_gout();
            }
            lds_barrier();  // keeps pace with the ring: one barrier per step, and two more
        }
        wait_vmcnt_imm<0>();
        return;
    }
    if (wave >= (uint32_t)kPointWaves2) {
        // ------------------------------------------------ loader wavefronts ------------------------------------
        const uint32_t lwave = wave - kPointWaves2;
        const uint32_t lane = (uint32_t)tid & 63u;
        const char* xb = reinterpret_cast<const char*>(x + (int64_t)n * C * plane_elems);
        lds_barrier();  // the box is published
        const Box box = read_box();
        constexpr int32_t EPU = 16 / (int32_t)sizeof(T);
        const uint32_t row_units = (uint32_t)(box.wb / EPU);
        const uint32_t units = (uint32_t)box.rows * row_units;    // 16-byte units of the box
        const uint32_t instrs = (units + 63u) / 64u;              // copy instructions per plane, all loaders together
        const uint32_t my_instrs = (instrs > lwave) ? (instrs - lwave + kCopyWaves - 1) / kCopyWaves : 0u;
        auto ring_loop = [&](auto pp_tag, auto go_tag) {
            constexpr int PP = decltype(pp_tag)::value;  // copies per plane of this loader
            constexpr int GO = decltype(go_tag)::value;
            constexpr int PER_STEP = 2 * (PP + GO);
            // The lane's 16 bytes of its wavefront's j-th instruction: unit (j * loaders + lwave) * 64 + lane of the
            // box; a lane past the box's last unit copies the last unit again (its LDS place, behind the box, is
            // nobody's).
            uint32_t goffs[PP > 0 ? PP : 1];
#pragma unroll
            for (int j = 0; j < PP; j++) {
                uint32_t u = ((uint32_t)j * kCopyWaves + lwave) * 64u + lane;
                u = u < units ? u : units - 1u;
                const uint32_t row = u / row_units, col = u - row * row_units;
                goffs[j] = (((uint32_t)box.ylo + row) * (uint32_t)W + (uint32_t)box.xa + col * (uint32_t)EPU) *
                           (uint32_t)sizeof(T);
            }
            const char* src = xb;
            uint32_t slot_off = lwave * 1024u;
            // gradOutput of the block: per channel 256 values in point order, sixteen segments of sixteen points
            constexpr uint32_t GLANES = kPoints * sizeof(T) / 16u;
            const uint32_t p0 = lane * (uint32_t)EPU;  // the lane's first point
            const char* gsrc = reinterpret_cast<const char*>(
                gout + (int64_t)n * C * points + (int64_t)(trow * 16u + (p0 >> 4)) * Wo + tcol * 16u + (p0 & 15u));
            const bool glane = lane < GLANES;
            const size_t gstep = (size_t)points * sizeof(T);
            uint32_t gslot_off = GOUT_RING;
            int fill = 0;  // step slot being filled
            auto issue = [&]() {
#pragma unroll
                for (int h = 0; h < 2; h++) {
#pragma unroll
                    for (int j = 0; j < PP; j++) {
                        __builtin_amdgcn_global_load_lds(
                            (global_cptr_t)(src + (size_t)h * plane_bytes + goffs[j]),
                            (lds_ptr_t)(lds + slot_off + h * PITCH + j * (kCopyWaves * 1024)), 16, 0, 0);
                    }
                }
                if constexpr (GO) {
                    if (glane) {
                        __builtin_amdgcn_global_load_lds((global_cptr_t)gsrc, (lds_ptr_t)(lds + gslot_off), 16, 0, 0);
                        __builtin_amdgcn_global_load_lds((global_cptr_t)(gsrc + gstep),
                                                         (lds_ptr_t)(lds + gslot_off + GOUT_PITCH), 16, 0, 0);
                    }
                    gsrc += 2 * gstep;
                }
                src += (size_t)2 * plane_bytes;
                fill = (fill + 1 == SBUF) ? 0 : fill + 1;
                slot_off = (uint32_t)fill * (2 * PITCH) + lwave * 1024u;
                gslot_off = GOUT_RING + (uint32_t)fill * (2 * GOUT_PITCH);
            };
            for (int i = 0; i < DEPTH; i++) {
                issue();
            }
            for (int32_t s = 0; s < steps_real - DEPTH; s++) {
                wait_vmcnt_imm<(DEPTH - 1) * PER_STEP>();  // step s has landed: the DEPTH - 1 after it may be out
                lds_barrier();                             // ... and the slots of step s - 2 are free
                issue();
            }
            ring_rundown<DEPTH - 1, PER_STEP>();
            for (int32_t s = steps_real; s <= steps + 1; s++) {
                lds_barrier();
            }
        };
        auto with_pp = [&](auto pp_tag) {
            constexpr int PP = decltype(pp_tag)::value;
            if constexpr ((SBUF - 3) * 2 * (PP + 1) <= 63 && PP * kCopyWaves * 1024 + 16 <= PITCH + kCopyWaves * 1024) {
                if (lwave == 0) {
                    ring_loop(pp_tag, std::integral_constant<int, 1>{});
                } else {
                    ring_loop(pp_tag, std::integral_constant<int, 0>{});
                }
            } else {
                for (int32_t s = 0; s <= steps + 1; s++) {
                    lds_barrier();
                }
            }
        };
        switch (my_instrs) {  // at most plane_bytes / 4 KiB, which the launch plan limits to 4
            case 0: with_pp(std::integral_constant<int, 0>{}); break;
            case 1: with_pp(std::integral_constant<int, 1>{}); break;
            case 2: with_pp(std::integral_constant<int, 2>{}); break;
            case 3: with_pp(std::integral_constant<int, 3>{}); break;
            default: with_pp(std::integral_constant<int, 4>{}); break;
        }
        return;
    }

    // ---------------------------------------------------- point wavefronts -------------------------------------
    if (tid < NBUF * 4) {
        reinterpret_cast<uint32_t*>(lds + (tid >> 2) * PITCH + zero_off)[tid & 3] = 0u;
    }
    if (clear.count != 0u) {
        uint32_t* words = clear.base + (size_t)n * clear.item_words;
        const uint32_t share = (clear.count + tiles_per_n - 1u) / tiles_per_n;
        const uint32_t from = tile * share;
        const uint32_t to = (from + share < clear.count) ? from + share : clear.count;
        for (uint32_t i = from + (uint32_t)tid; i < to; i += (uint32_t)(kPointWaves2 * 64)) {
            words[clear.first + i] = 0u;
        }
        if (tile == 0u && tid == 0) {
            words[clear.single] = 0u;
        }
    }
    const uint32_t parity = (uint32_t)tid & 1u;  // the lane's sum: 0 the x component of the point's gradient, 1 the y
    const int32_t pt = tid >> 1;                 // its point inside the block: row pt / 16, column pt % 16
    const int32_t pix = (int32_t)((trow * 16u + (uint32_t)(pt >> 4)) * (uint32_t)Wo + tcol * 16u + (uint32_t)(pt & 15));
    // (whole blocks only -- launch plan -- so every lane's point exists)
    const int64_t idx = (int64_t)n * points + pix;
    GradTaps<T, 0> tp;
    decide_grad_taps<T, 0>(tp, ElemIO<T>::load(grid + 2 * idx), ElemIO<T>::load(grid + 2 * idx + 1), H, W, pad, align);
    // the rows and columns of the lane's corners inside the image, then of the wavefront's, for the box
    {
        const int32_t x1 = (tp.x0 == INT32_MAX) ? tp.x0 : tp.x0 + 1, y1 = (tp.y0 == INT32_MAX) ? tp.y0 : tp.y0 + 1;
        const bool in0 = tp.off[0] >= 0, in1 = tp.off[1] >= 0, in2 = tp.off[2] >= 0, in3 = tp.off[3] >= 0;
        int32_t ylo = INT32_MAX, yhi = -1, xlo = INT32_MAX, xhi = -1;
        if (in0 || in1) {
            ylo = tp.y0;
            yhi = tp.y0;
        }
        if (in2 || in3) {
            ylo = ylo < y1 ? ylo : y1;
            yhi = y1;
        }
        if (in0 || in2) {
            xlo = tp.x0;
            xhi = tp.x0;
        }
        if (in1 || in3) {
            xlo = xlo < x1 ? xlo : x1;
            xhi = x1;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const int32_t a = __shfl_xor(ylo, o), b2 = __shfl_xor(yhi, o), c2 = __shfl_xor(xlo, o), d2 = __shfl_xor(xhi, o);
            ylo = a < ylo ? a : ylo;
            yhi = b2 > yhi ? b2 : yhi;
            xlo = c2 < xlo ? c2 : xlo;
            xhi = d2 > xhi ? d2 : xhi;
        }
        if ((tid & 63) == 0) {
            int32_t* bw = reinterpret_cast<int32_t*>(lds + BOX) + wave * 4u;
            bw[0] = ylo;
            bw[1] = yhi;
            bw[2] = xlo;
            bw[3] = xhi;
        }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    lds_barrier();  // every wavefront's ranges are in LDS
    const Box box = read_box();
    const float dxe = (float)(tp.x0 == INT32_MAX ? tp.x0 : tp.x0 + 1) - tp.fx, dxw = tp.fx - (float)tp.x0;
    const float dys = (float)(tp.y0 == INT32_MAX ? tp.y0 : tp.y0 + 1) - tp.fy, dyn = tp.fy - (float)tp.y0;
    uint32_t taddr[4], taddr_hi[4];  // in the first step slot, and in step slot SBUF / 2
    uint32_t keep[4];
    {
        uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
        asm volatile("" : "+s"(lds_base));
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const bool in = tp.off[k] >= 0;
            // the corner's place in the staged box
            const int32_t cy = (k < 2) ? tp.y0 : tp.y0 + 1, cx = (k & 1) ? tp.x0 + 1 : tp.x0;
            const uint32_t boff = (uint32_t)((cy - box.ylo) * box.wb + (cx - box.xa)) * (uint32_t)sizeof(T);
            taddr[k] = lds_base + (in ? boff : zero_off);
            asm volatile("" : "+v"(taddr[k]));
            taddr_hi[k] = taddr[k] + (SBUF / 2) * (2 * PITCH);
            asm volatile("" : "+v"(taddr_hi[k]));
            keep[k] = in ? 0xFFFFFFFFu : 0u;
        }
    }
    uint32_t gaddr;
    {
        uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
        asm volatile("" : "+s"(lds_base));
        gaddr = lds_base + GOUT_RING + (uint32_t)pt * (uint32_t)sizeof(T);
        asm volatile("" : "+v"(gaddr));
    }
    // The lane's four signed distances: its sum takes  -t0 +t1 -t2 +t3  of the products with the row distances (x
    // component) or  -t0 -t1 +t2 +t3  of those with the column distances (y component), grid_sampler2_d_grad_simt_det.h:
    // 150-185; the sign goes into the distance (a - b is a + (-b) bit for bit, and negating a factor negates the
    // rounded product), so that both lanes run the same instructions.
    float dk[4];
    dk[0] = parity ? -dxe : -dys;
    dk[1] = parity ? -dxw : dys;
    dk[2] = parity ? dxe : -dyn;
    dk[3] = parity ? dxw : dyn;
    float acc = 0.0f;
    // (v * d) * go as two fused multiply-adds onto -0: bit for bit the two rounded products
    auto term = [&](uint32_t vraw, float d, uint32_t gobits) -> float {
        const float t = __builtin_fmaf(tap_value<T>(vraw), d, neg_zero);
        return __builtin_fmaf(tap_value<T>(gobits), t, neg_zero);
    };
    // reads 0..4: the corners and the gradOutput value of the step's first plane, 5..9: of its second
    uint32_t r0[10], r1[10];
    auto read_one = [&](int slot, int k, uint32_t* r) {  // slot: step slot
        const int h = k / 5, c = k % 5;
        if (c == 4) {
            load_taps<T, 1>((uint32_t)((slot * 2 + h) * GOUT_PITCH), &gaddr, r + k);
        } else if (slot < SBUF / 2) {
            load_taps<T, 1>((uint32_t)((slot * 2 + h) * PITCH), taddr + c, r + k);
        } else {
            load_taps<T, 1>((uint32_t)(((slot - SBUF / 2) * 2 + h) * PITCH), taddr_hi + c, r + k);
        }
    };
    auto read_step = [&](int slot, uint32_t* r) {
#pragma unroll
        for (int k = 0; k < 10; k++) {
            read_one(slot, k, r);
        }
    };
    __builtin_amdgcn_s_waitcnt(0xC07F);  // the zero-slot writes, before the first barrier publishes them
    lds_barrier();                        // step 0 has landed
    read_step(0, r0);
    lds_barrier();                        // step 1 has landed
    read_step(1 % SBUF, r1);
    auto turn = [&](auto masked, int32_t b) {
#pragma unroll
        for (int u = 0; u < kUnrollSteps; u++) {
            const int32_t st = b + u;
            uint32_t cur[10];
#pragma unroll
            for (int k = 0; k < 10; k++) {
                cur[k] = r0[k];
            }
            uint32_t r2[10];
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xCA7F);  // lgkmcnt(10): the reads of step st are back
            lds_barrier();                       // step st + 2 has landed (or there is none)
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (decltype(masked)::value) {
                const uint32_t m = (st < steps_real) ? 0xFFFFFFFFu : 0u;
#pragma unroll
                for (int k = 0; k < 10; k++) {
                    cur[k] &= m;
                }
            }
            const int slot = (u + 2) % SBUF;
            // the reads of step st + 2 go out one or two at a time between the terms of step st
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const uint32_t g = cur[5 * h + 4];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    read_one(slot, 5 * h + k, r2);
                    if (k == 3) {
                        read_one(slot, 5 * h + 4, r2);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    acc += term(cur[5 * h + k], dk[k], g & keep[k]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int k = 0; k < 10; k++) {
                r0[k] = r1[k];
                r1[k] = r2[k];
            }
        }
    };
    int32_t b = 0;
    for (; b + kUnrollSteps <= steps_real; b += kUnrollSteps) {
        turn(std::false_type{}, b);
    }
    if (b < steps_real) {
        turn(std::true_type{}, b);
    }
    // products in fp32 first, then the conversion
    ElemIO<T>::store(dgrid + 2 * idx + parity, as_fp32_value((parity ? tp.my : tp.mx) * acc));
}

struct GridLdsPlan {
    bool ok = false;
    int cls = 0;
    uint32_t tiles_per_n = 0;
    int xcd_swizzle = 0;
};

// ring classes: plane pitch in LDS and slots (about 128 KiB of planes)
constexpr int kGradPitch[3] = {8208, 16400, 32784};
constexpr int kGradNbuf[3] = {16, 8, 4};

GridLdsPlan make_plan(const GridSamplerGradArgs& a)
{
    GridLdsPlan p;
    const int64_t esz = elem_size(a.elem);
    const int64_t plane_bytes = a.Hin * a.Win * esz;
    const int64_t points = a.Hout * a.Wout;
    // what the loaders' loop assumes: planes of whole KiB-chunks that divide evenly among the loaders, 16-byte
    // aligned; gradOutput rows (256 points of a channel) that are whole 16-byte units on 16-byte boundaries
    if (a.interp != 0 || plane_bytes % (kCopyWaves * 1024) != 0 || plane_bytes > 8 * kCopyWaves * 1024 ||
        reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || (points * esz) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(a.gout) % 16 != 0) {
        return p;
    }
    while (plane_bytes + 16 > kGradPitch[p.cls]) {
        p.cls++;
    }
    // Every workgroup streams all planes of its batch item: worth it when there are channels enough to fill the ring
    // and amortise its fill, and workgroups for a good part of the 256 CUs -- otherwise the one-lane-per-point
    // kernel, which has more of them, is the better one.
    const int64_t tiles = (points + kPoints - 1) / kPoints;
    if (a.C < 16 || a.C < kGradNbuf[p.cls] - 1 || a.N * tiles < 128 || a.N * tiles > INT32_MAX ||
        a.N * a.C > INT32_MAX) {
        return p;
    }
    p.tiles_per_n = (uint32_t)tiles;
    p.xcd_swizzle = (a.N % 8 == 0) ? 1 : 0;
    p.ok = true;
    return p;
}

template <typename T, int CLS>
hipError_t launch_cls2(const GridSamplerGradArgs& a, const GridLdsPlan& p, const GradClear& clear, hipStream_t stream)
{
    auto kernel = gs2d_grad_grid_lds2_kernel<T, kGradNbuf[CLS], kGradPitch[CLS]>;
    // the rings, the prefetch wavefront's dump area, and four words per point wavefront for the box
    constexpr int lds_bytes = kGradNbuf[CLS] * (kGradPitch[CLS] + kPoints * (int)sizeof(T)) + kDumpBytes + kPointWaves2 * 16;
    static_assert(lds_bytes <= kLdsLimit, "the rings fit a CU's LDS");
    static std::atomic<uint32_t> lds_allowed{0};
    const hipError_t ea = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), lds_bytes, lds_allowed);
    if (ea != hipSuccess) {
        return ea;
    }
    const uint32_t blocks = (uint32_t)(a.N * p.tiles_per_n);
    const int64_t plane_bytes = a.Hin * a.Win * (int64_t)sizeof(T);
    int64_t ahead = 262144 / plane_bytes;
    ahead = ahead > 64 ? 64 : ahead;
    if (ahead < kGradNbuf[CLS]) {
        ahead = kGradNbuf[CLS];
    }
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kThreadsLds2), lds_bytes, stream, (const T*)a.gout, (const T*)a.x,
                       (const T*)a.grid, (T*)a.dgrid, (int32_t)a.C, (int32_t)a.Hin, (int32_t)a.Win,
                       (int32_t)(a.Hout * a.Wout), p.tiles_per_n, (int32_t)a.pad, (int32_t)a.align, p.xcd_swizzle,
                       (int32_t)ahead, -0.0f, clear, (int32_t)a.Wout);
    return hipGetLastError();
}

template <typename T, int CLS>
hipError_t launch_cls(const GridSamplerGradArgs& a, const GridLdsPlan& p, const GradClear& clear, hipStream_t stream)
{
    if constexpr (CLS <= 1) {
        // two lanes per grid point and the planes' boxes only: an even channel count with steps enough to fill the
        // ring, an output of whole 16 x 16 blocks, input rows of whole 16-byte units
        if (a.C % 2 == 0 && a.C / 2 >= kGradNbuf[CLS] / 2 && a.Wout % 16 == 0 && a.Hout % 16 == 0 &&
            a.Win % (16 / (int)sizeof(T)) == 0 && a.Hin * a.Win * (int64_t)sizeof(T) <= 4 * kCopyWaves * 1024) {
            return launch_cls2<T, CLS>(a, p, clear, stream);
        }
    }
    auto kernel = gs2d_grad_grid_lds_kernel<T, kGradNbuf[CLS], kGradPitch[CLS]>;
    constexpr int lds_bytes = kGradNbuf[CLS] * (kGradPitch[CLS] + kPoints * (int)sizeof(T)) + kDumpBytes;
    static_assert(lds_bytes <= kLdsLimit, "the rings fit a CU's LDS");
    static std::atomic<uint32_t> lds_allowed{0};
    const hipError_t ea = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), lds_bytes, lds_allowed);
    if (ea != hipSuccess) {
        return ea;
    }
    const uint32_t blocks = (uint32_t)(a.N * p.tiles_per_n);
    // planes the L2 prefetch runs ahead of the ring: about 256 KiB of the item
    const int64_t plane_bytes = a.Hin * a.Win * (int64_t)sizeof(T);
    int64_t ahead = 262144 / plane_bytes;
    ahead = ahead > 64 ? 64 : ahead;
    if (ahead < kGradNbuf[CLS]) {
        ahead = kGradNbuf[CLS];
    }
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kThreadsLds), lds_bytes, stream, (const T*)a.gout, (const T*)a.x,
                       (const T*)a.grid, (T*)a.dgrid, (int32_t)a.C, (int32_t)a.Hin, (int32_t)a.Win,
                       (int32_t)(a.Hout * a.Wout), p.tiles_per_n, (int32_t)a.pad, (int32_t)a.align, p.xcd_swizzle,
                       (int32_t)ahead, -0.0f, clear);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_typed(const GridSamplerGradArgs& a, const GridLdsPlan& p, const GradClear& clear,
                        hipStream_t stream)
{
    switch (p.cls) {
        case 0: return launch_cls<T, 0>(a, p, clear, stream);
        case 1: return launch_cls<T, 1>(a, p, clear, stream);
        case 2: return launch_cls<T, 2>(a, p, clear, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

bool gs2d_grad_grid_uses_lds(const GridSamplerGradArgs& a) { return make_plan(a).ok; }

hipError_t run_gs2d_grad_grid_lds(const GridSamplerGradArgs& a, hipStream_t stream, bool* handled,
                                  const GradClear* clear_or_null)
{
    *handled = false;
    if (a.dgrid == nullptr) {
        return hipSuccess;
    }
    const GridLdsPlan p = make_plan(a);
    if (!p.ok) {
        return hipSuccess;
    }
    *handled = true;
    const GradClear clear = (clear_or_null != nullptr) ? *clear_or_null : GradClear{};  // count 0, base null: nothing
    switch (a.elem) {
        case Elem::F32: return launch_typed<float>(a, p, clear, stream);
        case Elem::F16: return launch_typed<_Float16>(a, p, clear, stream);
        case Elem::BF16: return launch_typed<__bf16>(a, p, clear, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
