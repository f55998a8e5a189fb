// Grid sampler 2-D forward, LDS-staged variant: plan selection (device code in gs2d_lds_kernel.hpp).
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>

#include "gs2d_lds_launch.hpp"
#include "options.hpp"

namespace opscv {

// CUs of the current device (256 on MI355X; also the answer where no device can be asked, as in host-only planning).
int compute_unit_count()
{
    static std::atomic<int> cached{0};
    int v = cached.load(std::memory_order_relaxed);
    if (v == 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
            (void)hipGetLastError();
            cus = 256;
        }
        v = cus;
        cached.store(v, std::memory_order_relaxed);
    }
    return v;
}

static LdsPlan make_lds_plan_rows(const GridSamplerArgs& a, bool pad_rows);

LdsPlan make_lds_plan(const GridSamplerArgs& a)
{
    // rows padded to a multiple of 128 bytes where that applies and the plan can keep the promise that goes with it
    // (the loaders' literal-count loop is the one that pads)
    const LdsPlan padded = make_lds_plan_rows(a, true);
    if (padded.ok && padded.chan_pairs) {
        return padded;
    }
    // Two channels per stage on the rows as they are rather than single channels on padded rows, where the padded
    // planes are too large for the former and an interleaved row is whole 128-byte lines (fp16 N16 C256 40x96: 12.3 us
    // padded, 10.8 in pairs; rows of 80 elements 12.6 and 12.0; rows of 72, which shift by eight banks a row in the
    // interleaved layout, 13.1 and 14.3).
    const LdsPlan as_is = make_lds_plan_rows(a, false);
    // (bicubic: sixteen reads per pixel and channel make the single-channel stages the slower choice whatever the rows:
    // fp16 N16 C256 48x80 51.0 us padded, 35.4 in pairs; 50x72 51.8 and 42.2; border padding 64.9 and 37.3)
    if (as_is.ok && as_is.chan_pairs && (a.Win % 32 == 0 || a.interp == 2)) {
        return as_is;
    }
    return padded.ok ? padded : as_is;
}

static LdsPlan make_lds_plan_rows(const GridSamplerArgs& a, bool pad_rows)
{
    LdsPlan p;
    const int64_t esz = elem_size(a.elem);
    const int64_t plane_bytes = a.Hin * a.Win * esz;
    // planes that start on 16-byte boundaries and are whole 16-byte units are copied as they are; every other
    // element-aligned plane in the shifted layout (gs2d_lds_kernel.hpp, issue_stage_copy), up to 14 bytes into its slot
    const uintptr_t xa = reinterpret_cast<uintptr_t>(a.x);
    const bool plain = plane_bytes % 16 == 0 && xa % 16 == 0;
    if (!plain && xa % esz != 0) {
        return p;  // a misaligned tensor: leave it to the direct variant
    }
    // staged rows: the plane's rows, or each padded to a multiple of 128 bytes (rows of whole 16-byte units that are
    // not one already; see the loaders' loop in gs2d_lds_kernel.hpp for why)
    const int64_t row_bytes = a.Win * esz;
    const bool padded = pad_rows && plain && row_bytes % 16 == 0 && row_bytes % 128 != 0;
    if (pad_rows && !padded) {
        return p;  // nothing to pad: the caller plans without
    }
    const int64_t lds_row_bytes = padded ? (row_bytes + 127) / 128 * 128 : row_bytes;
    const int64_t staged_bytes = a.Hin * lds_row_bytes;
    p.lds_w = (int32_t)(lds_row_bytes / esz);
    // a padded plane is copied in whole 1 KiB chunks that must stay in front of the slot of zeros
    const int64_t need = padded ? (staged_bytes + 1023) / 1024 * 1024 + 16
                                : ((plane_bytes + (plain ? 0 : 14) + 15) & ~(int64_t)15) + 16;
    const int64_t out_plane = a.Hout * a.Wout;
    // output-plane byte offsets are kept in 32 bits (and below the out-of-range marker 0x80000000)
    if (out_plane * esz >= ((int64_t)1 << 31) || need > kPitch[4]) {
        return p;
    }
    p.cls = 0;
    while (need > kPitch[p.cls]) {
        p.cls++;
    }
    const int cgs = kCgs[p.cls];
    p.lds_bytes = (uint32_t)(kNbuf[p.cls] * kPitch[p.cls] * cgs);
    // pixels per lane: every tile of an output plane streams all staged input planes through LDS again, so large
    // output planes over large input planes take eight (half the tiles, half the LDS fill traffic)
    p.ppt = (out_plane >= 2 * kThreads) ? 4 : 1;
    // (from 8192 output pixels on: fp16 N16 C128 96x96 -> 96x96 27.0 us with four, 22.1 with eight; 112x112 43.4 and
    // 28.4; fp32 N8 C128 96x96 34.7 and 25.1)
    if (p.cls >= 2 && out_plane >= 16 * kThreads) {
        p.ppt = 8;
    }
    if (a.interp == 2) {
        p.ppt = (out_plane >= 4 * kThreads) ? 2 : 1;  // sixteen tap offsets per pixel live in registers
    }
    // Two neighbouring pixels per lane and store for 16-bit elements: needs every output plane to start on a 4-byte
    // boundary and to hold whole pairs (fp16 N16 C256 64x64: 128-byte stores 17.1 us, 256-byte stores 16.2 us, and the
    // lanes of a wavefront then read taps two columns apart, which halves the LDS bank conflicts of a smooth grid)
    // Not for border padding: coordinates clamped to the first or last column then put both pixels of a lane on one
    // bank, next to their neighbours' (same case, border: 18.0 us with single pixels, 21.6 us with pairs).
    if (esz == 2 && p.ppt >= 4 && a.interp != 2 && a.pad != 1 && out_plane % 2 == 0 &&
        reinterpret_cast<uintptr_t>(a.y) % 4 == 0) {
        p.adj = 2;
    }
    const int64_t tile = (int64_t)kThreads * p.ppt;
    p.tiles_per_n = (uint32_t)((out_plane + tile - 1) / tile);
    // channels per workgroup: as many stages as possible (the pixel decisions are reused across them) while
    // still giving the 256 CUs at least two workgroups each -- one each where the ring takes more than half of a
    // CU's LDS and a second workgroup could not be resident anyway (bf16 N8 C128 128x128 -> 256x256 random grid:
    // 95 us with 32 channels per workgroup, 87 us with 64)
    const int64_t want_blocks = (p.lds_bytes > kLdsLimit / 2) ? 256 : 512;
    const int64_t base = a.N * p.tiles_per_n;
    const int64_t max_cblocks = (a.C + cgs - 1) / cgs;
    // Enough channel blocks to reach that count, or one block fewer where the count would spill into a second round
    // of workgroups: the cost of a choice is rounds times channels per block (fp16 N16 C128 96x96, 80 (item, tile)
    // pairs, one workgroup per CU: four channel blocks are 320 workgroups, a round and a quarter, 36.5 us; three are
    // 240).
    int64_t cblocks = 1, cpb = a.C;
    {
        int64_t best_cost = INT64_MAX;
        const int64_t up = (want_blocks + base - 1) / base;
        for (int64_t cand = up; cand >= up - 1; cand--) {
            int64_t cb = cand > max_cblocks ? max_cblocks : cand;
            cb = cb < 1 ? 1 : cb;
            int64_t per = (a.C + cb - 1) / cb;
            per = (per + cgs - 1) / cgs * cgs;
            // (16-bit bilinear and bicubic: an even count lets the kernel take two channels per stage; worth one more channel
            // where a block has eight or more)
            if (esz == 2 && a.interp != 1 && per >= 8 && per % 2 != 0 && a.C % 2 == 0) {
                per++;
            }
            cb = (a.C + per - 1) / per;
            const int64_t rounds = (base * cb + want_blocks - 1) / want_blocks;
            const int64_t cost = rounds * per;
            if (cost < best_cost) {
                best_cost = cost;
                cblocks = cb;
                cpb = per;
            }
        }
    }
    // Bicubic samples with two pixels per lane: sixteen tap offsets and sixteen tap values per pixel leave the CU room
    // for one workgroup of this kernel (87 registers a lane), so 512 workgroups run as two rounds of 256, and every
    // round pays the decisions of its pixels.  Where one workgroup per CU divides the channels evenly, that is the
    // launch: fp16 N16 C256 64x64 -> 64x64 in channel pairs 29.1 -> 25.3 us (reflection 36.7 -> 31.9), N16 C128
    // 64x128 33.3 -> 29.3, 128x64 33.7 -> 30.4.  (Other counts keep the finer blocks, which balance better than a
    // round and a fraction: N16 C256 72x72, 176 (item, tile) pairs, 63.3 us with three blocks against 77.1 with two.)
    // Likewise the bilinear channel pairs of the 16 KiB class (eight pixels per lane, 106 registers; the condition is
    // the one under which the plan below takes them): bf16 N8 C128 64x128 -> 128x256 22.3 -> 18.7 us, fp16 N16 C128
    // 38.7 -> 34.7, fp16 N16 C64 96x64 -> 256x128 20.9 -> 17.8.
    const bool large_pairs = esz == 2 && a.interp == 0 && p.cls == 2 && p.ppt == 8 && out_plane >= 2 * a.Hin * a.Win;
    if ((a.interp == 2 && p.ppt == 2 && cgs == 1) || large_pairs) {
        const int64_t cus = compute_unit_count();
        if (base <= cus && cus % base == 0 && a.C % (cus / base) == 0) {
            cblocks = cus / base;
            cpb = a.C / cblocks;
        }
    }
    p.chans_per_block = (int32_t)cpb;
    p.cblocks = (uint32_t)cblocks;
    if (a.N * p.tiles_per_n * cblocks > INT32_MAX) {
        return p;
    }
    // Exactly two workgroups per CU: the one that reaches a CU first keeps ahead of the one that joins it for the
    // whole kernel (its wavefronts are the older ones wherever the CU arbitrates), after which the CU runs half empty.
    // The launch hands out workgroups in index order and channel blocks are numbered with the index
    // (gs2d_lds_kernel.hpp), so the lower half of the channel blocks are those first workgroups and take more
    // channels than the upper half.  fp16 N16 C256 64x64, channels in contiguous ranges: 13.9 us with 16 + 16, 13.3
    // with 19 + 13, 12.9 with 20 + 12 (the stage rates measured while both ran were 2.2 and 1.45 per microsecond).
    // With the channels dealt out in turn (below) and the loaders' literal-count loop: 13.2 us with 16 + 16, 12.9
    // with 20 + 12, 12.5 with 22 + 10, 12.6 with 24 + 8, 13.1 with 26 + 6.
    // A wrong guess about who comes first costs balance, never correctness.
    if (cgs == 1 && cblocks % 2 == 0 && cpb >= 8 && a.C == cblocks * cpb &&
        a.N * p.tiles_per_n * cblocks == 2 * (int64_t)compute_unit_count() && (a.N * cblocks / 2) % 8 == 0) {
        int64_t wide = plain ? (cpb * 11 + 4) / 8 : (cpb * 5 + 2) / 4;
        // 16-bit bilinear and bicubic samples: even counts on both sides, so that the kernel can take two channels per
        // stage (below).  fp16 N16 C128 64x64 -> 64x64, eight channels per block on average: 11 + 5 in single stages
        // 7.9 us, 10 + 6 in pairs 7.4, 12 + 4 in pairs 7.1; bicubic 29.7, 19.6 and 19.5.
        if (esz == 2 && a.interp != 1 && plain && cpb % 2 == 0 && wide % 2 != 0 && a.force_variant != kGsRingSingle) {
            wide++;
        }
        const int64_t narrow = 2 * cpb - wide;
        if (narrow >= 1) {
            p.wide_blocks = (uint32_t)(cblocks / 2);
            p.chans_wide = (int32_t)wide;
            p.chans_per_block = (int32_t)narrow;
        }
    }
    // Channels dealt out to the channel blocks in turn rather than in contiguous ranges (single-plane stages, whole
    // aligned planes, every block's count exact): at any moment the workgroups of a batch item then read neighbouring
    // planes and write neighbouring planes, instead of sixteen streams 160 KB apart (fp16 N16 C256 64x64: 13.4 ->
    // 13.0 us before the split above was set again, 12.5 with it).
    if (cgs == 1 && plain && cblocks > 1 && a.C == cblocks * cpb) {
        p.chan_stride = (int32_t)cblocks;
    }
    p.copy_gran = plain ? 16 : 2;  // 2: 16-byte units in the shifted layout
    // Bank-spreading layout (gs2d_lds_kernel.hpp): rows of exactly 128 bytes, 16-byte copy granule.  Only for
    // border padding, where clamped coordinates pile up on the first and last column (one bank in the plain
    // layout).  Elsewhere the plain layout is the better one: the bank then depends on x alone and the lanes of a
    // wavefront have different x.
    if (a.pad == 1 && p.copy_gran == 16 && lds_row_bytes == 128) {
        p.row_shift = 7 | (2 << 8);  // rows of 128 bytes, rotated by two chunks per row
    }
    // all tiles of one (n, channel block) group on one XCD: needs the group count to be a multiple of 8
    p.xcd_swizzle = ((a.N * cblocks) % 8 == 0) ? 1 : 0;
    // Two channels per stage, interleaved in LDS (gs2d_lds_kernel.hpp, CHANNEL_PAIRS): bilinear samples of 16-bit
    // elements in the 8 KiB class with four pixels per lane, plain layout (rows padded or not), every block's channels
    // in pairs.
    {
        const int64_t last_block = a.C - (int64_t)(cblocks - 1) * cpb;
        const bool even_counts = p.wide_blocks != 0 ? (p.chans_wide % 2 == 0 && p.chans_per_block % 2 == 0)
                                                    : (cpb % 2 == 0 && last_block % 2 == 0);
        // (bicubic: one or two pixels per lane, sixteen 4-byte reads per pixel for both channels)
        const bool small = p.cls == 1 && (a.interp == 2 ? p.ppt <= 2 : p.ppt == 4) && 2 * staged_bytes + 16 <= kPairsPitch;
        // The 16 KiB class where there are at least two output pixels per input pixel (eight pixels per lane then):
        // fp16 N16 C128 96x64 -> 192x128 45.0 us with single channels, 29.3 in pairs (the pair layout of
        // gs2d_pair.hip: 55.8), bf16 N8 C128 64x128 -> 128x256 26.1 and 22.3 (24.4).  One output pixel per input
        // pixel is the loaders' game, and theirs is the better one with the copy engine: 96x64 -> 96x64 24.0 and 27.1.
        const bool large = p.cls == 2 && p.ppt == 8 && 2 * staged_bytes + 16 <= kPairsPitchLarge &&
                           out_plane >= 2 * a.Hin * a.Win;
        // (bicubic in that class: one or two pixels per lane again, whatever the output's size -- the LDS reads set the
        // pace there, not the loaders: fp16 N16 C256 96x80 -> 96x80 100.0 -> 63.7 us, border 181.9 -> 80.2; N16 C128
        // 128x64 57.5 -> 33.7; rows of 80 elements padded to 128 in this class rather than interleaved as they are in
        // the smaller one: 48x80 35.4 -> 32.6, 40x88 42.4 -> 31.4, border 37.3 -> 41.5 and 42.3 -> 37.5)
        const bool large_bicubic = a.interp == 2 && p.cls == 2 && p.ppt <= 2 && 2 * staged_bytes + 16 <= kPairsPitchLarge;
        if (a.interp != 1 && esz == 2 && (small || (large && a.interp == 0) || large_bicubic) && plain && p.copy_gran == 16 && a.C % 2 == 0 &&
            even_counts && a.force_variant != kGsRingSingle) {
            p.chan_pairs = true;
            p.pairs_pitch = small ? kPairsPitch : kPairsPitchLarge;
            p.lds_bytes = (uint32_t)(kPairsNbuf * p.pairs_pitch);
            if (p.row_shift != 0) {
                // an element is four bytes wide here: one chunk per row shifts a column by eight banks, as two do in
                // the single-channel layout
                p.row_shift = 7 | (1 << 8);
            }
        }
    }
    if (padded && !p.chan_pairs) {
        // Only the loaders' literal-count loop pads rows; what it asks for (gs2d_lds_kernel.hpp): single-plane
        // stages, every block with at least as many channels as the ring runs ahead, and a copy count per loader
        // that the loop is instantiated for.
        const int64_t last_block = a.C - (cblocks - 1) * cpb;  // channels of the last block (contiguous ranges)
        int64_t fewest = p.wide_blocks != 0 ? p.chans_per_block : (last_block < cpb ? last_block : cpb);
        const int64_t copies = ((staged_bytes + 1023) / 1024 + kLoaderWaves[p.cls] - 1) / kLoaderWaves[p.cls];
        if (cgs != 1 || fewest < kNbuf[p.cls] - 1 || copies > 16 || (kNbuf[p.cls] - 2) * copies > 63) {
            return p;
        }
    }
    p.ok = true;
    return p;
}

const char* gs2d_lds_variant_name(const GridSamplerArgs& a)
{
    const LdsPlan p = make_lds_plan(a);
    if (!p.ok) {
        return nullptr;
    }
    static const char* names[5] = {"lds_ring_p2064_4x4", "lds_ring_p8208_1x6", "lds_ring_p16400_1x4",
                                   "lds_ring_p32784_1x4", "lds_ring_p81904_1x2"};
    return p.chan_pairs ? (p.pairs_pitch == kPairsPitch ? "lds_ring_pairs_p16400_2x2" : "lds_ring_pairs_p32784_2x2")
                        : names[p.cls];
}

bool gs2d_lds_channel_pairs(const GridSamplerArgs& a)
{
    const LdsPlan p = make_lds_plan(a);
    return p.ok && p.chan_pairs;
}

int64_t gs2d_lds_channel_pairs_per_block(const GridSamplerArgs& a)
{
    const LdsPlan p = make_lds_plan(a);
    return (p.ok && p.chan_pairs) ? a.C / (int64_t)p.cblocks : 0;
}

hipError_t run_gs2d_lds(const GridSamplerArgs& a, hipStream_t stream, bool* handled)
{
    *handled = false;
    const LdsPlan p = make_lds_plan(a);
    if (!p.ok) {
        return hipSuccess;
    }
    *handled = true;
    if (p.chan_pairs) {
        return lds_launch_channel_pairs(a, p, stream);
    }
    const bool shifted = p.copy_gran == 2;
    switch (a.elem) {
        case Elem::F32:
            return shifted ? lds_launch_typed<float, true>(a, p, stream) : lds_launch_typed<float, false>(a, p, stream);
        case Elem::F16:
            return shifted ? lds_launch_typed<_Float16, true>(a, p, stream)
                           : lds_launch_typed<_Float16, false>(a, p, stream);
        case Elem::BF16:
            return shifted ? lds_launch_typed<__bf16, true>(a, p, stream)
                           : lds_launch_typed<__bf16, false>(a, p, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
