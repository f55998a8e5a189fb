/*
 * CPU oracle for the bilinear gather/interpolate path -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference arithmetic.  It is the checker for the HIP kernels
 * and the timed "cpu_baseline" of the benchmark; the shipped library never calls it.
 * Build: gcc -O2 -ffp-contract=off -fopenmp (see oracle/Makefile).  -ffp-contract=off is part
 * of the contract: the reference disables contraction file-wide and uses one explicit fmaf.
 *
 * Pinning status (how each function is checked by tests/, independent of this file's text):
 *   half/bf16 conversions        : exhaustive round trip over all 65536 patterns + numpy/torch casts
 *   oracle_unnormalize           : closed forms (g=-1,+1 -> -0.5,size-0.5 / 0,size-1), crafted fma-vs-mul point
 *   oracle_clip/reflect          : range/evenness/periodicity invariants + torch grid_sample at large |g|
 *   oracle_banker_round          : numpy rint on ties and near-ties
 *   oracle_grid_sampler2d        : known answers recorded for the reference's own example inputs
 *                                  (image/grid_sample/examples/test_aclnn_grid_sample2_d.cpp:96-98), identity
 *                                  grid of image/grid_sampler2_d/examples/arch35/test_geir_grid_sampler2_d.cpp:84-90,
 *                                  committed torch.nn.functional.grid_sample fixtures, live torch CPU comparison
 *   bicubic mode (interp 2)      : coefficient closed forms (t=0 -> 0,1,0,0; partition of unity; symmetry),
 *                                  identity grid, committed and live torch grid_sample(mode="bicubic") comparison,
 *                                  integer-coordinate samples reproduce the source pixel
 *   oracle_upsample_bilinear2d   : known answers for image/upsample_bilinear2d/examples/
 *                                  test_aclnn_upsample_bilinear2d.cpp:83-94, kernel-UT shapes (1,1,1,4)->(2,16),
 *                                  (3,16), committed torch interpolate fixtures, live torch CPU comparison
 *   oracle_resize_point_copy     : equals a strided numpy slice x[:, off::f, off::f, :] (off = 0 or (f-1)/2), equals the
 *                                  interpolating oracle on finite data (all weights there are exactly 0 or 1), and
 *                                  differs from it exactly where a sampled value is infinite (the formula multiplies
 *                                  it by its zero weight too)
 *   oracle_resize_nearest        : integer-factor upscales equal element repetition, committed and live
 *                                  torch interpolate(mode="nearest") comparison (bit-exact: a pure copy)
 *   oracle_nearest_nhwc_schedule : the strategies the reference's tiling UT names for its channels-last cases
 *                                  (test_resize_nearest_neighbor_v2_tiling.cpp, tests 03-07, 11, 14, 15, platform
 *                                  {64 cores, 253952 bytes}); the replicating rule it switches oracle_resize_nearest
 *                                  to: numpy repeat, and the one place it leaves the float rule (factor 41)
 *   oracle_upsample_bilinear2d_backward : adjointness with the forward oracle (<forward(x), g> = <x, backward(g)>),
 *                                  gradient mass conservation, x2 closed form, live torch autograd comparison
 *   oracle_grid_sampler3d        : identity grid reproduces the volume, a grid constant in z reduces to the 2-D
 *                                  sampler's geometry on one slice, reflection invariants, live torch
 *                                  grid_sample on 5-D inputs (both modes, all paddings); the reference's source
 *                                  does not fix whether its compiler contracts a*b+c in this file: restated with
 *                                  separate roundings, so bit-exactness to the reference is "parity unpinned",
 *                                  agreement with torch to 1e-5 is what is pinned
 *   oracle_grid_sampler2d_backward : live torch autograd of grid_sample (all modes, paddings, alignments; fp32 to
 *                                  1e-5), adjointness with the forward oracle (<forward(x), g> = <x, dx>), finite
 *                                  differences of the forward oracle for the grid gradient, the reference's example
 *                                  (examples/test_aclnn_grid_sampler2_d_backward.cpp) against torch.  The reference's
 *                                  source does not fix whether its compiler contracts a*b+c in these files and its
 *                                  default mode adds with atomics in arbitrary order: bit-level parity with the
 *                                  reference is "parity unpinned"; the accumulation order restated is that of its
 *                                  deterministic mode
 *   oracle_grid_sampler3d_backward : live torch autograd of grid_sample on 5-D inputs (both modes, all paddings
 *                                  and alignments; fp32 to 2e-5, both gradients), adjointness with the forward
 *                                  oracle, left-to-right sums in the element type for points piled on one voxel,
 *                                  with and without the chunk shift of several items per core.  Bit-level parity
 *                                  with the reference is "parity unpinned" for the reasons given for the 2-D
 *                                  backward; the accumulation order restated is that of its deterministic mode
 *   oracle_grid_sampler2d_arch35, oracle_upsample_a2_axis_taps, oracle_upsample_bilinear2d_a2 : restatements of two
 *                                  neighbouring implementations in the reference; the first is the checker of the
 *                                  library's second bilinear rule (option grid_sampler2d_rule = 1), the other two no
 *                                  HIP kernel follows (kept to show where they leave the mirrored kernels).  Pinned by closed forms (taps and
 *                                  weights at hand-computed coordinates, zero output for non-finite grid values,
 *                                  x2 upscale tap table) and by agreement with the mirrored oracle within tolerance
 *                                  on finite data
 *   oracle_resize_scale          : float bit patterns held by the reference's tiling UT
 *                                  (image/resize_bilinear_v2/tests/ut/op_host/arch35/test_resize_bilinear_v2_tiling.cpp)
 */
#include "cv_oracle.h"

#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------------------------
 * 16-bit float conversions (software, round-to-nearest-even; the reference converts through
 * __half2float/__float2half and static_cast: grid_sampler2_d_simt.h:84-102)
 * ---------------------------------------------------------------------------------------- */
static inline uint32_t f2u(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float u2f(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

float oracle_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) {
            return u2f(sign);
        }
        /* subnormal: value = man * 2^-24, exact in fp32 */
        float v = (float)man * 5.9604644775390625e-8f;
        return (sign != 0) ? -v : v;
    }
    if (exp == 31) {
        return u2f(sign | 0x7F800000u | (man << 13));
    }
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t oracle_float_to_half(float f)
{
    uint32_t u = f2u(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t abs = u & 0x7FFFFFFFu;
    if (abs >= 0x7F800000u) {
        if (abs > 0x7F800000u) {
            /* NaN: keep it a quiet NaN */
            return (uint16_t)(sign | 0x7E00u | ((abs >> 13) & 0x3FFu));
        }
        return (uint16_t)(sign | 0x7C00u);
    }
    if (abs >= 0x477FF000u) {
        /* >= 65520 rounds to infinity */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (abs < 0x38800000u) {
        /* result is subnormal (or zero): quantum is 2^-24 */
        if (abs < 0x33000000u) {
            /* < 2^-25 : rounds to zero (2^-25 itself ties to even = 0) */
            return sign;
        }
        uint32_t exp = abs >> 23;
        uint32_t man = (abs & 0x7FFFFFu) | 0x800000u;
        uint32_t shift = 126u - exp; /* 14..24 */
        uint32_t q = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) {
            q++;
        }
        return (uint16_t)(sign | q);
    }
    uint32_t man = abs & 0x7FFFFFu;
    uint32_t exp = (abs >> 23) - 112u;
    uint32_t q = (exp << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) {
        q++; /* carries into the exponent correctly */
    }
    return (uint16_t)(sign | q);
}

float oracle_bf16_to_float(uint16_t h) { return u2f((uint32_t)h << 16); }

uint16_t oracle_float_to_bf16(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
        return (uint16_t)((u >> 16) | 0x0040u);
    }
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

static inline float load_as_float(const void* p, int dtype, int64_t i)
{
    if (dtype == ORACLE_F32) {
        return ((const float*)p)[i];
    }
    if (dtype == ORACLE_F16) {
        return oracle_half_to_float(((const uint16_t*)p)[i]);
    }
    return oracle_bf16_to_float(((const uint16_t*)p)[i]);
}

static inline void store_from_float(void* p, int dtype, int64_t i, float v)
{
    if (dtype == ORACLE_F32) {
        ((float*)p)[i] = v;
    } else if (dtype == ORACLE_F16) {
        ((uint16_t*)p)[i] = oracle_float_to_half(v);
    } else {
        ((uint16_t*)p)[i] = oracle_float_to_bf16(v);
    }
}

/* ------------------------------------------------------------------------------------------
 * Grid sampler coordinate pipeline
 * ---------------------------------------------------------------------------------------- */

/* grid_sampler2_d_simt.h:125-132 : align -> ((g+1)/2)*(size-1); else ONE fused multiply-add */
float oracle_unnormalize(float coord, int32_t size, int32_t align_corners)
{
    if (align_corners != 0) {
        return ((coord + 1.0f) / 2.0f) * (float)(size - 1);
    }
    float scaling = (float)size / 2.0f;
    return fmaf(scaling, coord + 1.0f, -0.5f);
}

/* grid_sampler2_d_simt.h:136-143 */
float oracle_clip_coordinates(float coord, int32_t size)
{
    float max_val = (float)(size - 1);
    if (isnan(coord)) {
        return 0.0f;
    }
    return fminf(fmaxf(coord, 0.0f), max_val);
}

/* grid_sampler2_d_simt.h:171-185 : a - trunc(a/b)*b with product and difference rounded separately */
float oracle_reflect_coordinates(float coord, float low, float twice_span)
{
    if (twice_span == 0.0f) {
        return 0.0f;
    }
    float abs_in = fabsf(coord - low);
    float flips = truncf(abs_in / twice_span);
    float product = flips * twice_span;
    float extra = abs_in - product;
    float complement = twice_span - extra;
    return fminf(extra, complement) + low;
}

/* grid_sampler2_d_simt.h:187-200 */
float oracle_compute_coordinates(float coord, int32_t size, int32_t padding_mode, int32_t align_corners)
{
    if (padding_mode == 1) {
        coord = oracle_clip_coordinates(coord, size);
    } else if (padding_mode == 2) {
        if (align_corners != 0) {
            coord = oracle_reflect_coordinates(coord, 0.0f, 2.0f * (float)(size - 1));
        } else {
            coord = oracle_reflect_coordinates(coord, -0.5f, 2.0f * (float)size);
        }
        coord = oracle_clip_coordinates(coord, size);
    }
    return coord;
}

/* grid_sampler2_d_simt.h:202-207 */
float oracle_compute_source_index(float coord, int32_t size, int32_t padding_mode, int32_t align_corners)
{
    coord = oracle_unnormalize(coord, size, align_corners);
    return oracle_compute_coordinates(coord, size, padding_mode, align_corners);
}

/* grid_sampler2_d_simt.h:209-215 ; 2147483646.0f is 2^31 once rounded to fp32 */
float oracle_safe_downgrade(float x)
{
    if (x > 2147483646.0f || x < -2147483648.0f || isnan(x) || isinf(x)) {
        return -100.0f;
    }
    return x;
}

/* float -> int32 for values the guard above lets through; 2^31 itself saturates (it is out of
 * bounds for every legal tensor either way) */
static inline int32_t float_to_i32(float v)
{
    if (v >= 2147483648.0f) {
        return INT32_MAX;
    }
    if (v < -2147483648.0f) {
        return INT32_MIN;
    }
    return (int32_t)v;
}

/* grid_sampler2_d_simt.h:219-234 : round half to even built from floor, frac and parity */
int32_t oracle_banker_round(float x)
{
    float fl = floorf(x);
    float frac = x - fl;
    int32_t fi = float_to_i32(fl);
    if (frac < 0.5f) {
        return fi;
    }
    if (frac > 0.5f) {
        return (fi == INT32_MAX) ? fi : fi + 1;
    }
    if ((fi & 1) == 0) {
        return fi;
    }
    return (fi == INT32_MAX) ? fi : fi + 1;
}

static inline int within(int32_t h, int32_t w, int32_t H, int32_t W) { return h >= 0 && h < H && w >= 0 && w < W; }

/* the per-pixel decision of grid_sampler2_d_simt.h:479-498 (bilinear, nearest) */
static inline void gs_decide(float gx, float gy, int32_t Hin, int32_t Win, int interp, int pad, int align,
                             oracle_gs_tap* t)
{
    float ix = oracle_compute_source_index(gx, Win, pad, align);
    float iy = oracle_compute_source_index(gy, Hin, pad, align);
    t->flag = 0;
    t->w[0] = t->w[1] = t->w[2] = t->w[3] = 0.0f;
    if (interp == 0) {
        if (isnan(ix) || isinf(ix) || isnan(iy) || isinf(iy)) {
            t->flag = 1;
            t->ix0 = 0;
            t->iy0 = 0;
            return;
        }
        ix = oracle_safe_downgrade(ix);
        iy = oracle_safe_downgrade(iy);
        /* grid_sampler2_d_simt.h:307-316 */
        float ixf = floorf(ix);
        float iyf = floorf(iy);
        t->ix0 = float_to_i32(ixf);
        t->iy0 = float_to_i32(iyf);
        t->w[0] = (ixf + 1.0f - ix) * (iyf + 1.0f - iy);
        t->w[1] = (ix - ixf) * (iyf + 1.0f - iy);
        t->w[2] = (ixf + 1.0f - ix) * (iy - iyf);
        t->w[3] = (ix - ixf) * (iy - iyf);
    } else {
        ix = oracle_safe_downgrade(ix);
        iy = oracle_safe_downgrade(iy);
        t->ix0 = oracle_banker_round(ix);
        t->iy0 = oracle_banker_round(iy);
    }
}

/* ---- bicubic (A = -0.75) ---- */

/* grid_sampler2_d_simt.h:273-280 : every product, sum and difference rounded separately */
float oracle_cubic_convolution1(float x, float a)
{
    float t0 = (a + 2.0f) * x;
    float t1 = t0 - (a + 3.0f);
    float t2 = t1 * x;
    float t3 = t2 * x;
    return t3 + 1.0f;
}

/* grid_sampler2_d_simt.h:282-290 */
float oracle_cubic_convolution2(float x, float a)
{
    float t0 = a * x;
    float t1 = t0 - 5.0f * a;
    float t2 = t1 * x;
    float t3 = t2 + 8.0f * a;
    float t4 = t3 * x;
    return t4 - 4.0f * a;
}

/* grid_sampler2_d_simt.h:292-298 */
static inline int32_t safe_float_to_i32(float f)
{
    if (f >= 0.0f && f < 2147483648.0f) {
        return (int32_t)f;
    }
    return -1;
}

/* grid_sampler2_d_simt.h:362-371 : plain product, then three explicit fused multiply-adds */
static inline float bicubic_weighted_sum(float c0, float c1, float c2, float c3, float v0, float v1, float v2,
                                         float v3)
{
    float r = c0 * v0;
    r = fmaf(c1, v1, r);
    r = fmaf(c2, v2, r);
    r = fmaf(c3, v3, r);
    return r;
}

/* grid_sampler2_d_simt.h:499-503 (coordinates) and :379-412 (taps and coefficients) */
static inline void gs_decide_bicubic(float gx, float gy, int32_t Hin, int32_t Win, int pad, int align,
                                     oracle_gs_bicubic_tap* t)
{
    const float A = -0.75f;
    float ix = oracle_unnormalize(gx, Win, align);
    float iy = oracle_unnormalize(gy, Hin, align);
    memset(t, 0, sizeof(*t));
    if (isnan(ix) || isinf(ix) || isnan(iy) || isinf(iy)) {
        t->flag = 1;
        return;
    }
    float ixf = floorf(ix);
    float iyf = floorf(iy);
    float tx = ix - ixf;
    float ty = iy - iyf;
    for (int k = 0; k < 4; k++) {
        t->bx[k] = safe_float_to_i32(oracle_compute_coordinates(ixf + (float)(k - 1), Win, pad, align));
        t->by[k] = safe_float_to_i32(oracle_compute_coordinates(iyf + (float)(k - 1), Hin, pad, align));
    }
    t->cx[0] = oracle_cubic_convolution2(tx + 1.0f, A);
    t->cx[1] = oracle_cubic_convolution1(tx, A);
    t->cx[2] = oracle_cubic_convolution1(1.0f - tx, A);
    t->cx[3] = oracle_cubic_convolution2(2.0f - tx, A);
    t->cy[0] = oracle_cubic_convolution2(ty + 1.0f, A);
    t->cy[1] = oracle_cubic_convolution1(ty, A);
    t->cy[2] = oracle_cubic_convolution1(1.0f - ty, A);
    t->cy[3] = oracle_cubic_convolution2(2.0f - ty, A);
}

int oracle_grid_sampler2d_bicubic_taps(const void* grid, oracle_gs_bicubic_tap* taps, int dtype, int64_t N,
                                       int64_t Hin, int64_t Win, int64_t Hout, int64_t Wout, int padding_mode,
                                       int align_corners)
{
    if (padding_mode < 0 || padding_mode > 2 || dtype < 0 || dtype > 2) {
        return -1;
    }
    int64_t total = N * Hout * Wout;
    for (int64_t p = 0; p < total; p++) {
        float gx = load_as_float(grid, dtype, 2 * p);
        float gy = load_as_float(grid, dtype, 2 * p + 1);
        gs_decide_bicubic(gx, gy, (int32_t)Hin, (int32_t)Win, padding_mode, align_corners, &taps[p]);
    }
    return 0;
}

int oracle_grid_sampler2d_taps(const void* grid, oracle_gs_tap* taps, int dtype, int64_t N, int64_t Hin,
                               int64_t Win, int64_t Hout, int64_t Wout, int interp_mode, int padding_mode,
                               int align_corners)
{
    if (interp_mode < 0 || interp_mode > 1 || padding_mode < 0 || padding_mode > 2 || dtype < 0 || dtype > 2) {
        return -1;
    }
    int64_t total = N * Hout * Wout;
    for (int64_t p = 0; p < total; p++) {
        float gx = load_as_float(grid, dtype, 2 * p);
        float gy = load_as_float(grid, dtype, 2 * p + 1);
        gs_decide(gx, gy, (int32_t)Hin, (int32_t)Win, interp_mode, padding_mode, align_corners, &taps[p]);
    }
    return 0;
}

int oracle_grid_sampler2d(const void* x, const void* grid, void* y, int dtype, int64_t N, int64_t C, int64_t Hin,
                          int64_t Win, int64_t Hout, int64_t Wout, int interp_mode, int padding_mode,
                          int align_corners, int num_threads)
{
    if (interp_mode < 0 || interp_mode > 2 || padding_mode < 0 || padding_mode > 2 || dtype < 0 || dtype > 2) {
        return -1;
    }
    if (Hin <= 0 || Win <= 0 || Hin > INT32_MAX || Win > INT32_MAX) {
        return -2;
    }
    const int64_t total = N * Hout * Wout;
    const int64_t x_step = Hin * Win;
    const int64_t y_step = Hout * Wout;
    const int32_t H = (int32_t)Hin;
    const int32_t W = (int32_t)Win;
    (void)num_threads;
#ifdef _OPENMP
    if (num_threads <= 0) {
        num_threads = omp_get_max_threads();
    }
#pragma omp parallel for schedule(static) num_threads(num_threads)
#endif
    for (int64_t p = 0; p < total; p++) {
        /* pixel decode of grid_sampler2_d_simt.h:473-479 */
        int64_t hw = p / Wout;
        int64_t w_out = p - hw * Wout;
        int64_t n = hw / Hout;
        int64_t h_out = hw - n * Hout;
        float gx = load_as_float(grid, dtype, 2 * p);
        float gy = load_as_float(grid, dtype, 2 * p + 1);
        int64_t x_base = n * C * x_step;
        int64_t y_base = n * C * y_step + h_out * Wout + w_out;
        if (interp_mode == 2) {
            oracle_gs_bicubic_tap b;
            gs_decide_bicubic(gx, gy, H, W, padding_mode, align_corners, &b);
            if (b.flag) {
                for (int64_t c = 0; c < C; c++) {
                    store_from_float(y, dtype, y_base, NAN);
                    y_base += y_step;
                }
                continue;
            }
            /* grid_sampler2_d_simt.h:418-455 : a row outside the image contributes 0, a column outside reads 0 */
            for (int64_t c = 0; c < C; c++) {
                float r[4];
                for (int j = 0; j < 4; j++) {
                    r[j] = 0.0f;
                    if (b.by[j] >= 0 && b.by[j] < H) {
                        int64_t off = x_base + (int64_t)b.by[j] * W;
                        float v[4];
                        for (int k = 0; k < 4; k++) {
                            v[k] = (b.bx[k] >= 0 && b.bx[k] < W) ? load_as_float(x, dtype, off + b.bx[k]) : 0.0f;
                        }
                        r[j] = bicubic_weighted_sum(b.cx[0], b.cx[1], b.cx[2], b.cx[3], v[0], v[1], v[2], v[3]);
                    }
                }
                float out = bicubic_weighted_sum(b.cy[0], b.cy[1], b.cy[2], b.cy[3], r[0], r[1], r[2], r[3]);
                store_from_float(y, dtype, y_base, out);
                x_base += x_step;
                y_base += y_step;
            }
            continue;
        }
        oracle_gs_tap t;
        gs_decide(gx, gy, H, W, interp_mode, padding_mode, align_corners, &t);
        if (t.flag) {
            /* grid_sampler2_d_simt.h:236-247 */
            float nan_val = NAN;
            for (int64_t c = 0; c < C; c++) {
                store_from_float(y, dtype, y_base, nan_val);
                y_base += y_step;
            }
            continue;
        }
        if (interp_mode == 0) {
            /* grid_sampler2_d_simt.h:321-338 : taps added in nw, ne, sw, se order, each skipped when outside */
            int32_t x0 = t.ix0, y0 = t.iy0;
            int32_t x1 = (x0 == INT32_MAX) ? x0 : x0 + 1;
            int32_t y1 = (y0 == INT32_MAX) ? y0 : y0 + 1;
            int in_nw = within(y0, x0, H, W), in_ne = within(y0, x1, H, W);
            int in_sw = within(y1, x0, H, W), in_se = within(y1, x1, H, W);
            for (int64_t c = 0; c < C; c++) {
                float out = 0.0f;
                if (in_nw) {
                    out += load_as_float(x, dtype, x_base + (int64_t)y0 * W + x0) * t.w[0];
                }
                if (in_ne) {
                    out += load_as_float(x, dtype, x_base + (int64_t)y0 * W + x1) * t.w[1];
                }
                if (in_sw) {
                    out += load_as_float(x, dtype, x_base + (int64_t)y1 * W + x0) * t.w[2];
                }
                if (in_se) {
                    out += load_as_float(x, dtype, x_base + (int64_t)y1 * W + x1) * t.w[3];
                }
                store_from_float(y, dtype, y_base, out);
                x_base += x_step;
                y_base += y_step;
            }
        } else {
            /* grid_sampler2_d_simt.h:341-360 */
            int in = within(t.iy0, t.ix0, H, W);
            for (int64_t c = 0; c < C; c++) {
                float out = 0.0f;
                if (in) {
                    out = load_as_float(x, dtype, x_base + (int64_t)t.iy0 * W + t.ix0);
                }
                store_from_float(y, dtype, y_base, out);
                x_base += x_step;
                y_base += y_step;
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Upsample (resize_bilinear_v2, NCHW SIMT template)
 * ---------------------------------------------------------------------------------------- */

/* resize_bilinear_v2_tiling_arch35.cpp:175-184 (user scale -> reciprocal, else size ratio) and :228-243 */
float oracle_resize_scale(int64_t len_src, int64_t len_dst, int align_corners, float user_scale)
{
    if (align_corners == 0) {
        if (user_scale > 0.0f) {
            return 1.0f / user_scale;
        }
        return (float)len_src / (float)len_dst;
    }
    if (len_dst > 1) {
        return (float)(len_src - 1) / (float)(len_dst - 1);
    }
    return (float)len_src / (float)len_dst;
}

/* resize_bilinear_v2_simt_nchw.h:108-134 for one axis */
static inline void axis_tap(int64_t d, float scale, int half_pixel, int64_t len_src, int32_t* i0, int32_t* i1,
                            float* lambda)
{
    float orig;
    if (half_pixel) {
        orig = ((float)d + 0.5f) * scale - 0.5f;
    } else {
        orig = (float)d * scale;
    }
    if (orig < 0.0f) {
        orig = 0.0f;
    }
    float fl = floorf(orig);
    float lo = (orig > 0.0f) ? fl : 0.0f;
    float hi = (orig > 0.0f) ? ceilf(orig) : 0.0f;
    float last = (float)(len_src - 1);
    /* the reference assigns the float to an unsigned index and then clamps; clamping first is the
     * same for every in-range value and keeps the conversion defined for huge coordinates */
    int64_t a = (lo < last) ? (int64_t)lo : len_src - 1;
    int64_t b = (hi < last) ? (int64_t)hi : len_src - 1;
    *i0 = (int32_t)a;
    *i1 = (int32_t)b;
    *lambda = orig - fl;
}

/* The template for large NCHW outputs, one axis: resize_bilinear_v2_simt_hw.h:76-86.  The coordinate is not clamped at
 * zero before the fraction is taken.  floor and ceil are converted to the unsigned index type and capped at
 * len_src - 1; for the coordinates in [-0.5, 0) that half-pixel centres produce the floor is -1, whose conversion to
 * unsigned the language leaves undefined: taken as index 0, which is what the max(..., 0) written around it intends
 * (ceil is -0 -> 0 there). */
static inline void axis_tap_hw(int64_t d, float scale, int half_pixel, int64_t len_src, int32_t* i0, int32_t* i1,
                               float* lambda)
{
    const float offset = half_pixel ? 0.5f : 0.0f;
    const float orig = ((float)d + offset) * scale - offset;
    const float fl = floorf(orig), ce = ceilf(orig);
    const float last = (float)(len_src - 1);
    *i0 = (int32_t)((fl < 0.0f) ? 0 : ((fl < last) ? (int64_t)fl : len_src - 1));
    *i1 = (int32_t)((ce < 0.0f) ? 0 : ((ce < last) ? (int64_t)ce : len_src - 1));
    *lambda = orig - fl;
}

static int64_t g_reference_cores = 64;

/* Vector cores of the device the reference would run on (64 in the compile info of its tiling unit test); the NCHW
 * template choice depends on it: resize_bilinear_v2_tiling_arch35.cpp:606-615,877 */
void oracle_set_reference_cores(int64_t cores)
{
    g_reference_cores = cores > 0 ? cores : 64;
}

/* resize_bilinear_v2_tiling_arch35.cpp:592-595,606-615: 1 when the H*W-split template is chosen for an NCHW resize
 * that reached the interpolating templates */
int oracle_resize_uses_hw_split(int64_t N, int64_t C, int64_t Hs, int64_t Ws, int64_t Hd, int64_t Wd)
{
    const int64_t x_elems = N * C * Hs * Ws, y_elems = N * C * Hd * Wd;
    const int idx32 = y_elems < (int64_t)UINT32_MAX && x_elems < (int64_t)UINT32_MAX;
    const int64_t threshold = g_reference_cores * (idx32 ? 1024 : 512);
    return x_elems != 1 && (Ws != Wd || Hs != Hd) && Hd * Wd >= threshold;
}

int oracle_upsample_axis_taps(int64_t len_src, int64_t len_dst, int align_corners, float user_scale, int32_t* i0,
                              int32_t* i1, float* lambda)
{
    float scale = oracle_resize_scale(len_src, len_dst, align_corners, user_scale);
    for (int64_t d = 0; d < len_dst; d++) {
        axis_tap(d, scale, !align_corners, len_src, &i0[d], &i1[d], &lambda[d]);
    }
    return 0;
}

int oracle_upsample_bilinear2d(const void* x, void* y, int dtype, int64_t N, int64_t C, int64_t Hs, int64_t Ws,
                               int64_t Hd, int64_t Wd, int align_corners, double scales_h, double scales_w,
                               int num_threads)
{
    if (dtype < 0 || dtype > 2 || Hs <= 0 || Ws <= 0) {
        return -1;
    }
    const int64_t planes = N * C;
    const int64_t esz = (dtype == ORACLE_F32) ? 4 : 2;
    (void)num_threads;
#ifdef _OPENMP
    if (num_threads <= 0) {
        num_threads = omp_get_max_threads();
    }
#endif
    /* template selection of resize_bilinear_v2_tiling_arch35.cpp:592-623 + resize_bilinear_v2_apt.cpp:91-115:
     * same size -> copy; 1x1 source -> broadcast (always for align_corners, from 128 output bytes per plane
     * otherwise); 1x1 destination with align_corners -> element (0,0) */
    int mode = 0;
    if (Hs == Hd && Ws == Wd) {
        mode = 1;
    } else if (Hs == 1 && Ws == 1 && (align_corners || Hd * Wd * esz >= 128)) {
        mode = 2;
    } else if (Hd == 1 && Wd == 1 && align_corners) {
        mode = 3;
    }
    if (mode != 0) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(num_threads)
#endif
        for (int64_t pl = 0; pl < planes; pl++) {
            for (int64_t i = 0; i < Hd * Wd; i++) {
                int64_t src = (mode == 1) ? pl * Hs * Ws + i : pl * Hs * Ws;
                if (esz == 4) {
                    ((uint32_t*)y)[pl * Hd * Wd + i] = ((const uint32_t*)x)[src];
                } else {
                    ((uint16_t*)y)[pl * Hd * Wd + i] = ((const uint16_t*)x)[src];
                }
            }
        }
        return 0;
    }
    /* aclnn_upsample_bilinear_2d.cpp:411-412 narrows the user scales to float before they reach the tiling */
    const float scale_h = oracle_resize_scale(Hs, Hd, align_corners, (float)scales_h);
    const float scale_w = oracle_resize_scale(Ws, Wd, align_corners, (float)scales_w);
    const int half_pixel = !align_corners;
    const int64_t rows = planes * Hd;
    const int hw_split = oracle_resize_uses_hw_split(N, C, Hs, Ws, Hd, Wd);
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(num_threads)
#endif
    for (int64_t r = 0; r < rows; r++) {
        int64_t pl = r / Hd;
        int64_t h = r - pl * Hd;
        int32_t top, bottom;
        float dy;
        if (hw_split) {
            axis_tap_hw(h, scale_h, half_pixel, Hs, &top, &bottom, &dy);
        } else {
            axis_tap(h, scale_h, half_pixel, Hs, &top, &bottom, &dy);
        }
        const int64_t base = pl * Hs * Ws;
        for (int64_t w = 0; w < Wd; w++) {
            int32_t left, right;
            float dx;
            if (hw_split) {
                axis_tap_hw(w, scale_w, half_pixel, Ws, &left, &right, &dx);
            } else {
                axis_tap(w, scale_w, half_pixel, Ws, &left, &right, &dx);
            }
            float tl = load_as_float(x, dtype, base + (int64_t)top * Ws + left);
            float tr = load_as_float(x, dtype, base + (int64_t)top * Ws + right);
            float bl = load_as_float(x, dtype, base + (int64_t)bottom * Ws + left);
            float br = load_as_float(x, dtype, base + (int64_t)bottom * Ws + right);
            /* resize_bilinear_v2_simt_nchw.h:143-144 and resize_bilinear_v2_simt_hw.h:96-97 */
            float out = (1.0f - dy) * ((1.0f - dx) * tl + dx * tr) + dy * ((1.0f - dx) * bl + dx * br);
            store_from_float(y, dtype, r * Wd + w, out);
        }
    }
    return 0;
}

/* resize_nearest_neighbor_v2_simt.h:103-124 (the !align_corner && !half_pixel branch) */
static inline int64_t nearest_src(int64_t d, float scale, int64_t len_src)
{
    float f = floorf((float)d * scale);
    int64_t i = (int64_t)f;
    return (i < len_src - 1) ? i : len_src - 1;
}

static int64_t g_reference_ub_bytes = 253952;

void oracle_set_reference_ub_bytes(int64_t bytes)
{
    g_reference_ub_bytes = bytes > 0 ? bytes : 253952;
}

static int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

/* resize_nearest_neighbor_v2_tiling_base.cpp:640-665 (IsMatchTiling_NHWC_UB2UB), 476-494 (IsMatchTiling_NHWC) and
 * 667-713 (MatchTilingStrategyAndSetTilingKey) for a channels-last tensor with align_corners = half_pixel_centers =
 * false and no scales given, which is how aclnnResize calls the operator (aclnn_resize.cpp:278). */
int oracle_nearest_nhwc_schedule(int dtype, int64_t N, int64_t C, int64_t Hs, int64_t Ws, int64_t Hd, int64_t Wd)
{
    const int64_t esz = (dtype == ORACLE_F32) ? 4 : 2;
    const int64_t block = 32; /* bytes of a unified-buffer block */
    const int64_t ub = g_reference_ub_bytes, cores = g_reference_cores;
    const int aligned = (C * esz) % block == 0;                     /* :233-236 */
    const int64_t c_align = ceil_div64(C * esz, block) * block / esz; /* :237 */
    int ub2ub = 1;
    if (Wd <= Ws || Hd < Hs || Wd % Ws != 0 || Hd % Hs != 0) {
        ub2ub = 0; /* an upscale by whole factors only */
    } else if ((c_align * Ws * esz < 128 * 2 && c_align == C) || (C * esz < 128 && c_align != C)) {
        ub2ub = 0; /* few channels */
    } else if ((Ws + Wd) * c_align * esz * 2 > ub) {
        ub2ub = 0; /* a source row and an output row, double-buffered, do not fit */
    } else if (N * C * Hs * Ws >= (int64_t)UINT32_MAX || N * C * Hd * Wd >= (int64_t)UINT32_MAX) {
        ub2ub = 0;
    } else if (aligned && Wd * C * esz < 4096) {
        ub2ub = 0; /* short rows */
    }
    if (ub2ub) {
        const int64_t in_ub = Ws * c_align * esz * 2;
        const int64_t out_ub = (Hd / Hs) * Wd * c_align * esz * 2;
        int sch = (in_ub + out_ub <= ub) ? 6 : 7;
        const int64_t n_factor = ceil_div64(N, cores), n_cores = ceil_div64(N, n_factor);
        const int64_t h_factor = ceil_div64(Hs, cores), h_cores = ceil_div64(Hs, h_factor);
        if (n_cores < cores && h_cores < cores) {
            sch = 8;
        }
        return sch;
    }
    if (C * esz >= 128) {
        const int64_t max_ub_num = ((ub / 2) / block) * block / esz;
        if (aligned && (N * c_align < max_ub_num || C * esz < 256)) {
            return 2;
        }
        return (c_align <= max_ub_num) ? 0 : 1;
    }
    if (Hs == Hd && Ws == Wd) {
        return 4;
    }
    return (Hs == 1 && Ws == 1) ? 5 : 3;
}

int oracle_resize_nearest(const void* x, void* y, int dtype, int64_t N, int64_t C, int64_t Hs, int64_t Ws,
                          int64_t Hd, int64_t Wd, int channels_last)
{
    if (dtype < 0 || dtype > 2 || Hs <= 0 || Ws <= 0 || Hd <= 0 || Wd <= 0) {
        return -1;
    }
    const int64_t esz = (dtype == ORACLE_F32) ? 4 : 2;
    /* resize_nearest_neighbor_v2_tiling_base.cpp:257,262 */
    const float scale_h = (float)Hs / (float)Hd;
    const float scale_w = (float)Ws / (float)Wd;
    /* Schedules 6-8 replicate every source pixel Hd / Hs times down and Wd / Ws times across
     * (resize_nearest_neighbor_v2_data_copy_nhwc.h:110-111,205-231): output (h, w) is source (h / kh, w / kw) in
     * integer arithmetic, which floor(float(w) * scale) first misses at a factor of 41 (w = 41 gives 0). */
    int64_t rep_h = 0, rep_w = 0;
    if (channels_last) {
        const int sch = oracle_nearest_nhwc_schedule(dtype, N, C, Hs, Ws, Hd, Wd);
        if (sch >= 6 && sch <= 8) {
            rep_h = Hd / Hs;
            rep_w = Wd / Ws;
        }
    }
    const char* src = (const char*)x;
    char* dst = (char*)y;
    for (int64_t n = 0; n < N; n++) {
        for (int64_t c = 0; c < C; c++) {
            for (int64_t h = 0; h < Hd; h++) {
                const int64_t sy = rep_h ? h / rep_h : nearest_src(h, scale_h, Hs);
                for (int64_t w = 0; w < Wd; w++) {
                    const int64_t sx = rep_w ? w / rep_w : nearest_src(w, scale_w, Ws);
                    int64_t so, dof;
                    if (channels_last) {
                        so = ((n * Hs + sy) * Ws + sx) * C + c;
                        dof = ((n * Hd + h) * Wd + w) * C + c;
                    } else {
                        so = ((n * C + c) * Hs + sy) * Ws + sx;
                        dof = ((n * C + c) * Hd + h) * Wd + w;
                    }
                    memcpy(dst + dof * esz, src + so * esz, (size_t)esz);
                }
            }
        }
    }
    return 0;
}

/* resize_bilinear_v2_grad_tiling_arch35.cpp:352-394 (deterministic templates) */
static float grad_scale(int64_t len_src, int64_t len_dst, int align_corners, float user_scale)
{
    if (align_corners) {
        if (len_src > 1 && len_dst > 1) {
            return (float)(len_src - 1) / (float)(len_dst - 1);
        }
        return (float)len_src / (float)len_dst;
    }
    if (user_scale > 0.0f) {
        return 1.0f / user_scale;
    }
    return (float)len_src / (float)len_dst;
}

/* resize_bilinear_v2_grad_simt_determine_scales.h:55-63 */
static float grad_source_index(float scale, int64_t i, int half_pixel)
{
    return half_pixel ? scale * ((float)i + 0.5f) - 0.5f : scale * (float)i;
}

int oracle_upsample_bilinear2d_backward(const void* grads, void* y, int dtype_in, int dtype_out, int64_t N, int64_t C,
                                        int64_t Hs, int64_t Ws, int64_t Hd, int64_t Wd, int align_corners,
                                        int channels_last, double scales_h, double scales_w)
{
    if (dtype_in < 0 || dtype_in > 2 || dtype_out < 0 || dtype_out > 2 || Hs <= 0 || Ws <= 0 || Hd <= 0 || Wd <= 0) {
        return -1;
    }
    /* equal sizes: the entry point hands the incoming gradient on without running the operator, whatever the scales
     * (image/resize_bilinear_v2_grad/op_api/aclnn_upsample_bilinear_2d_backward.cpp:251-252; the operator's own
     * all-copy template says the same, resize_bilinear_v2_grad_tiling_arch35.cpp:310-313) */
    if (Hs == Hd && Ws == Wd && dtype_in == dtype_out) {
        memcpy(y, grads, (size_t)(N * C * Hs * Ws) * (size_t)((dtype_in == ORACLE_F32) ? 4 : 2));
        return 0;
    }
    const float scale_h = grad_scale(Hs, Hd, align_corners, (float)scales_h);
    const float scale_w = grad_scale(Ws, Wd, align_corners, (float)scales_w);
    const float inv_h = 1.0f / scale_h, inv_w = 1.0f / scale_w;
    const int half_pixel = !align_corners;
    const float offset = half_pixel ? 0.5f : 0.0f;
    /* template choice: resize_bilinear_v2_grad_tiling_arch35.cpp:422-436 */
    const int user_scales = !align_corners && (fabsf((float)Hs / (float)Hd - scale_h) >= 1.1920929e-7f ||
                                               fabsf((float)Ws / (float)Wd - scale_w) >= 1.1920929e-7f);
    for (int64_t n = 0; n < N; n++) {
        for (int64_t c = 0; c < C; c++) {
            for (int64_t H = 0; H < Hs; H++) {
                for (int64_t W = 0; W < Ws; W++) {
                    /* start of the walk: resize_bilinear_v2_grad_simt_determine.h:83-91 (both templates) */
                    float fy0 = ceilf(((float)H - 1.0f + offset) * inv_h - offset);
                    float fx0 = ceilf(((float)W - 1.0f + offset) * inv_w - offset);
                    int64_t in_y_start = (fy0 > 0.0f) ? (int64_t)fy0 : 0;
                    int64_t in_x_start = (fx0 > 0.0f) ? (int64_t)fx0 : 0;
                    float out_y_start = ((float)in_y_start + offset) * scale_h - offset;
                    float out_x_start = ((float)in_x_start + offset) * scale_w - offset;
                    /* first/last row or column: only in the user-scale template (…determine_scales.h:264-282) */
                    int hb = user_scales && (H == 0 || H == Hs - 1);
                    int wb = user_scales && (W == 0 || W == Ws - 1);
                    float acc = 0.0f;
                    float out_y = out_y_start;
                    int64_t in_y = in_y_start;
                    while ((hb || out_y < (float)H + 1.0f) && in_y < Hd) {
                        float out_x = out_x_start;
                        int64_t in_x = in_x_start;
                        while ((wb || out_x < (float)W + 1.0f) && in_x < Wd) {
                            int64_t gi = channels_last ? ((n * Hd + in_y) * Wd + in_x) * C + c
                                                       : ((n * C + c) * Hd + in_y) * Wd + in_x;
                            float g = load_as_float(grads, dtype_in, gi);
                            float yc = fmaxf(0.0f, fminf(out_y, (float)Hs - 1.0f));
                            float xc = fmaxf(0.0f, fminf(out_x, (float)Ws - 1.0f));
                            float y_lerp = 1.0f - fabsf(yc - (float)H);
                            float x_lerp = 1.0f - fabsf(xc - (float)W);
                            if (!hb && !wb) {
                                acc += g * y_lerp * x_lerp;
                            } else {
                                float yt = fminf(floorf(yc), (float)(Hs - 1));
                                float xt = fminf(floorf(xc), (float)(Ws - 1));
                                float lepy[2] = {y_lerp, yc - yt};
                                float lepx[2] = {x_lerp, xc - xt};
                                if (!hb) {
                                    for (int j = 0; j < 2; j++) {
                                        if (xt + (float)j == (float)W) {
                                            acc += g * lepx[j] * y_lerp;
                                        }
                                    }
                                } else if (!wb) {
                                    for (int i = 0; i < 2; i++) {
                                        if (yt + (float)i == (float)H) {
                                            acc += g * lepy[i] * x_lerp;
                                        }
                                    }
                                } else {
                                    for (int i = 0; i < 2; i++) {
                                        for (int j = 0; j < 2; j++) {
                                            if (yt + (float)i == (float)H && xt + (float)j == (float)W) {
                                                acc += g * lepx[j] * lepy[i];
                                            }
                                        }
                                    }
                                }
                            }
                            in_x++;
                            /* the plain template accumulates the coordinate, the user-scale one recomputes it */
                            out_x = user_scales ? grad_source_index(scale_w, in_x, half_pixel) : out_x + scale_w;
                        }
                        in_y++;
                        out_y = user_scales ? grad_source_index(scale_h, in_y, half_pixel) : out_y + scale_h;
                    }
                    int64_t yi = channels_last ? ((n * Hs + H) * Ws + W) * C + c : ((n * C + c) * Hs + H) * Ws + W;
                    store_from_float(y, dtype_out, yi, acc);
                }
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Point-copy template of the bilinear resize (channels-last only)
 *   selection: image/resize_bilinear_v2/op_host/arch35/resize_bilinear_v2_tiling_arch35.cpp:254-303
 *   indices  : image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_point_copy.h:117-124
 * Returns 1 and fills y (N,Hd,Wd,C) when the template applies, 0 when the interpolating templates apply.
 * ---------------------------------------------------------------------------------------- */
int oracle_resize_point_copy(const void* x, void* y, int dtype, int64_t N, int64_t C, int64_t Hs, int64_t Ws,
                             int64_t Hd, int64_t Wd, int align_corners, double scales_h, double scales_w)
{
    const int64_t esz = (dtype == ORACLE_F32) ? 4 : 2;
    if (Hs == Hd && Ws == Wd) {
        return 0; /* the all-copy template comes first */
    }
    if (C * esz < 128) {
        return 0;
    }
    const float scale_h = oracle_resize_scale(Hs, Hd, align_corners, (float)scales_h);
    const float scale_w = oracle_resize_scale(Ws, Wd, align_corners, (float)scales_w);
    if (scale_h < 1.0 || scale_w < 1.0) {
        return 0;
    }
    const int64_t fh = (int64_t)(scale_h + 1.1920928955078125e-7f);
    const int64_t fw = (int64_t)(scale_w + 1.1920928955078125e-7f);
    if (fabsf(scale_h - (float)fh) >= 1.1920928955078125e-7f || fabsf(scale_w - (float)fw) >= 1.1920928955078125e-7f) {
        return 0;
    }
    const int half_pixel = !align_corners;
    if (half_pixel && !(fh % 2 == 1 && fw % 2 == 1)) {
        return 0;
    }
    for (int64_t n = 0; n < N; n++) {
        for (int64_t h = 0; h < Hd; h++) {
            int64_t hs = half_pixel ? ((2 * h + 1) * fh - 1) / 2 : h * fh;
            hs = hs < Hs - 1 ? hs : Hs - 1;
            for (int64_t w = 0; w < Wd; w++) {
                int64_t ws = half_pixel ? ((2 * w + 1) * fw - 1) / 2 : w * fw;
                ws = ws < Ws - 1 ? ws : Ws - 1;
                memcpy((char*)y + ((n * Hd + h) * Wd + w) * C * esz, (const char*)x + ((n * Hs + hs) * Ws + ws) * C * esz,
                       (size_t)(C * esz));
            }
        }
    }
    return 1;
}

/* ------------------------------------------------------------------------------------------
 * Channels-last bilinear resize: x (N,Hs,Ws,C) -> y (N,Hd,Wd,C)
 *   template order : image/resize_bilinear_v2/op_host/arch35/resize_bilinear_v2_tiling_arch35.cpp:592-623
 *                    (all copy, point copy, broadcast from C * esz >= 128, channel-parallel from C * esz >= 128
 *                    and both scales >= 2, else the per-element template)
 *   channel-parallel arithmetic : image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_c_parallel.h:122-147
 *                    (taps and weights) and :190-232 (four products, top sum, bottom sum, total)
 *   per-element template : image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_simt_nhwc.h:60-150 with the
 *                    special cases picked in image/resize_bilinear_v2/op_kernel/resize_bilinear_v2_apt.cpp:117-142
 * Returns the template that produced y: 0 per-element, 1 all copy, 2 broadcast, 3 first pixel, 4 point copy,
 * 5 channel-parallel; -1 on bad arguments.
 * ---------------------------------------------------------------------------------------- */
int oracle_upsample_bilinear2d_nhwc(const void* x, void* y, int dtype, int64_t N, int64_t C, int64_t Hs, int64_t Ws,
                                    int64_t Hd, int64_t Wd, int align_corners, double scales_h, double scales_w)
{
    if (dtype < 0 || dtype > 2 || Hs <= 0 || Ws <= 0) {
        return -1;
    }
    const int64_t esz = (dtype == ORACLE_F32) ? 4 : 2;
    const int half_pixel = !align_corners;
    const float scale_h = oracle_resize_scale(Hs, Hd, align_corners, (float)scales_h);
    const float scale_w = oracle_resize_scale(Ws, Wd, align_corners, (float)scales_w);
    const int wide = C * esz >= 128;
    int mode = 0;
    if (Hs == Hd && Ws == Wd) {
        mode = 1;
    } else if (oracle_resize_point_copy(x, y, dtype, N, C, Hs, Ws, Hd, Wd, align_corners, scales_h, scales_w) == 1) {
        return 4;
    } else if (wide && Hs == 1 && Ws == 1) {
        mode = 2;
    } else if (wide && scale_w >= 2.0f && scale_h >= 2.0f) {
        mode = 5;
    } else if (!half_pixel && Hs == 1 && Ws == 1) {
        mode = 2;
    } else if (!half_pixel && Hd == 1 && Wd == 1) {
        mode = 3;
    }
    for (int64_t n = 0; n < N; n++) {
        for (int64_t h = 0; h < Hd; h++) {
            int32_t top, bottom;
            float dy;
            axis_tap(h, scale_h, half_pixel, Hs, &top, &bottom, &dy);
            for (int64_t w = 0; w < Wd; w++) {
                int32_t left, right;
                float dx;
                axis_tap(w, scale_w, half_pixel, Ws, &left, &right, &dx);
                const int64_t dst = ((n * Hd + h) * Wd + w) * C;
                if (mode >= 1 && mode <= 3) {
                    const int64_t src = (mode == 1) ? dst : n * Hs * Ws * C;
                    memcpy((char*)y + dst * esz, (const char*)x + src * esz, (size_t)(C * esz));
                    continue;
                }
                const int64_t tl_i = ((n * Hs + top) * Ws + left) * C, tr_i = ((n * Hs + top) * Ws + right) * C;
                const int64_t bl_i = ((n * Hs + bottom) * Ws + left) * C, br_i = ((n * Hs + bottom) * Ws + right) * C;
                if (mode == 5) {
                    /* c_parallel.h:122-142.  Its source position is not clamped at zero, which cannot matter: with a
                     * scale of two or more the position is at least 0.5 (half pixel) or 0 (otherwise); from there on
                     * "floor, then +1 when the fraction is positive" and floor/ceil name the same taps */
                    const float w_nw = (1.0f - dy) * (1.0f - dx);
                    const float w_ne = (1.0f - dy) * dx;
                    const float w_sw = dy * (1.0f - dx);
                    const float w_se = dy * dx;
                    for (int64_t c = 0; c < C; c++) {
                        float nw = load_as_float(x, dtype, tl_i + c) * w_nw;
                        float ne = load_as_float(x, dtype, tr_i + c) * w_ne;
                        float sw = load_as_float(x, dtype, bl_i + c) * w_sw;
                        float se = load_as_float(x, dtype, br_i + c) * w_se;
                        float sum_top = nw + ne;
                        float sum_bot = sw + se;
                        store_from_float(y, dtype, dst + c, sum_top + sum_bot);
                    }
                    continue;
                }
                for (int64_t c = 0; c < C; c++) {
                    float tl = load_as_float(x, dtype, tl_i + c);
                    float tr = load_as_float(x, dtype, tr_i + c);
                    float bl = load_as_float(x, dtype, bl_i + c);
                    float br = load_as_float(x, dtype, br_i + c);
                    /* resize_bilinear_v2_simt_nhwc.h:147-148 */
                    float out = (1.0f - dy) * ((1.0f - dx) * tl + dx * tr) + dy * ((1.0f - dx) * bl + dx * br);
                    store_from_float(y, dtype, dst + c, out);
                }
            }
        }
    }
    return mode;
}

/* ------------------------------------------------------------------------------------------
 * Volumetric grid sampler (5-D)
 *   image/grid_sample/op_kernel/arch35/grid_sampler_3d_bilinear_smit.h:53-135,146-191
 *   image/grid_sample/op_kernel/arch35/grid_sampler_bilinear_smit_common.h:37-94
 * The reference's index types are unsigned (uint32_t/uint64_t) for sizes and signed for the corner
 * indices; sizes here are positive int32 so (size - 1) converts to the same float.  Conversions the
 * reference leaves undefined (a float beyond the index type) are treated as out of bounds.
 * ---------------------------------------------------------------------------------------- */
static float gs3_clip_coordinates(float coord, int32_t size)
{
    coord = coord < 0 ? 0 : coord;
    coord = coord > (float)(size - 1) ? (float)size - 1 : coord;
    if (isnan(coord) || isinf(coord)) {
        return 0.0f;
    }
    return coord;
}

static float gs3_reflect_coordinates(float coord, int64_t twice_low, int64_t twice_high)
{
    if (twice_low == twice_high) {
        return 0;
    }
    float min = (float)twice_low / 2;
    float span = (float)(twice_high - twice_low) / 2;
    coord = fabsf(coord - min);
    float extra = fmodf(coord, span);
    float fl = floorf(coord / span);
    /* parity of the quotient: floats of 2^24 and more are even integers */
    int odd = (fl < 16777216.0f) && (((int64_t)fl) % 2 != 0);
    if (!odd) {
        return extra + min;
    }
    return span - extra + min;
}

float oracle_gs3d_clip(float coord, int32_t size, int32_t padding_mode, int32_t align_corners)
{
    if (padding_mode == 1) {
        coord = gs3_clip_coordinates(coord, size);
    } else if (padding_mode == 2) {
        if (align_corners) {
            coord = gs3_reflect_coordinates(coord, 0, 2 * ((int64_t)size - 1));
        } else {
            coord = gs3_reflect_coordinates(coord, -1, 2 * (int64_t)size - 1);
        }
        coord = gs3_clip_coordinates(coord, size);
    }
    if (!isfinite(coord)) {
        return -100.0f;
    }
    return coord;
}

float oracle_gs3d_unnormalize(float g, int32_t size, int32_t align_corners)
{
    if (align_corners == 1) {
        return (g + 1) / 2 * (float)(size - 1);
    }
    return ((g + 1) * (float)size - 1) / 2;
}

static int64_t gs3_index(float f)
{
    if (!(f >= -2147483648.0f && f < 2147483648.0f)) {
        return -1; /* outside every volume */
    }
    return (int64_t)f;
}

static float gs3_point_value(const void* x, int dtype, int64_t base, int64_t d, int64_t h, int64_t w, int64_t D,
                             int64_t H, int64_t W)
{
    if (d >= 0 && h >= 0 && w >= 0 && d < D && h < H && w < W) {
        return load_as_float(x, dtype, base + d * H * W + h * W + w);
    }
    return 0.0f;
}

int oracle_grid_sampler3d(const void* x, const void* grid, void* y, int dtype, int64_t N, int64_t C, int64_t Din,
                          int64_t Hin, int64_t Win, int64_t Dout, int64_t Hout, int64_t Wout, int interp, int pad,
                          int align, int threads)
{
    if (x == NULL || grid == NULL || y == NULL || dtype < 0 || dtype > 2 || interp < 0 || interp > 1 || pad < 0 ||
        pad > 2 || Din <= 0 || Hin <= 0 || Win <= 0) {
        return -1;
    }
    const int64_t out_vol = Dout * Hout * Wout;
    const int64_t in_vol = Din * Hin * Win;
    const int64_t points = N * out_vol;
    (void)threads;
#ifdef _OPENMP
    int nt = threads > 0 ? threads : omp_get_max_threads();
#pragma omp parallel for num_threads(nt) schedule(static)
#endif
    for (int64_t p = 0; p < points; p++) {
        const int64_t n = p / out_vol;
        const int64_t sp = p - n * out_vol;
        float gd = load_as_float(grid, dtype, 3 * p + 2);
        float gh = load_as_float(grid, dtype, 3 * p + 1);
        float gw = load_as_float(grid, dtype, 3 * p);
        gd = oracle_gs3d_clip(oracle_gs3d_unnormalize(gd, (int32_t)Din, align), (int32_t)Din, pad, align);
        gw = oracle_gs3d_clip(oracle_gs3d_unnormalize(gw, (int32_t)Win, align), (int32_t)Win, pad, align);
        gh = oracle_gs3d_clip(oracle_gs3d_unnormalize(gh, (int32_t)Hin, align), (int32_t)Hin, pad, align);
        for (int64_t c = 0; c < C; c++) {
            const int64_t base = (n * C + c) * in_vol;
            const int64_t yo = (n * C + c) * out_vol + sp;
            if (interp == 1) {
                float v = gs3_point_value(x, dtype, base, gs3_index(rintf(gd)), gs3_index(rintf(gh)),
                                          gs3_index(rintf(gw)), Din, Hin, Win);
                store_from_float(y, dtype, yo, v);
                continue;
            }
            float df = floorf(gd), hf = floorf(gh), wf = floorf(gw);
            float dd = gd - df, dh = gh - hf, dw = gw - wf;
            float v, wgt, acc;
            v = gs3_point_value(x, dtype, base, gs3_index(df), gs3_index(hf), gs3_index(wf), Din, Hin, Win);
            wgt = (1.0f - dw) * (1.0f - dh) * (1.0f - dd);
            acc = v * wgt;
            v = gs3_point_value(x, dtype, base, gs3_index(df), gs3_index(hf), gs3_index(wf + 1), Din, Hin, Win);
            wgt = dw * (1.0f - dh) * (1.0f - dd);
            acc += v * wgt;
            v = gs3_point_value(x, dtype, base, gs3_index(df), gs3_index(hf + 1), gs3_index(wf), Din, Hin, Win);
            wgt = (1.0f - dw) * dh * (1.0f - dd);
            acc += v * wgt;
            v = gs3_point_value(x, dtype, base, gs3_index(df), gs3_index(hf + 1), gs3_index(wf + 1), Din, Hin, Win);
            wgt = dw * dh * (1.0f - dd);
            acc += v * wgt;
            v = gs3_point_value(x, dtype, base, gs3_index(df + 1), gs3_index(hf), gs3_index(wf), Din, Hin, Win);
            wgt = (1.0f - dw) * (1.0f - dh) * dd;
            acc += v * wgt;
            v = gs3_point_value(x, dtype, base, gs3_index(df + 1), gs3_index(hf), gs3_index(wf + 1), Din, Hin, Win);
            wgt = dw * (1.0f - dh) * dd;
            acc += v * wgt;
            v = gs3_point_value(x, dtype, base, gs3_index(df + 1), gs3_index(hf + 1), gs3_index(wf), Din, Hin, Win);
            wgt = (1.0f - dw) * dh * dd;
            acc += v * wgt;
            v = gs3_point_value(x, dtype, base, gs3_index(df + 1), gs3_index(hf + 1), gs3_index(wf + 1), Din, Hin,
                                Win);
            wgt = dw * dh * dd;
            acc += v * wgt;
            store_from_float(y, dtype, yo, acc);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Backward of grid_sampler2d, deterministic mode
 *   image/grid_sampler2_d_grad/op_kernel/arch35/grid_sampler2_d_grad_simt_det.h:75-413
 *   image/grid_sampler3_d_grad/op_kernel/arch35/grid_sampler3_d_grad_simt_base.h:50-311
 * Several intermediates of the reference live in the tensor's element type T; rt() rounds to it.
 * The reference assigns whole batch items to a core (one per core while N does not exceed the core
 * count) and walks the item's grid points in chunks of 256 threads; per chunk, channel and tap a
 * single thread adds the 256 staged contributions in thread order, each add in T.  That loop nest is
 * restated literally below.  Adds of a staged zero to element 0 for taps outside the image
 * (grid_sampler2_d_grad_simt_det.h:86-88,93-97) are left out: they can only turn a -0 into +0.
 * ---------------------------------------------------------------------------------------- */
static float rt(int dtype, float v)
{
    if (dtype == ORACLE_F16) {
        return oracle_half_to_float(oracle_float_to_half(v));
    }
    if (dtype == ORACLE_BF16) {
        return oracle_bf16_to_float(oracle_float_to_bf16(v));
    }
    return v;
}

static float gsg_unnormalize(int dtype, float coord, int32_t size, int align, float* mult)
{
    float c;
    if (align == 1) {
        c = (coord + 1) / 2 * (float)(size - 1);
        *mult = rt(dtype, (float)(size - 1) / 2);
    } else {
        c = ((coord + 1) * (float)size - 1) / 2;
        *mult = rt(dtype, (float)size / 2);
    }
    return rt(dtype, c);
}

static float gsg_clip(int dtype, float coord, int32_t limit, float* g)
{
    if (coord <= 0.0f) {
        *g = 0.0f;
        return 0.0f;
    }
    float max = rt(dtype, (float)(limit - 1));
    if (coord >= max) {
        *g = 0.0f;
        return max;
    }
    *g = 1.0f;
    return coord;
}

static float gsg_reflect(int dtype, float coord, int64_t twice_low, int64_t twice_high, float* g)
{
    if (twice_low == twice_high) {
        *g = 0.0f;
        return 0.0f;
    }
    float mult;
    float min = (float)twice_low / 2;
    float span = (float)(twice_high - twice_low) / 2;
    coord = rt(dtype, coord - min);
    if (coord < 0.0f) {
        mult = -1.0f;
        coord = -coord;
    } else {
        mult = 1.0f;
    }
    float extra = fmodf(coord, span);
    float fl = floorf(coord / span);
    int odd = (fl < 16777216.0f) && (((int64_t)fl) % 2 != 0);
    if (!odd) {
        *g = mult;
        return rt(dtype, extra + min);
    }
    *g = -mult;
    return rt(dtype, span - extra + min);
}

static float gsg_source_index(int dtype, float coord, int32_t size, int pad, int align, float* mult)
{
    float gc = 0, gr = 0;
    coord = gsg_unnormalize(dtype, coord, size, align, mult);
    if (pad == 1) {
        coord = gsg_clip(dtype, coord, size, &gc);
        *mult = rt(dtype, *mult * gc);
    } else if (pad == 2) {
        if (align) {
            coord = gsg_reflect(dtype, coord, 0, 2 * ((int64_t)size - 1), &gr);
        } else {
            coord = gsg_reflect(dtype, coord, -1, 2 * (int64_t)size - 1, &gr);
        }
        coord = gsg_clip(dtype, coord, size, &gc);
        *mult = rt(dtype, *mult * gr * gc);
    }
    if (!isfinite(coord)) {
        return -100.0f;
    }
    return coord;
}

static int32_t gsg_to_i32(float f)
{
    if (f >= 2147483648.0f) {
        return INT32_MAX;
    }
    if (f < -2147483648.0f) {
        return INT32_MIN;
    }
    return (int32_t)f;
}

/* plane offset of a bicubic tap after padding, -1 outside (simt_base.h:249-311, simt_det.h:239-277) */
static int64_t gsg_bounded(float x, float y, int32_t W, int32_t H, int pad, int align)
{
    if (pad == 0) {
        if (x < 0 || x >= (float)W || y < 0 || y >= (float)H) {
            return -1;
        }
    } else if (pad == 1) {
        x = x < 0 ? 0 : (x >= (float)W ? (float)W - 1 : x);
        y = y < 0 ? 0 : (y >= (float)H ? (float)H - 1 : y);
    } else {
        float g;
        if (align) {
            x = gsg_reflect(ORACLE_F32, x, 0, 2 * ((int64_t)W - 1), &g);
            y = gsg_reflect(ORACLE_F32, y, 0, 2 * ((int64_t)H - 1), &g);
        } else {
            x = gsg_reflect(ORACLE_F32, x, -1, 2 * (int64_t)W - 1, &g);
            y = gsg_reflect(ORACLE_F32, y, -1, 2 * (int64_t)H - 1, &g);
        }
        x = gsg_clip(ORACLE_F32, x, W, &g);
        y = gsg_clip(ORACLE_F32, y, H, &g);
    }
    int32_t ix = gsg_to_i32(isfinite(x) ? x : -100.0f);
    int32_t iy = gsg_to_i32(isfinite(y) ? y : -100.0f);
    if (ix >= 0 && ix < W && iy >= 0 && iy < H) {
        return (int64_t)iy * W + ix;
    }
    return -1;
}

static void gsg_cubic_coeffs(float c[4], float t)
{
    c[0] = oracle_cubic_convolution2(t + 1.0f, -0.75f);
    c[1] = oracle_cubic_convolution1(t, -0.75f);
    c[2] = oracle_cubic_convolution1(1.0f - t, -0.75f);
    c[3] = oracle_cubic_convolution2(2.0f - t, -0.75f);
}

static void gsg_cubic_coeffs_grad(float c[4], float t)
{
    float A = -0.75f;
    float x = t + 1.0f;
    c[0] = (3.0f * A * x - 10.0f * A) * x + 8.0f * A;
    x = t;
    c[1] = (3.0f * (A + 2.0f) * x - 2.0f * (A + 3.0f)) * x;
    x = 1.0f - t;
    c[2] = -((3.0f * (A + 2.0f) * x - 2.0f * (A + 3.0f)) * x);
    x = 2.0f - t;
    c[3] = -((3.0f * A * x - 10.0f * A) * x + 8.0f * A);
}

#define GSG_CHUNK 256

int oracle_grid_sampler2d_backward(const void* gout, const void* x, const void* grid, void* dx, void* dgrid,
                                   int dtype, int64_t N, int64_t C, int64_t H, int64_t W, int64_t Ho, int64_t Wo,
                                   int interp, int pad, int align)
{
    if (gout == NULL || x == NULL || grid == NULL || dtype < 0 || dtype > 2 || interp < 0 || interp > 2 || pad < 0 ||
        pad > 2 || H <= 0 || W <= 0) {
        return -1;
    }
    const int64_t points = Ho * Wo, plane = H * W;
    if (dx != NULL) {
        for (int64_t i = 0; i < N * C * plane; i++) {
            store_from_float(dx, dtype, i, 0.0f);
        }
    }
    /* staged contributions of one chunk: [tap][thread] */
    static _Thread_local int64_t st_idx[16][GSG_CHUNK];
    static _Thread_local float st_val[16][GSG_CHUNK];
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic)
#endif
    for (int64_t n = 0; n < N; n++) {
        for (int64_t base = 0; base < points; base += GSG_CHUNK) {
            const int64_t cnt = (points - base < GSG_CHUNK) ? points - base : GSG_CHUNK;
            float gix[GSG_CHUNK], giy[GSG_CHUNK], mx[GSG_CHUNK], my[GSG_CHUNK];
            for (int64_t t = 0; t < cnt; t++) {
                gix[t] = giy[t] = 0.0f;
            }
            for (int64_t c = 0; c < C; c++) {
                const int64_t xin = (n * C + c) * plane;
                int ntaps = 0;
                for (int64_t t = 0; t < cnt; t++) {
                    const int64_t p = base + t;
                    float fx = load_as_float(grid, dtype, (n * points + p) * 2);
                    float fy = load_as_float(grid, dtype, (n * points + p) * 2 + 1);
                    const float go = load_as_float(gout, dtype, (n * C + c) * points + p);
                    if (interp == 2) {
                        fy = gsg_unnormalize(dtype, fy, (int32_t)H, align, &my[t]);
                        fx = gsg_unnormalize(dtype, fx, (int32_t)W, align, &mx[t]);
                        float xf = floorf(fx), yf = floorf(fy);
                        float cx[4], cy[4], cxg[4], cyg[4];
                        gsg_cubic_coeffs(cy, fy - yf);
                        gsg_cubic_coeffs(cx, fx - xf);
                        gsg_cubic_coeffs_grad(cyg, fy - yf);
                        gsg_cubic_coeffs_grad(cxg, fx - xf);
                        ntaps = 16;
                        for (int i = 0; i < 4; i++) {
                            for (int j = 0; j < 4; j++) {
                                float nx = xf - 1 + i;
                                float ny = yf - 1 + j;
                                float weight = cx[i] * cy[j];
                                float delta = go * weight;
                                int64_t o = gsg_bounded(nx, ny, (int32_t)W, (int32_t)H, pad, align);
                                st_idx[i * 4 + j][t] = o;
                                st_val[i * 4 + j][t] = rt(dtype, delta);
                                float val = (o >= 0) ? load_as_float(x, dtype, xin + o) : 0.0f;
                                giy[t] += val * cyg[j] * cx[i] * go;
                                gix[t] += val * cxg[i] * cy[j] * go;
                            }
                        }
                        continue;
                    }
                    fy = gsg_source_index(dtype, fy, (int32_t)H, pad, align, &my[t]);
                    fx = gsg_source_index(dtype, fx, (int32_t)W, pad, align, &mx[t]);
                    if (interp == 1) {
                        int32_t xi = gsg_to_i32(rintf(fx)), yi = gsg_to_i32(rintf(fy));
                        ntaps = 1;
                        st_idx[0][t] = (yi >= 0 && xi >= 0 && yi < H && xi < W) ? (int64_t)yi * W + xi : -1;
                        st_val[0][t] = rt(dtype, go);
                        continue;
                    }
                    int32_t x0 = gsg_to_i32(floorf(fx)), y0 = gsg_to_i32(floorf(fy));
                    int32_t x1 = (x0 == INT32_MAX) ? x0 : x0 + 1, y1 = (y0 == INT32_MAX) ? y0 : y0 + 1;
                    float tnw = rt(dtype, ((float)x1 - fx) * ((float)y1 - fy));
                    float tne = rt(dtype, (fx - (float)x0) * ((float)y1 - fy));
                    float tsw = rt(dtype, ((float)x1 - fx) * (fy - (float)y0));
                    float tse = rt(dtype, (fx - (float)x0) * (fy - (float)y0));
                    const int32_t cxs[4] = {x0, x1, x0, x1}, cys[4] = {y0, y0, y1, y1};
                    const float ws[4] = {tnw, tne, tsw, tse};
                    ntaps = 4;
                    for (int k = 0; k < 4; k++) {
                        const int in = cys[k] >= 0 && cxs[k] >= 0 && cys[k] < H && cxs[k] < W;
                        st_idx[k][t] = in ? (int64_t)cys[k] * W + cxs[k] : -1;
                        st_val[k][t] = rt(dtype, ws[k] * go);
                    }
                    if (st_idx[0][t] >= 0) {
                        float v = load_as_float(x, dtype, xin + st_idx[0][t]);
                        gix[t] -= v * ((float)y1 - fy) * go;
                        giy[t] -= v * ((float)x1 - fx) * go;
                    }
                    if (st_idx[1][t] >= 0) {
                        float v = load_as_float(x, dtype, xin + st_idx[1][t]);
                        gix[t] += v * ((float)y1 - fy) * go;
                        giy[t] -= v * (fx - (float)x0) * go;
                    }
                    if (st_idx[2][t] >= 0) {
                        float v = load_as_float(x, dtype, xin + st_idx[2][t]);
                        gix[t] -= v * (fy - (float)y0) * go;
                        giy[t] += v * ((float)x1 - fx) * go;
                    }
                    if (st_idx[3][t] >= 0) {
                        float v = load_as_float(x, dtype, xin + st_idx[3][t]);
                        gix[t] += v * (fy - (float)y0) * go;
                        giy[t] += v * (fx - (float)x0) * go;
                    }
                }
                /* thread 0 of the reference: tap after tap, 256 sequential adds in the element type */
                if (dx != NULL) {
                    for (int k = 0; k < ntaps; k++) {
                        for (int64_t t = 0; t < cnt; t++) {
                            if (st_idx[k][t] >= 0) {
                                const int64_t e = xin + st_idx[k][t];
                                store_from_float(dx, dtype, e, load_as_float(dx, dtype, e) + st_val[k][t]);
                            }
                        }
                    }
                }
            }
            if (dgrid != NULL) {
                for (int64_t t = 0; t < cnt; t++) {
                    const int64_t o = (n * points + base + t) * 2;
                    if (interp == 1) {
                        store_from_float(dgrid, dtype, o, 0.0f);
                        store_from_float(dgrid, dtype, o + 1, 0.0f);
                    } else {
                        store_from_float(dgrid, dtype, o, mx[t] * gix[t]);
                        store_from_float(dgrid, dtype, o + 1, my[t] * giy[t]);
                    }
                }
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Backward of the 3-D grid sampler, deterministic mode
 *   image/grid_sampler3_d_grad/op_kernel/arch35/grid_sampler3_d_grad_simt_det.h:63-398
 *   image/grid_sampler3_d_grad/op_host/grid_sampler3_d_grad_tiling.cpp:175-192 (items per core)
 * A core owns `per_core` whole batch items (1 while N does not exceed the core count, else
 * ceil(N / cores)) and walks their grid points as one run of indices in chunks of 256 threads, so the
 * chunk boundaries inside the second and later items of a core are shifted by (item * points) mod 256.
 * Per chunk, channel and corner (tnw, tne, tsw, tse, bnw, bne, bsw, bse) one thread adds the staged
 * contributions in thread order, each add in the element type.  Staged zeros added to element 0 for
 * corners outside the volume are left out (they can only turn a -0 into +0).
 * ---------------------------------------------------------------------------------------- */
int oracle_grid_sampler3d_backward(const void* gout, const void* x, const void* grid, void* dx, void* dgrid,
                                   int dtype, int64_t N, int64_t C, int64_t D, int64_t H, int64_t W, int64_t Do,
                                   int64_t Ho, int64_t Wo, int interp, int pad, int align)
{
    if (gout == NULL || x == NULL || grid == NULL || dtype < 0 || dtype > 2 || interp < 0 || interp > 1 || pad < 0 ||
        pad > 2 || D <= 0 || H <= 0 || W <= 0) {
        return -1;
    }
    const int64_t points = Do * Ho * Wo, vol = D * H * W;
    if (dx != NULL) {
        for (int64_t i = 0; i < N * C * vol; i++) {
            store_from_float(dx, dtype, i, 0.0f);
        }
    }
    const int64_t per_core = (N > g_reference_cores) ? (N + g_reference_cores - 1) / g_reference_cores : 1;
    static _Thread_local int64_t st_idx[8][GSG_CHUNK];
    static _Thread_local float st_val[8][GSG_CHUNK];
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic)
#endif
    for (int64_t n = 0; n < N; n++) {
        const int64_t phase = ((n % per_core) * points) % GSG_CHUNK; /* thread of the item's first point */
        for (int64_t base = -phase; base < points; base += GSG_CHUNK) {
            const int64_t t_lo = (base < 0) ? -base : 0;
            const int64_t t_hi = (points - base < GSG_CHUNK) ? points - base : GSG_CHUNK;
            float gi[3][GSG_CHUNK], mult[3][GSG_CHUNK];
            for (int64_t t = t_lo; t < t_hi; t++) {
                gi[0][t] = gi[1][t] = gi[2][t] = 0.0f;
            }
            for (int64_t c = 0; c < C; c++) {
                const int64_t xin = (n * C + c) * vol;
                const int ntaps = (interp == 1) ? 1 : 8;
                for (int64_t t = t_lo; t < t_hi; t++) {
                    const int64_t p = base + t;
                    float fx = load_as_float(grid, dtype, (n * points + p) * 3);
                    float fy = load_as_float(grid, dtype, (n * points + p) * 3 + 1);
                    float fz = load_as_float(grid, dtype, (n * points + p) * 3 + 2);
                    const float go = load_as_float(gout, dtype, (n * C + c) * points + p);
                    fx = gsg_source_index(dtype, fx, (int32_t)W, pad, align, &mult[0][t]);
                    fy = gsg_source_index(dtype, fy, (int32_t)H, pad, align, &mult[1][t]);
                    fz = gsg_source_index(dtype, fz, (int32_t)D, pad, align, &mult[2][t]);
                    if (interp == 1) {
                        int32_t zi = gsg_to_i32(rintf(fz)), yi = gsg_to_i32(rintf(fy)), xi = gsg_to_i32(rintf(fx));
                        const int in = zi >= 0 && yi >= 0 && xi >= 0 && zi < D && yi < H && xi < W;
                        st_idx[0][t] = in ? ((int64_t)zi * H + yi) * W + xi : -1;
                        st_val[0][t] = rt(dtype, go);
                        continue;
                    }
                    const int32_t x0 = gsg_to_i32(floorf(fx)), y0 = gsg_to_i32(floorf(fy)),
                                  z0 = gsg_to_i32(floorf(fz));
                    const int32_t x1 = (x0 == INT32_MAX) ? x0 : x0 + 1, y1 = (y0 == INT32_MAX) ? y0 : y0 + 1,
                                  z1 = (z0 == INT32_MAX) ? z0 : z0 + 1;
                    /* distance to the far corner per axis: index 0 weighs the low corner, 1 the high one */
                    const float wx[2] = {(float)x1 - fx, fx - (float)x0};
                    const float wy[2] = {(float)y1 - fy, fy - (float)y0};
                    const float wz[2] = {(float)z1 - fz, fz - (float)z0};
                    for (int k = 0; k < 8; k++) {
                        const int xs = k & 1, ys = (k >> 1) & 1, zs = k >> 2;
                        const int32_t cx = xs ? x1 : x0, cy = ys ? y1 : y0, cz = zs ? z1 : z0;
                        const int in = cz >= 0 && cy >= 0 && cx >= 0 && cz < D && cy < H && cx < W;
                        const float w = rt(dtype, wx[xs] * wy[ys] * wz[zs]);
                        st_idx[k][t] = in ? ((int64_t)cz * H + cy) * W + cx : -1;
                        st_val[k][t] = rt(dtype, w * go);
                        if (in) {
                            const float v = load_as_float(x, dtype, xin + st_idx[k][t]);
                            const float tx = v * wy[ys] * wz[zs] * go;
                            const float ty = v * wx[xs] * wz[zs] * go;
                            const float tz = v * wx[xs] * wy[ys] * go;
                            gi[0][t] = xs ? gi[0][t] + tx : gi[0][t] - tx;
                            gi[1][t] = ys ? gi[1][t] + ty : gi[1][t] - ty;
                            gi[2][t] = zs ? gi[2][t] + tz : gi[2][t] - tz;
                        }
                    }
                }
                if (dx != NULL) {
                    for (int k = 0; k < ntaps; k++) {
                        for (int64_t t = t_lo; t < t_hi; t++) {
                            if (st_idx[k][t] >= 0) {
                                const int64_t e = xin + st_idx[k][t];
                                store_from_float(dx, dtype, e, load_as_float(dx, dtype, e) + st_val[k][t]);
                            }
                        }
                    }
                }
            }
            if (dgrid != NULL) {
                for (int64_t t = t_lo; t < t_hi; t++) {
                    const int64_t o = (n * points + base + t) * 3;
                    for (int a = 0; a < 3; a++) {
                        store_from_float(dgrid, dtype, o + a, (interp == 1 || C == 0) ? 0.0f : mult[a][t] * gi[a][t]);
                    }
                }
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Two neighbouring implementations of the same operators in the reference, restated to show where their results
 * leave those of the kernels this library mirrors by default (tests/test_oracle.py).  The first is also the checker
 * of the library's second bilinear rule; no HIP kernel follows the second.
 * ---------------------------------------------------------------------------------------- */

/* The 2-D bilinear kernel of the reference's GridSample operator, which is what its aclnnGridSampler2D launches on
 * its newest part (aclnn_grid_sampler2d.cpp:321-324):
 *   image/grid_sample/op_kernel/arch35/grid_sampler_2d_bilinear_smit.h:56-153 and
 *   image/grid_sample/op_kernel/arch35/grid_sampler_bilinear_smit_common.h:36-90.
 * It differs from grid_sampler2_d_simt.h (the source mirrored by oracle_grid_sampler2d) in four places: the
 * unnormalisation is ((g + 1) * size - 1) / 2 instead of one fused multiply-add; reflection uses fmodf and the parity
 * of the quotient; a non-finite coordinate becomes -100 also for bilinear, so that the sample lies outside and the
 * output is 0 where the mirrored kernel writes NaN to every channel; and the weights are (1 - dh) * (1 - dw) with
 * dh = y - floor(y), a tap outside contributing value 0 times its weight. */
int oracle_grid_sampler2d_arch35(const void* x, const void* grid, void* y, int dtype, int64_t N, int64_t C,
                                 int64_t Hin, int64_t Win, int64_t Hout, int64_t Wout, int padding_mode,
                                 int align_corners)
{
    if (dtype < 0 || dtype > 2 || Hin <= 0 || Win <= 0 || padding_mode < 0 || padding_mode > 2) {
        return -1;
    }
    for (int64_t n = 0; n < N; n++) {
        for (int64_t h = 0; h < Hout; h++) {
            for (int64_t w = 0; w < Wout; w++) {
                const int64_t goff = ((n * Hout + h) * Wout + w) * 2;
                float gw = load_as_float(grid, dtype, goff);
                float gh = load_as_float(grid, dtype, goff + 1);
                gh = oracle_gs3d_unnormalize(gh, (int32_t)Hin, align_corners);
                gw = oracle_gs3d_unnormalize(gw, (int32_t)Win, align_corners);
                gw = oracle_gs3d_clip(gw, (int32_t)Win, padding_mode, align_corners);
                gh = oracle_gs3d_clip(gh, (int32_t)Hin, padding_mode, align_corners);
                const float hf = floorf(gh), wf = floorf(gw);
                const float dh = gh - hf, dw = gw - wf;
                const int64_t h0 = gs3_index(hf), w0 = gs3_index(wf);
                const int64_t h1 = gs3_index(hf + 1), w1 = gs3_index(wf + 1);
                for (int64_t c = 0; c < C; c++) {
                    const int64_t base = (n * C + c) * Hin * Win;
                    float v = gs3_point_value(x, dtype, base, 0, h0, w0, 1, Hin, Win);
                    float out = v * ((1.0f - dh) * (1.0f - dw));
                    v = gs3_point_value(x, dtype, base, 0, h0, w1, 1, Hin, Win);
                    out += v * ((1.0f - dh) * dw);
                    v = gs3_point_value(x, dtype, base, 0, h1, w0, 1, Hin, Win);
                    out += v * (dh * (1.0f - dw));
                    v = gs3_point_value(x, dtype, base, 0, h1, w1, 1, Hin, Win);
                    out += v * (dh * dw);
                    store_from_float(y, dtype, ((n * C + c) * Hout + h) * Wout + w, out);
                }
            }
        }
    }
    return 0;
}

/* Index and coefficient rule of the reference's matmul upsample kernel for its older parts, one axis:
 *   image/upsample_bilinear2d/op_kernel/upsample_bilinear2d_common.h:37-51 (getCenterValue, getLambda),
 *   image/upsample_bilinear2d/op_kernel/upsample_bilinear2d_kernel.h:299-318 (the coefficient matrices),
 *   scale: image/upsample_bilinear2d/op_host/upsample_bilinear2d_tiling.cpp:142-157.
 * src = scale * d (align_corners) or max(scale * (d + 0.5) - 0.5, 0); i0 = min(int(src), len - 1);
 * i1 = min(i0 + 1, len - 1); i0 == i1 -> coefficient 1 on i0, else l1 = clamp(src - i0, 0, 1), l0 = 1 - l1. */
int oracle_upsample_a2_axis_taps(int64_t len_src, int64_t len_dst, int align_corners, float user_scale, int32_t* i0,
                                 int32_t* i1, float* l0, float* l1)
{
    float scale;
    if (len_dst == len_src) {
        scale = 1.0f;
    } else if (align_corners) {
        scale = (len_dst > 1) ? (float)(len_src - 1) / (float)(len_dst - 1) : 0.0f;
    } else {
        scale = (user_scale > 0.0f) ? user_scale : (float)len_src / (float)len_dst;
    }
    for (int64_t d = 0; d < len_dst; d++) {
        float src;
        if (align_corners) {
            src = scale * (float)d;
        } else {
            src = scale * ((float)d + 0.5f) - 0.5f;
            src = (src > 0.0f) ? src : 0.0f;
        }
        int64_t a = (int64_t)src;
        a = (a < len_src - 1) ? a : len_src - 1;
        int64_t b = (a + 1 < len_src - 1) ? a + 1 : len_src - 1;
        i0[d] = (int32_t)a;
        i1[d] = (int32_t)b;
        if (a == b) {
            l0[d] = 1.0f;
            l1[d] = 0.0f;
        } else {
            float lam = src - (float)a;
            lam = (lam > 0.0f) ? lam : 0.0f;
            lam = (lam < 1.0f) ? lam : 1.0f;
            l1[d] = lam;
            l0[d] = 1.0f - lam;
        }
    }
    return 0;
}

/* The result of that kernel with its two taps per axis (fp32; width first, then height, as its two matrix products
 * go: upsample_bilinear2d_kernel.h:284-370).  The products with the zero entries of its banded coefficient
 * matrices are not modelled: they add nothing for finite data and make more outputs NaN for non-finite data. */
int oracle_upsample_bilinear2d_a2(const float* x, float* y, int64_t N, int64_t C, int64_t Hs, int64_t Ws, int64_t Hd,
                                  int64_t Wd, int align_corners)
{
    if (Hs <= 0 || Ws <= 0 || Hd <= 0 || Wd <= 0 || Hd > 65536 || Wd > 65536) {
        return -1;
    }
    static int32_t h0[65536], h1[65536], w0[65536], w1[65536];
    static float hl0[65536], hl1[65536], wl0[65536], wl1[65536];
    oracle_upsample_a2_axis_taps(Hs, Hd, align_corners, 0.0f, h0, h1, hl0, hl1);
    oracle_upsample_a2_axis_taps(Ws, Wd, align_corners, 0.0f, w0, w1, wl0, wl1);
    for (int64_t pl = 0; pl < N * C; pl++) {
        const float* xp = x + pl * Hs * Ws;
        for (int64_t i = 0; i < Hd; i++) {
            for (int64_t j = 0; j < Wd; j++) {
                float top = wl0[j] * xp[h0[i] * Ws + w0[j]];
                float bot = wl0[j] * xp[h1[i] * Ws + w0[j]];
                if (w1[j] != w0[j]) {
                    top += wl1[j] * xp[h0[i] * Ws + w1[j]];
                    bot += wl1[j] * xp[h1[i] * Ws + w1[j]];
                }
                float out = hl0[i] * top;
                if (h1[i] != h0[i]) {
                    out += hl1[i] * bot;
                }
                y[(pl * Hd + i) * Wd + j] = out;
            }
        }
    }
    return 0;
}

int oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
