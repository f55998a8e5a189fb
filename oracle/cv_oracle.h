/*
 * CPU oracle for the bilinear gather/interpolate path (TEST INFRASTRUCTURE ONLY).
 *
 * This library restates, in plain C, the arithmetic of the reference kernels so that the
 * HIP kernels can be checked against it.  It is the checker, never the product: nothing
 * under the shipped package may include, link or load it.  Only the test-suite, the smoke
 * entry and the benchmark's "cpu_baseline" leg call it.
 *
 * Reference sources followed (paths relative to the reference tree):
 *   grid sample : image/grid_sampler2_d/op_kernel/arch35/grid_sampler2_d_simt.h (bilinear, nearest, bicubic)
 *   upsample    : image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_simt_nchw.h
 *   scale rules : image/resize_bilinear_v2/op_host/arch35/resize_bilinear_v2_tiling_arch35.cpp:175-243
 *
 * Pinning status of each exported function is listed in cv_oracle.c's header comment.
 */
#ifndef CV_ORACLE_H_
#define CV_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type codes shared by every oracle entry point */
enum { ORACLE_F32 = 0, ORACLE_F16 = 1, ORACLE_BF16 = 2 };

/* ---- scalar building blocks (exported so that tests can pin each one separately) ---- */
float oracle_half_to_float(uint16_t h);
uint16_t oracle_float_to_half(float f);
float oracle_bf16_to_float(uint16_t h);
uint16_t oracle_float_to_bf16(float f);

float oracle_unnormalize(float coord, int32_t size, int32_t align_corners);
float oracle_clip_coordinates(float coord, int32_t size);
float oracle_reflect_coordinates(float coord, float low, float twice_span);
float oracle_compute_source_index(float coord, int32_t size, int32_t padding_mode, int32_t align_corners);
float oracle_safe_downgrade(float x);
int32_t oracle_banker_round(float x);

/*
 * Per-pixel tap record of the grid sampler: what the kernel decides before the channel loop.
 * bilinear: ix0/iy0 = north-west corner, w[4] = nw,ne,sw,se weights, flag = 1 when the pixel
 * is written as NaN (non-finite source coordinate).  nearest: ix0/iy0 = the selected texel,
 * w unused (0), flag = 0.
 */
typedef struct {
    int32_t ix0;
    int32_t iy0;
    float w[4];
    int32_t flag;
} oracle_gs_tap;

/*
 * Per-pixel record of the bicubic mode (grid_sampler2_d_simt.h:375-403): the four tap columns and rows after
 * padding (-1 = outside), the four column and row coefficients, flag = 1 when the pixel is written as NaN.
 */
typedef struct {
    int32_t bx[4];
    int32_t by[4];
    float cx[4];
    float cy[4];
    int32_t flag;
} oracle_gs_bicubic_tap;

float oracle_compute_coordinates(float coord, int32_t size, int32_t padding_mode, int32_t align_corners);
float oracle_cubic_convolution1(float x, float a);
float oracle_cubic_convolution2(float x, float a);
int oracle_grid_sampler2d_bicubic_taps(const void* grid, oracle_gs_bicubic_tap* taps, int dtype, int64_t N,
                                       int64_t Hin, int64_t Win, int64_t Hout, int64_t Wout, int padding_mode,
                                       int align_corners);

/* ---- whole-tensor entry points; all tensors contiguous, NCHW, grid is (N,Ho,Wo,2) ---- */

/* returns 0 on success, <0 on invalid arguments */
int oracle_grid_sampler2d(const void* x, const void* grid, void* y, int dtype, int64_t N, int64_t C, int64_t Hin,
                          int64_t Win, int64_t Hout, int64_t Wout, int interp_mode, int padding_mode,
                          int align_corners, int num_threads);

/* fills taps[N*Hout*Wout]; same decision code as oracle_grid_sampler2d */
int oracle_grid_sampler2d_taps(const void* grid, oracle_gs_tap* taps, int dtype, int64_t N, int64_t Hin,
                               int64_t Win, int64_t Hout, int64_t Wout, int interp_mode, int padding_mode,
                               int align_corners);

/* scale handed to the kernel for one axis (align_corners / user scale / size ratio) */
float oracle_resize_scale(int64_t len_src, int64_t len_dst, int align_corners, float user_scale);

/*
 * The reference picks between two NCHW interpolating templates by the output size and the number of vector cores of
 * its device (image/resize_bilinear_v2/op_host/arch35/resize_bilinear_v2_tiling_arch35.cpp:606-615): from
 * cores * 1024 output pixels per plane on, the H*W-split template
 * (image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_simt_hw.h:76-97), which takes the fraction from the
 * unclamped source coordinate.  oracle_set_reference_cores sets the core count (default 64, that of the reference's
 * tiling unit test); oracle_resize_uses_hw_split tells which template oracle_upsample_bilinear2d restates for a shape.
 */
void oracle_set_reference_cores(int64_t cores);
int oracle_resize_uses_hw_split(int64_t N, int64_t C, int64_t Hs, int64_t Ws, int64_t Hd, int64_t Wd);

/* scales_h / scales_w are the user-facing multipliers (0 = derive from sizes) */
int oracle_upsample_bilinear2d(const void* x, void* y, int dtype, int64_t N, int64_t C, int64_t Hs, int64_t Ws,
                               int64_t Hd, int64_t Wd, int align_corners, double scales_h, double scales_w,
                               int num_threads);

/*
 * nearest-neighbour resize with align_corners = false and half_pixel_centers = false, scale = in / out:
 * src = min(floor(float(dst) * scale), in - 1)
 * (image/resize_nearest_neighbor_v2/op_kernel/arch35/resize_nearest_neighbor_v2_simt.h:103-124, scale rule
 * image/resize_nearest_neighbor_v2/op_host/arch35/resize_nearest_neighbor_v2_tiling_base.cpp:253-263).
 * channels_last = 0: x is (N,C,Hs,Ws); 1: x is (N,Hs,Ws,C).
 * One of the reference's channels-last templates does not use that rule: for an upscale by whole factors with
 * enough channels and rows that fit its unified buffer it replicates every source pixel (src = dst / factor in
 * integer arithmetic, resize_nearest_neighbor_v2_data_copy_nhwc.h:110-111,205-231); the float rule first differs from
 * that at a factor of 41.  oracle_nearest_nhwc_schedule restates the choice
 * (resize_nearest_neighbor_v2_tiling_base.cpp:476-494,640-713; returns the schedule id of
 * resize_nearest_neighbor_v2_tiling_key.h, 6-8 are the replicating template) for the core count of
 * oracle_set_reference_cores and the buffer size of oracle_set_reference_ub_bytes (default 253952, that of the
 * reference's tiling UT); oracle_resize_nearest follows it for channels_last = 1.
 */
int oracle_resize_nearest(const void* x, void* y, int dtype, int64_t N, int64_t C, int64_t Hs, int64_t Ws,
                          int64_t Hd, int64_t Wd, int channels_last);
int oracle_nearest_nhwc_schedule(int dtype, int64_t N, int64_t C, int64_t Hs, int64_t Ws, int64_t Hd, int64_t Wd);
void oracle_set_reference_ub_bytes(int64_t bytes);

/*
 * Backward of the bilinear resize, deterministic gather formulation
 * (image/resize_bilinear_v2_grad/op_kernel/arch35/resize_bilinear_v2_grad_simt_determine.h:56-117; scales
 * image/resize_bilinear_v2_grad/op_host/arch35/resize_bilinear_v2_grad_tiling_arch35.cpp:352-394).
 * scales_h/scales_w > 0 (align_corners false) that differ from Hd/Hs, Wd/Ws follow the user-scale template
 * resize_bilinear_v2_grad_simt_determine_scales.h:77-305.
 * grads: (N,C,Hd,Wd) or channels_last (N,Hd,Wd,C), dtype_in; y: (N,C,Hs,Ws) / (N,Hs,Ws,C), dtype_out.
 */
int oracle_upsample_bilinear2d_backward(const void* grads, void* y, int dtype_in, int dtype_out, int64_t N, int64_t C,
                                        int64_t Hs, int64_t Ws, int64_t Hd, int64_t Wd, int align_corners,
                                        int channels_last, double scales_h, double scales_w);

/* per-axis tap table of the upsample: i0[len_dst], i1[len_dst], lambda[len_dst] */
int oracle_upsample_axis_taps(int64_t len_src, int64_t len_dst, int align_corners, float user_scale, int32_t* i0,
                              int32_t* i1, float* lambda);

/*
 * Point-copy template of the bilinear resize, channels-last (N,H,W,C) tensors
 * (image/resize_bilinear_v2/op_host/arch35/resize_bilinear_v2_tiling_arch35.cpp:254-303).  Returns 1 and fills y when
 * the template applies, else 0.
 */
int oracle_resize_point_copy(const void* x, void* y, int dtype, int64_t N, int64_t C, int64_t Hs, int64_t Ws,
                             int64_t Hd, int64_t Wd, int align_corners, double scales_h, double scales_w);

/*
 * Bilinear resize of channels-last tensors, x (N,Hs,Ws,C) -> y (N,Hd,Wd,C), with the reference's template choice for
 * that layout (image/resize_bilinear_v2/op_host/arch35/resize_bilinear_v2_tiling_arch35.cpp:592-623): the
 * channel-parallel template (image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_c_parallel.h:122-232) sums
 * four weighted taps where the per-element template (resize_bilinear_v2_simt_nhwc.h:60-150) nests two blends.
 * Returns the template used: 0 per-element, 1 all copy, 2 broadcast, 3 first pixel, 4 point copy, 5 channel-parallel.
 */
int oracle_upsample_bilinear2d_nhwc(const void* x, void* y, int dtype, int64_t N, int64_t C, int64_t Hs, int64_t Ws,
                                    int64_t Hd, int64_t Wd, int align_corners, double scales_h, double scales_w);

/*
 * Volumetric grid sampler, forward (image/grid_sample/op_kernel/arch35/grid_sampler_3d_bilinear_smit.h:146-191).
 * x (N,C,Din,Hin,Win), grid (N,Dout,Hout,Wout,3) ordered x,y,z, y (N,C,Dout,Hout,Wout); interp 0 bilinear,
 * 1 nearest (round half to even, image/grid_sample/op_kernel/grid_sampler_3d_nearest.h:569-571).
 */
float oracle_gs3d_unnormalize(float g, int32_t size, int32_t align_corners);
float oracle_gs3d_clip(float coord, int32_t size, int32_t padding_mode, int32_t align_corners);
int oracle_grid_sampler3d(const void* x, const void* grid, void* y, int dtype, int64_t N, int64_t C, int64_t Din,
                          int64_t Hin, int64_t Win, int64_t Dout, int64_t Hout, int64_t Wout, int interp, int pad,
                          int align, int threads);

/*
 * Backward of grid_sampler2d in the accumulation order of the reference's deterministic mode
 * (image/grid_sampler2_d_grad/op_kernel/arch35/grid_sampler2_d_grad_simt_det.h).  gout (N,C,Ho,Wo), x (N,C,H,W),
 * grid (N,Ho,Wo,2); dx (N,C,H,W) and dgrid (N,Ho,Wo,2) may each be NULL.
 */
int oracle_grid_sampler2d_backward(const void* gout, const void* x, const void* grid, void* dx, void* dgrid,
                                   int dtype, int64_t N, int64_t C, int64_t H, int64_t W, int64_t Ho, int64_t Wo,
                                   int interp, int pad, int align);

/*
 * Backward of the 3-D grid sampler in the accumulation order of the reference's deterministic mode
 * (image/grid_sampler3_d_grad/op_kernel/arch35/grid_sampler3_d_grad_simt_det.h).  gout (N,C,Do,Ho,Wo),
 * x (N,C,D,H,W), grid (N,Do,Ho,Wo,3) ordered x,y,z; dx (N,C,D,H,W) and dgrid (N,Do,Ho,Wo,3) may each be NULL.
 * interp 0 bilinear, 1 nearest.  The chunking follows oracle_set_reference_cores().
 */
int oracle_grid_sampler3d_backward(const void* gout, const void* x, const void* grid, void* dx, void* dgrid,
                                   int dtype, int64_t N, int64_t C, int64_t D, int64_t H, int64_t W, int64_t Do,
                                   int64_t Ho, int64_t Wo, int interp, int pad, int align);

/* Neighbouring implementations in the reference (not mirrored by any HIP kernel; see cv_oracle.c) */
int oracle_grid_sampler2d_arch35(const void* x, const void* grid, void* y, int dtype, int64_t N, int64_t C,
                                 int64_t Hin, int64_t Win, int64_t Hout, int64_t Wout, int padding_mode,
                                 int align_corners);
int oracle_upsample_a2_axis_taps(int64_t len_src, int64_t len_dst, int align_corners, float user_scale, int32_t* i0,
                                 int32_t* i1, float* l0, float* l1);
int oracle_upsample_bilinear2d_a2(const float* x, float* y, int64_t N, int64_t C, int64_t Hs, int64_t Ws, int64_t Hd,
                                  int64_t Wd, int align_corners);

int oracle_max_threads(void);

#ifdef __cplusplus
}
#endif

#endif /* CV_ORACLE_H_ */
