/*
 * aclnnGridSampler2D -- two-phase C API, MI355X (gfx950) implementation.
 *
 * Drop-in for the reference interface image/grid_sample/op_api/aclnn_grid_sampler2d.h:53-82
 * (implementation image/grid_sample/op_api/aclnn_grid_sampler2d.cpp:263-351).
 *
 * out[n,c,h,w] = sample(input[n,c,:,:], grid[n,h,w,:]) with grid in normalized [-1,1] coordinates
 * (x first, then y).
 *   interpolationMode : 0 bilinear, 1 nearest, 2 bicubic (A = -0.75)
 *   paddingMode       : 0 zeros, 1 border, 2 reflection
 *   dtypes            : FLOAT, FLOAT16, BF16 (all three tensors equal); DOUBLE is rejected with 161002
 *   shapes            : input (N,C,Hin,Win), grid (N,Hout,Wout,2), out (N,C,Hout,Wout); formats are ignored
 *   views             : arbitrary strides/offsets are honoured (packed through the workspace)
 * Validation order and status codes follow aclnn_grid_sampler2d.cpp:159-175.
 *
 * Which of the reference's kernels the arithmetic follows: image/grid_sampler2_d/op_kernel/arch35/
 * grid_sampler2_d_simt.h (one fused multiply-add in the unnormalisation, non-finite source coordinates give NaN in
 * every channel for bilinear and bicubic, zero for nearest).  On its newest part the reference's own
 * aclnnGridSampler2D launches a different kernel for bilinear NCHW tensors (aclnn_grid_sampler2d.cpp:321-324 ->
 * image/grid_sample/op_kernel/arch35/grid_sampler_2d_bilinear_smit.h), which agrees with the one followed here within
 * the bilinear tolerance (1e-5 fp32, 1e-3 relative 16-bit) on finite grids but not beyond it in one case: a NaN or
 * infinite grid value under zeros padding gives 0 there (grid_sampler_bilinear_smit_common.h:67-90 turns every
 * non-finite coordinate into an out-of-range one) and NaN here.  It also unnormalises as ((g + 1) * size - 1) / 2,
 * which can pick the neighbouring pair of corner pixels for coordinates within an ulp of a pixel centre (results stay
 * within tolerance).
 *
 * A caller that replaces the reference library on that part and wants its results, non-finite grid values included,
 * selects that second kernel's arithmetic for the bilinear mode with the process-wide option "grid_sampler2d_rule" = 1
 * (opscvSetOption in opscv_ext.h, or OPSCV_GRID_SAMPLER2D_RULE=arch35 in the environment when the library is loaded):
 * unnormalisation ((g + 1) * size - 1) / 2, reflection with fmodf, every non-finite coordinate turned into -100 (a zero
 * sample), weights (1 - dh)(1 - dw) ..., grid_sampler_2d_bilinear_smit.h:67-153 and
 * grid_sampler_bilinear_smit_common.h:36-90.  The option is read by the first phase and kept in the executor; nearest
 * and bicubic are not affected (the reference serves them with other kernels on that part).  The default stays the
 * rule described above.
 */
#ifndef OPSCV_ACLNN_GRID_SAMPLER2D_H_
#define OPSCV_ACLNN_GRID_SAMPLER2D_H_

#include "opscv_acl_base.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Phase 1 (host only, touches no device): validate, plan, report workspace bytes, hand out the executor. */
ACLNN_API aclnnStatus aclnnGridSampler2DGetWorkspaceSize(const aclTensor* input, const aclTensor* grid,
                                                         int64_t interpolationMode, int64_t paddingMode,
                                                         bool alignCorners, aclTensor* out, uint64_t* workspaceSize,
                                                         aclOpExecutor** executor);

/* Phase 2: enqueue the kernels on `stream` (a hipStream_t) and free the executor.  Asynchronous. */
ACLNN_API aclnnStatus aclnnGridSampler2D(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                         aclrtStream stream);

#ifdef __cplusplus
}
#endif

#endif /* OPSCV_ACLNN_GRID_SAMPLER2D_H_ */
