/*
 * aclnnUpsampleBilinear2dBackward -- two-phase C API, MI355X (gfx950) implementation.
 *
 * Drop-in for the reference interface image/resize_bilinear_v2_grad/op_api/aclnn_upsample_bilinear_2d_backward.h:20-35
 * (implementation image/resize_bilinear_v2_grad/op_api/aclnn_upsample_bilinear_2d_backward.cpp:48-312).
 *
 *   gradOut    : gradient of the upsampled tensor, (N,C,outH,outW) or, for NHWC tensors, (N,outH,outW,C)
 *   outputSize : {outH, outW}
 *   inputSize  : the four extents of the tensor that was upsampled, in the order of the tensors' format
 *   out        : gradient of that tensor (inputSize); same format as gradOut (NCHW or NHWC)
 *   dtypes     : FLOAT, FLOAT16, BF16; out has gradOut's dtype, except that a FLOAT gradOut may be reduced into
 *                a FLOAT16 or BF16 out (aclnn_upsample_bilinear_2d_backward.cpp:118-134)
 *
 * The kernel is the reference's deterministic formulation
 * (image/resize_bilinear_v2_grad/op_kernel/arch35/resize_bilinear_v2_grad_simt_determine.h:56-117): every element of
 * `out` gathers the gradOut elements whose bilinear footprint covers it, in a fixed order, accumulating in fp32 --
 * run-to-run reproducible, no atomics.  It is the template the reference's tiling picks for up-scaling
 * (resize_bilinear_v2_grad_tiling_arch35.cpp:457-468).  User scales (scalesH/scalesW > 0, align_corners false) that
 * differ from the ratio of the sizes run the reference's user-scale template
 * (resize_bilinear_v2_grad_simt_determine_scales.h:77-305).  Equal sizes copy gradOut to out.
 */
#ifndef OPSCV_ACLNN_UPSAMPLE_BILINEAR_2D_BACKWARD_H_
#define OPSCV_ACLNN_UPSAMPLE_BILINEAR_2D_BACKWARD_H_

#include "opscv_acl_base.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Phase 1 (host only, touches no device): validate, plan, report workspace bytes, hand out the executor. */
ACLNN_API aclnnStatus aclnnUpsampleBilinear2dBackwardGetWorkspaceSize(const aclTensor* gradOut,
                                                                      const aclIntArray* outputSize,
                                                                      const aclIntArray* inputSize, bool alignCorners,
                                                                      double scalesH, double scalesW, aclTensor* out,
                                                                      uint64_t* workspaceSize,
                                                                      aclOpExecutor** executor);

/* Phase 2: enqueue the kernels on `stream` (a hipStream_t) and free the executor.  Asynchronous. */
ACLNN_API aclnnStatus aclnnUpsampleBilinear2dBackward(void* workspace, uint64_t workspaceSize,
                                                      aclOpExecutor* executor, aclrtStream stream);

#ifdef __cplusplus
}
#endif

#endif /* OPSCV_ACLNN_UPSAMPLE_BILINEAR_2D_BACKWARD_H_ */
