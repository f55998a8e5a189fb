/*
 * aclnnGridSampler2DBackward -- two-phase C API, MI355X (gfx950) implementation.
 *
 * Drop-in for the reference interface
 * image/grid_sampler2_d_grad/op_host/op_api/aclnn_grid_sampler2d_backward.h:58-91 (implementation
 * image/grid_sampler2_d_grad/op_host/op_api/aclnn_grid_sampler2d_backward.cpp:214-357; device arithmetic
 * image/grid_sampler2_d_grad/op_kernel/arch35/grid_sampler2_d_grad_simt_det.h).
 *
 * Given gradOutput (N,C,Hout,Wout), input (N,C,Hin,Win) and grid (N,Hout,Wout,2) of one forward aclnnGridSampler2D
 * call, writes inputGrad (N,C,Hin,Win) when outputMask[0] and gridGrad (N,Hout,Wout,2) when outputMask[1].
 *   interpolationMode : 0 bilinear, 1 nearest (gridGrad is all zeros), 2 bicubic
 *   paddingMode       : 0 zeros, 1 border, 2 reflection
 *   dtypes            : FLOAT, FLOAT16, BF16 (all five tensors equal); DOUBLE is rejected with 161002
 *   outputMask        : exactly two flags; a NULL mask or two false flags make the call a successful no-op
 *   views             : arbitrary strides/offsets are honoured (packed through the workspace)
 * The result is deterministic: every element of inputGrad is the sum of its contributions in the order of the
 * reference's deterministic mode (grid points of a batch item in chunks of 256; per chunk tap after tap, per tap
 * point after point; every add rounded to the tensor's element type).
 * Validation order and status codes follow aclnn_grid_sampler2d_backward.cpp:195-240.
 */
#ifndef OPSCV_ACLNN_GRID_SAMPLER2D_BACKWARD_H_
#define OPSCV_ACLNN_GRID_SAMPLER2D_BACKWARD_H_

#include "opscv_acl_base.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Phase 1 (host only, touches no device): validate, plan, report workspace bytes, hand out the executor. */
ACLNN_API aclnnStatus aclnnGridSampler2DBackwardGetWorkspaceSize(const aclTensor* gradOutput, const aclTensor* input,
                                                                 const aclTensor* grid, int64_t interpolationMode,
                                                                 int64_t paddingMode, bool alignCorners,
                                                                 const aclBoolArray* outputMask, aclTensor* inputGrad,
                                                                 aclTensor* gridGrad, uint64_t* workspaceSize,
                                                                 aclOpExecutor** executor);

/* Phase 2: enqueue the kernels on `stream` (a hipStream_t) and free the executor.  Asynchronous. */
ACLNN_API aclnnStatus aclnnGridSampler2DBackward(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                 aclrtStream stream);

#ifdef __cplusplus
}
#endif

#endif /* OPSCV_ACLNN_GRID_SAMPLER2D_BACKWARD_H_ */
