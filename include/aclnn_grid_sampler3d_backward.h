/*
 * aclnnGridSampler3DBackward -- two-phase C API, MI355X (gfx950) implementation.
 *
 * Drop-in for the reference interface
 * image/grid_sampler3_d_grad/op_host/op_api/aclnn_grid_sampler3d_backward.h:24-36 (implementation
 * image/grid_sampler3_d_grad/op_host/op_api/aclnn_grid_sampler3d_backward.cpp:202-362; device arithmetic
 * image/grid_sampler3_d_grad/op_kernel/arch35/grid_sampler3_d_grad_simt_det.h).
 *
 * Given gradOutput (N,C,Dout,Hout,Wout), input (N,C,Din,Hin,Win) and grid (N,Dout,Hout,Wout,3; x, y, z) of one
 * forward aclnnGridSampler3D call, writes inputGrad (shape of input) when outputMask[0] and gridGrad (shape of grid)
 * when outputMask[1].
 *   interpolationMode : 0 bilinear (eight corners), 1 nearest (gridGrad is all zeros)
 *   paddingMode       : 0 zeros, 1 border, 2 reflection
 *   dtypes            : FLOAT, FLOAT16, BF16 (all five tensors equal); DOUBLE is rejected with 161002
 *   formats           : the format of input decides how input, gradOutput and inputGrad are read: NDHWC means
 *                       (N,D,H,W,C) extents, anything else (N,C,D,H,W)
 *   outputMask        : exactly two flags; a NULL mask or two false flags make the call a successful no-op
 *   views             : arbitrary strides/offsets are honoured (packed through the workspace)
 *   workspace         : also asked for with dense tensors when inputGrad is wanted (scratch of the kernels: cell slots,
 *                       corner weights and regrouped gradOutput of the bilinear gather, voxel spans of the chunks)
 * The result is deterministic: every element of inputGrad is the sum of its contributions in the order of the
 * reference's deterministic mode (grid points in chunks of 256; per chunk corner after corner, per corner point after
 * point; every add rounded to the tensor's element type).
 * Validation order and status codes follow aclnn_grid_sampler3d_backward.cpp:174-238.
 */
#ifndef OPSCV_ACLNN_GRID_SAMPLER3D_BACKWARD_H_
#define OPSCV_ACLNN_GRID_SAMPLER3D_BACKWARD_H_

#include "opscv_acl_base.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Phase 1 (host only, touches no device): validate, plan, report workspace bytes, hand out the executor. */
ACLNN_API aclnnStatus aclnnGridSampler3DBackwardGetWorkspaceSize(const aclTensor* gradOutput, const aclTensor* input,
                                                                 const aclTensor* grid, int64_t interpolationMode,
                                                                 int64_t paddingMode, bool alignCorners,
                                                                 const aclBoolArray* outputMask, aclTensor* inputGrad,
                                                                 aclTensor* gridGrad, uint64_t* workspaceSize,
                                                                 aclOpExecutor** executor);

/* Phase 2: enqueue the kernels on `stream` (a hipStream_t) and free the executor.  Asynchronous. */
ACLNN_API aclnnStatus aclnnGridSampler3DBackward(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                                 aclrtStream stream);

#ifdef __cplusplus
}
#endif

#endif /* OPSCV_ACLNN_GRID_SAMPLER3D_BACKWARD_H_ */
