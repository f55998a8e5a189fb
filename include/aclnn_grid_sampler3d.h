/*
 * aclnnGridSampler3D -- two-phase C API, MI355X (gfx950) implementation.
 *
 * Drop-in for the reference interface image/grid_sample/op_api/aclnn_grid_sampler3d.h:23-38
 * (implementation image/grid_sample/op_api/aclnn_grid_sampler3d.cpp:314-380; device arithmetic
 * image/grid_sample/op_kernel/arch35/grid_sampler_3d_bilinear_smit.h).
 *
 * out[n,c,d,h,w] = sample(input[n,c,:,:,:], grid[n,d,h,w,:]) with grid in normalized [-1,1] coordinates
 * ordered x (width), y (height), z (depth).
 *   interpolationMode : 0 bilinear (blend of the eight surrounding voxels), 1 nearest
 *   paddingMode       : 0 zeros, 1 border, 2 reflection
 *   dtypes            : FLOAT, FLOAT16, BF16 (all three tensors equal); DOUBLE is rejected with 161002
 *   formats           : NCDHW or ND: input (N,C,Din,Hin,Win), out (N,C,Dout,Hout,Wout);
 *                       NDHWC: input (N,Din,Hin,Win,C), out (N,Dout,Hout,Wout,C); grid (N,Dout,Hout,Wout,3)
 *   views             : arbitrary strides/offsets are honoured (packed through the workspace)
 * Validation order and status codes follow aclnn_grid_sampler3d.cpp:194-208.
 */
#ifndef OPSCV_ACLNN_GRID_SAMPLER3D_H_
#define OPSCV_ACLNN_GRID_SAMPLER3D_H_

#include "opscv_acl_base.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Phase 1 (host only, touches no device): validate, plan, report workspace bytes, hand out the executor. */
ACLNN_API aclnnStatus aclnnGridSampler3DGetWorkspaceSize(const aclTensor* input, const aclTensor* grid,
                                                         int64_t interpolationMode, int64_t paddingMode,
                                                         bool alignCorners, aclTensor* out, uint64_t* workspaceSize,
                                                         aclOpExecutor** executor);

/* Phase 2: enqueue the kernels on `stream` (a hipStream_t) and free the executor.  Asynchronous. */
ACLNN_API aclnnStatus aclnnGridSampler3D(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                         aclrtStream stream);

#ifdef __cplusplus
}
#endif

#endif /* OPSCV_ACLNN_GRID_SAMPLER3D_H_ */
