/*
 * aclnnResize -- two-phase C API, MI355X (gfx950) implementation.
 *
 * Drop-in for the reference interface image/resize_bilinear_v2/op_api/aclnn_resize.h:29-46
 * (implementation image/resize_bilinear_v2/op_api/aclnn_resize.cpp:251-321, the branch taken on the newest
 * parts: plain 4-D tensors, no blocked-format round trip).
 *
 *   self, out : 4-D, equal dtype (FLOAT, FLOAT16, BF16), equal format (NCHW or NHWC), equal N and C
 *   scales    : 4 floats in the order of the tensor's dimensions; out H and W must equal
 *               trunc(in * scale) within scale +- 1e-5 (aclnn_resize.cpp:100-118)
 *   mode      : a string starting with "nearest" or "bilinear" (aclnn_resize.cpp:147-155)
 *     bilinear : align_corners = false, half-pixel centres, scale = in / out -- the same kernel as
 *                aclnnUpsampleBilinear2d with alignCorners = false and zero user scales
 *     nearest  : src = min(floor(dst * (in / out)), in - 1)
 *                (image/resize_nearest_neighbor_v2/op_kernel/arch35/resize_nearest_neighbor_v2_simt.h:103-124);
 *                NHWC upscales by whole factors with at least 128 bytes of channels per pixel and rows that fit the
 *                reference device's unified buffer take the reference's replicating template instead,
 *                src = dst / factor (.../op_host/arch35/resize_nearest_neighbor_v2_tiling_base.cpp:640-665,
 *                .../op_kernel/arch35/resize_nearest_neighbor_v2_data_copy_nhwc.h:205-231): the same result up to
 *                a factor of 40, different from the float rule from 41 on.  The buffer size mirrored is 253952
 *                bytes unless the environment variable OPSCV_REFERENCE_UB_BYTES gives another.
 *   views     : arbitrary strides/offsets are honoured (packed through the workspace)
 */
#ifndef OPSCV_ACLNN_RESIZE_H_
#define OPSCV_ACLNN_RESIZE_H_

#include "opscv_acl_base.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Phase 1 (host only, touches no device): validate, plan, report workspace bytes, hand out the executor. */
ACLNN_API aclnnStatus aclnnResizeGetWorkspaceSize(const aclTensor* self, const aclFloatArray* scales,
                                                  const char* mode, aclTensor* out, uint64_t* workspaceSize,
                                                  aclOpExecutor** executor);

/* Phase 2: enqueue the kernels on `stream` (a hipStream_t) and free the executor.  Asynchronous. */
ACLNN_API aclnnStatus aclnnResize(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                  aclrtStream stream);

#ifdef __cplusplus
}
#endif

#endif /* OPSCV_ACLNN_RESIZE_H_ */
