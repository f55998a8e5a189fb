/*
 * aclnnUpsampleBilinear2d -- two-phase C API, MI355X (gfx950) implementation.
 *
 * Drop-in for the reference interface image/upsample_bilinear2d/op_host/op_api/aclnn_upsample_bilinear_2d.h:25-34
 * (implementation image/upsample_bilinear2d/op_host/op_api/aclnn_upsample_bilinear_2d.cpp:384-467).  The
 * arithmetic is the resize_bilinear_v2 NCHW rule the reference dispatches to on its newest parts
 * (image/resize_bilinear_v2/op_kernel/arch35/resize_bilinear_v2_simt_nchw.h:77-146):
 * half_pixel_centers = !alignCorners.
 *
 *   self / out  : FLOAT, FLOAT16 or BF16, equal dtypes, equal storage format (NCHW or NHWC), 4-D, equal N and C
 *   outputSize  : {Hout, Wout}, must equal out's spatial sizes
 *   scalesH/W   : user multipliers (>= 0); 0 derives the ratio from the sizes.  Ignored when alignCorners.
 * Validation order and status codes follow aclnn_upsample_bilinear_2d.cpp:170-195 (NULL self/out -> 561103).
 *
 * The reference's kernel for its older parts (two matrix products with banded coefficient matrices,
 * image/upsample_bilinear2d/op_kernel/upsample_bilinear2d_kernel.h:284-370, index rule
 * upsample_bilinear2d_common.h:37-51) takes the same taps and weights, except that its second tap is the next pixel
 * also at integer source coordinates, where the rule followed here blends the pixel with itself.  The two agree
 * on finite data; next to an infinite or NaN pixel the matrix products turn 0 * inf into NaN where this
 * implementation returns the pixel.
 */
#ifndef OPSCV_ACLNN_UPSAMPLE_BILINEAR_2D_H_
#define OPSCV_ACLNN_UPSAMPLE_BILINEAR_2D_H_

#include "opscv_acl_base.h"

#ifdef __cplusplus
extern "C" {
#endif

ACLNN_API aclnnStatus aclnnUpsampleBilinear2dGetWorkspaceSize(const aclTensor* self, const aclIntArray* outputSize,
                                                              const bool alignCorners, const double scalesH,
                                                              const double scalesW, aclTensor* out,
                                                              uint64_t* workspaceSize, aclOpExecutor** executor);

ACLNN_API aclnnStatus aclnnUpsampleBilinear2d(void* workspace, uint64_t workspaceSize, aclOpExecutor* executor,
                                              aclrtStream stream);

#ifdef __cplusplus
}
#endif

#endif /* OPSCV_ACLNN_UPSAMPLE_BILINEAR_2D_H_ */
