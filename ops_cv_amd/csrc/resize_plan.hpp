// Host-side planning of the bilinear resize: scale factors and kernel-template selection.
#pragma once

#include "acl_types.hpp"

namespace opscv {

// Scale handed to the kernel for one axis; user_scale <= 0 means "derive from the sizes".
// image/resize_bilinear_v2/op_host/arch35/resize_bilinear_v2_tiling_arch35.cpp:175-184,228-243
float resize_axis_scale(int64_t len_src, int64_t len_dst, bool align_corners, float user_scale);

// Fills mode / half_pixel / scales of `a` from its shape fields (elem, channels_last, N, C, Hs, Ws, Hd, Wd).
// Template choice follows resize_bilinear_v2_tiling_arch35.cpp:245-335,592-623 and
// image/resize_bilinear_v2/op_kernel/resize_bilinear_v2_apt.cpp:91-140.
void plan_resize(ResizeArgs* a, bool align_corners, float user_scale_h, float user_scale_w);

// Vector cores of the device the reference would run on.  Its choice between the per-plane and the H*W-split NCHW
// template depends on that number (resize_bilinear_v2_tiling_arch35.cpp:606-609,877), and the two templates differ in
// the border pixels of fp32 half-pixel upscales.  Option "reference_cores" (options.hpp), 64 unless set.
int64_t reference_vector_cores();

// Nearest-neighbour resize with align_corners = false and half_pixel_centers = false, the only combination
// aclnnResize requests (image/resize_bilinear_v2/op_api/aclnn_resize.cpp:286-288): scale = in / out
// (image/resize_nearest_neighbor_v2/op_host/arch35/resize_nearest_neighbor_v2_tiling_base.cpp:253-263).
// Sets rep_h / rep_w where the reference would take its replicating channels-last template (:640-665), whose index is
// destination / factor; that choice reads the size of the reference device's unified buffer, option
// "reference_ub_bytes" (253952 bytes unless set).
// Both planning functions also copy the kernel-variant overrides of the moment into `a`.
void plan_resize_nearest(ResizeArgs* a);

}  // namespace opscv
