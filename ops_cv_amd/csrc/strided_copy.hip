// Packing of non-contiguous views of up to five dimensions into contiguous workspace slices and back.
//
// Takes the place of the reference's l0op::Contiguous (inputs) and l0op::ViewCopy (output) steps,
// image/grid_sample/op_api/aclnn_grid_sampler2d.cpp:288-293,337-338.
#include <hip/hip_runtime.h>

#include "kernels.hpp"

namespace opscv {

namespace {

constexpr int kThreads = 256;

struct View5 {
    int64_t d1, d2, d3, d4;      // extents of dims 1..4 (dim 0 follows from the total)
    int64_t s0, s1, s2, s3, s4;  // element strides
};

template <typename U, bool GATHER>
__global__ __launch_bounds__(kThreads) void strided_copy_kernel(U* __restrict__ strided, U* __restrict__ packed,
                                                                 int64_t total, View5 v)
{
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
        int64_t r = i;
        const int64_t i4 = r % v.d4;
        r /= v.d4;
        const int64_t i3 = r % v.d3;
        r /= v.d3;
        const int64_t i2 = r % v.d2;
        r /= v.d2;
        const int64_t i1 = r % v.d1;
        const int64_t i0 = r / v.d1;
        const int64_t off = i0 * v.s0 + i1 * v.s1 + i2 * v.s2 + i3 * v.s3 + i4 * v.s4;
        if (GATHER) {
            packed[i] = strided[off];
        } else {
            strided[off] = packed[i];
        }
    }
}

template <typename U>
hipError_t run(const StridedView& sv, void* contiguous, bool gather, hipStream_t stream)
{
    const int64_t total = sv.dims[0] * sv.dims[1] * sv.dims[2] * sv.dims[3] * sv.dims[4];
    if (total == 0) {
        return hipSuccess;
    }
    View5 v{sv.dims[1],    sv.dims[2],    sv.dims[3],    sv.dims[4],   sv.strides[0],
            sv.strides[1], sv.strides[2], sv.strides[3], sv.strides[4]};
    int64_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 256 * 64) {
        blocks = 256 * 64;
    }
    if (gather) {
        hipLaunchKernelGGL((strided_copy_kernel<U, true>), dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                           (U*)sv.base, (U*)contiguous, total, v);
    } else {
        hipLaunchKernelGGL((strided_copy_kernel<U, false>), dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                           (U*)sv.base, (U*)contiguous, total, v);
    }
    return hipGetLastError();
}

}  // namespace

hipError_t launch_strided_copy(const StridedView& v, void* contiguous, int elem_bytes, bool gather,
                               hipStream_t stream)
{
    if (v.base == nullptr || contiguous == nullptr) {
        return hipErrorInvalidValue;
    }
    for (int i = 0; i < kViewDims; i++) {
        if (v.dims[i] < 0) {
            return hipErrorInvalidValue;
        }
    }
    if (elem_bytes == 4) {
        return run<uint32_t>(v, contiguous, gather, stream);
    }
    if (elem_bytes == 2) {
        return run<uint16_t>(v, contiguous, gather, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
