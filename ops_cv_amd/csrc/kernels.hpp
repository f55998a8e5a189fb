// Launch interface between the aclnn host layer and the HIP kernels.
#pragma once

#include <hip/hip_runtime_api.h>

#include <atomic>

#include "acl_types.hpp"

namespace opscv {

// Raises a kernel's dynamic-LDS limit once per device.  `done` is a bit mask of the devices served (one static
// object per kernel at the call site); setting the attribute twice is harmless, so concurrent first calls need no
// lock, only the atomic mask.
inline hipError_t allow_dynamic_lds(const void* kernel, int bytes, std::atomic<uint32_t>& done)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        return e;
    }
    const uint32_t bit = 1u << (dev & 31);
    if (done.load(std::memory_order_acquire) & bit) {
        return hipSuccess;
    }
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) {
        done.fetch_or(bit, std::memory_order_release);
    }
    return e;
}

// Record written per output pixel by the tap-dump kernel (28 bytes, no padding).
struct TapRecord {
    int32_t x0;
    int32_t y0;
    float w[4];
    int32_t flag;
};

// Record of the bicubic mode (68 bytes, no padding).
struct BicubicTapRecord {
    int32_t bx[4];
    int32_t by[4];
    float cx[4];
    float cy[4];
    int32_t flag;
};

// All tensors contiguous.  Each launcher validates the shapes against what its kernels assume and
// returns hipErrorInvalidValue instead of launching when they do not fit.
hipError_t launch_grid_sampler2d(const GridSamplerArgs& a, hipStream_t stream);
hipError_t launch_grid_sampler2d_taps(const GridSamplerArgs& a, TapRecord* taps, hipStream_t stream);
hipError_t launch_grid_sampler2d_bicubic_taps(const GridSamplerArgs& a, BicubicTapRecord* taps, hipStream_t stream);
hipError_t launch_resize(const ResizeArgs& a, hipStream_t stream);
hipError_t launch_resize_grad(const ResizeGradArgs& a, hipStream_t stream);
const char* resize_grad_variant(const ResizeGradArgs& a);  // which kernel launch_resize_grad picks (x may be null)
hipError_t launch_grid_sampler2d_grad(const GridSamplerGradArgs& a, hipStream_t stream);
// grid gradient of the 2-D sampler with the input planes staged through LDS (gs2d_grad_lds.hip); *handled is false
// when the shape does not qualify.  gs2d_grad_grid_uses_lds: whether it would run (pointers may still be null).
// Words of scratch memory that one kernel zeroes on its way for a later one: per batch item (item_words apart) `count`
// words from `first` on, and the word `single`.
struct GradClear {
    uint32_t* base;
    uint32_t item_words;
    uint32_t first;
    uint32_t count;
    uint32_t single;
};
// `clear`, when not null, is zeroed by the kernel if it runs (*handled).
hipError_t run_gs2d_grad_grid_lds(const GridSamplerGradArgs& a, hipStream_t stream, bool* handled,
                                  const GradClear* clear);
bool gs2d_grad_grid_uses_lds(const GridSamplerGradArgs& a);
// input gradient of the 2-D sampler as a gather over per-element contribution lists (gs2d_grad_csr.hip): 32-bit words
// of GridSamplerGradArgs::scratch it needs, 0 when the shape does not qualify; *handled is false when it did not run
int64_t gs2d_grad_csr_words(const GridSamplerGradArgs& a);
// whether run_gs2d_grad_input_csr would run, and the words it wants zeroed first: `cleared` says that an earlier kernel
// on the stream has done that, else it launches a kernel of its own for it
bool gs2d_grad_csr_clear(const GridSamplerGradArgs& a, GradClear* clear);
hipError_t run_gs2d_grad_input_csr(const GridSamplerGradArgs& a, hipStream_t stream, bool* handled, bool cleared);
hipError_t launch_grid_sampler3d(const GridSampler3DArgs& a, hipStream_t stream);
hipError_t launch_grid_sampler3d_grad(const GridSampler3DGradArgs& a, hipStream_t stream);
// 32-bit words of GridSampler3DGradArgs::chunk_ranges that make the input gradient faster; 0 when it would not help
int64_t gs3d_grad_range_words(const GridSampler3DGradArgs& a);
// 32-bit words of GridSampler3DGradArgs::lists that the gather variant of the input gradient needs; 0 when the shape
// does not qualify (gs3d_grad_lists.hip)
int64_t gs3d_grad_list_words(const GridSampler3DGradArgs& a);
// one scratch region holds both: the chunk spans at its start, the lists from this byte offset
inline uint64_t gs3d_grad_lists_offset(int64_t range_words) { return ((uint64_t)range_words * 4 + 255) / 256 * 256; }

// gather == true : strided view -> contiguous buffer;  false : contiguous buffer -> strided view
hipError_t launch_strided_copy(const StridedView& v, void* contiguous, int elem_bytes, bool gather,
                               hipStream_t stream);

// LDS-staged row-band resize (resize_band_lds.hip); *handled is false when the shape does not qualify.
hipError_t run_resize_band_lds(const ResizeArgs& a, hipStream_t stream, bool* handled);
// name of the LDS-staged variant that would run, or nullptr when neither applies
const char* resize_lds_variant(const ResizeArgs& a);

// Name of the kernel variant the launcher would pick for these arguments (for benchmarks and tests).
const char* grid_sampler2d_variant(const GridSamplerArgs& a);
const char* resize_variant(const ResizeArgs& a);

// CUs of the current device (256 on MI355X; also the answer where no device can be asked); gs2d_lds.hip
int compute_unit_count();

}  // namespace opscv
