// Scratch memory that belongs to the library instead of the caller: a file-scope device array that stands in for the
// workspace argument in the entry point that must not allocate (opscvGridSampler2DNoAlloc).  Every device the library
// runs on holds its own copy of the array, at its own address, from the moment the code object is loaded until the
// process ends.  All calls on one device share that copy: calls that overlap in time on one device race on it.
#include <hip/hip_runtime.h>

#include <atomic>

#include "executor.hpp"
#include "opscv_ext.h"

namespace opscv {

namespace {

constexpr uint64_t kScratchBytes = OPSCV_NOALLOC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// The array's name is a host-side stand-in, not a device address: the address of each device's copy is asked for
// once, with that device current, and kept.
std::atomic<void*> g_scratch_ptr[kMaxDevices];

}  // namespace

hipError_t static_scratch(void** ptr, uint64_t* bytes)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        return e;
    }
    if (dev < 0 || dev >= kMaxDevices) {
        return hipErrorInvalidDevice;
    }
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) {
            return e;
        }
        if (p == nullptr) {
            return hipErrorInvalidSymbol;
        }
        g_scratch_ptr[dev].store(p, std::memory_order_release);  // two first calls at once store the same address
    }
    *ptr = p;
    *bytes = kScratchBytes;
    return hipSuccess;
}

}  // namespace opscv
