// Streaming reference for the benchmark (built into libopscv_bench.so, used by bench.py only): a kernel that
// reads `in_bytes` once and writes `out_bytes` once with 16-byte vector accesses and no arithmetic, timed with
// events on the same stream and with the same buffer rotation as the measured operator.  It is what the memory
// system gives a kernel of this size that does nothing but move the operator's bytes.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

__device__ __forceinline__ uint4 xor4(uint4 a, uint4 b) { return make_uint4(a.x ^ b.x, a.y ^ b.y, a.z ^ b.z, a.w ^ b.w); }

// Every input chunk is loaded exactly once and every output chunk stored exactly once, all accesses coalesced.
// out >= in: chunk i of the input goes to output chunks i, i + in, i + 2 in, ...; out < in: output chunk i is the
// xor of input chunks i, i + out, i + 2 out, ... (the xor only keeps the loads alive).
__global__ __launch_bounds__(256) void stream_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                     uint64_t in_chunks, uint64_t out_chunks)
{
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    const uint64_t first = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (out_chunks >= in_chunks) {
        for (uint64_t i = first; i < in_chunks; i += stride) {
            const uint4 v = src[i];
            for (uint64_t j = i; j < out_chunks; j += in_chunks) {
                dst[j] = v;
            }
        }
    } else {
        for (uint64_t i = first; i < out_chunks; i += stride) {
            uint4 v = src[i];
            for (uint64_t j = i + out_chunks; j < in_chunks; j += out_chunks) {
                v = xor4(v, src[j]);
            }
            dst[i] = v;
        }
    }
}

}  // namespace

extern "C" __attribute__((visibility("default"))) int opscv_bench_stream(
    const void* const* srcs, void* const* dsts, int sets, uint64_t in_bytes, uint64_t out_bytes, int steps,
    void* stream, double* event_ms)
{
    hipStream_t s = (hipStream_t)stream;
    const uint64_t in_chunks = in_bytes / 16, out_chunks = out_bytes / 16;
    if (in_chunks == 0 || out_chunks == 0 || sets <= 0) {
        return -1;
    }
    const uint64_t work = (out_chunks < in_chunks) ? out_chunks : in_chunks;
    uint64_t blocks = (work + 255) / 256;
    if (blocks > 256 * 32) {
        blocks = 256 * 32;
    }
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        return -1;
    }
    // a few untimed launches right in front of the timed region, as the operator loops do
    for (int k = 0; k < 10; k++) {
        const int i = (steps + k) % sets;
        hipLaunchKernelGGL(stream_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const uint4*)srcs[i],
                           (uint4*)dsts[i], in_chunks, out_chunks);
    }
    if (hipStreamSynchronize(s) != hipSuccess) {
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        return -1;
    }
    (void)hipEventRecord(e0, s);
    for (int k = 0; k < steps; k++) {
        const int i = k % sets;
        hipLaunchKernelGGL(stream_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const uint4*)srcs[i],
                           (uint4*)dsts[i], in_chunks, out_chunks);
    }
    (void)hipEventRecord(e1, s);
    if (hipEventSynchronize(e1) != hipSuccess || hipGetLastError() != hipSuccess) {
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        return -1;
    }
    float ms = 0.0f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    *event_ms = ms;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return 0;
}
