// Streaming reference for the benchmark (built into libopscv_bench.so, used by bench.py only): a kernel that
// reads `in_bytes` once and writes `out_bytes` once with 16-byte vector accesses and no arithmetic, timed with
// events on the same stream and with the same buffer rotation as the measured operator.  It is what the memory
// system gives a well-tuned kernel of this size that does nothing but move the operator's bytes.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef uint32_t chunk_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ chunk_t xor4(chunk_t a, chunk_t b) { return a ^ b; }

// Every input chunk is loaded from memory once and every output chunk stored exactly once, all accesses coalesced.
//   MODE 0  out == in: chunk i to chunk i.
//   MODE 1  out = r * in: one lane per output chunk j, which takes input chunk j >> shift or j / r (contiguous stores;
//           the r neighbouring lanes that share an input chunk ask for it with one instruction).
//   MODE 2  any other out >= in: input chunk i goes to output chunks i, i + in, i + 2 in, ...
//   MODE 3  out < in: output chunk i is the xor of input chunks i, i + out, i + 2 out, ... (the xor only keeps the
//           loads alive).
// Tuned to be a ceiling rather than a strawman: U independent 16-byte loads in flight per lane before the first store,
// non-temporal stores (the lines are written through instead of being left dirty in L2 for the end of the kernel to
// write back: 13.2 -> 10.7 us for 33.5 MB in and out), and the caller tries several grid sizes and keeps the best.
template <int U, int MODE>
__global__ __launch_bounds__(256) void stream_kernel(const chunk_t* __restrict__ src, chunk_t* __restrict__ dst,
                                                     uint64_t in_chunks, uint64_t out_chunks, uint32_t ratio)
{
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    const uint64_t first = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (MODE == 0 || MODE == 1) {
        const bool pow2 = (ratio & (ratio - 1u)) == 0u;
        const uint32_t shift = 31u - (uint32_t)__builtin_clz(ratio);
        for (uint64_t j = first; j < out_chunks; j += U * stride) {
            chunk_t v[U];
#pragma unroll
            for (int k = 0; k < U; k++) {
                const uint64_t jk = j + (uint64_t)k * stride;
                if (jk < out_chunks) {
                    v[k] = src[MODE == 0 ? jk : (pow2 ? (jk >> shift) : jk / ratio)];
                }
            }
#pragma unroll
            for (int k = 0; k < U; k++) {
                const uint64_t jk = j + (uint64_t)k * stride;
                if (jk < out_chunks) {
                    __builtin_nontemporal_store(v[k], dst + jk);
                }
            }
        }
    } else if constexpr (MODE == 2) {
        for (uint64_t i = first; i < in_chunks; i += U * stride) {
            chunk_t v[U];
#pragma unroll
            for (int k = 0; k < U; k++) {
                const uint64_t ik = i + (uint64_t)k * stride;
                if (ik < in_chunks) {
                    v[k] = src[ik];
                }
            }
#pragma unroll
            for (int k = 0; k < U; k++) {
                const uint64_t ik = i + (uint64_t)k * stride;
                if (ik < in_chunks) {
                    for (uint64_t jj = ik; jj < out_chunks; jj += in_chunks) {
                        __builtin_nontemporal_store(v[k], dst + jj);
                    }
                }
            }
        }
    } else {
        for (uint64_t i = first; i < out_chunks; i += stride) {
            chunk_t v = src[i];
            for (uint64_t j = i + out_chunks; j < in_chunks; j += out_chunks) {
                v = xor4(v, src[j]);
            }
            __builtin_nontemporal_store(v, dst + i);
        }
    }
}

typedef void (*stream_fn_t)(const chunk_t*, chunk_t*, uint64_t, uint64_t, uint32_t);

template <int MODE>
stream_fn_t pick_unroll(int unroll)
{
    switch (unroll) {
        case 1: return stream_kernel<1, MODE>;
        case 2: return stream_kernel<2, MODE>;
        default: return stream_kernel<4, MODE>;
    }
}

}  // namespace

// Times `steps` launches of the streaming kernel; `unroll` (1, 2, 4) loads in flight per lane and `groups_per_cu`
// workgroups of 256 lanes per CU (256 CUs assumed for the grid size; 0 = one lane per unit of work).  The caller
// sweeps a few settings and reports the fastest.
extern "C" __attribute__((visibility("default"))) int opscv_bench_stream(
    const void* const* srcs, void* const* dsts, int sets, uint64_t in_bytes, uint64_t out_bytes, int steps,
    void* stream, int unroll, int groups_per_cu, double* event_ms)
{
    hipStream_t s = (hipStream_t)stream;
    const uint64_t in_chunks = in_bytes / 16, out_chunks = out_bytes / 16;
    if (in_chunks == 0 || out_chunks == 0 || sets <= 0) {
        return -1;
    }
    int mode;
    uint64_t ratio = 1;
    if (out_chunks == in_chunks) {
        mode = 0;
    } else if (out_chunks > in_chunks && out_chunks % in_chunks == 0 && out_chunks / in_chunks <= 0x7FFFFFFFu) {
        mode = 1;
        ratio = out_chunks / in_chunks;
    } else if (out_chunks > in_chunks) {
        mode = 2;
    } else {
        mode = 3;
    }
    stream_fn_t kernel = mode == 0 ? pick_unroll<0>(unroll)
                       : mode == 1 ? pick_unroll<1>(unroll)
                       : mode == 2 ? pick_unroll<2>(unroll)
                                   : pick_unroll<3>(1);
    const uint64_t per_lane = (mode == 3) ? 1 : (uint64_t)(unroll == 1 || unroll == 2 ? unroll : 4);
    const uint64_t work = ((mode == 2) ? in_chunks : out_chunks) / per_lane + 1;
    uint64_t blocks = (work + 255) / 256;
    if (groups_per_cu > 0 && blocks > (uint64_t)256 * groups_per_cu) {
        blocks = (uint64_t)256 * groups_per_cu;
    }
    if (blocks > 0x7FFFFFFFu) {
        return -1;
    }
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        return -1;
    }
    // a few untimed launches right in front of the timed region, as the operator loops do
    for (int k = 0; k < 10; k++) {
        const int i = (steps + k) % sets;
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const chunk_t*)srcs[i], (chunk_t*)dsts[i],
                           in_chunks, out_chunks, (uint32_t)ratio);
    }
    if (hipStreamSynchronize(s) != hipSuccess) {
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        return -1;
    }
    (void)hipEventRecord(e0, s);
    for (int k = 0; k < steps; k++) {
        const int i = k % sets;
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const chunk_t*)srcs[i], (chunk_t*)dsts[i],
                           in_chunks, out_chunks, (uint32_t)ratio);
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
