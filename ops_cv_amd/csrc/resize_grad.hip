// Backward of the bilinear resize for gfx950, deterministic gather formulation.
//
// Replaces the reference device kernel
// image/resize_bilinear_v2_grad/op_kernel/arch35/resize_bilinear_v2_grad_simt_determine.h:56-117 and the scale rules
// of image/resize_bilinear_v2_grad/op_host/arch35/resize_bilinear_v2_grad_tiling_arch35.cpp:352-394.
//
// One lane per element (n, c, H, W) of the outgoing gradient.  It visits the incoming-gradient rows inY whose
// source coordinate outY = (inY + o) * scale - o lies in (H - 1, H + 1), starting at
// ceil((H - 1 + o) / scale - o) and advancing outY by repeated addition of the scale (as the reference does, so
// the rounding of every coordinate is the same), and likewise the columns; each visited element contributes
// g * (1 - |clamp(outY) - H|) * (1 - |clamp(outX) - W|), summed in fp32 in row-major visiting order.  No atomics:
// the result does not depend on scheduling.  The translation unit is compiled with -ffp-contract=off.
#include <hip/hip_runtime.h>

#include "kernels.hpp"
#include "sampler_math.hpp"

namespace opscv {

namespace {

constexpr int kGradThreads = 256;

// User-scale template (resize_bilinear_v2_grad_simt_determine_scales.h:77-305), for scales that are not the ratio
// of the sizes.  Same walk, but the source coordinate of every visited row/column is recomputed as
// scale * (i + o) - o instead of accumulated, and an element on the first or last row (column) of the outgoing
// gradient scans the incoming rows (columns) to the end and takes, per visited element, the weights of the taps
// that land on it (floor tap: 1 - |c - H|; next tap: c - floor(c)).
template <typename TI, typename TO, bool HALF_PIXEL, bool NHWC>
__global__ __launch_bounds__(kGradThreads) void resize_grad_scales_kernel(const TI* __restrict__ g, TO* __restrict__ y,
                                                                           int64_t total, int32_t C, int32_t Hs,
                                                                           int32_t Ws, int32_t Hd, int32_t Wd,
                                                                           float scale_h, float scale_w,
                                                                           float inv_scale_h, float inv_scale_w)
{
    const int64_t stride = (int64_t)gridDim.x * kGradThreads;
    const float offset = HALF_PIXEL ? 0.5f : 0.0f;
    const float last_y = (float)Hs - 1.0f, last_x = (float)Ws - 1.0f;
    auto source_index = [](float scale, int64_t i) {
        return HALF_PIXEL ? scale * ((float)i + 0.5f) - 0.5f : scale * (float)i;
    };
    for (int64_t idx = (int64_t)blockIdx.x * kGradThreads + threadIdx.x; idx < total; idx += stride) {
        int64_t t = idx;
        int32_t c, W, H;
        if (NHWC) {
            c = (int32_t)(t % C);
            t /= C;
            W = (int32_t)(t % Ws);
            t /= Ws;
            H = (int32_t)(t % Hs);
            t /= Hs;
        } else {
            W = (int32_t)(t % Ws);
            t /= Ws;
            H = (int32_t)(t % Hs);
            t /= Hs;
            c = (int32_t)(t % C);
            t /= C;
        }
        const int64_t n = t;
        const float fy0 = __builtin_ceilf(((float)H - 1.0f + offset) * inv_scale_h - offset);
        const float fx0 = __builtin_ceilf(((float)W - 1.0f + offset) * inv_scale_w - offset);
        const int64_t in_y_start = (fy0 > 0.0f) ? (int64_t)fy0 : 0;
        const int64_t in_x_start = (fx0 > 0.0f) ? (int64_t)fx0 : 0;
        const float out_y_start = ((float)in_y_start + offset) * scale_h - offset;
        const float out_x_start = ((float)in_x_start + offset) * scale_w - offset;
        const float fh = (float)H, fw = (float)W;
        const bool hb = (H == 0 || H == Hs - 1), wb = (W == 0 || W == Ws - 1);
        float acc = 0.0f;
        float out_y = out_y_start;
        for (int64_t in_y = in_y_start; (hb || out_y < fh + 1.0f) && in_y < Hd;) {
            const float yc = __builtin_fmaxf(0.0f, __builtin_fminf(out_y, last_y));
            const float y_lerp = 1.0f - __builtin_fabsf(yc - fh);
            const float yt = __builtin_fminf(__builtin_floorf(yc), last_y);
            const float lepy[2] = {y_lerp, yc - yt};
            float out_x = out_x_start;
            for (int64_t in_x = in_x_start; (wb || out_x < fw + 1.0f) && in_x < Wd;) {
                const int64_t gi = NHWC ? ((n * Hd + in_y) * Wd + in_x) * C + c : ((n * C + c) * Hd + in_y) * Wd + in_x;
                const float gv = ElemIO<TI>::load(g + gi);
                const float xc = __builtin_fmaxf(0.0f, __builtin_fminf(out_x, last_x));
                const float x_lerp = 1.0f - __builtin_fabsf(xc - fw);
                const float xt = __builtin_fminf(__builtin_floorf(xc), last_x);
                const float lepx[2] = {x_lerp, xc - xt};
                if (!hb && !wb) {
                    acc += gv * y_lerp * x_lerp;
                } else if (!hb) {
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        if (xt + (float)j == fw) {
                            acc += gv * lepx[j] * y_lerp;
                        }
                    }
                } else if (!wb) {
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        if (yt + (float)i == fh) {
                            acc += gv * lepy[i] * x_lerp;
                        }
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 2; i++) {
#pragma unroll
                        for (int j = 0; j < 2; j++) {
                            if (yt + (float)i == fh && xt + (float)j == fw) {
                                acc += gv * lepx[j] * lepy[i];
                            }
                        }
                    }
                }
                in_x++;
                out_x = source_index(scale_w, in_x);
            }
            in_y++;
            out_y = source_index(scale_h, in_y);
        }
        ElemIO<TO>::store(y + idx, acc);
    }
}

template <typename TI, typename TO, bool HALF_PIXEL, bool NHWC>
__global__ __launch_bounds__(kGradThreads) void resize_grad_kernel(const TI* __restrict__ g, TO* __restrict__ y,
                                                                    int64_t total, int32_t C, int32_t Hs, int32_t Ws,
                                                                    int32_t Hd, int32_t Wd, float scale_h,
                                                                    float scale_w, float inv_scale_h,
                                                                    float inv_scale_w)
{
    const int64_t stride = (int64_t)gridDim.x * kGradThreads;
    const float offset = HALF_PIXEL ? 0.5f : 0.0f;
    const float last_y = (float)Hs - 1.0f, last_x = (float)Ws - 1.0f;
    for (int64_t idx = (int64_t)blockIdx.x * kGradThreads + threadIdx.x; idx < total; idx += stride) {
        int64_t t = idx;
        int32_t c, W, H;
        if (NHWC) {
            c = (int32_t)(t % C);
            t /= C;
            W = (int32_t)(t % Ws);
            t /= Ws;
            H = (int32_t)(t % Hs);
            t /= Hs;
        } else {
            W = (int32_t)(t % Ws);
            t /= Ws;
            H = (int32_t)(t % Hs);
            t /= Hs;
            c = (int32_t)(t % C);
            t /= C;
        }
        const int64_t n = t;
        const float fy0 = __builtin_ceilf(((float)H - 1.0f + offset) * inv_scale_h - offset);
        const float fx0 = __builtin_ceilf(((float)W - 1.0f + offset) * inv_scale_w - offset);
        const int64_t in_y_start = (fy0 > 0.0f) ? (int64_t)fy0 : 0;
        const int64_t in_x_start = (fx0 > 0.0f) ? (int64_t)fx0 : 0;
        const float out_y_start = ((float)in_y_start + offset) * scale_h - offset;
        const float out_x_start = ((float)in_x_start + offset) * scale_w - offset;
        const float fh = (float)H, fw = (float)W;
        float acc = 0.0f;
        float out_y = out_y_start;
        for (int64_t in_y = in_y_start; out_y < fh + 1.0f && in_y < Hd; in_y++) {
            const float yc = __builtin_fmaxf(0.0f, __builtin_fminf(out_y, last_y));
            const float y_lerp = 1.0f - __builtin_fabsf(yc - fh);
            float out_x = out_x_start;
            for (int64_t in_x = in_x_start; out_x < fw + 1.0f && in_x < Wd; in_x++) {
                const int64_t gi = NHWC ? ((n * Hd + in_y) * Wd + in_x) * C + c : ((n * C + c) * Hd + in_y) * Wd + in_x;
                const float xc = __builtin_fmaxf(0.0f, __builtin_fminf(out_x, last_x));
                const float x_lerp = 1.0f - __builtin_fabsf(xc - fw);
                acc += ElemIO<TI>::load(g + gi) * y_lerp * x_lerp;
                out_x += scale_w;
            }
            out_y += scale_h;
        }
        ElemIO<TO>::store(y + idx, acc);
    }
}

template <typename TI, typename TO>
hipError_t run(const ResizeGradArgs& a, hipStream_t stream)
{
    const int64_t total = a.N * a.C * a.Hs * a.Ws;
    int64_t blocks = (total + kGradThreads - 1) / kGradThreads;
    if (blocks > 256 * 256) {
        blocks = 256 * 256;
    }
#define OPSCV_RG(HP, CL)                                                                                              \
    if (a.user_scales) {                                                                                              \
        hipLaunchKernelGGL((resize_grad_scales_kernel<TI, TO, HP, CL>), dim3((unsigned)blocks), dim3(kGradThreads),   \
                           0, stream, (const TI*)a.x, (TO*)a.y, total, (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws,    \
                           (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h, a.scale_w, a.inv_scale_h, a.inv_scale_w);         \
    } else {                                                                                                          \
        hipLaunchKernelGGL((resize_grad_kernel<TI, TO, HP, CL>), dim3((unsigned)blocks), dim3(kGradThreads), 0,       \
                           stream, (const TI*)a.x, (TO*)a.y, total, (int32_t)a.C, (int32_t)a.Hs, (int32_t)a.Ws,       \
                           (int32_t)a.Hd, (int32_t)a.Wd, a.scale_h, a.scale_w, a.inv_scale_h, a.inv_scale_w);         \
    }
    if (a.half_pixel) {
        if (a.channels_last) {
            OPSCV_RG(true, true);
        } else {
            OPSCV_RG(true, false);
        }
    } else {
        if (a.channels_last) {
            OPSCV_RG(false, true);
        } else {
            OPSCV_RG(false, false);
        }
    }
#undef OPSCV_RG
    return hipGetLastError();
}

}  // namespace

hipError_t launch_resize_grad(const ResizeGradArgs& a, hipStream_t stream)
{
    const int64_t lim = INT32_MAX;
    if (a.N < 0 || a.C < 0 || a.Hs <= 0 || a.Ws <= 0 || a.Hd <= 0 || a.Wd <= 0 || a.Hs > lim || a.Ws > lim ||
        a.Hd > lim || a.Wd > lim || a.C > lim || a.N > lim) {
        return hipErrorInvalidValue;
    }
    if (a.N == 0 || a.C == 0) {
        return hipSuccess;
    }
    if (a.x == nullptr || a.y == nullptr) {
        return hipErrorInvalidValue;
    }
    if (a.copy) {
        if (a.elem_in != a.elem_out) {
            return hipErrorInvalidValue;
        }
        return hipMemcpyAsync(a.y, a.x, (size_t)(a.N * a.C * a.Hs * a.Ws) * elem_size(a.elem_in),
                              hipMemcpyDeviceToDevice, stream);
    }
    if (a.elem_in == Elem::F32) {
        switch (a.elem_out) {
            case Elem::F32: return run<float, float>(a, stream);
            case Elem::F16: return run<float, _Float16>(a, stream);
            case Elem::BF16: return run<float, __bf16>(a, stream);
        }
    }
    if (a.elem_in == Elem::F16 && a.elem_out == Elem::F16) {
        return run<_Float16, _Float16>(a, stream);
    }
    if (a.elem_in == Elem::BF16 && a.elem_out == Elem::BF16) {
        return run<__bf16, __bf16>(a, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace opscv
