// Reproducible fp32 2-D convolution (forward, grad-input, grad-kernel), NCHW.
//
// Contract (RepDL backend/cpu/convolution.cpp:12-128): one accumulator per
// output element, starting at +0.0f, one fused multiply-add per contributing
// tap in the reference's lexicographic loop order; taps that fall outside the
// image (or, for grad-input, between strides) are SKIPPED, not multiplied by a
// padded zero -- fma(0, w, acc) differs from a skip when acc is -0.0f or w is
// not finite.
//
// These kernels walk each output's chain directly, one lane per output element
// (grad-kernel: one lane per kernel element), with the spatially fastest index
// on the lane so that neighbouring lanes read neighbouring addresses.
#include "common.h"

namespace
{
struct ConvDims
{
    int N, IC, H, W, OC, KH, KW, OH, OW, sH, sW, pH, pW, groups;
};

// backend/cpu/convolution.cpp:26-50
__global__ __launch_bounds__(256) void conv2d_direct(const float *__restrict__ I,
                                                     const float *__restrict__ Kr,
                                                     float *__restrict__ O, ConvDims d,
                                                     int64_t total)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total)
        return;
    const int ow = (int)(idx % d.OW);
    int64_t t = idx / d.OW;
    const int oh = (int)(t % d.OH);
    t /= d.OH;
    const int oc = (int)(t % d.OC);
    const int n = (int)(t / d.OC);
    const int ICg = d.IC / d.groups, OCg = d.OC / d.groups;
    const int g = oc / OCg;
    float sum = 0.0f;
    for (int i = 0; i < ICg; i++)
    {
        const int ic = g * ICg + i;
        const float *ip = I + ((int64_t)n * d.IC + ic) * d.H * d.W;
        const float *kp = Kr + ((int64_t)oc * ICg + i) * d.KH * d.KW;
        for (int kh = 0; kh < d.KH; kh++)
        {
            const int h = oh * d.sH - d.pH + kh;
            if (h < 0 || h >= d.H)
                continue;
            for (int kw = 0; kw < d.KW; kw++)
            {
                const int w = ow * d.sW - d.pW + kw;
                if (w < 0 || w >= d.W)
                    continue;
                sum = __fmaf_rn(ip[h * d.W + w], kp[kh * d.KW + kw], sum);
            }
        }
    }
    O[idx] = sum;
}

// backend/cpu/convolution.cpp:65-88
__global__ __launch_bounds__(256) void conv2d_grad_input_direct(const float *__restrict__ GO,
                                                                const float *__restrict__ Kr,
                                                                float *__restrict__ GI, ConvDims d,
                                                                int64_t total)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total)
        return;
    const int w = (int)(idx % d.W);
    int64_t t = idx / d.W;
    const int h = (int)(t % d.H);
    t /= d.H;
    const int ic = (int)(t % d.IC);
    const int n = (int)(t / d.IC);
    float sum = 0.0f;
    for (int oc = 0; oc < d.OC; oc++)
    {
        const float *gp = GO + ((int64_t)n * d.OC + oc) * d.OH * d.OW;
        const float *kp = Kr + ((int64_t)oc * d.IC + ic) * d.KH * d.KW;
        for (int kh = 0; kh < d.KH; kh++)
        {
            // C semantics: '/' truncates toward zero and '%' takes the sign of
            // the dividend, as in the reference (:75-77).
            const int th = h - kh + d.pH;
            const int oh = th / d.sH;
            if (oh < 0 || oh >= d.OH || (th % d.sH) != 0)
                continue;
            for (int kw = 0; kw < d.KW; kw++)
            {
                const int tw = w - kw + d.pW;
                const int ow = tw / d.sW;
                if (ow < 0 || ow >= d.OW || (tw % d.sW) != 0)
                    continue;
                sum = __fmaf_rn(gp[oh * d.OW + ow], kp[kh * d.KW + kw], sum);
            }
        }
    }
    GI[idx] = sum;
}

// backend/cpu/convolution.cpp:103-126
__global__ __launch_bounds__(64) void conv2d_grad_kernel_direct(const float *__restrict__ GO,
                                                                const float *__restrict__ I,
                                                                float *__restrict__ GK, ConvDims d,
                                                                int64_t total)
{
    const int64_t idx = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (idx >= total)
        return;
    const int kw = (int)(idx % d.KW);
    int64_t t = idx / d.KW;
    const int kh = (int)(t % d.KH);
    t /= d.KH;
    const int ic = (int)(t % d.IC);
    const int oc = (int)(t / d.IC);
    float sum = 0.0f;
    for (int n = 0; n < d.N; n++)
    {
        const float *gp = GO + ((int64_t)n * d.OC + oc) * d.OH * d.OW;
        const float *ip = I + ((int64_t)n * d.IC + ic) * d.H * d.W;
        for (int oh = 0; oh < d.OH; oh++)
        {
            const int h = oh * d.sH - d.pH + kh;
            if (h < 0 || h >= d.H)
                continue;
            for (int ow = 0; ow < d.OW; ow++)
            {
                const int w = ow * d.sW - d.pW + kw;
                if (w < 0 || w >= d.W)
                    continue;
                sum = __fmaf_rn(gp[oh * d.OW + ow], ip[h * d.W + w], sum);
            }
        }
    }
    GK[idx] = sum;
}

inline bool fits_i32(int64_t v) { return v >= 0 && v <= REPDL_I32_MAX; }
} // namespace

REPDL_API int repdl_hip_conv2d(const float *input, const float *kernel, float *output, int64_t N,
                               int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW,
                               int64_t sH, int64_t sW, int64_t pH, int64_t pW, int64_t groups,
                               void *stream)
{
    REPDL_REQUIRE(N >= 0 && IC >= 0 && H >= 0 && W >= 0 && OC >= 0 && KH > 0 && KW > 0);
    REPDL_REQUIRE(sH > 0 && sW > 0 && pH >= 0 && pW >= 0 && groups > 0);
    REPDL_REQUIRE(IC % groups == 0 && OC % groups == 0);
    REPDL_REQUIRE(H + 2 * pH >= KH && W + 2 * pW >= KW);
    const int64_t OH = (H + 2 * pH - KH) / sH + 1, OW = (W + 2 * pW - KW) / sW + 1;
    const int64_t total = N * OC * OH * OW;
    if (total == 0)
        return REPDL_OK;
    REPDL_REQUIRE(input != nullptr && kernel != nullptr && output != nullptr);
    REPDL_REQUIRE(fits_i32(H * W) && fits_i32(OH * OW) && fits_i32(IC * KH * KW) && fits_i32(N) && fits_i32(OC));
    const int64_t grid = repdl_cdiv(total, 256);
    REPDL_REQUIRE(fits_i32(grid));
    ConvDims d{(int)N, (int)IC, (int)H, (int)W, (int)OC, (int)KH, (int)KW, (int)OH,
               (int)OW, (int)sH, (int)sW, (int)pH, (int)pW, (int)groups};
    hipLaunchKernelGGL(conv2d_direct, dim3((unsigned)grid), dim3(256), 0, repdl_stream(stream), input, kernel,
                       output, d, total);
    return repdl_launch_status();
}

REPDL_API int repdl_hip_conv2d_grad_input(const float *grad_output, const float *kernel,
                                          float *grad_input, int64_t N, int64_t OC, int64_t OH,
                                          int64_t OW, int64_t IC, int64_t KH, int64_t KW, int64_t H,
                                          int64_t W, int64_t sH, int64_t sW, int64_t pH, int64_t pW,
                                          void *stream)
{
    REPDL_REQUIRE(N >= 0 && IC >= 0 && H >= 0 && W >= 0 && OC >= 0 && OH >= 0 && OW >= 0 && KH > 0 && KW > 0);
    REPDL_REQUIRE(sH > 0 && sW > 0 && pH >= 0 && pW >= 0);
    const int64_t total = N * IC * H * W;
    if (total == 0)
        return REPDL_OK;
    REPDL_REQUIRE(grad_input != nullptr);
    REPDL_REQUIRE(OC * OH * OW == 0 || (grad_output != nullptr && kernel != nullptr));
    REPDL_REQUIRE(fits_i32(H * W) && fits_i32(OH * OW) && fits_i32(OC * KH * KW) && fits_i32(N) && fits_i32(IC));
    REPDL_REQUIRE(fits_i32(H + pH) && fits_i32(W + pW));
    const int64_t grid = repdl_cdiv(total, 256);
    REPDL_REQUIRE(fits_i32(grid));
    ConvDims d{(int)N, (int)IC, (int)H, (int)W, (int)OC, (int)KH, (int)KW, (int)OH,
               (int)OW, (int)sH, (int)sW, (int)pH, (int)pW, 1};
    hipLaunchKernelGGL(conv2d_grad_input_direct, dim3((unsigned)grid), dim3(256), 0, repdl_stream(stream),
                       grad_output, kernel, grad_input, d, total);
    return repdl_launch_status();
}

REPDL_API int repdl_hip_conv2d_grad_kernel(const float *grad_output, const float *input,
                                           float *grad_kernel, int64_t N, int64_t IC, int64_t H,
                                           int64_t W, int64_t OC, int64_t OH, int64_t OW, int64_t KH,
                                           int64_t KW, int64_t sH, int64_t sW, int64_t pH, int64_t pW,
                                           void *stream)
{
    REPDL_REQUIRE(N >= 0 && IC >= 0 && H >= 0 && W >= 0 && OC >= 0 && OH >= 0 && OW >= 0 && KH > 0 && KW > 0);
    REPDL_REQUIRE(sH > 0 && sW > 0 && pH >= 0 && pW >= 0);
    const int64_t total = OC * IC * KH * KW;
    if (total == 0)
        return REPDL_OK;
    REPDL_REQUIRE(grad_kernel != nullptr);
    REPDL_REQUIRE(N * OH * OW == 0 || (grad_output != nullptr && input != nullptr));
    REPDL_REQUIRE(fits_i32(H * W) && fits_i32(OH * OW) && fits_i32(N) && fits_i32(IC) && fits_i32(OC));
    REPDL_REQUIRE(fits_i32(OH * sH + KH) && fits_i32(OW * sW + KW));
    const int64_t grid = repdl_cdiv(total, 64);
    REPDL_REQUIRE(fits_i32(grid));
    ConvDims d{(int)N, (int)IC, (int)H, (int)W, (int)OC, (int)KH, (int)KW, (int)OH,
               (int)OW, (int)sH, (int)sW, (int)pH, (int)pW, 1};
    hipLaunchKernelGGL(conv2d_grad_kernel_direct, dim3((unsigned)grid), dim3(64), 0, repdl_stream(stream),
                       grad_output, input, grad_kernel, d, total);
    return repdl_launch_status();
}
