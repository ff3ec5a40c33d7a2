// Elementwise correctly rounded operators for gfx950: exp, log, sqrt, div.
//
// Semantics: RepDL backend/cpu/math.cpp:14-17, 32-35 (exp, log: glibc's binary64
// routine followed by one rounding to binary32) and repdl/ops.py:98-103, 122-123
// (div, sqrt: the IEEE binary32 results).  The arithmetic lives in crmath.h and
// uses no approximate-function instruction and no '/' operator; this file only
// streams the data: 16-byte loads and stores, grid-stride, several loads in
// flight per lane; the exp/log tables (2 KiB / 4 KiB) are copied to LDS once per
// workgroup.  All four are HBM-bound: 8 bytes per element (12 for tensor/tensor
// division).
#include "common.h"
#include "crmath.h"

namespace
{
__device__ const uint64_t g_exp_tab[256] = CRM_EXP_TAB_INIT;
__device__ const double g_log_tab[512] = CRM_LOG_TAB_INIT;

constexpr int EW_THREADS = 256;
constexpr int EW_UNROLL = 4; // float4 per lane per iteration

enum Op
{
    OP_EXP,
    OP_LOG,
    OP_SQRT,
    OP_DIV_SCALAR
};

template <int OP>
struct Ctx
{
    const uint64_t *exp_tab;
    const double *log_tab;
    crm_divisor divisor;
    __device__ __forceinline__ float apply(float x) const
    {
        if (OP == OP_EXP)
            return crm_exp(x, exp_tab);
        if (OP == OP_LOG)
            return crm_log(x, log_tab);
        if (OP == OP_SQRT)
            return crm_sqrt(x);
        return crm_div_by(x, divisor);
    }
};

template <int OP>
__global__ __launch_bounds__(EW_THREADS) void unary_kernel(const float *__restrict__ in,
                                                           float *__restrict__ out, int64_t n,
                                                           float scalar, int vec_ok)
{
    __shared__ __attribute__((aligned(16))) uint64_t tab[512];
    Ctx<OP> ctx;
    ctx.exp_tab = tab;
    ctx.log_tab = reinterpret_cast<const double *>(tab);
    if (OP == OP_EXP)
    {
        for (int i = threadIdx.x; i < 256; i += EW_THREADS)
            tab[i] = g_exp_tab[i];
        __syncthreads();
    }
    if (OP == OP_LOG)
    {
        for (int i = threadIdx.x; i < 512; i += EW_THREADS)
            tab[i] = crm_d2u(g_log_tab[i]);
        __syncthreads();
    }
    if (OP == OP_DIV_SCALAR)
        ctx.divisor = crm_divisor_make(scalar);

    const int64_t tid = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x;
    const int64_t nthreads = (int64_t)gridDim.x * EW_THREADS;
    int64_t done = 0;
    if (vec_ok)
    {
        const int64_t n4 = n >> 2;
        const float4 *in4 = reinterpret_cast<const float4 *>(in);
        float4 *out4 = reinterpret_cast<float4 *>(out);
        int64_t i = tid;
        for (; i + (EW_UNROLL - 1) * nthreads < n4; i += EW_UNROLL * nthreads)
        {
            float4 v[EW_UNROLL];
#pragma unroll
            for (int u = 0; u < EW_UNROLL; u++)
                v[u] = in4[i + u * nthreads];
#pragma unroll
            for (int u = 0; u < EW_UNROLL; u++)
            {
                float4 r;
                r.x = ctx.apply(v[u].x);
                r.y = ctx.apply(v[u].y);
                r.z = ctx.apply(v[u].z);
                r.w = ctx.apply(v[u].w);
                out4[i + u * nthreads] = r;
            }
        }
        for (; i < n4; i += nthreads)
        {
            float4 v = in4[i], r;
            r.x = ctx.apply(v.x);
            r.y = ctx.apply(v.y);
            r.z = ctx.apply(v.z);
            r.w = ctx.apply(v.w);
            out4[i] = r;
        }
        done = n4 << 2;
    }
    for (int64_t i = done + tid; i < n; i += nthreads)
        out[i] = ctx.apply(in[i]);
}

__global__ __launch_bounds__(EW_THREADS) void div_kernel(const float *__restrict__ a,
                                                         const float *__restrict__ b,
                                                         float *__restrict__ out, int64_t n,
                                                         int vec_ok)
{
    const int64_t tid = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x;
    const int64_t nthreads = (int64_t)gridDim.x * EW_THREADS;
    int64_t done = 0;
    if (vec_ok)
    {
        const int64_t n4 = n >> 2;
        const float4 *a4 = reinterpret_cast<const float4 *>(a);
        const float4 *b4 = reinterpret_cast<const float4 *>(b);
        float4 *out4 = reinterpret_cast<float4 *>(out);
        int64_t i = tid;
        for (; i + nthreads < n4; i += 2 * nthreads)
        {
            float4 x0 = a4[i], y0 = b4[i], x1 = a4[i + nthreads], y1 = b4[i + nthreads], r;
            r.x = crm_div(x0.x, y0.x);
            r.y = crm_div(x0.y, y0.y);
            r.z = crm_div(x0.z, y0.z);
            r.w = crm_div(x0.w, y0.w);
            out4[i] = r;
            r.x = crm_div(x1.x, y1.x);
            r.y = crm_div(x1.y, y1.y);
            r.z = crm_div(x1.z, y1.z);
            r.w = crm_div(x1.w, y1.w);
            out4[i + nthreads] = r;
        }
        for (; i < n4; i += nthreads)
        {
            float4 x = a4[i], y = b4[i], r;
            r.x = crm_div(x.x, y.x);
            r.y = crm_div(x.y, y.y);
            r.z = crm_div(x.z, y.z);
            r.w = crm_div(x.w, y.w);
            out4[i] = r;
        }
        done = n4 << 2;
    }
    for (int64_t i = done + tid; i < n; i += nthreads)
        out[i] = crm_div(a[i], b[i]);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

inline unsigned ew_grid(int64_t n)
{
    // 8 workgroups per CU on 256 CUs, fewer for small inputs
    int64_t want = repdl_cdiv(repdl_cdiv(n, 4), EW_THREADS);
    if (want > 2048)
        want = 2048;
    if (want < 1)
        want = 1;
    return (unsigned)want;
}

template <int OP>
int launch_unary(const float *in, float *out, int64_t n, float scalar, void *stream)
{
    REPDL_REQUIRE(n >= 0);
    if (n == 0)
        return REPDL_OK;
    REPDL_REQUIRE(in != nullptr && out != nullptr);
    const int vec_ok = aligned16(in) && aligned16(out);
    hipLaunchKernelGGL((unary_kernel<OP>), dim3(ew_grid(n)), dim3(EW_THREADS), 0, repdl_stream(stream), in,
                       out, n, scalar, vec_ok);
    return repdl_launch_status();
}
} // namespace

REPDL_API int repdl_hip_exp(const float *in, float *out, int64_t n, void *stream)
{
    return launch_unary<OP_EXP>(in, out, n, 0.0f, stream);
}

REPDL_API int repdl_hip_log(const float *in, float *out, int64_t n, void *stream)
{
    return launch_unary<OP_LOG>(in, out, n, 0.0f, stream);
}

REPDL_API int repdl_hip_sqrt(const float *in, float *out, int64_t n, void *stream)
{
    return launch_unary<OP_SQRT>(in, out, n, 0.0f, stream);
}

REPDL_API int repdl_hip_div_scalar(const float *a, float b, float *out, int64_t n, void *stream)
{
    return launch_unary<OP_DIV_SCALAR>(a, out, n, b, stream);
}

REPDL_API int repdl_hip_div(const float *a, const float *b, float *out, int64_t n, void *stream)
{
    REPDL_REQUIRE(n >= 0);
    if (n == 0)
        return REPDL_OK;
    REPDL_REQUIRE(a != nullptr && b != nullptr && out != nullptr);
    const int vec_ok = aligned16(a) && aligned16(b) && aligned16(out);
    hipLaunchKernelGGL(div_kernel, dim3(ew_grid(n)), dim3(EW_THREADS), 0, repdl_stream(stream), a, b, out, n,
                       vec_ok);
    return repdl_launch_status();
}
