// Elementwise correctly rounded operators for gfx950: exp, log, sqrt, div.
//
// Semantics: RepDL backend/cpu/math.cpp:14-17, 32-35 (exp, log: glibc's binary64
// routine followed by one rounding to binary32) and repdl/ops.py:98-103, 122-123
// (div, sqrt: the IEEE binary32 results).  The arithmetic lives in crmath.h and
// uses no approximate-function instruction and no '/' operator; this file only
// streams the data: 16-byte non-temporal loads and stores, one small contiguous
// chunk per workgroup, four loads in flight per lane; the exp/log tables (2 KiB each) are copied to LDS once per
// workgroup.  All four are HBM-bound: 8 bytes per element (12 for tensor/tensor
// division).
#include "common.h"
#include "crmath.h"

namespace
{
__device__ const uint64_t g_exp_tab[256] = CRM_EXP_TAB_INIT;
__device__ const float g_log_invc[128] = CRM_LOG_INVC_INIT;
__device__ const double g_log_hi[128] = CRM_LOG_HI_INIT;
__device__ const float g_log_lo[128] = CRM_LOG_LO_INIT;

constexpr int EW_THREADS = 256;
constexpr int EW_UNROLL = 4;                     // 16-byte accesses in flight per lane
constexpr int EW_CHUNK = EW_THREADS * EW_UNROLL; // float4 per workgroup (16 KiB in, 16 KiB out)

typedef float v4f __attribute__((ext_vector_type(4)));

// Streaming accesses: every byte is touched once, so loads and stores carry the
// non-temporal hint and each workgroup owns one small contiguous chunk (many small
// workgroups keep more independent loads in flight than few long-running ones).
__device__ __forceinline__ v4f ld_stream(const v4f *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st_stream(v4f v, v4f *p) { __builtin_nontemporal_store(v, p); }

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
    crm_log_tables_wide log_tab;
    crm_divisor divisor;
    __device__ __forceinline__ float apply(float x) const
    {
        if (OP == OP_EXP)
            return crm_exp(x, exp_tab);
        if (OP == OP_LOG)
            return crm_log_wide(x, log_tab);
        if (OP == OP_SQRT)
            return crm_sqrt(x);
        return crm_div_by(x, divisor);
    }
    __device__ __forceinline__ v4f apply4(v4f v) const
    {
        v4f r;
        r.x = apply(v.x);
        r.y = apply(v.y);
        r.z = apply(v.z);
        r.w = apply(v.w);
        return r;
    }
};

template <int OP>
__global__ __launch_bounds__(EW_THREADS) void unary_kernel(const float *__restrict__ in,
                                                           float *__restrict__ out, int64_t n,
                                                           float scalar, int vec_ok)
{
    // exp: 256 words (tail, sbits pairs); log: logc_hi[128], invc[128], logc_lo[128], all binary64
    __shared__ __attribute__((aligned(16))) uint64_t tab[OP == OP_LOG ? 384 : 256];
    Ctx<OP> ctx;
    ctx.exp_tab = tab;
    double *lhi = reinterpret_cast<double *>(tab);
    double *linvc = lhi + 128, *llo = lhi + (OP == OP_LOG ? 256 : 128);
    ctx.log_tab.invc = linvc;
    ctx.log_tab.logc_hi = lhi;
    ctx.log_tab.logc_lo = llo;
    if (OP == OP_DIV_SCALAR)
        ctx.divisor = crm_divisor_make(scalar);

    const int64_t n4 = n >> 2;
    const int64_t b0 = (int64_t)blockIdx.x * EW_CHUNK;
    const bool full = vec_ok && b0 + EW_CHUNK <= n4;
    const v4f *in4 = reinterpret_cast<const v4f *>(in);
    v4f *out4 = reinterpret_cast<v4f *>(out);

    // the streaming loads go out first, then the table fill, so that both are in flight
    // together
    v4f v[EW_UNROLL];
    if (full)
    {
#pragma unroll
        for (int u = 0; u < EW_UNROLL; u++)
            v[u] = ld_stream(&in4[b0 + threadIdx.x + u * EW_THREADS]);
    }
    if (OP == OP_EXP)
    {
        for (int i = threadIdx.x; i < 256; i += EW_THREADS)
            tab[i] = g_exp_tab[i];
        __syncthreads();
    }
    if (OP == OP_LOG)
    {
        if (threadIdx.x < 128)
        {
            lhi[threadIdx.x] = g_log_hi[threadIdx.x];
            linvc[threadIdx.x] = (double)g_log_invc[threadIdx.x];
            llo[threadIdx.x] = (double)g_log_lo[threadIdx.x];
        }
        __syncthreads();
    }
    if (full)
    {
#pragma unroll
        for (int u = 0; u < EW_UNROLL; u++)
            st_stream(ctx.apply4(v[u]), &out4[b0 + threadIdx.x + u * EW_THREADS]);
        return;
    }
    // partial last chunk, the (n mod 4) tail, or unaligned pointers: element by element
    const int64_t e0 = b0 * 4;
    const int64_t e1 = e0 + EW_CHUNK * 4 < n ? e0 + EW_CHUNK * 4 : n;
    for (int64_t i = e0 + threadIdx.x; i < e1; i += EW_THREADS)
        out[i] = ctx.apply(in[i]);
}

__device__ __forceinline__ v4f div4(v4f a, v4f b)
{
    v4f r;
    r.x = crm_div(a.x, b.x);
    r.y = crm_div(a.y, b.y);
    r.z = crm_div(a.z, b.z);
    r.w = crm_div(a.w, b.w);
    return r;
}

__global__ __launch_bounds__(EW_THREADS) void div_kernel(const float *__restrict__ a,
                                                         const float *__restrict__ b,
                                                         float *__restrict__ out, int64_t n,
                                                         int vec_ok)
{
    const int64_t n4 = n >> 2;
    const int64_t b0 = (int64_t)blockIdx.x * EW_CHUNK;
    if (vec_ok && b0 + EW_CHUNK <= n4)
    {
        const v4f *a4 = reinterpret_cast<const v4f *>(a);
        const v4f *b4 = reinterpret_cast<const v4f *>(b);
        v4f *out4 = reinterpret_cast<v4f *>(out);
        v4f x[EW_UNROLL], y[EW_UNROLL];
#pragma unroll
        for (int u = 0; u < EW_UNROLL; u++)
        {
            x[u] = ld_stream(&a4[b0 + threadIdx.x + u * EW_THREADS]);
            y[u] = ld_stream(&b4[b0 + threadIdx.x + u * EW_THREADS]);
        }
#pragma unroll
        for (int u = 0; u < EW_UNROLL; u++)
            st_stream(div4(x[u], y[u]), &out4[b0 + threadIdx.x + u * EW_THREADS]);
        return;
    }
    const int64_t e0 = b0 * 4;
    const int64_t e1 = e0 + EW_CHUNK * 4 < n ? e0 + EW_CHUNK * 4 : n;
    for (int64_t i = e0 + threadIdx.x; i < e1; i += EW_THREADS)
        out[i] = crm_div(a[i], b[i]);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// one workgroup per EW_CHUNK float4 (4 * EW_CHUNK elements)
inline int64_t ew_grid(int64_t n) { return repdl_cdiv(n, 4 * (int64_t)EW_CHUNK); }

template <int OP>
int launch_unary(const float *in, float *out, int64_t n, float scalar, void *stream)
{
    REPDL_REQUIRE(n >= 0);
    if (n == 0)
        return REPDL_OK;
    REPDL_REQUIRE(in != nullptr && out != nullptr);
    const int vec_ok = aligned16(in) && aligned16(out);
    const int64_t grid = ew_grid(n);
    REPDL_REQUIRE(grid <= REPDL_I32_MAX);
    hipLaunchKernelGGL((unary_kernel<OP>), dim3((unsigned)grid), dim3(EW_THREADS), 0, repdl_stream(stream), in,
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
    const int64_t grid = ew_grid(n);
    REPDL_REQUIRE(grid <= REPDL_I32_MAX);
    hipLaunchKernelGGL(div_kernel, dim3((unsigned)grid), dim3(EW_THREADS), 0, repdl_stream(stream), a, b, out, n,
                       vec_ok);
    return repdl_launch_status();
}
