// softmax and cross_entropy for gfx950.
//
// Semantics: RepDL backend/cpu/softmax.cpp:15-21 and cross_entropy.cpp:15-24 --
// compositions of a row maximum, exp, the SERIAL row sum, log / division and (for
// the loss) a serial mean over the rows.  One wave owns one row: the maximum is a
// wave reduction (max is exact, so its order is free), exp / division are done
// lane-parallel, and the row sum is a strict j = 0..N-1 chain that every lane
// evaluates redundantly from LDS broadcasts, so all lanes hold the same sum.
// NaN logits are outside the contract (NaN-ness propagates, payload unspecified).
#include "common.h"
#include "crmath.h"

namespace
{
__device__ const uint64_t g_exp_tab2[256] = CRM_EXP_TAB_INIT;
__device__ const float g_log_invc2[128] = CRM_LOG_INVC_INIT;
__device__ const double g_log_hi2[128] = CRM_LOG_HI_INIT;
__device__ const float g_log_lo2[128] = CRM_LOG_LO_INIT;

constexpr int CH = 256; // columns staged per pass

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
    {
        float o = __shfl_xor(v, off, 64);
        // NaN-propagating maximum
        v = (o != o) ? o : ((v != v) ? v : (o > v ? o : v));
    }
    return v;
}

__device__ __forceinline__ float row_max(const float *x, int64_t N, int lane)
{
    float m = -__builtin_inff();
    bool has = false;
    for (int64_t j = lane; j < N; j += 64)
    {
        float v = x[j];
        m = (v != v) ? v : ((m != m) ? m : (v > m ? v : m));
        has = true;
    }
    (void)has;
    return wave_max(m);
}

// e_j = exp(x_j - m) for one row, written to e_out (if not null); returns the
// serial sum over j, identical in every lane.
__device__ __forceinline__ float row_exp_sum(const float *x, float *e_out, int64_t N, float m,
                                             int lane, float *stage, const uint64_t *exp_tab)
{
    float acc = 0.0f;
    for (int64_t c0 = 0; c0 < N; c0 += CH)
    {
#pragma unroll
        for (int u = 0; u < CH / 64; u++)
        {
            int64_t j = c0 + lane + 64 * u;
            float e = 0.0f;
            if (j < N)
            {
                e = crm_exp(x[j] - m, exp_tab);
                if (e_out)
                    e_out[j] = e;
            }
            stage[lane + 64 * u] = e;
        }
        __syncthreads();
        const int cnt = (N - c0 < CH) ? (int)(N - c0) : CH;
        for (int c = 0; c < cnt; c++)
            acc = acc + stage[c];
        __syncthreads();
    }
    return acc;
}

__global__ __launch_bounds__(64) void softmax_kernel(const float *__restrict__ in,
                                                     float *__restrict__ out, int64_t M, int64_t N)
{
    __shared__ uint64_t exp_tab[256];
    __shared__ float stage[CH];
    const int lane = threadIdx.x;
    for (int i = lane; i < 256; i += 64)
        exp_tab[i] = g_exp_tab2[i];
    __syncthreads();
    const int64_t row = blockIdx.x;
    const float *x = in + row * N;
    float *o = out + row * N;
    const float m = row_max(x, N, lane);
    const float sum = row_exp_sum(x, o, N, m, lane, stage, exp_tab);
    const crm_divisor d = crm_divisor_make(sum);
    __syncthreads();
    for (int64_t j = lane; j < N; j += 64)
        o[j] = crm_div_by(o[j], d);
}

__global__ __launch_bounds__(64) void cross_entropy_rows_kernel(const float *__restrict__ in,
                                                                const int64_t *__restrict__ target,
                                                                float *__restrict__ loss, int64_t M,
                                                                int64_t N)
{
    __shared__ uint64_t exp_tab[256];
    __shared__ double log_hi[128];
    __shared__ float log_invc[128], log_lo[128];
    __shared__ float stage[CH];
    const int lane = threadIdx.x;
    for (int i = lane; i < 256; i += 64)
        exp_tab[i] = g_exp_tab2[i];
    for (int i = lane; i < 128; i += 64)
    {
        log_hi[i] = g_log_hi2[i];
        log_invc[i] = g_log_invc2[i];
        log_lo[i] = g_log_lo2[i];
    }
    __syncthreads();
    const int64_t row = blockIdx.x;
    const float *x = in + row * N;
    const float m = row_max(x, N, lane);
    const float sum = row_exp_sum(x, nullptr, N, m, lane, stage, exp_tab);
    if (lane == 0)
    {
        crm_log_tables lt;
        lt.invc = log_invc;
        lt.logc_hi = log_hi;
        lt.logc_lo = log_lo;
        float l = crm_log(sum, lt);
        int64_t t = target[row];
        float shifted = (t >= 0 && t < N) ? x[t] - m : __builtin_nanf("");
        loss[row] = l - shifted;
    }
}
} // namespace

REPDL_API int repdl_hip_softmax(const float *in, float *out, int64_t M, int64_t N, void *stream)
{
    REPDL_REQUIRE(M >= 0 && N >= 0);
    if (M == 0 || N == 0)
        return REPDL_OK;
    REPDL_REQUIRE(in != nullptr && out != nullptr && M <= REPDL_I32_MAX);
    hipLaunchKernelGGL(softmax_kernel, dim3((unsigned)M), dim3(64), 0, repdl_stream(stream), in, out, M, N);
    return repdl_launch_status();
}

REPDL_API int repdl_hip_cross_entropy(const float *in, const int64_t *target, float *out, int64_t M,
                                      int64_t N, float *workspace, void *stream)
{
    REPDL_REQUIRE(M >= 0 && N > 0 && out != nullptr);
    if (M > 0)
    {
        REPDL_REQUIRE(in != nullptr && target != nullptr && M <= REPDL_I32_MAX);
        if (workspace == nullptr)
            return REPDL_E_WORKSPACE;
        hipLaunchKernelGGL(cross_entropy_rows_kernel, dim3((unsigned)M), dim3(64), 0, repdl_stream(stream),
                           in, target, workspace, M, N);
        int rc = repdl_launch_status();
        if (rc != REPDL_OK)
            return rc;
    }
    return repdl_hip_sum1d(workspace, out, M, 1, stream);
}
