// Optimizer updates as one fused elementwise pass over a list of tensors.
//
// RepDL's optimizers are Python sequences of tensor operations (repdl/optim.py:56-83 for
// Adam): every operation rounds once, and the reproducible operators are ops.sqrt and a
// true division.  Here the same sequence is evaluated per element in registers, with each
// rounding written out (the file is compiled with -ffp-contract=off, so only the explicit
// fmaf calls fuse), and the tensors of a parameter group share launches: the kernel
// argument carries up to OPT_MAX_TENSORS tensor descriptors and a block -> tensor map, so a
// model with many small parameters costs one launch instead of a dozen per parameter.
//
// Adam, per element (b1, b2, 1-b1, 1-b2, eps, wd, sqrt(1-b2^t) and -(lr/(1-b1^t)) are
// computed by the caller in binary64 and rounded to binary32 once, as PyTorch rounds a
// Python number that meets a float32 tensor):
//   g' = wd != 0 ? fma(wd, p, g) : g              grad.add(param, alpha=wd)        optim.py:64-66
//   m  = fma(1-b1, g', RN(m * b1))                exp_avg.mul_(b1).add_(g', alpha) optim.py:68
//   v  = RN(RN(v * b2) + RN(RN(g' * g') * (1-b2)))                                 optim.py:69
//   s  = amsgrad ? (vmax = max(vmax, v)) : v      torch.maximum, NaN if either is  optim.py:71-74
//   d  = RN(div(sqrt(s), sqrt(1-b2^t)) + eps)     ops.div(ops.sqrt(.), .).add_     optim.py:75-81
//   p  = RN(p + RN(div(m, d) * -(lr/(1-b1^t))))   param.add_(div(m, d).mul(-step)) optim.py:82-83
// SGD: p = RN(p - RN(g * lr)).
// All of it is HBM-bound streaming: Adam moves 28 bytes per element (36 with amsgrad),
// SGD 12.
#include "common.h"
#include "crmath.h"

namespace
{
constexpr int OPT_THREADS = 256;
constexpr int OPT_UNROLL = 2;                       // 16-byte accesses in flight per lane and stream
constexpr int OPT_CHUNK = OPT_THREADS * OPT_UNROLL; // float4 per workgroup
constexpr int OPT_ELEMS = OPT_CHUNK * 4;            // elements per workgroup
constexpr int OPT_MAX_TENSORS = 32;                 // descriptors per launch (kernel argument < 4 KiB)

typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4f ld_stream(const v4f *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st_stream(v4f v, v4f *p) { __builtin_nontemporal_store(v, p); }

struct AdamHyper
{
    float beta1, one_minus_beta1, beta2, one_minus_beta2, eps, weight_decay;
};

template <typename T>
struct Batch
{
    T t[OPT_MAX_TENSORS];
    int first_block[OPT_MAX_TENSORS + 1]; // first_block[i] .. first_block[i+1]: workgroups of tensor i
    unsigned vec_mask;                    // bit i: every pointer of tensor i is 16-byte aligned
    int count;
};

// the tensor that owns this workgroup (uniform over the workgroup)
template <typename T>
__device__ __forceinline__ int owner(const Batch<T> &b)
{
    int lo = 0, hi = b.count;
    while (hi - lo > 1)
    {
        const int mid = (lo + hi) >> 1;
        if (b.first_block[mid] <= (int)blockIdx.x)
            lo = mid;
        else
            hi = mid;
    }
    return lo;
}

// torch.maximum: NaN if either operand is
__device__ __forceinline__ float max_nan(float a, float b)
{
    if (a != a)
        return a;
    if (b != b)
        return b;
    return a > b ? a : b;
}

struct AdamCtx
{
    AdamHyper h;
    crm_divisor root_bc2;
    float step_scale;
    bool amsgrad, decay;

    __device__ __forceinline__ void apply(float &p, float g, float &m, float &v, float &vmax) const
    {
        if (decay)
            g = fmaf(h.weight_decay, p, g);
        m = fmaf(h.one_minus_beta1, g, m * h.beta1);
        v = (v * h.beta2) + ((g * g) * h.one_minus_beta2);
        float second = v;
        if (amsgrad)
        {
            vmax = max_nan(vmax, v);
            second = vmax;
        }
        const float denom = crm_div_by(crm_sqrt(second), root_bc2) + h.eps;
        p = p + crm_div(m, denom) * step_scale;
    }
    __device__ __forceinline__ void apply4(v4f &p, v4f g, v4f &m, v4f &v, v4f &vmax) const
    {
#pragma unroll
        for (int k = 0; k < 4; k++)
        {
            float pk = p[k], mk = m[k], vk = v[k], xk = vmax[k];
            apply(pk, g[k], mk, vk, xk);
            p[k] = pk;
            m[k] = mk;
            v[k] = vk;
            vmax[k] = xk;
        }
    }
};

__global__ __launch_bounds__(OPT_THREADS) void adam_kernel(const Batch<repdl_adam_tensor> b, const AdamHyper h)
{
    const int ti = owner(b);
    const repdl_adam_tensor t = b.t[ti];
    AdamCtx c;
    c.h = h;
    c.root_bc2 = crm_divisor_make(t.sqrt_bias_correction2);
    c.step_scale = t.step_scale;
    c.amsgrad = t.max_exp_avg_sq != nullptr;
    c.decay = h.weight_decay != 0.0f;

    const int64_t n4 = t.n >> 2;
    const int64_t b0 = (int64_t)((int)blockIdx.x - b.first_block[ti]) * OPT_CHUNK;
    if (((b.vec_mask >> ti) & 1u) && b0 + OPT_CHUNK <= n4)
    {
        v4f *p4 = reinterpret_cast<v4f *>(t.param);
        const v4f *g4 = reinterpret_cast<const v4f *>(t.grad);
        v4f *m4 = reinterpret_cast<v4f *>(t.exp_avg);
        v4f *v4 = reinterpret_cast<v4f *>(t.exp_avg_sq);
        v4f *x4 = reinterpret_cast<v4f *>(t.max_exp_avg_sq);
        v4f p[OPT_UNROLL], g[OPT_UNROLL], m[OPT_UNROLL], v[OPT_UNROLL], x[OPT_UNROLL];
#pragma unroll
        for (int u = 0; u < OPT_UNROLL; u++)
        {
            const int64_t i = b0 + threadIdx.x + u * OPT_THREADS;
            p[u] = ld_stream(&p4[i]);
            g[u] = ld_stream(&g4[i]);
            m[u] = ld_stream(&m4[i]);
            v[u] = ld_stream(&v4[i]);
            if (c.amsgrad)
                x[u] = ld_stream(&x4[i]);
            else
                x[u] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int u = 0; u < OPT_UNROLL; u++)
        {
            const int64_t i = b0 + threadIdx.x + u * OPT_THREADS;
            c.apply4(p[u], g[u], m[u], v[u], x[u]);
            st_stream(p[u], &p4[i]);
            st_stream(m[u], &m4[i]);
            st_stream(v[u], &v4[i]);
            if (c.amsgrad)
                st_stream(x[u], &x4[i]);
        }
        return;
    }
    // partial last chunk, the (n mod 4) tail, or unaligned pointers: element by element
    const int64_t e0 = b0 * 4;
    const int64_t e1 = e0 + OPT_ELEMS < t.n ? e0 + OPT_ELEMS : t.n;
    for (int64_t i = e0 + threadIdx.x; i < e1; i += OPT_THREADS)
    {
        float p = t.param[i], m = t.exp_avg[i], v = t.exp_avg_sq[i];
        float x = c.amsgrad ? t.max_exp_avg_sq[i] : 0.0f;
        c.apply(p, t.grad[i], m, v, x);
        t.param[i] = p;
        t.exp_avg[i] = m;
        t.exp_avg_sq[i] = v;
        if (c.amsgrad)
            t.max_exp_avg_sq[i] = x;
    }
}

__global__ __launch_bounds__(OPT_THREADS) void sgd_kernel(const Batch<repdl_sgd_tensor> b, const float lr)
{
    const int ti = owner(b);
    const repdl_sgd_tensor t = b.t[ti];
    const int64_t n4 = t.n >> 2;
    const int64_t b0 = (int64_t)((int)blockIdx.x - b.first_block[ti]) * OPT_CHUNK;
    if (((b.vec_mask >> ti) & 1u) && b0 + OPT_CHUNK <= n4)
    {
        v4f *p4 = reinterpret_cast<v4f *>(t.param);
        const v4f *g4 = reinterpret_cast<const v4f *>(t.grad);
        v4f p[OPT_UNROLL], g[OPT_UNROLL];
#pragma unroll
        for (int u = 0; u < OPT_UNROLL; u++)
        {
            p[u] = ld_stream(&p4[b0 + threadIdx.x + u * OPT_THREADS]);
            g[u] = ld_stream(&g4[b0 + threadIdx.x + u * OPT_THREADS]);
        }
#pragma unroll
        for (int u = 0; u < OPT_UNROLL; u++)
        {
            v4f r;
            r.x = p[u].x - g[u].x * lr;
            r.y = p[u].y - g[u].y * lr;
            r.z = p[u].z - g[u].z * lr;
            r.w = p[u].w - g[u].w * lr;
            st_stream(r, &p4[b0 + threadIdx.x + u * OPT_THREADS]);
        }
        return;
    }
    const int64_t e0 = b0 * 4;
    const int64_t e1 = e0 + OPT_ELEMS < t.n ? e0 + OPT_ELEMS : t.n;
    for (int64_t i = e0 + threadIdx.x; i < e1; i += OPT_THREADS)
        t.param[i] = t.param[i] - t.grad[i] * lr;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

inline bool pointers_ok(const repdl_adam_tensor &t)
{
    return t.param != nullptr && t.grad != nullptr && t.exp_avg != nullptr && t.exp_avg_sq != nullptr;
}
inline bool pointers_ok(const repdl_sgd_tensor &t) { return t.param != nullptr && t.grad != nullptr; }

inline bool vector_ok(const repdl_adam_tensor &t)
{
    return aligned16(t.param) && aligned16(t.grad) && aligned16(t.exp_avg) && aligned16(t.exp_avg_sq) &&
           aligned16(t.max_exp_avg_sq);
}
inline bool vector_ok(const repdl_sgd_tensor &t) { return aligned16(t.param) && aligned16(t.grad); }

// Packs the non-empty tensors into batches of at most OPT_MAX_TENSORS descriptors (and
// fewer than 2^31 workgroups) and hands each batch to `launch`.
template <typename T, typename Launch>
int for_batches(const T *tensors, int count, Launch launch)
{
    REPDL_REQUIRE(count >= 0);
    REPDL_REQUIRE(count == 0 || tensors != nullptr);
    for (int i = 0; i < count; i++)
    {
        REPDL_REQUIRE(tensors[i].n >= 0);
        REPDL_REQUIRE(tensors[i].n == 0 || pointers_ok(tensors[i]));
        REPDL_REQUIRE(repdl_cdiv(tensors[i].n, OPT_ELEMS) <= REPDL_I32_MAX);
    }
    Batch<T> b;
    b.count = 0;
    b.vec_mask = 0;
    b.first_block[0] = 0;
    for (int i = 0; i < count; i++)
    {
        if (tensors[i].n == 0)
            continue;
        const int64_t blocks = repdl_cdiv(tensors[i].n, OPT_ELEMS);
        if (b.count == OPT_MAX_TENSORS || (int64_t)b.first_block[b.count] + blocks > REPDL_I32_MAX)
        {
            const int rc = launch(b);
            if (rc != REPDL_OK)
                return rc;
            b.count = 0;
            b.vec_mask = 0;
        }
        b.t[b.count] = tensors[i];
        if (vector_ok(tensors[i]))
            b.vec_mask |= 1u << b.count;
        b.first_block[b.count + 1] = b.first_block[b.count] + (int)blocks;
        b.count++;
    }
    return b.count ? launch(b) : REPDL_OK;
}
} // namespace

REPDL_API int repdl_hip_adam_step(const repdl_adam_tensor *tensors, int count, float beta1, float one_minus_beta1,
                                  float beta2, float one_minus_beta2, float eps, float weight_decay, void *stream)
{
    const AdamHyper h{beta1, one_minus_beta1, beta2, one_minus_beta2, eps, weight_decay};
    return for_batches(tensors, count, [&](const Batch<repdl_adam_tensor> &b) {
        hipLaunchKernelGGL(adam_kernel, dim3((unsigned)b.first_block[b.count]), dim3(OPT_THREADS), 0,
                           repdl_stream(stream), b, h);
        return repdl_launch_status();
    });
}

REPDL_API int repdl_hip_sgd_step(const repdl_sgd_tensor *tensors, int count, float lr, void *stream)
{
    return for_batches(tensors, count, [&](const Batch<repdl_sgd_tensor> &b) {
        hipLaunchKernelGGL(sgd_kernel, dim3((unsigned)b.first_block[b.count]), dim3(OPT_THREADS), 0,
                           repdl_stream(stream), b, lr);
        return repdl_launch_status();
    });
}
