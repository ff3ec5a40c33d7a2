// The elementwise passes of batch normalisation, fused.
//
// RepDL's batch norm (repdl/nn/batchnorm.py:12-66) is a composition of PyTorch elementwise
// operations around its reproducible sums, divisions and square root; every operation rounds
// once.  The three compositions that run over the whole activation tensor are evaluated here
// per element in registers with the same roundings in the same order (compiled with
// -ffp-contract=off: nothing fuses), one pass over memory each instead of three or four:
//   apply     y = RN(RN(RN(RN(x - mean[c]) / std[c]) * weight[c]) + bias[c])   forward, batchnorm.py:25-32
//   gvar      t = RN(RN(gy * RN(mean[c] - x)) * coef[c])                        integrand of grad_var, :56-58
//   gweight   t = RN(RN(RN(x - mean[c]) / std[c]) * gy)                         integrand of grad_weight, :60-61
// The tensors are [outer][channels][inner] (NCHW: outer = N, inner = H*W; [B,F]: inner = 1).
// All HBM-bound streaming: 8 B/element for apply, 12 for the two integrands.
#include "common.h"
#include "crmath.h"

namespace
{
constexpr int BN_THREADS = 256;
constexpr int BN_UNROLL = 4;
constexpr int BN_CHUNK = BN_THREADS * BN_UNROLL * 4; // elements per workgroup

typedef float v4f __attribute__((ext_vector_type(4)));

enum BnMode
{
    BN_APPLY,
    BN_GVAR,
    BN_GWEIGHT
};

// per-channel constants of one mode
struct BnChannel
{
    float mean, w, b, coef;
    crm_divisor std;
};

template <int MODE>
__device__ __forceinline__ BnChannel bn_channel(const float *mean, const float *p1, const float *p2, const float *p3, int64_t c)
{
    // APPLY: p1 = std, p2 = weight, p3 = bias;  GVAR: p1 = coef;  GWEIGHT: p1 = std
    BnChannel ch;
    ch.mean = mean[c];
    ch.w = ch.b = ch.coef = 0.0f;
    if (MODE == BN_APPLY)
    {
        ch.std = crm_divisor_make(p1[c]);
        ch.w = p2[c];
        ch.b = p3[c];
    }
    else if (MODE == BN_GVAR)
    {
        ch.std = crm_divisor_make(1.0f);
        ch.coef = p1[c];
    }
    else
        ch.std = crm_divisor_make(p1[c]);
    return ch;
}

// a: x (APPLY, GWEIGHT) or gy (GVAR);  b: unused (APPLY), x (GVAR), gy (GWEIGHT)
template <int MODE>
__device__ __forceinline__ float bn_value(float a, float b, const BnChannel &ch)
{
    if (MODE == BN_APPLY)
        return (crm_div_by(a - ch.mean, ch.std) * ch.w) + ch.b;
    if (MODE == BN_GVAR)
        return (a * (ch.mean - b)) * ch.coef;
    return crm_div_by(a - ch.mean, ch.std) * b;
}

// Rows of at least one chunk: a workgroup stays inside one (outer, channel) row, so the channel's
// constants (the reciprocal of the divisor among them) are computed once per workgroup.
template <int MODE>
__global__ __launch_bounds__(BN_THREADS) void bn_rows_kernel(const float *__restrict__ A, const float *__restrict__ B,
                                                             float *__restrict__ out, const float *__restrict__ mean,
                                                             const float *__restrict__ p1, const float *__restrict__ p2,
                                                             const float *__restrict__ p3, int64_t channels, int64_t inner,
                                                             int chunks, int vec_ok)
{
    const int64_t rowi = blockIdx.x / chunks;
    const int chunk = blockIdx.x - (int)(rowi * chunks);
    const BnChannel ch = bn_channel<MODE>(mean, p1, p2, p3, rowi % channels);
    const float *a = A + rowi * inner;
    const float *b = MODE == BN_APPLY ? nullptr : B + rowi * inner;
    float *o = out + rowi * inner;
    const int64_t e0 = (int64_t)chunk * BN_CHUNK;
    if (vec_ok && e0 + BN_CHUNK <= inner)
    {
        const v4f *a4 = reinterpret_cast<const v4f *>(a + e0);
        const v4f *b4 = reinterpret_cast<const v4f *>(b + e0);
        v4f *o4 = reinterpret_cast<v4f *>(o + e0);
        v4f x[BN_UNROLL], y[BN_UNROLL];
#pragma unroll
        for (int u = 0; u < BN_UNROLL; u++)
        {
            x[u] = __builtin_nontemporal_load(&a4[threadIdx.x + u * BN_THREADS]);
            if (MODE != BN_APPLY)
                y[u] = __builtin_nontemporal_load(&b4[threadIdx.x + u * BN_THREADS]);
            else
                y[u] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int u = 0; u < BN_UNROLL; u++)
        {
            v4f r;
            r.x = bn_value<MODE>(x[u].x, y[u].x, ch);
            r.y = bn_value<MODE>(x[u].y, y[u].y, ch);
            r.z = bn_value<MODE>(x[u].z, y[u].z, ch);
            r.w = bn_value<MODE>(x[u].w, y[u].w, ch);
            __builtin_nontemporal_store(r, &o4[threadIdx.x + u * BN_THREADS]);
        }
        return;
    }
    const int64_t e1 = e0 + BN_CHUNK < inner ? e0 + BN_CHUNK : inner;
    for (int64_t i = e0 + threadIdx.x; i < e1; i += BN_THREADS)
        o[i] = bn_value<MODE>(a[i], MODE == BN_APPLY ? 0.0f : b[i], ch);
}

// Short rows (inner below one chunk; [B,F] tensors have inner = 1): one element per thread, its
// channel from the flat index.
template <int MODE>
__global__ __launch_bounds__(BN_THREADS) void bn_flat_kernel(const float *__restrict__ A, const float *__restrict__ B,
                                                             float *__restrict__ out, const float *__restrict__ mean,
                                                             const float *__restrict__ p1, const float *__restrict__ p2,
                                                             const float *__restrict__ p3, int64_t channels, int64_t inner,
                                                             int64_t total)
{
    const int64_t i = (int64_t)blockIdx.x * BN_THREADS + threadIdx.x;
    if (i >= total)
        return;
    const int64_t c = (i / inner) % channels;
    const BnChannel ch = bn_channel<MODE>(mean, p1, p2, p3, c);
    out[i] = bn_value<MODE>(A[i], MODE == BN_APPLY ? 0.0f : B[i], ch);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <int MODE>
int bn_launch(const float *A, const float *B, float *out, const float *mean, const float *p1, const float *p2,
              const float *p3, int64_t outer, int64_t channels, int64_t inner, void *stream)
{
    REPDL_REQUIRE(outer >= 0 && channels >= 0 && inner >= 0);
    if (outer == 0 || channels == 0 || inner == 0)
        return REPDL_OK;
    REPDL_REQUIRE(outer <= REPDL_I32_MAX && channels <= REPDL_I32_MAX && inner <= REPDL_I32_MAX);
    const int64_t rows = outer * channels;
    REPDL_REQUIRE(rows <= ((int64_t)1 << 62) / inner);
    REPDL_REQUIRE(A != nullptr && out != nullptr && mean != nullptr && p1 != nullptr);
    REPDL_REQUIRE(MODE == BN_APPLY ? (p2 != nullptr && p3 != nullptr) : B != nullptr);
    hipStream_t s = repdl_stream(stream);
    if (inner >= BN_CHUNK / 4)
    {
        const int64_t chunks = repdl_cdiv(inner, BN_CHUNK);
        REPDL_REQUIRE(rows * chunks <= REPDL_I32_MAX);
        const int vec_ok = inner % 4 == 0 && aligned16(A) && aligned16(out) && (MODE == BN_APPLY || aligned16(B));
        hipLaunchKernelGGL((bn_rows_kernel<MODE>), dim3((unsigned)(rows * chunks)), dim3(BN_THREADS), 0, s, A, B, out, mean, p1,
                           p2, p3, channels, inner, (int)chunks, vec_ok);
        return repdl_launch_status();
    }
    const int64_t total = rows * inner;
    const int64_t grid = repdl_cdiv(total, BN_THREADS);
    REPDL_REQUIRE(grid <= REPDL_I32_MAX);
    hipLaunchKernelGGL((bn_flat_kernel<MODE>), dim3((unsigned)grid), dim3(BN_THREADS), 0, s, A, B, out, mean, p1, p2, p3,
                       channels, inner, total);
    return repdl_launch_status();
}
} // namespace

REPDL_API int repdl_hip_bn_apply(const float *x, const float *mean, const float *std, const float *weight,
                                 const float *bias, float *y, int64_t outer, int64_t channels, int64_t inner,
                                 void *stream)
{
    return bn_launch<BN_APPLY>(x, nullptr, y, mean, std, weight, bias, outer, channels, inner, stream);
}

REPDL_API int repdl_hip_bn_gvar_term(const float *grad_y, const float *x, const float *mean, const float *coef,
                                     float *out, int64_t outer, int64_t channels, int64_t inner, void *stream)
{
    return bn_launch<BN_GVAR>(grad_y, x, out, mean, coef, nullptr, nullptr, outer, channels, inner, stream);
}

REPDL_API int repdl_hip_bn_gweight_term(const float *x, const float *mean, const float *std, const float *grad_y,
                                        float *out, int64_t outer, int64_t channels, int64_t inner, void *stream)
{
    return bn_launch<BN_GWEIGHT>(x, grad_y, out, mean, std, nullptr, nullptr, outer, channels, inner, stream);
}
