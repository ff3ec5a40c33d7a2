/*
 * repdl_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C (C11 + OpenMP) CPU restatement of the arithmetic of RepDL's CPU
 * backend, operator by operator.  It exists only so that tests, the smoke
 * check and the benchmark's cpu_baseline leg can compare the HIP kernels with
 * an independent implementation of the same fixed evaluation order.  Nothing
 * in the shipped package may link, load or call it.
 *
 * Every function cites the reference lines it restates (paths relative to the
 * RepDL source tree).  The contract in one place:
 *   - binary32, round-to-nearest-even, subnormals kept;
 *   - every multiply-accumulate is ONE fused fmaf (single rounding);
 *   - every output element owns one accumulator that starts at +0.0f and is
 *     updated in the reference's loop order; taps that fall outside the image
 *     are skipped, never multiplied by a padded zero;
 *   - sums are strict left-to-right chains, result multiplied once by
 *     (float)(average ? 1.0/count : 1.0);
 *   - exp/log are glibc's binary64 routine followed by one rounding to
 *     binary32; sqrt is binary64 sqrt followed by one rounding; div is the
 *     IEEE binary32 quotient.
 * Loop nests may be blocked or vectorised ACROSS output elements for speed
 * (the order of operations inside one output element is never touched), which
 * is why this file must be built with -ffp-contract=off and without
 * -ffast-math: the only fused operations are the explicit fmaf calls.
 *
 * Pinning status (what proves each function equals the reference):
 *   mm, conv2d, conv2d_grad_input, conv2d_grad_kernel, sum1d, sum2d_dim0,
 *   sum2d_dim1, sum4d_dim023, exp2d/log1d (as exp/log), softmax,
 *   cross_entropy: golden SHA-256 vectors written by the reference's own C++
 *   CPU backend compiled from its sources (tests/golden/), plus exact-rational
 *   brute force on tiny inputs and integer-valued cases that must equal
 *   torch's results exactly.
 *   div, sqrt: the reference composes these from PyTorch CPU operators
 *   (repdl/ops.py:98-103, 122-123); pinned against torch CPU on the host and
 *   against exact rational arithmetic.  glibc exp/log are third-party code
 *   not held by the reference and not correctly rounded: their float-rounded
 *   results are whatever the host's glibc returns -- "parity unpinned" by any
 *   reference-held vector, pinned here by calling the same libm.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

static inline uint32_t f2u(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float u2f(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

ORACLE_API int repdl_oracle_threads(void)
{
#if defined(_OPENMP)
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------
 * mm -- backend/cpu/matrix_multiplication.cpp:12-36
 *   M,K from A (swapped when transA), N from B (:15-17);
 *   C[i][j] = fmaf chain over k = 0..K-1 starting from +0 (:26-33).
 * A is [M,K] row-major (or [K,M] when transA), B is [K,N] (or [N,K] when
 * transB), C is [M,N] row-major.
 *
 * Blocked so that a panel of IB rows x JB columns of accumulators lives in
 * L1 while k runs over the whole K range: each C element still sees exactly
 * k = 0,1,...,K-1 in order with one fmaf per step.
 * ---------------------------------------------------------------------- */
#define MM_IB 8
#define MM_JB 512

ORACLE_API void repdl_oracle_mm(const float *A, const float *B, float *C, int64_t M, int64_t N,
                                int64_t K, int transA, int transB)
{
    const float *Bn = B; /* B as [K,N] */
    float *Bt = NULL;
    if (transB)
    {
        Bt = (float *)malloc((size_t)(K > 0 ? K : 1) * (size_t)(N > 0 ? N : 1) * sizeof(float));
#pragma omp parallel for schedule(static)
        for (int64_t k = 0; k < K; k++)
            for (int64_t j = 0; j < N; j++)
                Bt[k * N + j] = B[j * K + k];
        Bn = Bt;
    }
    int64_t nib = (M + MM_IB - 1) / MM_IB, njb = (N + MM_JB - 1) / MM_JB;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int64_t ib = 0; ib < nib; ib++)
        for (int64_t jb = 0; jb < njb; jb++)
        {
            float acc[MM_IB][MM_JB];
            int64_t i0 = ib * MM_IB, j0 = jb * MM_JB;
            int64_t ni = (M - i0 < MM_IB) ? M - i0 : MM_IB;
            int64_t nj = (N - j0 < MM_JB) ? N - j0 : MM_JB;
            for (int64_t ii = 0; ii < ni; ii++)
                for (int64_t jj = 0; jj < nj; jj++)
                    acc[ii][jj] = 0.0f;
            for (int64_t k = 0; k < K; k++)
            {
                const float *brow = Bn + k * N + j0;
                for (int64_t ii = 0; ii < ni; ii++)
                {
                    float a = !transA ? A[(i0 + ii) * K + k] : A[k * M + (i0 + ii)];
                    float *arow = acc[ii];
#pragma omp simd
                    for (int64_t jj = 0; jj < nj; jj++)
                        arow[jj] = fmaf(a, brow[jj], arow[jj]);
                }
            }
            for (int64_t ii = 0; ii < ni; ii++)
                memcpy(C + (i0 + ii) * N + j0, acc[ii], (size_t)nj * sizeof(float));
        }
    free(Bt);
}

/* ------------------------------------------------------------------------
 * conv2d -- backend/cpu/convolution.cpp:12-52  (NCHW, groups supported)
 *   OH,OW (:17-18); group of an output channel (:31); accumulation order
 *   (i, kh, kw) lexicographic with out-of-image taps skipped (:32-47);
 *   fmaf(input, kernel, sum) (:45).
 * ---------------------------------------------------------------------- */
ORACLE_API void repdl_oracle_conv2d(const float *I, const float *Kr, float *O, int64_t N,
                                    int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH,
                                    int64_t KW, int64_t sH, int64_t sW, int64_t pH, int64_t pW,
                                    int64_t groups)
{
    int64_t OH = (H + 2 * pH - KH) / sH + 1, OW = (W + 2 * pW - KW) / sW + 1;
    int64_t ICg = IC / groups, OCg = OC / groups;
#pragma omp parallel for collapse(3) schedule(static)
    for (int64_t n = 0; n < N; n++)
        for (int64_t oc = 0; oc < OC; oc++)
            for (int64_t oh = 0; oh < OH; oh++)
                for (int64_t ow = 0; ow < OW; ow++)
                {
                    float sum = 0.0f;
                    int64_t g = oc / OCg;
                    for (int64_t i = 0; i < ICg; i++)
                    {
                        int64_t ic = g * ICg + i;
                        for (int64_t kh = 0; kh < KH; kh++)
                        {
                            int64_t h = oh * sH - pH + kh;
                            if (h < 0 || h >= H)
                                continue;
                            for (int64_t kw = 0; kw < KW; kw++)
                            {
                                int64_t w = ow * sW - pW + kw;
                                if (w < 0 || w >= W)
                                    continue;
                                sum = fmaf(I[((n * IC + ic) * H + h) * W + w],
                                           Kr[((oc * ICg + i) * KH + kh) * KW + kw], sum);
                            }
                        }
                    }
                    O[((n * OC + oc) * OH + oh) * OW + ow] = sum;
                }
}

/* ------------------------------------------------------------------------
 * conv2d_grad_input -- backend/cpu/convolution.cpp:54-90  (groups == 1)
 *   order (oc, kh, kw) (:72-86); a tap contributes iff (h-kh+pH) is a
 *   multiple of sH and the quotient lies in [0,OH) -- C truncating '/' and
 *   '%' on possibly negative ints exactly as written there (:75-77, :80-82);
 *   fmaf(grad_output, kernel, sum) (:83).
 * ---------------------------------------------------------------------- */
ORACLE_API void repdl_oracle_conv2d_grad_input(const float *GO, const float *Kr, float *GI,
                                               int64_t N, int64_t OC, int64_t OH, int64_t OW,
                                               int64_t IC, int64_t KH, int64_t KW, int64_t H,
                                               int64_t W, int64_t sH, int64_t sW, int64_t pH,
                                               int64_t pW)
{
#pragma omp parallel for collapse(3) schedule(static)
    for (int64_t n = 0; n < N; n++)
        for (int64_t ic = 0; ic < IC; ic++)
            for (int64_t h = 0; h < H; h++)
                for (int64_t w = 0; w < W; w++)
                {
                    float sum = 0.0f;
                    for (int64_t oc = 0; oc < OC; oc++)
                        for (int64_t kh = 0; kh < KH; kh++)
                        {
                            int64_t th = h - kh + pH;
                            int64_t oh = th / sH;
                            if (oh < 0 || oh >= OH || (th % sH))
                                continue;
                            for (int64_t kw = 0; kw < KW; kw++)
                            {
                                int64_t tw = w - kw + pW;
                                int64_t ow = tw / sW;
                                if (ow < 0 || ow >= OW || (tw % sW))
                                    continue;
                                sum = fmaf(GO[((n * OC + oc) * OH + oh) * OW + ow],
                                           Kr[((oc * IC + ic) * KH + kh) * KW + kw], sum);
                            }
                        }
                    GI[((n * IC + ic) * H + h) * W + w] = sum;
                }
}

/* ------------------------------------------------------------------------
 * conv2d_grad_kernel -- backend/cpu/convolution.cpp:92-128
 *   order (n, oh, ow) with out-of-image taps skipped (:109-124);
 *   fmaf(grad_output, input, sum) (:121).
 * ---------------------------------------------------------------------- */
ORACLE_API void repdl_oracle_conv2d_grad_kernel(const float *GO, const float *I, float *GK,
                                                int64_t N, int64_t IC, int64_t H, int64_t W,
                                                int64_t OC, int64_t OH, int64_t OW, int64_t KH,
                                                int64_t KW, int64_t sH, int64_t sW, int64_t pH,
                                                int64_t pW)
{
#pragma omp parallel for collapse(4) schedule(dynamic, 4)
    for (int64_t oc = 0; oc < OC; oc++)
        for (int64_t ic = 0; ic < IC; ic++)
            for (int64_t kh = 0; kh < KH; kh++)
                for (int64_t kw = 0; kw < KW; kw++)
                {
                    float sum = 0.0f;
                    for (int64_t n = 0; n < N; n++)
                        for (int64_t oh = 0; oh < OH; oh++)
                        {
                            int64_t h = oh * sH - pH + kh;
                            if (h < 0 || h >= H)
                                continue;
                            for (int64_t ow = 0; ow < OW; ow++)
                            {
                                int64_t w = ow * sW - pW + kw;
                                if (w < 0 || w >= W)
                                    continue;
                                sum = fmaf(GO[((n * OC + oc) * OH + oh) * OW + ow],
                                           I[((n * IC + ic) * H + h) * W + w], sum);
                            }
                        }
                    GK[((oc * IC + ic) * KH + kh) * KW + kw] = sum;
                }
}

/* ------------------------------------------------------------------------
 * sums -- backend/cpu/summation.cpp
 *   factor is computed in double and rounded to float once (:15, :27, :46,
 *   :64); the result is factor * sum even when not averaging (:19, :36, :55,
 *   :75).  The volatile keeps the compiler from folding 1.0f * x.
 * ---------------------------------------------------------------------- */
static inline float sum_factor(int average, int64_t count)
{
    float factor = average ? 1.0 / (double)(int)count : 1.0;
    return factor;
}

/* sum1d -- summation.cpp:12-20: single serial chain (:17-18). */
ORACLE_API float repdl_oracle_sum1d(const float *I, int64_t N, int average)
{
    float sum = 0.0f, factor = sum_factor(average, N);
    for (int64_t i = 0; i < N; i++)
        sum += I[i];
    return factor * sum;
}

/* sum2d_dim0 -- summation.cpp:22-39: one chain per column over rows (:33-36). */
ORACLE_API void repdl_oracle_sum2d_dim0(const float *I, float *O, int64_t M, int64_t N, int average)
{
    float factor = sum_factor(average, M);
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < N; j++)
    {
        float sum = 0.0f;
        for (int64_t i = 0; i < M; i++)
            sum += I[i * N + j];
        O[j] = factor * sum;
    }
}

/* sum2d_dim1 -- summation.cpp:41-58: one chain per row over columns (:52-55). */
ORACLE_API void repdl_oracle_sum2d_dim1(const float *I, float *O, int64_t M, int64_t N, int average)
{
    float factor = sum_factor(average, N);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; i++)
    {
        float sum = 0.0f;
        for (int64_t j = 0; j < N; j++)
            sum += I[i * N + j];
        O[i] = factor * sum;
    }
}

/* sum4d_dim023 -- summation.cpp:59-78: per channel, order (n, h, w) (:71-74). */
ORACLE_API void repdl_oracle_sum4d_dim023(const float *I, float *O, int64_t N, int64_t C,
                                          int64_t H, int64_t W, int average)
{
    float factor = average ? 1.0 / (double)((int)N * (int)H * (int)W) : 1.0;
#pragma omp parallel for schedule(static)
    for (int64_t c = 0; c < C; c++)
    {
        float sum = 0.0f;
        for (int64_t n = 0; n < N; n++)
            for (int64_t h = 0; h < H; h++)
                for (int64_t w = 0; w < W; w++)
                    sum += I[((n * C + c) * H + h) * W + w];
        O[c] = factor * sum;
    }
}

/* ------------------------------------------------------------------------
 * exp / log -- backend/cpu/math.cpp:14-17 and :32-35:
 *   (float)std::exp((double)x), (float)std::log((double)x), any shape here
 *   (the reference only has the 2-D and 1-D drivers :19-30, :37-47).
 * ---------------------------------------------------------------------- */
ORACLE_API void repdl_oracle_exp(const float *I, float *O, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++)
        O[i] = (float)exp((double)I[i]);
}

ORACLE_API void repdl_oracle_log(const float *I, float *O, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++)
        O[i] = (float)log((double)I[i]);
}

/* ------------------------------------------------------------------------
 * sqrt -- repdl/ops.py:122-123: input.to(float64).sqrt().to(float32).
 *   The square root of a negative number (including -inf) is the POSITIVE
 *   quiet NaN 0x7FC00000 in PyTorch's CPU kernel (not the x86 "indefinite"
 *   0xFFC00000 that a bare sqrtsd gives); NaN inputs keep sign and payload and
 *   are quieted; sqrt(-0) = -0.
 * ---------------------------------------------------------------------- */
static inline float ieee_sqrt(float x)
{
    uint32_t u = f2u(x);
    if ((u & 0x7fffffffu) > 0x7f800000u)
        return u2f(u | 0x00400000u);
    if ((u >> 31) && (u & 0x7fffffffu))
        return u2f(0x7fc00000u);
    return (float)sqrt((double)x);
}

ORACLE_API void repdl_oracle_sqrt(const float *I, float *O, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++)
        O[i] = ieee_sqrt(I[i]);
}

/* ------------------------------------------------------------------------
 * div -- repdl/ops.py:98-103: input.div(other); a Python-float divisor is
 *   first made a float32 0-dim tensor, so it is the IEEE binary32 quotient in
 *   both cases.  x86 divss semantics for NaNs: a NaN dividend wins (quieted),
 *   else a NaN divisor (quieted); 0/0 and inf/inf give 0xFFC00000.
 * ---------------------------------------------------------------------- */
static inline float ieee_div(float a, float b)
{
    uint32_t ua = f2u(a), ub = f2u(b);
    if ((ua & 0x7fffffffu) > 0x7f800000u)
        return u2f(ua | 0x00400000u);
    if ((ub & 0x7fffffffu) > 0x7f800000u)
        return u2f(ub | 0x00400000u);
    volatile float q = a / b;
    if (q != q)
        return u2f(0xffc00000u);
    return q;
}

ORACLE_API void repdl_oracle_div(const float *A, const float *B, float *O, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++)
        O[i] = ieee_div(A[i], B[i]);
}

ORACLE_API void repdl_oracle_div_scalar(const float *A, float b, float *O, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++)
        O[i] = ieee_div(A[i], b);
}

/* row maximum as torch.max(dim=1) computes it: a NaN in the row wins. */
static inline float row_max(const float *x, int64_t n)
{
    float m = x[0];
    for (int64_t j = 1; j < n; j++)
    {
        float v = x[j];
        if (v != v)
        {
            if (m == m)
                m = v;
        }
        else if (v > m)
            m = v;
    }
    return m;
}

/* ------------------------------------------------------------------------
 * softmax -- backend/cpu/softmax.cpp:15-21:
 *   x - rowmax (:17), exp2d (:18), divide by the serial row sum (:19).
 * ---------------------------------------------------------------------- */
ORACLE_API void repdl_oracle_softmax(const float *I, float *O, int64_t M, int64_t N)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; i++)
    {
        const float *x = I + i * N;
        float *o = O + i * N;
        float m = row_max(x, N);
        for (int64_t j = 0; j < N; j++)
            o[j] = (float)exp((double)(x[j] - m));
        float sum = 0.0f;
        for (int64_t j = 0; j < N; j++)
            sum += o[j];
        volatile float one = 1.0f;
        sum = one * sum;
        for (int64_t j = 0; j < N; j++)
            o[j] = o[j] / sum;
    }
}

/* ------------------------------------------------------------------------
 * cross_entropy -- backend/cpu/cross_entropy.cpp:15-24:
 *   shifted = x - rowmax (:17); exp2d (:18); serial row sum (:19); log1d
 *   (:20); minus shifted[target] (:21); sum1d with average (:22).
 * scratch must hold M floats.
 * ---------------------------------------------------------------------- */
ORACLE_API float repdl_oracle_cross_entropy(const float *I, const int64_t *target, int64_t M,
                                            int64_t N, float *scratch)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; i++)
    {
        const float *x = I + i * N;
        float m = row_max(x, N);
        float sum = 0.0f;
        for (int64_t j = 0; j < N; j++)
            sum += (float)exp((double)(x[j] - m));
        volatile float one = 1.0f;
        sum = one * sum;
        float l = (float)log((double)sum);
        l -= x[target[i]] - m;
        scratch[i] = l;
    }
    return repdl_oracle_sum1d(scratch, M, 1);
}

/* ------------------------------------------------------------------------
 * Optimizer steps.  repdl/optim.py:56-83 writes Adam as PyTorch tensor
 *   operations, each rounding once; this is that sequence per element, with
 *   the scalars already rounded to binary32 as PyTorch rounds a Python number
 *   that meets a float32 tensor:
 *     :64-66  grad.add(param, alpha=wd)       -> fmaf(wd, p, g)   [only if wd != 0]
 *     :68     exp_avg.mul_(b1).add_(g, alpha) -> fmaf(c1, g, m * b1)
 *             (Tensor.add with alpha is one fused multiply-add in PyTorch's CPU
 *             kernels, vector body and scalar tail alike; checked against torch
 *             in tests/test_oracle_pin.py)
 *     :69     exp_avg_sq.mul_(b2).add_(mul(g, g).mul(c2)): four roundings
 *     :71-74  torch.maximum: NaN if either operand is
 *     :75-81  ops.div(ops.sqrt(s), sqrt(bc2)).add_(eps)
 *     :82-83  param.add_(div(exp_avg, denom).mul(-step_size))
 *   vmax == NULL: amsgrad off.  Pinning: against the same sequence of torch
 *   CPU operators over several steps (tests/test_oracle_pin.py).
 * ---------------------------------------------------------------------- */
static inline float max_nan(float a, float b)
{
    if (a != a)
        return a;
    if (b != b)
        return b;
    return a > b ? a : b;
}

ORACLE_API void repdl_oracle_adam_step(float *P, const float *G, float *M, float *V, float *VMAX, int64_t n,
                                       float b1, float c1, float b2, float c2, float eps, float wd,
                                       float sqrt_bc2, float step_scale)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++)
    {
        float g = G[i];
        if (wd != 0.0f)
            g = fmaf(wd, P[i], g);
        const float mb = M[i] * b1;
        const float m = fmaf(c1, g, mb);
        const float vb = V[i] * b2;
        const float gg = g * g;
        const float ggc = gg * c2;
        const float v = vb + ggc;
        float s = v;
        if (VMAX)
        {
            s = max_nan(VMAX[i], v);
            VMAX[i] = s;
        }
        const float root = ieee_sqrt(s);
        const float scaled = ieee_div(root, sqrt_bc2);
        const float denom = scaled + eps;
        const float q = ieee_div(m, denom);
        const float upd = q * step_scale;
        P[i] = P[i] + upd;
        M[i] = m;
        V[i] = v;
    }
}

/* p <- p - RN(g * lr): two roundings (the product, then the difference). */
ORACLE_API void repdl_oracle_sgd_step(float *P, const float *G, int64_t n, float lr)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++)
    {
        const float step = G[i] * lr;
        P[i] = P[i] - step;
    }
}
