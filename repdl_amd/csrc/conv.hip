// Reproducible fp32 2-D convolution (forward, grad-input, grad-kernel), NCHW.
//
// Contract (RepDL backend/cpu/convolution.cpp:12-128): one accumulator per
// output element, starting at +0.0f, one fused multiply-add per contributing
// tap in the reference's lexicographic loop order; taps that fall outside the
// image (or, for grad-input, between strides) are SKIPPED, not multiplied by a
// padded zero.
//
// Forward and grad-input run as implicit GEMMs on the tiling of the mm kernel
// (k-major LDS tiles, 8x8 register micro-tiles of v_fma_f32, K never split):
//     forward     C[oc, pixel]  = sum_k W[oc, k] * im2col(X)[k, pixel],     k = (ic, kh, kw)
//     grad-input  C[ic, pixel]  = sum_k W^T[ic, k] * col(GO)[k, pixel],     k = (oc, kh, kw)
// with k running in exactly the reference's order.  The gathered operand holds a
// zero where the reference skips a tap.  For finite data fma(0, w, acc) = acc
// unless acc is -0.0f, and a chain can hold -0.0f only after a product so small
// that it rounds to zero; with non-finite data the padded product is a NaN that
// sticks.  So the epilogue recomputes with the literal skip-the-tap chain (the
// *_exact functions below) every NaN result, and the zero results only when the
// operands can produce such a product (see "the guard of the zero results" below).
//
// grad-kernel has only OC*IC*KH*KW outputs, each a chain as long as the batch
// (N*OH*OW): it is limited by chain length and parallelism, not by FMA rate.
#include <type_traits>

#include "common.h"

namespace
{
struct ConvDims
{
    int N, IC, H, W, OC, KH, KW, OH, OW, sH, sW, pH, pW, groups;
    const float *bias; // forward only: [OC], added once to each output after its chain; null = none
};

// repdl/nn/conv.py:27-28: the bias is one rounded addition to the finished chain
__device__ __forceinline__ float with_bias(float v, const ConvDims &d, int oc) { return d.bias != nullptr ? v + d.bias[oc] : v; }

// ---------------------------------------------------------------------------
// The literal chains (exact by construction).
// ---------------------------------------------------------------------------

// backend/cpu/convolution.cpp:30-48
__device__ __forceinline__ float conv2d_exact(const float *__restrict__ I, const float *__restrict__ Kr,
                                              const ConvDims &d, int n, int oc, int oh, int ow)
{
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
    return sum;
}

// backend/cpu/convolution.cpp:71-86.  '/' truncates toward zero and '%' takes the
// sign of the dividend, as in the reference (:75-77).
__device__ __forceinline__ float conv2d_grad_input_exact(const float *__restrict__ GO,
                                                         const float *__restrict__ Kr, const ConvDims &d,
                                                         int n, int ic, int h, int w)
{
    float sum = 0.0f;
    for (int oc = 0; oc < d.OC; oc++)
    {
        const float *gp = GO + ((int64_t)n * d.OC + oc) * d.OH * d.OW;
        const float *kp = Kr + ((int64_t)oc * d.IC + ic) * d.KH * d.KW;
        for (int kh = 0; kh < d.KH; kh++)
        {
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
    return sum;
}

// backend/cpu/convolution.cpp:108-124
__device__ __forceinline__ float conv2d_grad_kernel_exact(const float *__restrict__ GO,
                                                          const float *__restrict__ I, const ConvDims &d,
                                                          int oc, int ic, int kh, int kw)
{
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
    return sum;
}

// ---------------------------------------------------------------------------
// The guard of the zero results.  A chain that multiplies padded zeros where the
// reference skips a tap can differ from the reference's only while its accumulator
// is -0.0f (x + (+-0) = x for every other x).  The accumulator starts at +0.0f; an
// exact cancellation gives +0.0f, and (+0) + (+-0) = +0, so the first -0.0f of a
// chain can only come from a nonzero sum g*x + acc that rounds to zero.  acc is a
// multiple of 2^-149, so that needs a product with bits below 2^-149, and a product
// of two binary32 values has at most 48 significant bits: |g*x| < 2^-101.  If
//     (smallest nonzero |value| of one operand) * (that of the other) >= 2^-101
// no such product exists, no chain ever holds -0.0f, and the padded chain equals the
// literal one on all finite data, zero results included.  guard[0..1] hold the two
// minima (as bit patterns; GUARD_NONE when an operand has no nonzero value), found
// in one extra pass over the operands (or in the pass that pads them); the kernels
// recompute a zero result with the literal chain only when guard_tiny() says a tiny
// product is possible, and a NaN result always (0 * inf of a padded tap).
// Without it, data with whole dead channels or zero borders (every ReLU network)
// sent each of its zero results through a serial literal chain.
// ---------------------------------------------------------------------------
constexpr unsigned GUARD_NONE = 0x7f800000u;
// Workspace of the guard: words 0 and 1 are the two minima, then (from word 64) GUARD_PARTS
// per-workgroup minima for each operand.  No atomics: thousands of them on one address
// would cost more than the pass itself.
constexpr int GUARD_PARTS = 2048;
constexpr size_t GUARD_BYTES = (64 + 2 * GUARD_PARTS) * sizeof(unsigned);
static_assert(GUARD_BYTES % 256 == 0, "what follows the guard in a workspace stays aligned");

inline unsigned *guard_parts(unsigned *guard, int operand) { return guard + 64 + operand * GUARD_PARTS; }

__device__ __forceinline__ unsigned guard_bits(float v)
{
    const unsigned b = __float_as_uint(v) & 0x7fffffffu;
    return b == 0u ? GUARD_NONE : b; // NaN patterns are above GUARD_NONE and never the minimum
}

__device__ __forceinline__ unsigned guard_min(unsigned a, unsigned b) { return b < a ? b : a; }

// Minimum over the 256 threads of a workgroup (all of them call), valid in thread 0.
__device__ __forceinline__ unsigned guard_block_min(unsigned m)
{
    __shared__ unsigned wave_min[4];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        m = guard_min(m, (unsigned)__shfl_xor((int)m, o));
    __syncthreads(); // a previous use of wave_min has been read
    if ((threadIdx.x & 63) == 0)
        wave_min[threadIdx.x >> 6] = m;
    __syncthreads();
    return guard_min(guard_min(wave_min[0], wave_min[1]), guard_min(wave_min[2], wave_min[3]));
}

// A null guard: the geometry skips no tap (no padding, whole rows), nothing to decide.
__device__ __forceinline__ bool guard_tiny(const unsigned *__restrict__ guard)
{
    return guard != nullptr && (double)__uint_as_float(guard[0]) * (double)__uint_as_float(guard[1]) < 0x1p-101;
}

__device__ __forceinline__ bool guard_suspect(float v, bool tiny)
{
    return (v != v) || (tiny && (__float_as_uint(v) << 1) == 0u);
}

// Workgroup blk of nblk: the minimum over its grid-stride share of p[0..n) into parts[blk].
__device__ __forceinline__ void guard_scan_block(const float *__restrict__ p, int64_t n, int blk, int nblk,
                                                 unsigned *__restrict__ parts)
{
    typedef float v4f __attribute__((ext_vector_type(4)));
    const int64_t stride = (int64_t)nblk * 256;
    const int64_t first = (int64_t)blk * 256 + threadIdx.x;
    unsigned m = GUARD_NONE;
    int64_t done = 0;
    if ((reinterpret_cast<uintptr_t>(p) & 15) == 0)
    {
        const v4f *__restrict__ p4 = reinterpret_cast<const v4f *>(p);
        const int64_t n4 = n / 4;
        for (int64_t i = first; i < n4; i += stride)
        {
            const v4f v = p4[i];
            m = guard_min(guard_min(m, guard_bits(v.x)),
                          guard_min(guard_bits(v.y), guard_min(guard_bits(v.z), guard_bits(v.w))));
        }
        done = n4 * 4;
    }
    for (int64_t i = done + first; i < n; i += stride)
        m = guard_min(m, guard_bits(p[i]));
    m = guard_block_min(m);
    if (threadIdx.x == 0)
        parts[blk] = m;
}

// Blocks [0, nblk_a) take the minimum over a[0..na) into the parts of operand 0, the
// others over b[0..nb) into those of operand 1; either range of blocks may be empty.
__global__ __launch_bounds__(256) void conv_guard_kernel(const float *__restrict__ a, int64_t na,
                                                         const float *__restrict__ b, int64_t nb, int nblk_a,
                                                         unsigned *__restrict__ parts_a,
                                                         unsigned *__restrict__ parts_b)
{
    if ((int)blockIdx.x < nblk_a)
        guard_scan_block(a, na, (int)blockIdx.x, nblk_a, parts_a);
    else
        guard_scan_block(b, nb, (int)blockIdx.x - nblk_a, (int)gridDim.x - nblk_a, parts_b);
}

// guard[op] = minimum of the first count[op] parts of operand op (GUARD_NONE for none)
__global__ __launch_bounds__(256) void conv_guard_final_kernel(unsigned *__restrict__ guard, int count_a, int count_b)
{
#pragma unroll
    for (int op = 0; op < 2; op++)
    {
        const unsigned *__restrict__ parts = guard + 64 + op * GUARD_PARTS;
        const int count = op == 0 ? count_a : count_b;
        unsigned m = GUARD_NONE;
        for (int i = threadIdx.x; i < count; i += 256)
            m = guard_min(m, parts[i]);
        m = guard_block_min(m);
        if (threadIdx.x == 0)
            guard[op] = m;
    }
}

inline int guard_blocks(int64_t n)
{
    const int64_t b = (n + 4095) / 4096; // 16 values per thread
    return (int)(b < 1 ? 1 : (b > 1024 ? 1024 : b));
}

// Scans the operands given (a null one is left to the padding pass of its caller, which
// then sets its own count of parts); returns the counts of parts written.
inline void launch_guard_scan(const float *a, int64_t na, const float *b, int64_t nb, unsigned *guard, hipStream_t s,
                              int &count_a, int &count_b)
{
    count_a = a ? guard_blocks(na) : 0;
    count_b = b ? guard_blocks(nb) : 0;
    if (count_a + count_b > 0)
        REPDL_LAUNCH(conv_guard_kernel, dim3((unsigned)(count_a + count_b)), dim3(256), 0, s, a, a ? na : 0, b,
                           b ? nb : 0, count_a, guard_parts(guard, 0), guard_parts(guard, 1));
}

inline void launch_guard_final(unsigned *guard, int count_a, int count_b, hipStream_t s)
{
    REPDL_LAUNCH(conv_guard_final_kernel, dim3(1), dim3(256), 0, s, guard, count_a, count_b);
}

// ---------------------------------------------------------------------------
// Implicit GEMM for forward (MODE_FWD) and grad-input (MODE_DGRAD).
// Tile BM x 128 outputs (BM = 64 or 128 rows = output / input channels, 128
// columns = pixels of one image), BK = 16, 2*BM threads, 8x8 micro-tile per lane.
// ---------------------------------------------------------------------------
constexpr int BN = 128, BK = 16, LDB = BN + 4;
enum
{
    MODE_FWD = 0,
    MODE_DGRAD = 1
};

// position of a k index in the (channel, kh, kw) mixed radix, advanced by BK per
// k-tile without divisions
struct KPos
{
    int c, kh, kw;
};

struct KStep
{
    int dc, dkh, dkw; // BK = dc*KH*KW + dkh*KW + dkw
};

__device__ __forceinline__ void kpos_advance(KPos &p, const KStep &s, int KH, int KW)
{
    p.kw += s.dkw;
    if (p.kw >= KW)
    {
        p.kw -= KW;
        p.kh++;
    }
    p.kh += s.dkh;
    if (p.kh >= KH)
    {
        p.kh -= KH;
        p.c++;
    }
    p.c += s.dc;
}

typedef float f16v __attribute__((ext_vector_type(16)));

template <int BM, int MODE, bool MFMA>
__global__ __launch_bounds__(2 * BM) void conv_gemm_kernel(const float *__restrict__ Xg, // gathered operand: input (FWD) / grad_output (DGRAD)
                                                           const float *__restrict__ Wt, // kernel
                                                           float *__restrict__ Out, ConvDims d, int wvec,
                                                           int ovec, const unsigned *__restrict__ guard)
{
    constexpr int NT = 2 * BM;
    constexpr int LDA = BM + 4;
    constexpr int NA = BM * BK / 4 / NT;  // float4 slots of A per thread (2)
    constexpr int NB = BN * BK / 4 / NT;  // float4 slots of B per thread (4 or 2)
    constexpr int KSTRIDE_B = NT / 32;    // k rows between two B slots of a thread
    __shared__ __attribute__((aligned(16))) float As[2][BK * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int KHW = d.KH * d.KW;
    const int ICg = d.IC / d.groups, OCg = d.OC / d.groups;
    // GEMM extents
    const int M = MODE == MODE_FWD ? OCg : d.IC;
    const int K = (MODE == MODE_FWD ? ICg : d.OC) * KHW;
    const int P = MODE == MODE_FWD ? d.OH * d.OW : d.H * d.W; // pixels (columns) per image
    const int PW = MODE == MODE_FWD ? d.OW : d.W;
    const int n = MODE == MODE_FWD ? blockIdx.z / d.groups : blockIdx.z;
    const int g = MODE == MODE_FWD ? blockIdx.z % d.groups : 0;
    const int m0 = blockIdx.y * BM, p0 = blockIdx.x * BN;

    // forward with a bias: the values of this tile's rows, read from LDS in the epilogue
    __shared__ float bias_s[BM];
    if (MODE == MODE_FWD && d.bias != nullptr)
    {
        if (tid < BM)
            bias_s[tid] = m0 + tid < M ? d.bias[g * OCg + m0 + tid] : 0.0f;
        __syncthreads();
    }

    KStep kstep;
    kstep.dc = BK / KHW;
    kstep.dkh = (BK % KHW) / d.KW;
    kstep.dkw = (BK % KHW) % d.KW;

    // ---- B (gathered) operand: this thread's four pixels ----
    const int p4 = (tid & 31) << 2;
    int pb_h[4], pb_w[4]; // FWD: oh*sH-pH, ow*sW-pW;  DGRAD: h+pH, w+pW
    bool pvalid[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
    {
        const int pix = p0 + p4 + j;
        pvalid[j] = pix < P;
        const int ph = pix / PW, pw = pix - ph * PW;
        if (MODE == MODE_FWD)
        {
            pb_h[j] = ph * d.sH - d.pH;
            pb_w[j] = pw * d.sW - d.pW;
        }
        else
        {
            pb_h[j] = ph + d.pH;
            pb_w[j] = pw + d.pW;
        }
    }
    KPos bpos[NB];
    int bk[NB];
#pragma unroll
    for (int i = 0; i < NB; i++)
    {
        const int k = (tid >> 5) + KSTRIDE_B * i;
        bk[i] = k;
        bpos[i].c = k / KHW;
        const int rem = k - bpos[i].c * KHW;
        bpos[i].kh = rem / d.KW;
        bpos[i].kw = rem - bpos[i].kh * d.KW;
    }
    // ---- A (kernel) operand ----
    // FWD: element (m, k) = Wg[m*K + k] (k contiguous): slot = (row idx>>2, 4 k's).
    // DGRAD: element (m=ic, k=(oc,kh,kw)) = W[(oc*IC + ic)*KHW + kh*KW + kw]: slot =
    // (k row, 4 consecutive ic), gathered with stride KHW.
    const float *Wg = MODE == MODE_FWD ? Wt + (int64_t)g * OCg * K : Wt;
    constexpr int A_R4 = BM / 4;             // DGRAD: float4 groups per k row
    constexpr int KSTRIDE_A = NT / A_R4;     // DGRAD: k rows between two A slots (8)
    KPos apos[NA];
    int ak[NA];
    if (MODE == MODE_DGRAD)
    {
#pragma unroll
        for (int i = 0; i < NA; i++)
        {
            const int k = tid / A_R4 + KSTRIDE_A * i;
            ak[i] = k;
            apos[i].c = k / KHW;
            const int rem = k - apos[i].c * KHW;
            apos[i].kh = rem / d.KW;
            apos[i].kw = rem - apos[i].kh * d.KW;
        }
    }

    float4 fa[NA], fb[NB];

    // Positions k >= K hold -0.0f here and +0.0f in the gathered operand: the product is -0
    // and x + (-0) = x for every x, so the matrix kernel can run whole k-tiles.
    auto load_a = [&](int k0) {
#pragma unroll
        for (int i = 0; i < NA; i++)
        {
            float4 v = make_float4(-0.0f, -0.0f, -0.0f, -0.0f);
            if (MODE == MODE_FWD)
            {
                const int idx = tid + NT * i;
                const int r = m0 + (idx >> 2), k = k0 + ((idx & 3) << 2);
                if (r < M)
                {
                    const float *p = Wg + (int64_t)r * K + k;
                    if (wvec && k + 3 < K)
                        v = *reinterpret_cast<const float4 *>(p);
                    else
                    {
                        if (k + 0 < K) v.x = p[0];
                        if (k + 1 < K) v.y = p[1];
                        if (k + 2 < K) v.z = p[2];
                        if (k + 3 < K) v.w = p[3];
                    }
                }
            }
            else
            {
                const int r = m0 + ((tid % A_R4) << 2);
                if (ak[i] < K)
                {
                    const float *p = Wg + ((int64_t)apos[i].c * d.IC + r) * KHW + apos[i].kh * d.KW + apos[i].kw;
                    if (r + 0 < M) v.x = p[0];
                    if (r + 1 < M) v.y = p[KHW];
                    if (r + 2 < M) v.z = p[2 * KHW];
                    if (r + 3 < M) v.w = p[3 * KHW];
                }
                ak[i] += BK;
                kpos_advance(apos[i], kstep, d.KH, d.KW);
            }
            fa[i] = v;
        }
    };
    auto store_a = [&](float *S) {
#pragma unroll
        for (int i = 0; i < NA; i++)
        {
            if (MODE == MODE_FWD)
            {
                const int idx = tid + NT * i;
                const int r = idx >> 2, k = (idx & 3) << 2;
                S[(k + 0) * LDA + r] = fa[i].x;
                S[(k + 1) * LDA + r] = fa[i].y;
                S[(k + 2) * LDA + r] = fa[i].z;
                S[(k + 3) * LDA + r] = fa[i].w;
            }
            else
            {
                const int k = tid / A_R4 + KSTRIDE_A * i, r = (tid % A_R4) << 2;
                *reinterpret_cast<float4 *>(&S[k * LDA + r]) = fa[i];
            }
        }
    };
    auto load_b = [&]() {
#pragma unroll
        for (int i = 0; i < NB; i++)
        {
            float v[4] = {0.f, 0.f, 0.f, 0.f};
            if (bk[i] < K)
            {
                if (MODE == MODE_FWD)
                {
                    const float *base = Xg + ((int64_t)n * d.IC + g * ICg + bpos[i].c) * d.H * d.W;
#pragma unroll
                    for (int j = 0; j < 4; j++)
                    {
                        const int h = pb_h[j] + bpos[i].kh, w = pb_w[j] + bpos[i].kw;
                        if (pvalid[j] && (unsigned)h < (unsigned)d.H && (unsigned)w < (unsigned)d.W)
                            v[j] = base[h * d.W + w];
                    }
                }
                else
                {
                    const float *base = Xg + ((int64_t)n * d.OC + bpos[i].c) * d.OH * d.OW;
#pragma unroll
                    for (int j = 0; j < 4; j++)
                    {
                        const int th = pb_h[j] - bpos[i].kh, tw = pb_w[j] - bpos[i].kw;
                        int oh = th, ow = tw;
                        bool ok = pvalid[j] && th >= 0 && tw >= 0;
                        if (d.sH != 1)
                        {
                            oh = th / d.sH;
                            ok = ok && (th - oh * d.sH) == 0;
                        }
                        if (d.sW != 1)
                        {
                            ow = tw / d.sW;
                            ok = ok && (tw - ow * d.sW) == 0;
                        }
                        if (ok && oh < d.OH && ow < d.OW)
                            v[j] = base[oh * d.OW + ow];
                    }
                }
            }
            bk[i] += BK;
            kpos_advance(bpos[i], kstep, d.KH, d.KW);
            fb[i] = make_float4(v[0], v[1], v[2], v[3]);
        }
    };
    auto store_b = [&](float *S) {
#pragma unroll
        for (int i = 0; i < NB; i++)
        {
            const int k = (tid >> 5) + KSTRIDE_B * i;
            *reinterpret_cast<float4 *>(&S[k * LDB + p4]) = fb[i];
        }
    };

    float *Oimg = Out + (int64_t)n * (MODE == MODE_FWD ? d.OC : d.IC) * P;
    const int nkt = (K + BK - 1) / BK;
    if constexpr (MFMA)
    {
        // Matrix-instruction form: each wave owns 64 rows x 64 pixels as 2 x 2 blocks of
        // v_mfma_f32_32x32x2_f32 (lane l supplies row / pixel l%32 at k = l/32, the k = 0
        // product is added first).  BM = 64: two waves side by side; BM = 128: 2 x 2 waves.
        const int lane = tid & 63, l32 = lane & 31, half = lane >> 5;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wm = BM == 64 ? 0 : (wave & 1), wn = BM == 64 ? wave : (wave >> 1);
        f16v acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    acc[i][j][r] = 0.0f;
        const int a_off = half * LDA + wm * 64 + l32, b_off = half * LDB + wn * 64 + l32;
        if (nkt > 0)
        {
            load_a(0);
            load_b();
            store_a(As[0]);
            store_b(Bs[0]);
        }
        __syncthreads();
        for (int kt = 0; kt < nkt; kt++)
        {
            const int cur = kt & 1;
            const bool more = kt + 1 < nkt;
            if (more)
            {
                load_a((kt + 1) * BK);
                load_b();
            }
            const float *as = As[cur] + a_off, *bs = Bs[cur] + b_off;
            float a[BK / 2][2], b[BK / 2][2];
#pragma unroll
            for (int kp = 0; kp < BK / 2; kp++)
            {
                a[kp][0] = as[2 * kp * LDA];
                a[kp][1] = as[2 * kp * LDA + 32];
                b[kp][0] = bs[2 * kp * LDB];
                b[kp][1] = bs[2 * kp * LDB + 32];
            }
#pragma unroll
            for (int kp = 0; kp < BK / 2; kp++)
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kp][i], b[kp][j], acc[i][j], 0, 0, 0);
            if (more)
            {
                store_a(As[cur ^ 1]);
                store_b(Bs[cur ^ 1]);
            }
            __syncthreads();
        }
        // register r of a block: row 8*(r/4) + 4*(lane/32) + r%4, pixel lane%32
        const bool tiny = guard_tiny(guard);
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
            {
                const int m = m0 + wm * 64 + 32 * i + 8 * (r >> 2) + 4 * half + (r & 3);
                if (m >= M)
                    continue;
                const int ch = MODE == MODE_FWD ? g * OCg + m : m;
#pragma unroll
                for (int j = 0; j < 2; j++)
                {
                    const int pix = p0 + wn * 64 + 32 * j + l32;
                    if (pix >= P)
                        continue;
                    float v = acc[i][j][r];
                    if (guard_suspect(v, tiny))
                    {
                        const int ph = pix / PW, pw = pix - ph * PW;
                        v = MODE == MODE_FWD ? conv2d_exact(Xg, Wt, d, n, ch, ph, pw)
                                             : conv2d_grad_input_exact(Xg, Wt, d, n, ch, ph, pw);
                    }
                    if (MODE == MODE_FWD && d.bias != nullptr)
                        v = v + bias_s[m - m0];
                    Oimg[(int64_t)ch * P + pix] = v;
                }
            }
    }
    else
    {
        float acc[8][8];
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int j = 0; j < 8; j++)
                acc[i][j] = 0.0f;

        auto fma_step = [&](const float *A, const float *B, int kk) {
            const float4 a0 = *reinterpret_cast<const float4 *>(&A[kk * LDA + ty * 4]);
            const float4 a1 = *reinterpret_cast<const float4 *>(&A[kk * LDA + BM / 2 + ty * 4]);
            const float4 b0 = *reinterpret_cast<const float4 *>(&B[kk * LDB + tx * 4]);
            const float4 b1 = *reinterpret_cast<const float4 *>(&B[kk * LDB + 64 + tx * 4]);
            const float a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
            const float b[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
            for (int i = 0; i < 8; i++)
#pragma unroll
                for (int j = 0; j < 8; j++)
                    acc[i][j] = __fmaf_rn(a[i], b[j], acc[i][j]);
        };

        if (nkt > 0)
        {
            load_a(0);
            load_b();
            store_a(As[0]);
            store_b(Bs[0]);
        }
        __syncthreads();
        for (int kt = 0; kt < nkt; kt++)
        {
            const int cur = kt & 1;
            const bool more = kt + 1 < nkt;
            if (more)
            {
                load_a((kt + 1) * BK);
                load_b();
            }
            const int krem = K - kt * BK;
            if (krem >= BK)
            {
#pragma unroll
                for (int kk = 0; kk < BK; kk++)
                    fma_step(As[cur], Bs[cur], kk);
            }
            else
            {
                for (int kk = 0; kk < krem; kk++)
                    fma_step(As[cur], Bs[cur], kk);
            }
            if (more)
            {
                store_a(As[cur ^ 1]);
                store_b(Bs[cur ^ 1]);
            }
            __syncthreads();
        }

        // ---- epilogue: literal recompute of the suspect results (see the guard), then store ----
        const bool tiny = guard_tiny(guard);
#pragma unroll
        for (int i = 0; i < 8; i++)
        {
            const int m = m0 + ty * 4 + (i & 3) + (i >> 2) * (BM / 2);
            if (m >= M)
                continue;
            const int ch = MODE == MODE_FWD ? g * OCg + m : m; // output channel (FWD) / input channel (DGRAD)
#pragma unroll
            for (int jh = 0; jh < 2; jh++)
            {
                const int pix = p0 + tx * 4 + jh * 64;
                float v[4];
#pragma unroll
                for (int j = 0; j < 4; j++)
                {
                    v[j] = acc[i][jh * 4 + j];
                    const bool suspect = guard_suspect(v[j], tiny);
                    if (suspect && pix + j < P)
                    {
                        const int ph = (pix + j) / PW, pw = (pix + j) - ph * PW;
                        v[j] = MODE == MODE_FWD ? conv2d_exact(Xg, Wt, d, n, ch, ph, pw)
                                                : conv2d_grad_input_exact(Xg, Wt, d, n, ch, ph, pw);
                    }
                    if (MODE == MODE_FWD && d.bias != nullptr)
                        v[j] = v[j] + bias_s[m - m0];
                }
                float *p = Oimg + (int64_t)ch * P + pix;
                if (ovec && pix + 3 < P)
                    *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
                else
                {
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        if (pix + j < P)
                            p[j] = v[j];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Implicit GEMM without address arithmetic in the loop (matrix path, the common
// shapes).  While a matrix instruction runs, its SIMD issues no vector ALU
// instruction of any wave, so the index arithmetic and bounds checks of a gather are
// paid in matrix time.  Here the gathered operand is first copied into a zero-padded
// workspace tensor ([C][Hp][Wp] per image, by conv_pad_kernel; skipped when there is
// nothing to pad), after which the element of k-row k at pixel p sits at
//     image base + tab[k] + pix_off[p]
// with tab[k] depending only on k = (channel, kh, kw) (a table written once per call
// by conv_ktab_kernel, read with scalar loads) and pix_off[p] only on the pixel (one
// per-thread constant).  A load is then: scalar base, constant vector offset.
//   forward     tab[k] = c*Hp*Wp + kh*Wp + kw,                  pix_off = oh*sH*Wp + ow*sW
//   grad-input  tab[k] = oc*Hp*Wp + (pH+PT-kh)*Wp + (pW+PL-kw), pix_off = h*Wp + w      (stride 1)
// The kernel operand is read as [M][K] panels with k contiguous: the kernel itself for forward,
// for grad-input a copy WT[ic][(oc, kh, kw)] that conv_ktab_kernel writes next to the table.
// Lanes map to pixels, k-rows to instructions, so every table entry is wave-uniform.
// Requires K % 16 == 0 and M % BM == 0; pixels
// past the end of the image repeat the last pixel and are not stored.  The padded
// zeros play the role of the skipped taps exactly as in conv_gemm_kernel, with the same
// epilogue.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void conv_pad_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                       int64_t planes, int H, int W, int Hp, int Wp, int PT, int PL,
                                                       int dH, int dW, unsigned *__restrict__ parts)
{
    // A workgroup takes whole planes (grid-stride: at most GUARD_PARTS workgroups, each leaves
    // the minimum of what it copied); a wave takes rows, a lane columns: no divisions.
    unsigned m = GUARD_NONE;
    const int plane = Hp * Wp;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int64_t pl = blockIdx.x; pl < planes; pl += gridDim.x)
    {
        const float *__restrict__ sp = src + pl * H * W;
        float *__restrict__ dp = dst + pl * plane;
        // eight rows per wave and pass: their loads are all issued before the first store (one
        // row in flight per wave left the copy at 3.2 TB/s)
        constexpr int U = 8;
        for (int wp = lane; wp < Wp; wp += 64)
        {
            // source element (h, w) lands at (PT + h*dH, PL + w*dW); everything else is zero
            const int wd = wp - PL;
            const int w = dW == 1 ? wd : wd / dW;
            const bool win = wd >= 0 && w < W && (dW == 1 || w * dW == wd);
            for (int hp0 = wave; hp0 < Hp; hp0 += 4 * U)
            {
                float v[U];
#pragma unroll
                for (int u = 0; u < U; u++)
                {
                    const int hp = hp0 + 4 * u;
                    const int hd = hp - PT;
                    const int h = dH == 1 ? hd : hd / dH;
                    const bool hin = hp < Hp && hd >= 0 && h < H && (dH == 1 || h * dH == hd);
                    v[u] = (hin && win) ? sp[h * W + w] : 0.0f;
                }
#pragma unroll
                for (int u = 0; u < U; u++)
                {
                    const int hp = hp0 + 4 * u;
                    if (hp < Hp)
                    {
                        dp[hp * Wp + wp] = v[u];
                        m = guard_min(m, guard_bits(v[u]));
                    }
                }
            }
        }
    }
    m = guard_block_min(m);
    if (threadIdx.x == 0)
        parts[blockIdx.x] = m;
}

inline unsigned pad_blocks(int64_t planes)
{
    return (unsigned)(planes < 1 ? 1 : (planes > GUARD_PARTS ? GUARD_PARTS : planes)); // 2048 x 256 threads fill the chip
}

// The small jobs of a call in one launch.  Blocks [0, ceil(Kp / 256)) write the table (entries
// past K repeat the last one: their kernel values are -0.0f).  The panel_blocks after them write
// the kernel operand as the panels the matrix kernel reads, [groups][Mp][Kp] with k contiguous,
// rows past M zero and columns past K -0.0f (a product of -0.0f and finite data is a zero, and
// adding a zero of either sign changes no accumulator that is not -0.0f: see the guard):
//   forward     panel[g][m][k] = W[g*M + m][k],                     k = (ic, kh, kw)
//   grad-input  panel[0][m][k] = W[oc][m][kh][kw],                  k = (oc, kh, kw)
// (forward with whole tiles reads the kernel itself and has no such blocks).  The scan_blocks
// after those take the kernel's part of the guard of the zero results.
__global__ __launch_bounds__(256) void conv_ktab_kernel(int *__restrict__ tabB, int K, int Kp, int M, int Mp, int groups,
                                                        int KH, int KW, int plane, int Wp, int mode, int IC, int baseH,
                                                        int baseW, const float *__restrict__ W,
                                                        float *__restrict__ panel, int panel_blocks,
                                                        int64_t kernel_count, int scan_blocks,
                                                        unsigned *__restrict__ parts)
{
    const int KHW = KH * KW;
    const int tab_blocks = (Kp + 255) / 256;
    if ((int)blockIdx.x >= tab_blocks + panel_blocks)
    {
        guard_scan_block(W, kernel_count, (int)blockIdx.x - tab_blocks - panel_blocks, scan_blocks, parts);
        return;
    }
    if ((int)blockIdx.x >= tab_blocks)
    {
        const int64_t idx = (int64_t)(blockIdx.x - tab_blocks) * 256 + threadIdx.x; // = (g * Mp + m) * Kp + k
        if (idx >= (int64_t)groups * Mp * Kp)
            return;
        const int k = (int)(idx % Kp);
        const int64_t gm = idx / Kp;
        const int m = (int)(gm % Mp), g = (int)(gm / Mp);
        float v;
        if (k >= K)
            v = -0.0f;
        else if (m >= M)
            v = 0.0f;
        else if (mode == MODE_FWD)
            v = W[((int64_t)g * M + m) * K + k];
        else
        {
            const int oc = k / KHW, rem = k - oc * KHW;
            v = W[((int64_t)oc * IC + m) * KHW + rem];
        }
        panel[idx] = v;
        return;
    }
    const int k = blockIdx.x * 256 + threadIdx.x;
    if (k >= Kp)
        return;
    const int kk = k < K ? k : K - 1;
    const int c = kk / KHW, rem = kk - c * KHW;
    const int kh = rem / KW, kw = rem - kh * KW;
    tabB[k] = mode == MODE_FWD ? c * plane + kh * Wp + kw : c * plane + (baseH - kh) * Wp + (baseW - kw);
}

// PB: 32-pixel blocks per wave (2: tiles of 128 pixels; 1, only with BM = 64: tiles of 64 pixels,
// twice the workgroups at half the duration, for layers whose 128-pixel tiles fill the chip unevenly);
// RAGGED: the last row tile has rows past M (not stored)
template <int BM, int MODE, int PB, bool RAGGED>
__global__ __launch_bounds__(2 * BM) void conv_gemm_fast_kernel(const float *__restrict__ Gp,   // padded gathered operand
                                                                const float *__restrict__ Xg,   // the original one (epilogue)
                                                                const float *__restrict__ Wt,   // the kernel (epilogue)
                                                                const float *__restrict__ Wa,   // kernel operand as [M][K] panels
                                                                float *__restrict__ Out, ConvDims d,
                                                                const int *__restrict__ tabB, int plane, int Wp,
                                                                int64_t img_stride, const unsigned *__restrict__ guard,
                                                                int Mp, int Kp) // panel extents (multiples of BM, BK)
{
    constexpr int NT = 2 * BM;
    constexpr int LDA = BM + 4;
    static_assert(PB == 2 || (PB == 1 && BM == 64), "tiles of 64 pixels only with two waves");
    constexpr int TBN = PB == 2 ? BN : BN / 2;          // pixels per tile
    constexpr int NKR = BM == 64 && PB == 2 ? 16 : 8;   // k-rows of the gathered tile per wave
    typedef float v4f __attribute__((ext_vector_type(4)));
    // Two buffers for the gathered tile, no row pad (its rows are written and read by
    // consecutive lanes).  The kernel tile has two buffers with 128-pixel tiles (one barrier
    // per k-tile: 112x112 forward 0.807 -> 0.780 ms) and one with 64-pixel tiles, where the
    // LDS it saves is a tenth workgroup per CU and worth more than the barrier.
    constexpr int LDBF = TBN;
    constexpr int NA = PB == 2 ? 2 : 1;
    // 128-pixel tiles run the software-pipelined loop (112x112 forward 0.729 -> 0.697 ms, 128
    // channels at 28x28 0.219 -> 0.208); with 64-pixel tiles it needs the second kernel buffer
    // and loses more with the tenth workgroup than it gains (56x56 forward 0.203 -> 0.212 ms).
    constexpr bool PIPE = PB == 2;
    __shared__ __attribute__((aligned(16))) float As[NA][BK * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDBF];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int KHW = d.KH * d.KW;
    const int ICg = d.IC / d.groups, OCg = d.OC / d.groups;
    const int M = MODE == MODE_FWD ? OCg : d.IC; // rows that exist; the panels have Mp
    const int K = Kp;                            // k-steps of the panels and the table
    const int P = MODE == MODE_FWD ? d.OH * d.OW : d.H * d.W;
    const int PW = MODE == MODE_FWD ? d.OW : d.W;
    const int n = MODE == MODE_FWD ? blockIdx.z / d.groups : blockIdx.z;
    const int g = MODE == MODE_FWD ? blockIdx.z % d.groups : 0;
    const int m0 = blockIdx.y * BM, p0 = blockIdx.x * TBN;

    // gathered operand: this lane's pixel, this wave's k-rows
    const int b_half = PB == 1 ? 0 : (BM == 64 ? wave : (wave & 1));
    const int b_kr0 = PB == 1 ? 8 * wave : (BM == 64 ? 0 : 8 * (wave >> 1));
    const int pix_local = 64 * b_half + lane;
    const int pixc = p0 + pix_local < P ? p0 + pix_local : P - 1;
    const int pph = pixc / PW, ppw = pixc - pph * PW;
    const int pix_off = MODE == MODE_FWD ? pph * d.sH * Wp + ppw * d.sW : pph * Wp + ppw;
    const float *Gimg = Gp + (int64_t)n * img_stride + (MODE == MODE_FWD ? (int64_t)g * ICg * plane : 0);
    // kernel operand
    const float *Wg = Wa + (int64_t)g * Mp * K;
    uint32_t a_voff[2]; // byte offsets of this thread's two float4 slots in the [BM][K] panel
    int a_st[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
    {
        const int idx = tid + NT * i;
        const int r = idx >> 2, k4 = (idx & 3) << 2;
        a_voff[i] = (uint32_t)(r * K + k4) * 4u;
        a_st[i] = k4 * LDA + r;
    }

    v4f fa4[2];
    float fb[NKR];
    auto load_tiles = [&](int kt) {
        const int *tb = tabB + kt * BK + b_kr0;
#pragma unroll
        for (int j = 0; j < NKR; j++)
        {
            const float *rowp = Gimg + tb[j];
            fb[j] = rowp[pix_off];
        }
        const char *ab = reinterpret_cast<const char *>(Wg + (int64_t)m0 * K + kt * BK);
#pragma unroll
        for (int i = 0; i < 2; i++)
            fa4[i] = *reinterpret_cast<const v4f *>(ab + a_voff[i]);
    };
    auto store_tiles = [&](int buf) {
        float *as = As[NA == 2 ? buf : 0], *bs = Bs[buf];
#pragma unroll
        for (int j = 0; j < NKR; j++)
            bs[(b_kr0 + j) * LDBF + pix_local] = fb[j];
#pragma unroll
        for (int i = 0; i < 2; i++)
        {
            as[a_st[i] + 0 * LDA] = fa4[i][0];
            as[a_st[i] + 1 * LDA] = fa4[i][1];
            as[a_st[i] + 2 * LDA] = fa4[i][2];
            as[a_st[i] + 3 * LDA] = fa4[i][3];
        }
    };

    const int l32 = lane & 31, half = lane >> 5;
    const int wm = BM == 64 ? 0 : (wave & 1), wn = BM == 64 ? wave : (wave >> 1);
    f16v acc[2][PB];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < PB; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0.0f;
    const int a_off = half * LDA + wm * 64 + l32, b_off = half * LDBF + wn * (32 * PB) + l32;

    // forward with a bias: the values of this tile's rows go to LDS behind the first tiles (the
    // barrier that publishes those publishes them) and are read back in the epilogue
    __shared__ float bias_s[BM];
    const bool has_bias = MODE == MODE_FWD && d.bias != nullptr;
    float bias_r = 0.0f;
    const int nkt = K / BK;
    if (nkt > 0)
        load_tiles(0);
    if (has_bias && tid < BM && m0 + tid < M)
        bias_r = d.bias[g * OCg + m0 + tid];
    if (nkt > 0)
        store_tiles(0);
    if (has_bias && tid < BM)
        bias_s[tid] = bias_r;
    __syncthreads();
    if constexpr (PIPE)
    {
        // Software pipeline over the k-pairs of a k-tile: the operands of pair kp + 1 are read
        // while the matrix instructions of pair kp run, the next k-tile goes to the other LDS
        // buffers mid-way, and the barrier sits before the last pair, whose instructions cover
        // the first operand reads of the next k-tile.  Every read of a buffer is issued before
        // the barrier that precedes the next stores into it, so one barrier per k-tile is enough.
        float pa[2][2], pb[2][PB];
        auto read_ops = [&](int buf, int kp, float(&a)[2], float(&b)[PB]) {
            const float *as = As[buf] + a_off, *bs = Bs[buf] + b_off;
            a[0] = as[2 * kp * LDA];
            a[1] = as[2 * kp * LDA + 32];
#pragma unroll
            for (int j = 0; j < PB; j++)
                b[j] = bs[2 * kp * LDBF + 32 * j];
        };
        if (nkt > 0)
            read_ops(0, 0, pa[0], pb[0]);
        for (int kt = 0; kt < nkt; kt++)
        {
            const int cur = kt & 1;
            const bool more = kt + 1 < nkt;
            if (more)
                load_tiles(kt + 1);
#pragma unroll
            for (int kp = 0; kp < BK / 2; kp++)
            {
                if (kp + 1 < BK / 2)
                    read_ops(cur, kp + 1, pa[(kp + 1) & 1], pb[(kp + 1) & 1]);
                else if (more)
                    read_ops(cur ^ 1, 0, pa[0], pb[0]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < PB; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[kp & 1][i], pb[kp & 1][j], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (kp == 4 && more)
                    store_tiles(cur ^ 1);
                if (kp == BK / 2 - 2)
                    __syncthreads();
            }
        }
    }
    else
    for (int kt = 0; kt < nkt; kt++)
    {
        const int cur = kt & 1;
        const bool more = kt + 1 < nkt;
        if (more)
            load_tiles(kt + 1);
        const float *as = As[NA == 2 ? cur : 0] + a_off, *bs = Bs[cur] + b_off;
        float a[BK / 2][2], b[BK / 2][PB];
#pragma unroll
        for (int kp = 0; kp < BK / 2; kp++)
        {
            a[kp][0] = as[2 * kp * LDA];
            a[kp][1] = as[2 * kp * LDA + 32];
#pragma unroll
            for (int j = 0; j < PB; j++)
                b[kp][j] = bs[2 * kp * LDBF + 32 * j];
        }
#pragma unroll
        for (int kp = 0; kp < BK / 2; kp++)
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < PB; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kp][i], b[kp][j], acc[i][j], 0, 0, 0);
        if (NA == 1)
            __syncthreads(); // every wave has read the kernel tile
        if (more)
            store_tiles(cur ^ 1); // (NA == 2: last read before the barrier that ended the previous k-tile)
        __syncthreads();
    }

    float *Oimg = Out + (int64_t)n * (MODE == MODE_FWD ? d.OC : d.IC) * P;
    const bool tiny = guard_tiny(guard);
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int r = 0; r < 16; r++)
        {
            const int m = m0 + wm * 64 + 32 * i + 8 * (r >> 2) + 4 * half + (r & 3);
            if (RAGGED && m >= M)
                continue;
            const int ch = MODE == MODE_FWD ? g * OCg + m : m;
#pragma unroll
            for (int j = 0; j < PB; j++)
            {
                const int pix = p0 + wn * (32 * PB) + 32 * j + l32;
                if (pix >= P)
                    continue;
                float v = acc[i][j][r];
                if (guard_suspect(v, tiny))
                {
                    const int ph = pix / PW, pw = pix - ph * PW;
                    v = MODE == MODE_FWD ? conv2d_exact(Xg, Wt, d, n, ch, ph, pw)
                                         : conv2d_grad_input_exact(Xg, Wt, d, n, ch, ph, pw);
                }
                if (has_bias)
                    v = v + bias_s[m - m0];
                Oimg[(int64_t)ch * P + pix] = v;
            }
        }
}

// ---------------------------------------------------------------------------
// grad-kernel.  GK[oc][ic][kh][kw] is a chain over k = (n, oh, ow): there are
// only OC*IC*KH*KW chains and K = N*OH*OW cannot be split, so one LANE owns one
// chain (one dependent v_fma_f32 per k) and the kernel is shaped to make a k
// step cost little more than that FMA:
//   * a wave = one oc x 64 consecutive (ic,kh,kw) columns.  Its grad_output
//     value is wave-uniform: lane l loads element l of a 64-wide piece of an
//     output row (one coalesced load, issued a whole chunk ahead), and step k
//     broadcasts lane k with v_readlane_b32 into an SGPR that feeds the FMA;
//   * a workgroup = 4 waves (4 oc) sharing the same columns; the input rows
//     those columns touch are staged once per workgroup in LDS, zero-padded
//     left and right, so a lane's tap for consecutive ow is a ds_read_b32 at a
//     fixed offset (+ow*sW) and out-of-image taps read a zero;
//   * a chunk = R output rows of one image; the next chunk's input rows and
//     grad_output pieces are loaded into registers before the FMAs of the
//     current one (two LDS buffers).
// Every piece runs PIECE (16/32/64) steps: steps beyond the end of the row read
// the zero pad and a zero grad_output.  These padded zeros make the same +-0 /
// NaN results suspect as in the implicit GEMMs; those are recomputed with the
// literal chain.
// ---------------------------------------------------------------------------
// A step of a chain is an instruction pair: the FMA of this step and, next to it, the
// broadcast for the step eight ahead.  v_readlane_b32 has a long latency before its SGPR
// result can feed a VALU operand (about 12 clocks measured), short enough to hide behind
// eight dependent FMAs but not behind one.
// Eight steps as ONE asm block (the compiler pads every separate asm statement with an
// s_nop, which would cost a third issue slot per step): FMAs with the broadcast values gc
// and the taps xv[XO..XO+7]; meanwhile gn receives lanes LANE0..LANE0+7 of gsrc, the
// broadcast values of the eight steps after.
template <int LANE0, int XO>
__device__ __forceinline__ float wgrad_steps8(int gsrc, const int (&gc)[8], int (&gn)[8], const float (&xv)[16],
                                              float acc)
{
    asm volatile("v_readlane_b32 %0, %9, %10\n\tv_fmac_f32_e32 %8, %18, %26\n\t"
                 "v_readlane_b32 %1, %9, %11\n\tv_fmac_f32_e32 %8, %19, %27\n\t"
                 "v_readlane_b32 %2, %9, %12\n\tv_fmac_f32_e32 %8, %20, %28\n\t"
                 "v_readlane_b32 %3, %9, %13\n\tv_fmac_f32_e32 %8, %21, %29\n\t"
                 "v_readlane_b32 %4, %9, %14\n\tv_fmac_f32_e32 %8, %22, %30\n\t"
                 "v_readlane_b32 %5, %9, %15\n\tv_fmac_f32_e32 %8, %23, %31\n\t"
                 "v_readlane_b32 %6, %9, %16\n\tv_fmac_f32_e32 %8, %24, %32\n\t"
                 "v_readlane_b32 %7, %9, %17\n\tv_fmac_f32_e32 %8, %25, %33"
                 : "=&s"(gn[0]), "=&s"(gn[1]), "=&s"(gn[2]), "=&s"(gn[3]), "=&s"(gn[4]), "=&s"(gn[5]), "=&s"(gn[6]),
                   "=&s"(gn[7]), "+v"(acc)
                 : "v"(gsrc), "n"(LANE0 + 0), "n"(LANE0 + 1), "n"(LANE0 + 2), "n"(LANE0 + 3), "n"(LANE0 + 4),
                   "n"(LANE0 + 5), "n"(LANE0 + 6), "n"(LANE0 + 7), "s"(gc[0]), "s"(gc[1]), "s"(gc[2]), "s"(gc[3]),
                   "s"(gc[4]), "s"(gc[5]), "s"(gc[6]), "s"(gc[7]), "v"(xv[XO + 0]), "v"(xv[XO + 1]), "v"(xv[XO + 2]),
                   "v"(xv[XO + 3]), "v"(xv[XO + 4]), "v"(xv[XO + 5]), "v"(xv[XO + 6]), "v"(xv[XO + 7]));
    return acc;
}

template <bool UNIT>
__device__ __forceinline__ void wgrad_read16(const float *__restrict__ xr, int k0, int sW, float (&xv)[16])
{
#pragma unroll
    for (int u = 0; u < 16; u++)
        xv[u] = UNIT ? xr[k0 + u] : xr[(k0 + u) * sW];
}

// The software pipeline across the pieces of a chunk.  Invariant on entry to a piece: sa
// holds the broadcast values of its steps 0..7 and xa the taps of its steps 0..15; on exit
// the same holds for the next piece (g1 / x1).  Within the piece the taps are read sixteen
// steps ahead and the broadcasts eight steps ahead of their use.
template <int PIECE, bool UNIT>
struct WgradPipe
{
    int sa[8], sb[8];
    float xa[16], xb[16];

    __device__ __forceinline__ void prime(int g0, const float *x0, int sW)
    {
#pragma unroll
        for (int u = 0; u < 8; u++)
            sa[u] = __builtin_amdgcn_readlane(g0, u);
        wgrad_read16<UNIT>(x0, 0, sW, xa);
    }

    // PIECE = 32 or 64
    __device__ __forceinline__ float piece(int g, const float *x, int g1, const float *x1, int sW, float acc)
    {
        if (PIECE == 64)
        {
            wgrad_read16<UNIT>(x, 16, sW, xb);
            acc = wgrad_steps8<8, 0>(g, sa, sb, xa, acc);
            acc = wgrad_steps8<16, 8>(g, sb, sa, xa, acc);
            wgrad_read16<UNIT>(x, 32, sW, xa);
            acc = wgrad_steps8<24, 0>(g, sa, sb, xb, acc);
            acc = wgrad_steps8<32, 8>(g, sb, sa, xb, acc);
            wgrad_read16<UNIT>(x, 48, sW, xb);
            acc = wgrad_steps8<40, 0>(g, sa, sb, xa, acc);
            acc = wgrad_steps8<48, 8>(g, sb, sa, xa, acc);
            wgrad_read16<UNIT>(x1, 0, sW, xa);
            acc = wgrad_steps8<56, 0>(g, sa, sb, xb, acc);
            acc = wgrad_steps8<0, 8>(g1, sb, sa, xb, acc);
        }
        else
        {
            wgrad_read16<UNIT>(x, 16, sW, xb);
            acc = wgrad_steps8<8, 0>(g, sa, sb, xa, acc);
            acc = wgrad_steps8<16, 8>(g, sb, sa, xa, acc);
            wgrad_read16<UNIT>(x1, 0, sW, xa);
            acc = wgrad_steps8<24, 0>(g, sa, sb, xb, acc);
            acc = wgrad_steps8<0, 8>(g1, sb, sa, xb, acc);
        }
        return acc;
    }

    // PIECE = 16: two pieces at a time (the second may be a dummy that only prefetches), so
    // that the tap registers are back in xa at the end
    __device__ __forceinline__ float pair16(int g, const float *x, int g1, const float *x1, int g2,
                                            const float *x2, bool second, int sW, float acc)
    {
        wgrad_read16<UNIT>(x1, 0, sW, xb);
        acc = wgrad_steps8<8, 0>(g, sa, sb, xa, acc);
        acc = wgrad_steps8<0, 8>(g1, sb, sa, xa, acc);
        if (second)
        {
            wgrad_read16<UNIT>(x2, 0, sW, xa);
            acc = wgrad_steps8<8, 0>(g1, sa, sb, xb, acc);
            acc = wgrad_steps8<0, 8>(g2, sb, sa, xb, acc);
        }
        return acc;
    }
};

constexpr int WG_SLOTS = 16; // float4 staging slots per thread (16 rows x 64 floats per pass)
constexpr int WG_Q = 16;    // row pieces per chunk (one register of grad_output each)

template <int PIECE>
__global__ __launch_bounds__(256) void conv_wgrad_kernel(const float *__restrict__ GO,
                                                         const float *__restrict__ X,
                                                         float *__restrict__ GK, ConvDims d, int R, int NP,
                                                         int Wp, int CP, int hrows, int bufsz, int xvec,
                                                         const unsigned *__restrict__ guard)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int KHW = d.KH * d.KW, NC = d.IC * KHW;
    const int c0 = blockIdx.x * 64;
    const int col = c0 + lane;
    const bool cvalid = col < NC;
    const int colc = cvalid ? col : NC - 1;
    const int ic = colc / KHW;
    const int rem = colc - ic * KHW;
    const int kh = rem / d.KW, kw = rem - kh * d.KW;
    const int ic_first = c0 / KHW;
    const int last_col = (c0 + 63 < NC) ? c0 + 63 : NC - 1;
    const int nic = last_col / KHW - ic_first + 1;
    const int nrows = nic * hrows; // staged rows per chunk
    const int oc = blockIdx.y * 4 + wave;
    const bool ovalid = oc < d.OC;
    const int occ = ovalid ? oc : d.OC - 1;
    const int lane_off = (ic - ic_first) * CP + kh * Wp + kw;

    // both buffers start as zeros; staging only ever writes [pW, pW + roundup4(W)) of a
    // row, with zeros beyond W, so the left and right pads stay zero
    for (int i = tid; i < 2 * bufsz; i += 256)
        lds[i] = 0.0f;

    // staging slots of this thread: slot q covers row (tid>>4) + 16*(q / nseg), floats
    // [64*(q % nseg) + 4*(tid&15), +4) of that row
    const int nseg = (d.W + 63) >> 6;
    const int npass = (nrows + 15) >> 4;
    int s_goff[WG_SLOTS], s_hr[WG_SLOTS], s_w[WG_SLOTS], s_loff[WG_SLOTS];
#pragma unroll
    for (int q = 0; q < WG_SLOTS; q++)
    {
        const int pass = q / nseg, seg = q - pass * nseg;
        const int row = (tid >> 4) + 16 * pass;
        const int w = 64 * seg + 4 * (tid & 15);
        const bool on = pass < npass && row < nrows && w < d.W;
        const int icl = row / hrows, hr = row - icl * hrows;
        s_goff[q] = (ic_first + icl) * d.H * d.W + w;
        s_hr[q] = hr;
        s_w[q] = w;
        s_loff[q] = on ? icl * CP + hr * Wp + d.pW + w : -1;
    }
    __syncthreads();

    float4 stage[WG_SLOTS];
    float gnext[WG_Q], gcur[WG_Q];
    // input rows and grad_output pieces of chunk (n, oh0) -> registers
    auto chunk_load = [&](int n, int oh0) {
        const float *Xn = X + (int64_t)n * d.IC * d.H * d.W;
        const int hbase = oh0 * d.sH - d.pH;
#pragma unroll
        for (int q = 0; q < WG_SLOTS; q++)
        {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            const int h = hbase + s_hr[q];
            if (s_loff[q] >= 0 && h >= 0 && h < d.H)
            {
                const float *p = Xn + s_goff[q] + h * d.W;
                if (xvec && s_w[q] + 3 < d.W)
                    v = *reinterpret_cast<const float4 *>(p);
                else
                {
                    if (s_w[q] + 0 < d.W) v.x = p[0];
                    if (s_w[q] + 1 < d.W) v.y = p[1];
                    if (s_w[q] + 2 < d.W) v.z = p[2];
                    if (s_w[q] + 3 < d.W) v.w = p[3];
                }
            }
            stage[q] = v;
        }
        const float *gp = GO + (((int64_t)n * d.OC + occ) * d.OH + oh0) * d.OW;
        const int Rc = (d.OH - oh0 < R) ? d.OH - oh0 : R;
        int r = 0, pc = 0;
#pragma unroll
        for (int q = 0; q < WG_Q; q++)
        {
            float g = 0.0f;
            const int ow = pc * PIECE + lane;
            if (r < Rc && lane < PIECE && ow < d.OW)
                g = gp[r * d.OW + ow];
            gnext[q] = g;
            if (++pc == NP)
            {
                pc = 0;
                r++;
            }
        }
    };
    auto stage_store = [&](int buf) {
#pragma unroll
        for (int q = 0; q < WG_SLOTS; q++)
            if (s_loff[q] >= 0)
            {
                float *p = &lds[buf * bufsz + s_loff[q]];
                p[0] = stage[q].x;
                p[1] = stage[q].y;
                p[2] = stage[q].z;
                p[3] = stage[q].w;
            }
    };

    float acc = 0.0f;
    int n = 0, oh0 = 0;
    const bool any = d.N > 0 && d.OH > 0 && d.OW > 0;
    if (any)
    {
        chunk_load(0, 0);
        stage_store(0);
    }
    __syncthreads();
    int buf = 0;
    while (any)
    {
#pragma unroll
        for (int q = 0; q < WG_Q; q++)
            gcur[q] = gnext[q];
        int n1 = n, oh1 = oh0 + R;
        if (oh1 >= d.OH)
        {
            oh1 = 0;
            n1 = n + 1;
        }
        const bool more = n1 < d.N;
        if (more)
            chunk_load(n1, oh1);
        {
            const int nq = ((d.OH - oh0 < R) ? d.OH - oh0 : R) * NP;
            const float *xs = lds + buf * bufsz + lane_off;
            // tap pointer of piece q (row q / NP, piece q % NP of that row), clamped to the last
            // real piece so that the prefetch past the end stays inside the staged rows
            auto xptr = [&](int q) {
                const int qq = q < nq ? q : nq - 1;
                const int r = qq / NP, pc = qq - r * NP;
                return xs + r * d.sH * Wp + pc * PIECE * d.sW;
            };
            const int sW = d.sW;
            if (sW == 1)
            {
                WgradPipe<PIECE, true> pipe;
                pipe.prime(__float_as_int(gcur[0]), xptr(0), 1);
                if (PIECE == 16)
                {
#pragma unroll
                    for (int q = 0; q < WG_Q; q += 2)
                        if (q < nq)
                            acc = pipe.pair16(__float_as_int(gcur[q]), xptr(q), __float_as_int(gcur[q + 1]), xptr(q + 1),
                                              __float_as_int(gcur[q + 2 < WG_Q ? q + 2 : q]), xptr(q + 2), q + 1 < nq, 1, acc);
                }
                else
                {
#pragma unroll
                    for (int q = 0; q < WG_Q; q++)
                        if (q < nq)
                            acc = pipe.piece(__float_as_int(gcur[q]), xptr(q), __float_as_int(gcur[q + 1 < WG_Q ? q + 1 : q]),
                                             xptr(q + 1), 1, acc);
                }
            }
            else
            {
                WgradPipe<PIECE, false> pipe;
                pipe.prime(__float_as_int(gcur[0]), xptr(0), sW);
                if (PIECE == 16)
                {
#pragma unroll
                    for (int q = 0; q < WG_Q; q += 2)
                        if (q < nq)
                            acc = pipe.pair16(__float_as_int(gcur[q]), xptr(q), __float_as_int(gcur[q + 1]), xptr(q + 1),
                                              __float_as_int(gcur[q + 2 < WG_Q ? q + 2 : q]), xptr(q + 2), q + 1 < nq, sW, acc);
                }
                else
                {
#pragma unroll
                    for (int q = 0; q < WG_Q; q++)
                        if (q < nq)
                            acc = pipe.piece(__float_as_int(gcur[q]), xptr(q), __float_as_int(gcur[q + 1 < WG_Q ? q + 1 : q]),
                                             xptr(q + 1), sW, acc);
                }
            }
        }
        if (more)
            stage_store(buf ^ 1);
        __syncthreads();
        if (!more)
            break;
        buf ^= 1;
        n = n1;
        oh0 = oh1;
    }
    if (ovalid && cvalid)
    {
        if (guard_suspect(acc, guard_tiny(guard)))
            acc = conv2d_grad_kernel_exact(GO, X, d, oc, ic, kh, kw);
        GK[(int64_t)oc * NC + col] = acc;
    }
}

// ---------------------------------------------------------------------------
// grad-kernel on the matrix instruction v_mfma_f32_16x16x4_f32 (four k per
// instruction, ascending, each a single-rounding FMA; see mfma_check.hip).
// A wave owns ONE 16 (oc) x 16 (columns) block: the chains are as long as the batch
// and cannot be split, so what counts is the time per step of a chain, and a
// dependent sequence of these instructions advances 256 chains by four steps in 32
// clocks with two operand registers per instruction.  While a matrix instruction
// runs, the SIMD issues no vector ALU instruction of any wave (measured), so every
// VALU instruction on that SIMD lengthens the chain: the work is split by wave.
//
// A workgroup is four waves, one workgroup per CU, one wave per SIMD.  Waves 0 and 1
// compute (2 x 16 oc over the same 16 columns): LDS reads and matrix instructions,
// next to no VALU.  Waves 2 and 3 stage: per chunk (R output rows of one image) they
// bring
//   * grad_output[n][oc0..oc0+31][oh0..oh0+R)[*]: R*OW consecutive floats per oc, at
//     pitch GP (GP = 4 mod 32: the 64 lanes of an operand read hit every bank twice);
//   * the input rows the 16 columns touch, zero-padded left and right as in
//     conv_wgrad_kernel, so that a tap is an LDS word at a fixed per-lane offset
// into the LDS buffer that is not being computed from, and then issue the global
// loads of the chunk after, which stay in flight across the barrier.
// Lane l of a computing wave supplies, for the four steps ow..ow+3 of one
// instruction, grad_output of oc l%16 and the tap of column l%16, both at step l/16.
// Operands are read a piece (QP instructions) ahead.  Out-of-image taps read staged
// zeros, so +-0 / NaN results are recomputed with the literal chain, as everywhere
// in this file.  Widths that are not multiples of 4 are first rounded up in copies whose rows
// end in zeros (conv_pad_kernel): for grad_output the added steps multiply a zero, for the
// input the added columns fall into the zero pad of the staged rows.
// Requires OH % R == 0 and 16-byte aligned grad_output and input; other shapes take
// conv_wgrad_kernel.
// ---------------------------------------------------------------------------
typedef float f4v __attribute__((ext_vector_type(4)));
constexpr int MW_GS = 32; // most float4 staging slots of grad_output per staging thread
constexpr int MW_XS = 8;  // most float4 staging slots of input per staging thread
constexpr int MW_OC = 32; // oc per workgroup
constexpr int MW_ST = 128; // staging threads

// QP: instructions per piece; SW: the stride along a row, 0 when it is neither 1 nor 2 (the taps of a piece
// then sit at offsets the instructions cannot carry: an addition per read, and no two words per read --
// 7x7 at stride 2, 3 -> 64 at 224x224, took 18 clocks per step that way); XS, GS: staging slots per thread
// (input, grad_output); XV: the staged input rows are 16-byte aligned in LDS (1x1 kernels without padding:
// see the launcher)
template <int QP, int SW, int XS, int GS, bool XV>
__global__ __launch_bounds__(256) void conv_wgrad_mfma_kernel(const float *__restrict__ GOs, // grad_output, rows of 4*QP*NP floats
                                                              const float *__restrict__ Xs,  // input, rows of xW floats
                                                              const float *__restrict__ GO,  // both as given (epilogue)
                                                              const float *__restrict__ X,
                                                              float *__restrict__ GK, ConvDims d, int R, int NP,
                                                              int GP, int Wp, int CP, int hrows, int xoff, int bufsz,
                                                              int xW, const unsigned *__restrict__ guard)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x;
    const bool stager = __builtin_amdgcn_readfirstlane(tid >> 7) != 0;
    const int KHW = d.KH * d.KW, NC = d.IC * KHW;
    const int c0 = blockIdx.x * 16;
    const int ic_first = c0 / KHW;
    const int oc0 = blockIdx.y * MW_OC;
    const int OWp = 4 * QP * NP; // steps per output row: OW, or OW rounded up to 4 in a zero-padded copy
    const int nchunks = d.N * (d.OH / R);

    for (int i = tid; i < 2 * bufsz; i += 256)
        lds[i] = 0.0f;
    __syncthreads();

    if (stager)
    {
        const int st = tid & (MW_ST - 1);
        const int last_col = (c0 + 15 < NC) ? c0 + 15 : NC - 1;
        const int nic = last_col / KHW - ic_first + 1;
        // Slots, fixed for the whole kernel.  Slots past the data repeat the last slot (same words,
        // same values), so that no load or store sits behind a branch or a mask (the compiler waits
        // for every outstanding load where branches that contain loads merge).
        // Input: slot = (staged row, 4 floats of it); W % 4 == 0 and 16-byte alignment are given.
        const int nw4 = xW >> 2;
        const int nxs = nic * hrows * nw4;
        int x_goff[XS], x_hr[XS], x_loff[XS];
#pragma unroll
        for (int i = 0; i < XS; i++)
        {
            int s = st + MW_ST * i;
            s = s < nxs ? s : nxs - 1;
            const int row = s / nw4, w = (s - row * nw4) << 2;
            const int icl = row / hrows, hr = row - icl * hrows;
            x_goff[i] = (ic_first + icl) * d.H * xW + w;
            x_hr[i] = hr;
            x_loff[i] = xoff + icl * CP + hr * Wp + d.pW + w;
        }
        // grad_output: slot = (oc, 4 consecutive steps of the chunk)
        const int spo = (R * OWp) >> 2; // float4 per oc and chunk
        uint32_t g_goff[GS];
        int g_loff[GS];
#pragma unroll
        for (int i = 0; i < GS; i++)
        {
            int s = st + MW_ST * i;
            s = s < MW_OC * spo ? s : MW_OC * spo - 1;
            const int o = s / spo, t = (s - o * spo) << 2;
            const int oc = oc0 + o < d.OC ? oc0 + o : d.OC - 1; // rows of missing oc repeat the last one
            g_goff[i] = (uint32_t)((oc - oc0) * d.OH * OWp + t) * 4u;
            g_loff[i] = 64 + o * GP + t;
        }
        f4v xst[XS], gst[GS]; // plain vectors: they must stay in registers
        // Bit i: slot i of the chunk in xst is a row of the image (else a row of padding: zeros).  The
        // zeros go in when the slot is stored, a chunk later: a select on the loaded value at the load
        // makes the wave wait for the load it has just issued, in front of the barrier the computing
        // waves are waiting at (3x3, 64 -> 64 at 56x56, batch 64: 0.99 -> 0.955 ms).
        // (A second set of staging registers, the loads issued two chunks ahead of their store, was
        // slower: 1.03 ms.  Memory latency is not what the chunks wait for.)
        unsigned x_ok = 0;
        auto chunk_load = [&](int n, int oh0) {
            const float *Xn = Xs + (int64_t)n * d.IC * d.H * xW;
            const int hbase = oh0 * d.sH - d.pH;
            x_ok = 0;
#pragma unroll
            for (int i = 0; i < XS; i++)
            {
                const int h = hbase + x_hr[i];
                const bool ok = h >= 0 && h < d.H;
                const int hc = h < 0 ? 0 : (h >= d.H ? d.H - 1 : h);
                xst[i] = *reinterpret_cast<const f4v *>(Xn + x_goff[i] + hc * xW);
                x_ok |= ok ? 1u << i : 0u;
            }
            const char *Gn = reinterpret_cast<const char *>(GOs + (((int64_t)n * d.OC + oc0) * d.OH + oh0) * OWp);
#pragma unroll
            for (int i = 0; i < GS; i++)
                gst[i] = *reinterpret_cast<const f4v *>(Gn + g_goff[i]);
        };
        auto stage_store = [&](int buf) {
            float *base = lds + buf * bufsz;
#pragma unroll
            for (int i = 0; i < XS; i++)
            {
                float *p = base + x_loff[i];
                const bool ok = (x_ok >> i) & 1u;
                f4v v;
                v[0] = ok ? xst[i][0] : 0.0f;
                v[1] = ok ? xst[i][1] : 0.0f;
                v[2] = ok ? xst[i][2] : 0.0f;
                v[3] = ok ? xst[i][3] : 0.0f;
                if (XV)
                    *reinterpret_cast<f4v *>(p) = v;
                else
                {
                    p[0] = v[0];
                    p[1] = v[1];
                    p[2] = v[2];
                    p[3] = v[3];
                }
            }
#pragma unroll
            for (int i = 0; i < GS; i++)
                *reinterpret_cast<f4v *>(base + g_loff[i]) = gst[i];
        };
        int n1 = 0, oh1 = 0; // the chunk the next chunk_load fetches
        auto advance = [&]() {
            oh1 += R;
            if (oh1 >= d.OH)
            {
                oh1 = 0;
                n1++;
            }
        };
        if (nchunks > 0)
        {
            chunk_load(n1, oh1);
            advance();
            stage_store(0);
        }
        if (nchunks > 1)
        {
            chunk_load(n1, oh1);
            advance();
        }
        __syncthreads();
        for (int c = 0; c < nchunks; c++)
        {
            // registers hold chunk c + 1; buffer (c + 1) & 1 was last read in iteration c - 1
            if (c + 1 < nchunks)
                stage_store((c + 1) & 1);
            if (c + 2 < nchunks)
            {
                chunk_load(n1, oh1);
                advance();
            }
            __syncthreads();
        }
        return;
    }

    // ---- computing waves ----
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = c0 + (lane & 15);
    const int colc = col < NC ? col : NC - 1;
    const int ic = colc / KHW;
    const int rem = colc - ic * KHW;
    const int kh = rem / d.KW, kw = rem - kh * d.KW;
    const int q = lane >> 4;
    const int sW = SW > 0 ? SW : d.sW;
    const int a_lane = 64 + (wave * 16 + (lane & 15)) * GP + q; // 64 zero words lead each buffer
    const int x_lane = xoff + (ic - ic_first) * CP + kh * Wp + kw + q * sW;
    const int npieces = R * NP;

    f4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
    __syncthreads(); // chunk 0 is staged
    for (int c = 0; c < nchunks; c++)
    {
        const int buf = c & 1;
        const float *ab = lds + buf * bufsz + a_lane;
        const float *xb = lds + buf * bufsz + x_lane;
        // A piece is QP consecutive instructions of an output row.  The operands of the next
        // piece are read while the current one runs; the pointers of the piece being read advance
        // by one vector addition each: the grad_output words of consecutive pieces follow each
        // other without a gap (4*QP per piece), the taps advance by 4*QP*sW inside a row and jump
        // to the next staged row after the last piece of a row.  The read behind the last piece
        // of the chunk fetches words that are never used (inside the buffer, or the slack behind it).
        const float *ap = ab, *xp = xb;
        int rp = 0;
        const int xstep_in = 4 * QP * sW, xstep_row = d.sH * Wp - (NP - 1) * 4 * QP * sW;
        auto advance_piece = [&]() {
            ap += 4 * QP;
            const bool last = ++rp == NP;
            xp += last ? xstep_row : xstep_in;
            rp = last ? 0 : rp;
        };
        // runs the piece in (ca, cb) and reads the next one into (na, nb): one pair of reads
        // behind every instruction, pinned there (left alone, the scheduler moves the reads
        // behind the last instructions of the piece, too late for the next one)
        auto step_piece = [&](const float (&ca)[QP], const float (&cb)[QP], float (&na)[QP], float (&nb)[QP]) {
            // (reads in pairs: two words 16 bytes apart come with one ds_read2_b32, and the wave,
            // alone on its SIMD, issues an instruction only every 8 clocks or so -- three
            // instructions per 32-clock matrix instruction were one too many)
#pragma unroll
            for (int u = 0; u < QP; u += 2)
            {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ca[u], cb[u], acc, 0, 0, 0);
                if (u == 0)
                    advance_piece(); // under the first instruction
                na[u] = ap[4 * u];
                if (u + 1 < QP)
                    na[u + 1] = ap[4 * u + 4];
                nb[u] = xp[4 * u * sW];
                if (u + 1 < QP)
                    nb[u + 1] = xp[(4 * u + 4) * sW];
                __builtin_amdgcn_sched_barrier(0);
                if (u + 1 < QP)
                {
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ca[u + 1], cb[u + 1], acc, 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        float a0[QP], b0[QP], a1[QP], b1[QP];
#pragma unroll
        for (int u = 0; u < QP; u++)
        {
            a0[u] = ap[4 * u];
            b0[u] = xp[4 * u * sW];
        }
        __builtin_amdgcn_sched_barrier(0);
        for (int p = 0; p + 1 < npieces; p += 2)
        {
            step_piece(a0, b0, a1, b1);
            step_piece(a1, b1, a0, b0);
        }
        if (npieces & 1) // the operands of the last piece are in (a0, b0)
        {
#pragma unroll
            for (int u = 0; u < QP; u++)
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[u], b0[u], acc, 0, 0, 0);
        }
        __syncthreads();
    }
    // register r of the block: oc 4*(lane/16) + r of the wave's 16, column lane%16
    const bool tiny = guard_tiny(guard);
#pragma unroll
    for (int r = 0; r < 4; r++)
    {
        const int oc = oc0 + wave * 16 + 4 * q + r;
        if (oc < d.OC && col < NC)
        {
            float v = acc[r];
            if (guard_suspect(v, tiny))
                v = conv2d_grad_kernel_exact(GO, X, d, oc, ic, kh, kw);
            GK[(int64_t)oc * NC + col] = v;
        }
    }
}

// ---------------------------------------------------------------------------
// grad-kernel as one matrix product, for layers with MANY SHORT chains (the late layers of
// a network: 512 x 512 x 3 x 3 chains of 64 x 7 x 7 steps).  The chain kernel above is built
// for the opposite case; there it pays its per-workgroup start-up a dozen times over.
//     GK[oc][(ic,kh,kw)] = sum_k GOt[k][oc] * col[k][(ic,kh,kw)],   k = (n, oh, ow) ascending
// with GOt the grad_output with k outermost and col the im2col of the input (a zero where the
// tap falls outside the image), both written into a workspace; the product is repdl_hip_mm
// (transA), whose chains run over k in exactly this order.  The zeros stand for skipped taps
// as everywhere: a pass over the result recomputes the NaN results, and the zero results when
// the guard asks, with the literal chain.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void wgrad_got_kernel(const float *__restrict__ GO, float *__restrict__ GOt, int64_t total,
                                                        int OC, int OHW)
{
    // (the launcher takes this route only below 2^31 elements: 32-bit divisions, a fraction of the cost of 64-bit ones)
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x; // = k * OC + oc
    if ((int64_t)idx >= total)
        return;
    const uint32_t k = idx / (uint32_t)OC, oc = idx - k * (uint32_t)OC;
    const uint32_t n = k / (uint32_t)OHW, p = k - n * (uint32_t)OHW;
    GOt[idx] = GO[((int64_t)n * OC + oc) * OHW + p];
}

__global__ __launch_bounds__(256) void wgrad_col_kernel(const float *__restrict__ X, float *__restrict__ col, int64_t total,
                                                        ConvDims d, int NC)
{
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x; // = k * NC + (ic, kh, kw); below 2^31, as above
    if ((int64_t)idx >= total)
        return;
    const uint32_t k = idx / (uint32_t)NC, c = idx - k * (uint32_t)NC;
    const uint32_t KHW = (uint32_t)(d.KH * d.KW);
    const uint32_t ic = c / KHW, rem = c - ic * KHW;
    const uint32_t kh = rem / (uint32_t)d.KW, kw = rem - kh * (uint32_t)d.KW;
    const uint32_t t = k / (uint32_t)d.OW, ow = k - t * (uint32_t)d.OW;
    const uint32_t n = t / (uint32_t)d.OH, oh = t - n * (uint32_t)d.OH;
    const int h = (int)oh * d.sH - d.pH + (int)kh, w = (int)ow * d.sW - d.pW + (int)kw;
    col[idx] = (h >= 0 && h < d.H && w >= 0 && w < d.W) ? X[(((int64_t)n * d.IC + ic) * d.H + h) * d.W + w] : 0.0f;
}

__global__ __launch_bounds__(256) void wgrad_fixup_kernel(const float *__restrict__ GO, const float *__restrict__ X,
                                                          float *__restrict__ GK, ConvDims d, int64_t total,
                                                          const unsigned *__restrict__ guard)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total)
        return;
    const float v = GK[idx];
    if (!guard_suspect(v, guard_tiny(guard)))
        return;
    const int kw = (int)(idx % d.KW);
    int64_t t = idx / d.KW;
    const int kh = (int)(t % d.KH);
    t /= d.KH;
    const int ic = (int)(t % d.IC);
    const int oc = (int)(t / d.IC);
    GK[idx] = conv2d_grad_kernel_exact(GO, X, d, oc, ic, kh, kw);
}

// Rough times of the two grad-kernel routes (seconds), from measurements on the layers of a
// ResNet at batch 64: the chain kernel needs 12 clocks per step of a chain at stride 1 and 18 at
// stride 2 (64 -> 128, 3x3, stride 2 at 56x56: 0.38 ms for 50176 steps), and about 34 us per round of
// 256 workgroups (one per CU) on top; the product runs at about 100 TFLOP/s once it has enough
// tiles, never faster than its own k-chain on small tiles (about 20 clocks per step: 128 x 64 x 50176
// 0.43 ms), plus the passes that write its operands.  (128 -> 256, 3x3, stride 2 at 28x28: chain
// 0.37 ms, product 0.26; 256 -> 256 at 14x14: 0.49 / 0.36; 128 -> 128 at 28x28: 0.52 / 0.63.)  On output rows
// of fewer than 16 pixels the chain kernel's pieces are one or two instructions long and mostly
// overhead: 256 -> 512, 1x1 at 7x7, 3136 steps, 0.19 ms against 0.065 for the product.  With a 1x1
// kernel the sixteen columns of a block are sixteen channels, whose rows all have to be staged: about
// 90 us per round instead of 34 (1024 -> 256 at 14x14, two rounds of 12544 steps: 0.33 ms, product 0.20).
inline bool wgrad_prefers_gemm(int64_t OC, int64_t NC, int64_t K, int64_t sW, int64_t OW, int64_t KHW)
{
    const double clk = 1.0 / 2.35e9;
    const double rounds = (double)repdl_cdiv(repdl_cdiv(NC, 16) * repdl_cdiv(OC, 32), 256);
    const int64_t OWr = (OW + 3) / 4 * 4;
    const double step = (double)K * (sW > 2 ? 18.0 : 12.5) * (OWr < 16 ? 16.0 / (double)OWr : 1.0) * clk;
    const double t_chain = (rounds < 1.0 ? 1.0 : rounds) * (step + (KHW == 1 ? 90e-6 : 34e-6));
    const double flop = 2.0 * (double)OC * (double)NC * (double)K;
    const double t_mm = flop / 100e12 > (double)K * 20.0 * clk ? flop / 100e12 : (double)K * 20.0 * clk;
    const double t_gemm = t_mm + (double)K * (double)(NC + OC) * 8.0 / 3e12 + 40e-6;
    return t_gemm < 0.8 * t_chain;
}

// X'[n][c][oh][ow] = X[n][c][oh * sH][ow * sW]: what a 1x1 kernel at a stride reads of its input
// (I: uint32_t where the tensors have fewer than 2^31 elements -- 64-bit divisions cost several times more)
template <typename I>
__global__ __launch_bounds__(256) void conv_subsample_kernel(const float *__restrict__ X, float *__restrict__ Xs, int64_t total,
                                                             int H, int W, int OH, int OW, int sH, int sW)
{
    const I idx = (I)blockIdx.x * 256 + threadIdx.x;
    if ((int64_t)idx >= total)
        return;
    const I t = idx / (I)OW;
    const int ow = (int)(idx - t * (I)OW);
    const I plane = t / (I)OH;
    const int oh = (int)(t - plane * (I)OH);
    Xs[idx] = X[((int64_t)plane * H + (int64_t)oh * sH) * W + (int64_t)ow * sW];
}

// G[n][c][h][w] = G'[n][c][h / sH][w / sW] where a 1x1 kernel at a stride reads (h, w), +0 elsewhere:
// the grad-input of that layer from the grad-input G' of the same layer at stride 1
template <typename I>
__global__ __launch_bounds__(256) void conv_upsample_kernel(const float *__restrict__ Gs, float *__restrict__ G, int64_t total,
                                                            int H, int W, int OH, int OW, int sH, int sW)
{
    const I idx = (I)blockIdx.x * 256 + threadIdx.x;
    if ((int64_t)idx >= total)
        return;
    const I t = idx / (I)W;
    const int w = (int)(idx - t * (I)W);
    const I plane = t / (I)H;
    const int h = (int)(t - plane * (I)H);
    const int oh = h / sH, ow = w / sW;
    float v = 0.0f;
    if (oh * sH == h && ow * sW == w && oh < OH && ow < OW)
        v = Gs[((int64_t)plane * OH + oh) * OW + ow];
    __builtin_nontemporal_store(v, &G[idx]);
}

// Strided grad-input by phases.  Input position h takes the taps kh with (h + pH - kh) a multiple of sH,
// that is kh = r + a * sH with r = (h + pH) % sH: the positions of one residue pair (rh, rw) are the
// grad-input of a STRIDE-1 layer without padding whose kernel is the taps of that residue,
//     G'[n][ic][h'][w'] = sum over (oc, a, b) of GO[n][oc][h' - a][w' - b] * Ws[oc][ic][a][b],
//     Ws[oc][ic][a][b] = W[oc][ic][rh + a * sH][rw + b * sW],   h = sH * h' + rh - pH,
// with (oc, a, b) ascending exactly the reference's (oc, kh, kw) over the taps that count.  No product
// with a zero of a dilated grad_output: a quarter of the work at stride 2.
__global__ __launch_bounds__(256) void conv_phase_taps_kernel(const float *__restrict__ Wk, float *__restrict__ Ws, int total, int KH,
                                                                int KW, int A, int B, int rh, int rw, int sH, int sW)
{
    const int idx = blockIdx.x * 256 + threadIdx.x; // = (oc * IC + ic) * A * B + a * B + b
    if (idx >= total)
        return;
    const int b = idx % B, t = idx / B;
    const int a = t % A, plane = t / A;
    Ws[idx] = Wk[((int64_t)plane * KH + rh + a * sH) * KW + rw + b * sW];
}

// G[n][ic][sH * h' + rh - pH][sW * w' + rw - pW] = Gp[n][ic][h'][w'] (Gp == nullptr: +0, a residue without taps)
__global__ __launch_bounds__(256) void conv_phase_scatter_kernel(const float *__restrict__ Gp, float *__restrict__ G, int64_t total, int HP,
                                                                 int WP, int H, int W, int sH, int sW, int oh0, int ow0)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; // index into Gp: (plane, h', w')
    if (idx >= total)
        return;
    const int wp = (int)(idx % WP);
    const int64_t t = idx / WP;
    const int hp = (int)(t % HP);
    const int64_t plane = t / HP;
    const int h = sH * hp + oh0, w = sW * wp + ow0;
    if (h >= 0 && h < H && w >= 0 && w < W)
        G[(plane * H + h) * W + w] = Gp != nullptr ? Gp[idx] : 0.0f;
}

// ---------------------------------------------------------------------------
// Forward and grad-input of 3x3 kernels at stride 1 from an INPUT PATCH in LDS, both operands moved
// from global memory straight into LDS (global_load_lds, see mm.hip), v_mfma_f32_16x16x4_f32.
//
// The implicit GEMM above fetches the gathered operand tap by tap: nine global loads and nine LDS
// stores per input value, from a zero-padded copy of the whole tensor that a separate pass writes
// first.  Here a workgroup owns 64 rows x TN consecutive pixels of one image (2 x WGN waves of
// 32 x 32; rows past the last channel repeat it and are not stored) and brings the patch of the
// source those pixels touch into LDS once per chunk of four source channels (36 k = nine quads of
// the matrix instruction, k running in the reference's order (c, kh, kw)):
//   * the kernel operand A[64][36], k contiguous (the kernel itself for forward, a transposed copy
//     for grad-input), lands as [quad][row][4];
//   * the source patch lands as [channel][patch row][pitch] with pitch = source width + 4: DMA lane
//     s brings 16 bytes (four columns of one source row) to words 4s .. 4s+3, lanes whose row lies
//     outside the image or whose columns lie past the row's end are switched off, and their words
//     keep the zeros written once before the first chunk.  So the four cells after each row are
//     the zeros right of the image, and -- one row further on -- the zeros left of it; rows above
//     and below the image are rows of zeros.  (Widths that are not multiples of 4, or a tensor off
//     16-byte boundaries: 4 bytes per DMA lane, pitch = width + 2.)  Tap (c, kh, kw) of pixel (y, x)
//     is the patch word c * plane + (y - y0 + dy(kh)) * pitch + x + dx(kw), dy(kh) = kh, dx(kw) = kw
//     for forward and 2 - kh, 2 - kw for grad-input: a per-lane constant for each (quad, lane group),
//     18 address registers, every operand read a ds_read_b32 with an immediate.
// Three LDS buffers, operands read two quads ahead, one barrier per chunk, no vector arithmetic in
// the loop: the schedule of mm_dma_kernel.  Padded zeros stand where the reference skips a tap, as
// in the implicit GEMM, with the same epilogue (NaN results, and zero results when the guard asks,
// recomputed with the literal chain).  The guard's minima are reduced by every workgroup from the
// per-block parts of the scan launch.
// ---------------------------------------------------------------------------
namespace tapdma
{
// words per patch row: the source row and the zero cells after it -- four where the DMA moves 16
// bytes per lane (source width in fours), two where it moves 4 (any width).  (Rows padded so that
// the four lane groups of an operand read fall on different banks were measured too: no difference.)
__host__ __device__ inline int patch_pitch(int SW, int vec) { return SW + (vec == 4 ? 4 : 2); }
constexpr int CCH = 4, NQ = 9, D = 2, R = D + 1, NB = 3;
constexpr int QSA = 4 * 64;        // words per quad of the kernel operand
constexpr int OPA = NQ * QSA;      // words per chunk
constexpr int BLEAD = 4;           // zero words before the first patch row (the cells left of row 0)
constexpr int BWORDS = 2048;       // patch words per chunk, at most
constexpr int BSTR = BLEAD + BWORDS + 12; // words between patch buffers (a multiple of 4)

__device__ __forceinline__ void dma16(const void *base, uint32_t voff, uint32_t lds_byte)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base), "s"(lds_byte)
                 : "memory", "m0");
}
__device__ __forceinline__ void dma4(const void *base, uint32_t voff, uint32_t lds_byte)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(voff), "s"(base), "s"(lds_byte)
                 : "memory", "m0");
}

template <int MODE, int WGN, int VEC>
__global__ __launch_bounds__(128 * WGN) void conv_tapdma_kernel(const float *__restrict__ Src, // gathered tensor [N][C][SH][SW]
                                                                const float *__restrict__ Wt,  // the kernel (epilogue)
                                                                const float *__restrict__ PA,  // kernel operand [M][C * 9]
                                                                float *__restrict__ Out, ConvDims d, const unsigned *__restrict__ parts_a,
                                                                int count_a, const unsigned *__restrict__ parts_b, int count_b,
                                                                int use_guard, int PR)
{
    constexpr bool FLIP = MODE == MODE_DGRAD;
    constexpr int NW = 2 * WGN, NTH = 64 * NW, TN = 32 * WGN;
    constexpr int NIB = BWORDS / VEC / 64; // DMA instructions of a patch, at most
    constexpr int CA = (NQ + NW - 1) / NW, CB = (NIB + NW - 1) / NW;
    typedef float v4f __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) float smem[]; // [NB][OPA] then [NB][BSTR]
    __shared__ float bias_s[64];
    __shared__ unsigned gmin_s[NW][2];
    float *const As = smem, *const Bs = smem + NB * OPA;
    // where the dynamic LDS starts (the arrays above lie before it): DMA destinations are LDS byte addresses
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)smem;
    const int tid = threadIdx.x, lane = tid & 63, l16 = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int C = MODE == MODE_FWD ? d.IC : d.OC, M = MODE == MODE_FWD ? d.OC : d.IC;
    const int SH = MODE == MODE_FWD ? d.H : d.OH, SW = MODE == MODE_FWD ? d.W : d.OW; // source plane
    const int PH = MODE == MODE_FWD ? d.OH : d.H, PW = MODE == MODE_FWD ? d.OW : d.W; // output plane
    const int P = PH * PW, K = C * 9;
    const int dymin = MODE == MODE_FWD ? -d.pH : d.pH - 2, dxmin = MODE == MODE_FWD ? -d.pW : d.pW - 2;
    // The row tiles of one pixel tile read the same patch: ids 8 apart, i.e. the same XCD, back to back
    // (workgroup ids go to the XCDs round-robin), so that only the first brings it in from memory.
    const int mtiles = (M + 63) / 64, ptiles = (P + TN - 1) / TN;
    const int group = blockIdx.x / (8 * mtiles), rest = blockIdx.x % (8 * mtiles);
    const int pt = group * 8 + rest % 8;
    if (pt >= ptiles * d.N)
        return;
    const int n = pt / ptiles, m0 = (rest / 8) * 64, p0 = (pt % ptiles) * TN;
    const int y0 = p0 / PW;
    const int pitch = patch_pitch(SW, VEC), gpr = pitch / VEC, plane = PR * pitch; // gpr: DMA lanes per patch row
    const int nslot = CCH * PR * gpr, nib = (nslot + 63) / 64;
    const int nkt = C / CCH;

    // the guard's parts, requested now and reduced after the main loop
    unsigned ga = GUARD_NONE, gb = GUARD_NONE;
    if (use_guard)
    {
        for (int i = tid; i < count_a; i += NTH)
            ga = guard_min(ga, parts_a[i]);
        for (int i = tid; i < count_b; i += NTH)
            gb = guard_min(gb, parts_b[i]);
    }
    const bool has_bias = MODE == MODE_FWD && d.bias != nullptr;
    if (has_bias && tid < 64)
        bias_s[tid] = m0 + tid < M ? d.bias[m0 + tid] : 0.0f;
    // the patch buffers start as zeros; the DMA only ever writes cells that hold image data
    for (int i = tid; i < NB * BSTR / 4; i += NTH)
        reinterpret_cast<v4f *>(Bs)[i] = (v4f){0.f, 0.f, 0.f, 0.f};

    // DMA lanes.  Kernel operand: instruction e = quad e, lane = row.  Patch: slot s = (c * PR + i) * gpr + gi.
    uint32_t va[CA], vb[CB];
    bool okb[CB];
    const int arow = m0 + lane < M ? lane : M - 1 - m0; // rows past the last: the last one again, never stored
#pragma unroll
    for (int t = 0; t < CA; t++)
        va[t] = (uint32_t)((arow * K + 4 * (wave + NW * t)) * 4);
#pragma unroll
    for (int t = 0; t < CB; t++)
    {
        const int sl = 64 * (wave + NW * t) + lane;
        const int c = sl / (PR * gpr), rem = sl - c * (PR * gpr), i = rem / gpr, gi = rem - i * gpr;
        const int ys = y0 + dymin + i;
        okb[t] = sl < nslot && ys >= 0 && ys < SH && VEC * gi < SW;
        vb[t] = okb[t] ? (uint32_t)(((c * SH + ys) * SW + VEC * gi) * 4) : 0u;
    }
    const char *a_base = reinterpret_cast<const char *>(PA + (int64_t)m0 * K);
    const char *b_base = reinterpret_cast<const char *>(Src + (int64_t)n * C * SH * SW);
    const int64_t b_step = (int64_t)CCH * SH * SW * 4;
    auto issue = [&](int buf) {
#pragma unroll
        for (int t = 0; t < CA; t++)
            if (wave + NW * t < NQ)
                dma16(a_base, va[t], lds0 + (uint32_t)((buf * OPA + (wave + NW * t) * QSA) * 4));
#pragma unroll
        for (int t = 0; t < CB; t++)
            if (wave + NW * t < nib)
            {
                if (okb[t])
                {
                    if (VEC == 4)
                        dma16(b_base, vb[t], lds0 + (uint32_t)((NB * OPA + buf * BSTR + BLEAD + 256 * (wave + NW * t)) * 4));
                    else
                        dma4(b_base, vb[t], lds0 + (uint32_t)((NB * OPA + buf * BSTR + BLEAD + 64 * (wave + NW * t)) * 4));
                }
            }
        a_base += CCH * 9 * 4;
        b_base += b_step;
    };

    // operand read addresses
    const float *ra = As + (wm * 32 + l16) * 4 + g;
    const float *rbp[2][NQ];
    int pix[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
    {
        pix[j] = p0 + wn * 32 + 16 * j + l16;
        const int pc = pix[j] < P ? pix[j] : P - 1;
        const int y = pc / PW, x = pc - y * PW;
        const int base = BLEAD + (y - y0) * pitch + x + dxmin;
#pragma unroll
        for (int q = 0; q < NQ; q++)
        {
            const int k = 4 * q + g, c = k / 9, kh = (k % 9) / 3, kw = k % 3;
            rbp[j][q] = Bs + base + c * plane + (FLIP ? 2 - kh : kh) * pitch + (FLIP ? 2 - kw : kw);
        }
    }

    v4f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
            acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
    float xa[R][2], xb[R][2];
    auto read_q = [&](int buf, int q, float(&a)[2], float(&b)[2]) {
#pragma unroll
        for (int i = 0; i < 2; i++)
            a[i] = ra[buf * OPA + q * QSA + 64 * i];
#pragma unroll
        for (int j = 0; j < 2; j++)
            b[j] = rbp[j][q][buf * BSTR];
    };
    auto mfma_q = [&](float(&a)[2], float(&b)[2]) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[j], acc[i][j], 0, 0, 0);
    };

    __syncthreads(); // the zeros are in place before any DMA
#pragma unroll
    for (int u = 0; u < NB - 1; u++)
        if (u < nkt)
            issue(u);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#pragma unroll
    for (int q = 0; q < D; q++)
        read_q(0, q, xa[q], xb[q]);
    for (int kt = 0; kt < nkt; kt += NB)
    {
#pragma unroll
        for (int u = 0; u < NB; u++)
        {
            if (kt + u >= nkt)
                break;
            const bool more1 = kt + u + 1 < nkt, more_dma = kt + u + NB - 1 < nkt;
#pragma unroll
            for (int q = 0; q < NQ; q++)
            {
                if (q == NQ - D)
                {
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    if (more_dma)
                        issue((u + NB - 1) % NB);
                }
                const int qq = q + D;
                if (qq < NQ)
                    read_q(u, qq, xa[qq % R], xb[qq % R]);
                else if (more1)
                    read_q((u + 1) % NB, qq - NQ, xa[qq % R], xb[qq % R]);
                __builtin_amdgcn_sched_barrier(0);
                mfma_q(xa[q % R], xb[q % R]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // the guard: minimum over the workgroup of each operand's parts
    bool tiny = false;
    if (use_guard)
    {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1)
        {
            ga = guard_min(ga, (unsigned)__shfl_xor((int)ga, o));
            gb = guard_min(gb, (unsigned)__shfl_xor((int)gb, o));
        }
        if (lane == 0)
        {
            gmin_s[wave][0] = ga;
            gmin_s[wave][1] = gb;
        }
        __syncthreads();
        ga = gmin_s[0][0];
        gb = gmin_s[0][1];
#pragma unroll
        for (int w = 1; w < NW; w++)
        {
            ga = guard_min(ga, gmin_s[w][0]);
            gb = guard_min(gb, gmin_s[w][1]);
        }
        tiny = (double)__uint_as_float(ga) * (double)__uint_as_float(gb) < 0x1p-101;
    }

    float *Oimg = Out + (int64_t)n * M * P;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int r = 0; r < 4; r++)
        {
            const int m = m0 + wm * 32 + 16 * i + 4 * g + r;
            if (m >= M)
                continue;
#pragma unroll
            for (int j = 0; j < 2; j++)
            {
                if (pix[j] >= P)
                    continue;
                float v = acc[i][j][r];
                if (guard_suspect(v, tiny))
                {
                    const int ph = pix[j] / PW, pw = pix[j] - ph * PW;
                    v = MODE == MODE_FWD ? conv2d_exact(Src, Wt, d, n, m, ph, pw) : conv2d_grad_input_exact(Src, Wt, d, n, m, ph, pw);
                }
                if (has_bias)
                    v = v + bias_s[m - m0];
                __builtin_nontemporal_store(v, &Oimg[(int64_t)m * P + pix[j]]);
            }
        }
}

// The small jobs of a call in one launch: blocks [0, ca) scan the gathered tensor for the guard,
// the next cb the kernel, the rest (grad-input only) write the kernel operand with k contiguous:
//   A[m][k = (oc, kh, kw)] = W[oc][m][kh][kw]
__global__ __launch_bounds__(256) void conv_tapdma_prep_kernel(const float *__restrict__ G, int64_t gcount, int ca,
                                                               const float *__restrict__ W, int64_t wcount, int cb,
                                                               unsigned *__restrict__ parts_a, unsigned *__restrict__ parts_b,
                                                               float *__restrict__ PA, int IC, int OC)
{
    const int b = blockIdx.x;
    if (b < ca)
    {
        guard_scan_block(G, gcount, b, ca, parts_a);
        return;
    }
    if (b < ca + cb)
    {
        guard_scan_block(W, wcount, b - ca, cb, parts_b);
        return;
    }
    const int64_t idx = (int64_t)(b - ca - cb) * 256 + threadIdx.x;
    if (idx >= wcount)
        return;
    const int K = OC * 9;
    const int m = (int)(idx / K), k = (int)(idx - (int64_t)m * K);
    const int oc = k / 9, rem = k - oc * 9;
    PA[idx] = W[((int64_t)oc * IC + m) * 9 + rem];
}

// rows of the patch of TN consecutive pixels: the image rows they span, and two more
inline int patch_rows(int TN, int PW) { return (TN + PW - 2) / PW + 1 + 2; }

template <int MODE>
bool applies(const ConvDims &d, const float *gathered, const float *kernel, int TN, int vec)
{
    const int C = MODE == MODE_FWD ? d.IC : d.OC, M = MODE == MODE_FWD ? d.OC : d.IC;
    const int SH = MODE == MODE_FWD ? d.H : d.OH, SW = MODE == MODE_FWD ? d.W : d.OW;
    const int PH = MODE == MODE_FWD ? d.OH : d.H, PW = MODE == MODE_FWD ? d.OW : d.W;
    if (!(d.groups == 1 && d.KH == 3 && d.KW == 3 && d.sH == 1 && d.sW == 1 && d.pH <= 2 && d.pW <= 2 && M >= 1 && (M + 63) / 64 <= 65535 &&
          C % CCH == 0 && C >= CCH && PH >= 1 && PW >= 1 && SH >= 1 && SW >= 1 && d.N <= 65535 &&
          (repdl_cdiv((int64_t)PH * PW, TN) * d.N + 8) * ((M + 63) / 64) < (1LL << 30)))
        return false;
    if ((reinterpret_cast<uintptr_t>(kernel) & 15) != 0)
        return false;
    if (vec == 4 && (SW % 4 != 0 || (reinterpret_cast<uintptr_t>(gathered) & 15) != 0))
        return false;
    return (int64_t)patch_rows(TN, PW) * patch_pitch(SW, vec) * CCH <= BWORDS && (int64_t)C * SH * SW * 4 < (1LL << 31) &&
           (int64_t)64 * C * 9 * 4 < (1LL << 31) && (int64_t)PH * PW < (1LL << 30);
}

template <int MODE, int WGN, int VEC>
int launch(const float *gathered, const float *kernel, float *out, const ConvDims &d, hipStream_t s)
{
    constexpr int TN = 32 * WGN;
    const int C = MODE == MODE_FWD ? d.IC : d.OC, M = MODE == MODE_FWD ? d.OC : d.IC;
    const int P = MODE == MODE_FWD ? d.OH * d.OW : d.H * d.W, PW = MODE == MODE_FWD ? d.OW : d.W;
    const int64_t gcount = (int64_t)d.N * C * (MODE == MODE_FWD ? (int64_t)d.H * d.W : (int64_t)d.OH * d.OW);
    const int64_t wcount = (int64_t)d.OC * d.IC * 9;
    // the reference skips taps at every border of a 3x3 kernel unless forward runs without padding
    const bool skips = MODE == MODE_DGRAD || d.pH > 0 || d.pW > 0;
    const size_t pa_bytes = MODE == MODE_DGRAD ? ((size_t)wcount * sizeof(float) + 255) / 256 * 256 : 0;
    char *ws = nullptr;
    const hipError_t e0 = repdl_ws_acquire(reinterpret_cast<void **>(&ws), GUARD_BYTES + pa_bytes, s);
    if (e0 != hipSuccess)
        return (int)e0;
    unsigned *guard = reinterpret_cast<unsigned *>(ws);
    float *PA = reinterpret_cast<float *>(ws + GUARD_BYTES);
    const int ca = skips ? guard_blocks(gcount) : 0, cb = skips ? guard_blocks(wcount) : 0;
    const int wb = MODE == MODE_DGRAD ? (int)repdl_cdiv(wcount, 256) : 0;
    if (ca + cb + wb > 0)
        REPDL_LAUNCH(conv_tapdma_prep_kernel, dim3((unsigned)(ca + cb + wb)), dim3(256), 0, s, gathered, gcount, ca, kernel, wcount,
                           cb, guard_parts(guard, 0), guard_parts(guard, 1), PA, d.IC, d.OC);
    constexpr size_t shmem = (size_t)NB * (OPA + BSTR) * sizeof(float);
    auto kern = &conv_tapdma_kernel<MODE, WGN, VEC>;
    if (shmem > 48 * 1024)
    {
        const hipError_t e = REPDL_FUNC_SET_ATTRIBUTE(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess)
        {
            (void)repdl_ws_release(ws, s);
            return (int)e;
        }
    }
    const dim3 grid((unsigned)(repdl_cdiv(repdl_cdiv(P, TN) * d.N, 8) * 8 * repdl_cdiv(M, 64)));
    REPDL_LAUNCH(kern, grid, dim3(128 * WGN), shmem, s, gathered, kernel, MODE == MODE_DGRAD ? PA : kernel, out, d,
                       guard_parts(guard, 0), ca, guard_parts(guard, 1), cb, skips ? 1 : 0, patch_rows(TN, PW));
    const int rc = repdl_launch_status();
    const hipError_t e = repdl_ws_release(ws, s);
    return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
}
} // namespace tapdma

// ---------------------------------------------------------------------------
// 1x1 kernels at stride 1 without padding: forward and grad-input are plain products per image,
//     Out[m][pixel] = sum_c A[m][c] * Src[c][pixel],
// and Src is already what the matrix instruction wants: lanes 0-31 of an operand register take 32
// consecutive pixels of channel c, lanes 32-63 those of channel c + 1 -- two coalesced 128-byte
// pieces.  So nothing goes through LDS and no wave waits for another: each of a workgroup's four
// waves computes 64 rows x 32 pixels, streaming Src from global memory PB pairs of channels ahead
// of their use and the kernel operand (register layout, as for the patch kernel) PA pairs ahead.
// The reference skips no tap here, so there is nothing to guard and nothing to recompute.
// ---------------------------------------------------------------------------
namespace point
{
constexpr int RING = 8; // pairs of channels per unrolled step; both streams run RING pairs ahead

template <int MODE>
__global__ __launch_bounds__(256, 6) void conv_point_kernel(const float *__restrict__ Src, // [N][C][P]
                                                            const float *__restrict__ PA,  // kernel operand, register layout
                                                            float *__restrict__ Out, ConvDims d)
{
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int C = MODE == MODE_FWD ? d.IC : d.OC, M = MODE == MODE_FWD ? d.OC : d.IC;
    const int P = d.H * d.W; // (1x1, stride 1, no padding: input and output planes coincide)
    // Workgroup ids go to the 8 XCDs round-robin.  The M / 64 row tiles of one pixel tile read the same
    // columns of Src: they get ids 8 apart -- the same XCD, dispatched back to back -- so that only the
    // first of them brings those columns in from memory (256 rows: 412 -> 2xx MB per call).
    const int mtiles = M / 64, ptiles = (P + 127) / 128;
    const int group = blockIdx.x / (8 * mtiles), rest = blockIdx.x % (8 * mtiles);
    const int pt = group * 8 + rest % 8, mt = rest / 8;
    if (pt >= ptiles * d.N)
        return;
    const int n = pt / ptiles, m0 = mt * 64, p0 = (pt % ptiles) * 128;
    const int pix = p0 + wave * 32 + l32;
    const int pc = pix < P ? pix : P - 1;
    const int npair = C / 2;
    const __amdgpu_buffer_rsrc_t brsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(Src + (int64_t)n * C * P), 0, C * P * 4, 0x00020000);
    // Forward: PA is the prepared copy (see conv_point_prep_kernel).  Grad-input: the kernel itself -- A[m][c] =
    // W[c][m] has m contiguous, so lanes 0-31 of an operand register read 32 consecutive words of row c and lanes
    // 32-63 those of row c + 1, two coalesced 128-byte pieces, exactly the register layout: no copy, no launch.
    const __amdgpu_buffer_rsrc_t arsrc =
        MODE == MODE_FWD ? __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(PA + (int64_t)mt * npair * 128), 0, npair * 128 * 4, 0x00020000)
                         : __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(PA), 0, C * M * 4, 0x00020000);
    const int b_voff = (half * P + pc) * 4, a_voff = MODE == MODE_FWD ? lane * 4 : (half * M + m0 + l32) * 4;
    const int pair_bytes = 2 * P * 4;
    const int a_pair = MODE == MODE_FWD ? 512 : 2 * M * 4, a_second = MODE == MODE_FWD ? 256 : 128;

    float ar[RING][2], br[RING];
    auto request = [&](int slot, int q) { // pair q of the stream
        br[slot] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(brsrc, b_voff, q * pair_bytes, 0));
        ar[slot][0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(arsrc, a_voff, q * a_pair, 0));
        ar[slot][1] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(arsrc, a_voff + a_second, q * a_pair, 0));
    };
    f16v acc[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            acc[i][r] = 0.0f;
#pragma unroll
    for (int q = 0; q < RING; q++)
        request(q, q);
    for (int q0 = 0; q0 < npair; q0 += RING)
    {
#pragma unroll
        for (int u = 0; u < RING; u++)
        {
            const float a0 = ar[u][0], a1 = ar[u][1], b0 = br[u];
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1], 0, 0, 0);
            if (q0 + u + RING < npair) // (uniform)
                request(u, q0 + u + RING);
        }
    }
    const bool has_bias = MODE == MODE_FWD && d.bias != nullptr;
    float *Oimg = Out + (int64_t)n * M * P;
    if (pix < P)
    {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
            {
                const int m = m0 + 32 * i + 8 * (r >> 2) + 4 * half + (r & 3);
                float v = acc[i][r];
                if (has_bias)
                    v = v + d.bias[m];
                __builtin_nontemporal_store(v, &Oimg[(int64_t)m * P + pix]);
            }
    }
}

// the kernel operand in register layout: word ((mt * npair + q) * 2 + i) * 64 + lane holds
// A[mt * 64 + 32 * i + lane % 32][2 * q + lane / 32];  forward A[m][c] = W[m][c], grad-input A[m][c] = W[c][m]
__global__ __launch_bounds__(256) void conv_point_prep_kernel(const float *__restrict__ W, float *__restrict__ PA, int64_t wcount,
                                                              int mode, int C, int M)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= wcount)
        return;
    const int lane = (int)(idx & 63), i = (int)((idx >> 6) & 1);
    const int64_t t = idx >> 7; // = mt * npair + q
    const int npair = C / 2;
    const int q = (int)(t % npair), mt = (int)(t / npair);
    const int m = mt * 64 + 32 * i + (lane & 31), c = 2 * q + (lane >> 5);
    PA[idx] = mode == MODE_FWD ? W[(int64_t)m * C + c] : W[(int64_t)c * M + m];
}

template <int MODE>
bool applies(const ConvDims &d)
{
    const int C = MODE == MODE_FWD ? d.IC : d.OC, M = MODE == MODE_FWD ? d.OC : d.IC;
    const int64_t P = (int64_t)d.H * d.W;
    // (the kernel takes the source plane for the output plane: a grad-input call whose input extents are not
    // those of grad_output -- the residues of a strided layer make such calls -- has to go elsewhere)
    return d.groups == 1 && d.KH == 1 && d.KW == 1 && d.sH == 1 && d.sW == 1 && d.pH == 0 && d.pW == 0 && d.H == d.OH && d.W == d.OW &&
           M % 64 == 0 && M / 64 <= 65535 &&
           C % (2 * RING) == 0 && C >= 2 * RING && P >= 1 && d.N <= 65535 && (int64_t)C * P * 4 < (1LL << 31) && (int64_t)M * C * 4 < (1LL << 31) &&
           (repdl_cdiv(P, 128) * d.N + 8) * (M / 64) < (1LL << 30) &&
           P >= 1024; // (small images: the products over all images at once, see conv_prefers_mm)
}

template <int MODE>
int launch(const float *gathered, const float *kernel, float *out, const ConvDims &d, hipStream_t s)
{
    const int C = MODE == MODE_FWD ? d.IC : d.OC, M = MODE == MODE_FWD ? d.OC : d.IC;
    const int P = d.H * d.W;
    const int64_t wcount = (int64_t)M * C;
    const int64_t ptiles = repdl_cdiv(P, 128) * d.N;
    const dim3 grid((unsigned)(repdl_cdiv(ptiles, 8) * 8 * (M / 64)));
    if (MODE == MODE_DGRAD)
    {
        // (the kernel is read where it lies: 256 -> 64 at 56x56, batch 64, 0.0723 -> ... ms per call without the copy's launch)
        REPDL_LAUNCH((conv_point_kernel<MODE>), grid, dim3(256), 0, s, gathered, kernel, out, d);
        return repdl_launch_status();
    }
    float *PA = nullptr;
    const hipError_t e0 = repdl_ws_acquire(reinterpret_cast<void **>(&PA), (size_t)wcount * sizeof(float), s);
    if (e0 != hipSuccess)
        return (int)e0;
    REPDL_LAUNCH(conv_point_prep_kernel, dim3((unsigned)repdl_cdiv(wcount, 256)), dim3(256), 0, s, kernel, PA, wcount, MODE, C, M);
    REPDL_LAUNCH((conv_point_kernel<MODE>), grid, dim3(256), 0, s, gathered, PA, out, d);
    const int rc = repdl_launch_status();
    const hipError_t e = repdl_ws_release(PA, s);
    return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
}
} // namespace point

inline bool fits_i32(int64_t v) { return v >= 0 && v <= REPDL_I32_MAX; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Which pixel-tile width for the two-wave kernel?  Tiles of 128 pixels keep the matrix pipes
// busier (73 against 71 TFLOP/s on launches of 6000 workgroups), but with 152 registers per
// lane only 1536 of their workgroups are resident at a time, and a launch of one or two rounds
// leaves much of the chip idle at its end.  Tiles of 64 pixels make twice the workgroups of
// half the duration, 2560 resident.  Measured (batch 64, 64 -> 64 channels, 3x3, forward /
// grad-input): 28x28 0.127 / 0.121 -> 0.087 / 0.087 ms, 56x56 0.247 / 0.241 -> 0.226 / 0.224,
// 80x80 0.431 / 0.414 -> 0.423 / 0.412, 112x112 0.818 / 0.751 -> 0.818 / 0.773.
inline bool conv_small_tiles(int64_t workgroups128) { return workgroups128 < 4096; }

template <int MODE>
int launch_conv_gemm(const float *gathered, const float *kernel, float *out, const ConvDims &d, void *stream)
{
    const int KHW = d.KH * d.KW;
    const int M = MODE == MODE_FWD ? d.OC / d.groups : d.IC;
    const int64_t K = (int64_t)(MODE == MODE_FWD ? d.IC / d.groups : d.OC) * KHW;
    const int64_t P = MODE == MODE_FWD ? (int64_t)d.OH * d.OW : (int64_t)d.H * d.W;
    const int64_t gz = MODE == MODE_FWD ? (int64_t)d.N * d.groups : d.N;
    const int64_t gx = repdl_cdiv(P, BN);
    REPDL_REQUIRE(gz <= 65535 && fits_i32(gx) && fits_i32(K));
    const int wvec = MODE == MODE_FWD && aligned16(kernel) && (K % 4 == 0);
    const int ovec = aligned16(out) && (P % 4 == 0);
    hipStream_t s = repdl_stream(stream);
    const bool mfma = repdl_mfma_exact();
    // 3x3 at stride 1: the input-patch kernel (batch 64: 64 -> 64 at 56x56 0.213 -> 0.149 ms, 128 -> 128 at
    // 28x28 0.208 -> 0.143, 256 -> 256 at 14x14 0.28 -> 0.18)
    // Tiles of 128 pixels (eight waves) or of 64 (four)?  On the wider tile the kernel operand serves twice the
    // pixels and twice the waves share the DMA -- 3 to 12 % faster where both widths cover the image with the same
    // waste -- but its last tile of an image wastes more: 28x28 = 784 pixels are 7 tiles of 128 or 13 of 64, and
    // the narrow tile is 5 % faster there once the launch is large (1664 tiles); small launches take the wide tile
    // whatever the waste (64 x 64 channels at 28x28, 832 tiles: 11 % faster), images of one narrow tile never (7x7:
    // 63 % slower).  Measured at batch 64, forward / grad-input alike: 64 -> 64 at 56x56 0.147 -> 0.143 ms, 256 ->
    // 256 at 14x14 0.167 -> 0.153, 64 -> 64 at 64x64 0.181 -> 0.166, 32 -> 32 at 56x56 0.089 -> 0.081.
    const int64_t c128 = repdl_cdiv(P, 128), c64 = repdl_cdiv(P, 64);
    const int64_t tiles64 = c64 * d.N * repdl_cdiv(MODE == MODE_FWD ? d.OC : d.IC, 64);
    const bool wide = P > 64 && (tiles64 < 1024 || 186 * c128 < 100 * c64);
    if (mfma && wide && tapdma::applies<MODE>(d, gathered, kernel, 128, 4))
    {
        repdl_route_note(REPDL_ROUTE_CONV_PATCH_16_WIDE);
        return tapdma::launch<MODE, 4, 4>(gathered, kernel, out, d, s);
    }
    if (mfma && tapdma::applies<MODE>(d, gathered, kernel, 64, 4))
    {
        repdl_route_note(REPDL_ROUTE_CONV_PATCH_16);
        return tapdma::launch<MODE, 2, 4>(gathered, kernel, out, d, s);
    }
    // any other width, 4 bytes per DMA lane
    if (mfma && wide && tapdma::applies<MODE>(d, gathered, kernel, 128, 1))
    {
        repdl_route_note(REPDL_ROUTE_CONV_PATCH_4_WIDE);
        return tapdma::launch<MODE, 4, 1>(gathered, kernel, out, d, s);
    }
    if (mfma && tapdma::applies<MODE>(d, gathered, kernel, 64, 1))
    {
        repdl_route_note(REPDL_ROUTE_CONV_PATCH_4);
        return tapdma::launch<MODE, 2, 1>(gathered, kernel, out, d, s);
    }
    // (chains of 64 terms or fewer: the streaming kernel, which has no prologue to fill -- batch 64,
    // 56x56, 64 channels in, 256 out: 0.087 against 0.098 ms)
    const bool short_chain = K <= 64 && point::applies<MODE>(d);
    if (mfma && !short_chain && d.groups == 1 && KHW == 1 && d.sH == 1 && d.sW == 1 && d.pH == 0 && d.pW == 0 && d.H == d.OH && d.W == d.OW)
    {
        // a 1x1 kernel at stride 1: per image Out[M][P] = A[M][C] . Src[C][P], A = W (forward) or W^T
        // (grad-input) -- a batch of plain products, and the reference skips no tap here (batch 64:
        // 512 -> 128 at 28x28 0.096 -> 0.072 ms, 1024 -> 256 at 14x14 0.119 -> 0.080, 256 -> 64 at 56x56
        // 0.079 -> 0.072)
        const int rc = repdl_mm_batched(kernel, gathered, out, MODE == MODE_FWD ? d.bias : nullptr, M, P, K, MODE == MODE_DGRAD, 0,
                                        d.N, 0, (int64_t)K * P, (int64_t)M * P, s);
        if (rc != REPDL_E_UNSUPPORTED)
        {
            repdl_route_note(REPDL_ROUTE_CONV_POINT_MM);
            return rc;
        }
    }
    if (mfma && point::applies<MODE>(d))
    {
        repdl_route_note(REPDL_ROUTE_CONV_POINT);
        return point::launch<MODE>(gathered, kernel, out, d, s);
    }
    const int64_t gathered_count =
        (int64_t)d.N * (MODE == MODE_FWD ? (int64_t)d.IC * d.H * d.W : (int64_t)d.OC * d.OH * d.OW);
    const int64_t kernel_count = (int64_t)d.OC * (d.IC / d.groups) * KHW;
    // does the reference skip any tap?  (forward: only into the padding; grad-input: at the
    // borders of any kernel wider than one tap, and between strides)
    const bool skips_geom = MODE == MODE_FWD ? (d.pH > 0 || d.pW > 0)
                                             : (KHW > 1 || d.sH > 1 || d.sW > 1 || d.pH > 0 || d.pW > 0);
    // Fast path.  Rows and k-steps are rounded up to whole tiles in a padded copy of the kernel
    // operand (see conv_ktab_kernel); 128-row tiles when that rounds no further than 64-row ones.
    const int64_t M64 = repdl_cdiv(M, 64) * 64, M128 = repdl_cdiv(M, 128) * 128;
    const int bm = (M > 64 && M128 == M64) ? 128 : 64;
    const int64_t Mp = bm == 128 ? M128 : M64, Kp = repdl_cdiv(K, BK) * BK;
    const int groups = MODE == MODE_FWD ? d.groups : 1;
    const bool panel = MODE == MODE_DGRAD || Mp != M || Kp != K;
    // (forward with few, ragged k-steps -- a 3-channel stem layer -- stays with the gather kernel: copying
    // its large input into the workspace costs more than the gather, 0.39 against 0.45 ms for 3 -> 64, 3x3)
    const bool few_k = MODE == MODE_FWD && Kp != K && K < 256;
    if (mfma && M > 0 && K > 0 && !few_k && (MODE == MODE_FWD || (d.sH <= 4 && d.sW <= 4)))
    {
        // Strided grad-input: grad_output goes into the workspace DILATED (stride - 1 zeros between
        // its elements), after which it is the stride-1 case; the zeros take the place of the taps the
        // reference skips between the strides.  (The matrix instructions then spend 1 - 1/(sH*sW) of
        // their time on zeros, still well ahead of the gather with its divisions.)
        const int C = MODE == MODE_FWD ? d.IC : d.OC;                 // channels of the gathered tensor
        const int SH = MODE == MODE_FWD ? d.H : d.OH, SW = MODE == MODE_FWD ? d.W : d.OW; // source extents
        const int DH = MODE == MODE_FWD ? 1 : d.sH, DW = MODE == MODE_FWD ? 1 : d.sW;     // dilation
        const int GH = (SH - 1) * DH + 1, GW = (SW - 1) * DW + 1;
        const int PT = MODE == MODE_FWD ? d.pH : (d.KH - 1 - d.pH > 0 ? d.KH - 1 - d.pH : 0);
        const int PL = MODE == MODE_FWD ? d.pW : (d.KW - 1 - d.pW > 0 ? d.KW - 1 - d.pW : 0);
        int64_t Hp = GH + 2 * (int64_t)PT, Wp = GW + 2 * (int64_t)PL;
        if (MODE == MODE_DGRAD)
        { // rows / columns of the input that no output reaches still read (zeros) up to h + pH + PT
            Hp = Hp > d.H + d.pH + PT ? Hp : d.H + d.pH + PT;
            Wp = Wp > d.W + d.pW + PL ? Wp : d.W + d.pW + PL;
        }
        const int64_t plane = Hp * Wp, img = (int64_t)C * plane;
        if (SH > 0 && SW > 0 && img * 4 < (1LL << 31) && groups * Mp * Kp * 4 < (1LL << 31) && Mp / bm <= 65535 &&
            (int64_t)d.N * img / 256 < REPDL_I32_MAX)
        {
            // padded k-steps are zero products too: the guard decides about zero results
            const bool skips = skips_geom || Kp != K;
            const bool pad = PT > 0 || PL > 0 || DH > 1 || DW > 1 || Hp != GH || Wp != GW;
            // workspace: the guard words, the table, the kernel operand's panels (when not the kernel itself),
            // the padded copy of the gathered operand
            const size_t tab_bytes = ((size_t)Kp * sizeof(int) + 255) / 256 * 256;
            const size_t wt_bytes = panel ? ((size_t)(groups * Mp * Kp) * sizeof(float) + 255) / 256 * 256 : 0;
            const size_t ws_bytes = GUARD_BYTES + tab_bytes + wt_bytes + (pad ? (size_t)d.N * img * sizeof(float) : 0);
            char *ws = nullptr;
            hipError_t e = repdl_ws_acquire(reinterpret_cast<void **>(&ws), ws_bytes, s);
            if (e != hipSuccess)
                return (int)e;
            unsigned *guard = reinterpret_cast<unsigned *>(ws);
            int *tabB = reinterpret_cast<int *>(ws + GUARD_BYTES);
            float *WT = reinterpret_cast<float *>(ws + GUARD_BYTES + tab_bytes);
            float *Gp = reinterpret_cast<float *>(ws + GUARD_BYTES + tab_bytes + wt_bytes);
            const float *Wa = panel ? WT : kernel;
            // guard[0]: the gathered operand (in the padding pass when there is one), guard[1]: the kernel
            // guard: the kernel's part in the table launch, the gathered operand's in the padding pass
            // when there is one
            int ca = 0, cb = 0, unused = 0;
            if (skips && !pad)
                launch_guard_scan(gathered, gathered_count, nullptr, 0, guard, s, ca, unused);
            if (skips)
                cb = guard_blocks(kernel_count);
            const int64_t wt_blocks = panel ? repdl_cdiv(groups * Mp * Kp, 256) : 0;
            REPDL_LAUNCH(conv_ktab_kernel, dim3((unsigned)(repdl_cdiv(Kp, 256) + wt_blocks + cb)), dim3(256), 0, s, tabB,
                               (int)K, (int)Kp, M, (int)Mp, groups, d.KH, d.KW, (int)plane, (int)Wp, MODE, d.IC, d.pH + PT,
                               d.pW + PL, kernel, WT, (int)wt_blocks, kernel_count, cb, guard_parts(guard, 1));
            if (pad)
            {
                const int64_t planes = (int64_t)d.N * C;
                ca = (int)pad_blocks(planes);
                REPDL_LAUNCH(conv_pad_kernel, dim3((unsigned)ca), dim3(256), 0, s, gathered, Gp, planes, SH, SW,
                                   (int)Hp, (int)Wp, PT, PL, DH, DW, guard_parts(guard, 0));
            }
            if (skips)
                launch_guard_final(guard, ca, cb, s);
            else
                guard = nullptr;
            const float *src = pad ? Gp : gathered;
            // Tiles of 64 pixels when that fills the chip more evenly (see conv_small_tiles).
            const bool small_tiles = bm == 64 && conv_small_tiles(gx * (Mp / bm) * gz);
            dim3 grid((unsigned)(small_tiles ? repdl_cdiv(P, BN / 2) : gx), (unsigned)(Mp / bm), (unsigned)gz);
#define REPDL_CONV_FAST(BM_, PB_, RG_)                                                                                  \
    REPDL_LAUNCH((conv_gemm_fast_kernel<BM_, MODE, PB_, RG_>), grid, dim3(2 * BM_), 0, s, src, gathered, kernel, \
                       Wa, out, d, tabB, (int)plane, (int)Wp, img, guard, (int)Mp, (int)Kp)
            const bool ragged = Mp != M;
            repdl_route_note(bm == 64 && small_tiles ? REPDL_ROUTE_CONV_PADDED_64_HALF : bm == 64 ? REPDL_ROUTE_CONV_PADDED_64 : REPDL_ROUTE_CONV_PADDED_128);
            if (bm == 64 && small_tiles)
            {
                if (ragged)
                    REPDL_CONV_FAST(64, 1, true);
                else
                    REPDL_CONV_FAST(64, 1, false);
            }
            else if (bm == 64)
            {
                if (ragged)
                    REPDL_CONV_FAST(64, 2, true);
                else
                    REPDL_CONV_FAST(64, 2, false);
            }
            else
            {
                if (ragged)
                    REPDL_CONV_FAST(128, 2, true);
                else
                    REPDL_CONV_FAST(128, 2, false);
            }
#undef REPDL_CONV_FAST
            const int rc = repdl_launch_status();
            e = repdl_ws_release(ws, s);
            return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
        }
    }
    REPDL_REQUIRE(repdl_cdiv(M, 128) <= 65535);
    const bool skips = skips_geom;
    unsigned *guard = nullptr;
    hipError_t ge = hipSuccess;
    if (skips)
    {
        ge = repdl_ws_acquire(reinterpret_cast<void **>(&guard), GUARD_BYTES, s);
        if (ge != hipSuccess)
            return (int)ge;
        int ca = 0, cb = 0;
        launch_guard_scan(gathered, gathered_count, kernel, kernel_count, guard, s, ca, cb);
        launch_guard_final(guard, ca, cb, s);
    }
    repdl_route_note(M <= 64 ? REPDL_ROUTE_CONV_GATHER_64 : REPDL_ROUTE_CONV_GATHER_128);
    if (M <= 64)
    {
        dim3 grid((unsigned)gx, (unsigned)repdl_cdiv(M, 64), (unsigned)gz);
        if (mfma)
            REPDL_LAUNCH((conv_gemm_kernel<64, MODE, true>), grid, dim3(128), 0, s, gathered, kernel, out, d, wvec, ovec, guard);
        else
            REPDL_LAUNCH((conv_gemm_kernel<64, MODE, false>), grid, dim3(128), 0, s, gathered, kernel, out, d, wvec, ovec, guard);
    }
    else
    {
        dim3 grid((unsigned)gx, (unsigned)repdl_cdiv(M, 128), (unsigned)gz);
        if (mfma)
            REPDL_LAUNCH((conv_gemm_kernel<128, MODE, true>), grid, dim3(256), 0, s, gathered, kernel, out, d, wvec, ovec, guard);
        else
            REPDL_LAUNCH((conv_gemm_kernel<128, MODE, false>), grid, dim3(256), 0, s, gathered, kernel, out, d, wvec, ovec, guard);
    }
    const int rc = repdl_launch_status();
    if (skips)
        ge = repdl_ws_release(guard, s);
    return rc != REPDL_OK ? rc : (ge == hipSuccess ? REPDL_OK : (int)ge);
}
// ---------------------------------------------------------------------------
// Forward and grad-input as one matrix product, for layers with SMALL IMAGES and many
// channels (the late layers of a network: 512 channels at 7x7).  The implicit GEMM above tiles
// the pixels of one image at a time; 49 pixels fill no tile, and its few workgroups leave each
// SIMD a single wave that cannot hide its own load latency (0.51 ms for 512 -> 512, 3x3, batch
// 64).  Here the gathered operand is written out as a matrix with a row per output element of
// all images,
//     forward     col[(n, oh, ow)][(ic, kh, kw)] = X[n][ic][oh*sH - pH + kh][ow*sW - pW + kw]
//     grad-input  col[(n, h, w)][(oc, kh, kw)]   = GO[n][oc][(h + pH - kh) / sH][(w + pW - kw) / sW]
// (a zero where the reference skips the tap), the product C = col . Wp^T is repdl_hip_mm
// (transB), whose chains run over k in exactly the reference's order, and a last pass moves
// C[(n, pixel)][channel] to NCHW, recomputing NaN results (and zero results when the guard
// asks) with the literal chain.  Wp is the kernel itself for forward, a [IC][(oc, kh, kw)]
// copy for grad-input.
// ---------------------------------------------------------------------------
template <int MODE>
__global__ __launch_bounds__(256) void conv_col_kernel(const float *__restrict__ G, float *__restrict__ col, int64_t total,
                                                       ConvDims d, int K)
{
    // (conv_prefers_mm keeps this route below 2^31 elements: 32-bit divisions)
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x; // = row * K + k
    if ((int64_t)idx >= total)
        return;
    const uint32_t row = idx / (uint32_t)K;
    const int k = (int)(idx - row * (uint32_t)K);
    const int KHW = d.KH * d.KW;
    const int c = k / KHW, rem = k - c * KHW;
    const int kh = rem / d.KW, kw = rem - kh * d.KW;
    const uint32_t PW = (uint32_t)(MODE == MODE_FWD ? d.OW : d.W), PH = (uint32_t)(MODE == MODE_FWD ? d.OH : d.H);
    const uint32_t t = row / PW;
    const int pw = (int)(row - t * PW);
    const int64_t n = t / PH;
    const int ph = (int)(t - (uint32_t)n * PH);
    float v = 0.0f;
    if (MODE == MODE_FWD)
    {
        const int h = ph * d.sH - d.pH + kh, w = pw * d.sW - d.pW + kw;
        if (h >= 0 && h < d.H && w >= 0 && w < d.W)
            v = G[((n * d.IC + c) * d.H + h) * d.W + w];
    }
    else
    {
        const int th = ph + d.pH - kh, tw = pw + d.pW - kw;
        const int oh = th / d.sH, ow = tw / d.sW;
        if (th >= 0 && tw >= 0 && oh * d.sH == th && ow * d.sW == tw && oh < d.OH && ow < d.OW)
            v = G[((n * d.OC + c) * d.OH + oh) * d.OW + ow];
    }
    col[idx] = v;
}

// WT[ic][(oc, kh, kw)] = W[oc][ic][kh][kw]
__global__ __launch_bounds__(256) void conv_wt_kernel(const float *__restrict__ W, float *__restrict__ WT, int64_t total,
                                                      int IC, int KHW, int K)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; // = ic * K + k
    if (idx >= total)
        return;
    const int k = (int)(idx % K), ic = (int)(idx / K);
    const int oc = k / KHW, rem = k - oc * KHW;
    WT[idx] = W[((int64_t)oc * IC + ic) * KHW + rem];
}

template <int MODE>
__global__ __launch_bounds__(256) void conv_mm_out_kernel(const float *__restrict__ C, const float *__restrict__ Xg,
                                                          const float *__restrict__ Wt, float *__restrict__ Out, ConvDims d,
                                                          int64_t total, const unsigned *__restrict__ guard)
{
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x; // NCHW index of the output (below 2^31, as above)
    if ((int64_t)idx >= total)
        return;
    const int P = MODE == MODE_FWD ? d.OH * d.OW : d.H * d.W, PW = MODE == MODE_FWD ? d.OW : d.W;
    const int M = MODE == MODE_FWD ? d.OC : d.IC;
    const uint32_t t = idx / (uint32_t)P;
    const int p = (int)(idx - t * (uint32_t)P);
    const int64_t n = t / (uint32_t)M;
    const int ch = (int)(t - (uint32_t)n * (uint32_t)M);
    float v = C[(n * P + p) * M + ch];
    if (guard_suspect(v, guard_tiny(guard)))
    {
        const int ph = p / PW, pw = p - ph * PW;
        v = MODE == MODE_FWD ? conv2d_exact(Xg, Wt, d, (int)n, ch, ph, pw) : conv2d_grad_input_exact(Xg, Wt, d, (int)n, ch, ph, pw);
    }
    Out[idx] = MODE == MODE_FWD ? with_bias(v, d, ch) : v;
}

// Small images, many channels, one group, the matrix path on: see above.  (Measured at batch 64:
// 512 -> 512 3x3 at 7x7 0.51 -> 0.29 ms, 512 -> 2048 1x1 0.19 -> 0.13; at 14x14 the implicit GEMM
// is the faster one, 0.29 against 0.34 ms for 256 -> 256 3x3.)
inline bool conv_prefers_mm(const ConvDims &d, int64_t M, int64_t K, int64_t P)
{

    return d.groups == 1 && P <= 100 && K >= 512 && M >= 128 && (int64_t)d.N * P >= 2048 && (int64_t)d.N * P * K < (1LL << 31) &&
           (int64_t)d.N * P * M < (1LL << 31) && M * K < (1LL << 31) && repdl_mfma_exact();
}

template <int MODE>
int launch_conv_mm(const float *gathered, const float *kernel, float *out, const ConvDims &d, void *stream)
{
    const int KHW = d.KH * d.KW;
    const int64_t M = MODE == MODE_FWD ? d.OC : d.IC;
    const int64_t K = (int64_t)(MODE == MODE_FWD ? d.IC : d.OC) * KHW;
    const int64_t P = MODE == MODE_FWD ? (int64_t)d.OH * d.OW : (int64_t)d.H * d.W;
    const int64_t rows = (int64_t)d.N * P;
    hipStream_t s = repdl_stream(stream);
    repdl_route_note(REPDL_ROUTE_CONV_IM2COL);
    const bool skips = MODE == MODE_FWD ? (d.pH > 0 || d.pW > 0) : (KHW > 1 || d.sH > 1 || d.sW > 1 || d.pH > 0 || d.pW > 0);
    const size_t col_bytes = ((size_t)(rows * K) * sizeof(float) + 255) / 256 * 256;
    const size_t c_bytes = ((size_t)(rows * M) * sizeof(float) + 255) / 256 * 256;
    const size_t wt_bytes = MODE == MODE_FWD ? 0 : ((size_t)(M * K) * sizeof(float) + 255) / 256 * 256;
    char *ws = nullptr;
    hipError_t e = repdl_ws_acquire(reinterpret_cast<void **>(&ws), GUARD_BYTES + col_bytes + c_bytes + wt_bytes, s);
    if (e != hipSuccess)
        return (int)e;
    unsigned *guard = reinterpret_cast<unsigned *>(ws);
    float *col = reinterpret_cast<float *>(ws + GUARD_BYTES);
    float *C = reinterpret_cast<float *>(ws + GUARD_BYTES + col_bytes);
    float *WT = reinterpret_cast<float *>(ws + GUARD_BYTES + col_bytes + c_bytes);
    if (skips)
    {
        int ca = 0, cb = 0;
        const int64_t gathered_count = (int64_t)d.N * (MODE == MODE_FWD ? (int64_t)d.IC * d.H * d.W : (int64_t)d.OC * d.OH * d.OW);
        launch_guard_scan(gathered, gathered_count, kernel, (int64_t)d.OC * d.IC * KHW, guard, s, ca, cb);
        launch_guard_final(guard, ca, cb, s);
    }
    REPDL_LAUNCH((conv_col_kernel<MODE>), dim3((unsigned)repdl_cdiv(rows * K, 256)), dim3(256), 0, s, gathered, col,
                       rows * K, d, (int)K);
    if (MODE == MODE_DGRAD)
        REPDL_LAUNCH(conv_wt_kernel, dim3((unsigned)repdl_cdiv(M * K, 256)), dim3(256), 0, s, kernel, WT, M * K, d.IC, KHW,
                           (int)K);
    int rc = repdl_launch_status();
    if (rc == REPDL_OK)
        rc = repdl_hip_mm(col, MODE == MODE_FWD ? kernel : WT, C, rows, M, K, 0, 1, stream);
    if (rc == REPDL_OK)
    {
        const int64_t total = rows * M;
        REPDL_LAUNCH((conv_mm_out_kernel<MODE>), dim3((unsigned)repdl_cdiv(total, 256)), dim3(256), 0, s, C, gathered, kernel,
                           out, d, total, skips ? guard : static_cast<const unsigned *>(nullptr));
        rc = repdl_launch_status();
    }
    e = repdl_ws_release(ws, s);
    return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
}
} // namespace

REPDL_API int repdl_hip_conv2d(const float *input, const float *kernel, float *output, int64_t N,
                               int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW,
                               int64_t sH, int64_t sW, int64_t pH, int64_t pW, int64_t groups,
                               void *stream)
{
    return repdl_hip_conv2d_bias(input, kernel, nullptr, output, N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, groups, stream);
}

REPDL_API int repdl_hip_conv2d_bias(const float *input, const float *kernel, const float *bias, float *output,
                                    int64_t N, int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH,
                                    int64_t KW, int64_t sH, int64_t sW, int64_t pH, int64_t pW, int64_t groups,
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
    REPDL_REQUIRE(fits_i32(OH * sH + KH + pH) && fits_i32(OW * sW + KW + pW));
    ConvDims d{(int)N, (int)IC, (int)H, (int)W, (int)OC, (int)KH, (int)KW, (int)OH,
               (int)OW, (int)sH, (int)sW, (int)pH, (int)pW, (int)groups, bias};
    // (A 1x1 kernel at a stride gains nothing from a gathered input here, unlike its two gradients: the
    // implicit product below reads only the positions it needs; 64 -> 128 at 56x56, stride 2: 0.028 ms both ways.)
    // (3x3 kernels at stride 1 have a kernel of their own that is faster than the product also on small
    // images: 512 -> 512 at 7x7, batch 64, 0.26 -> 0.19 ms; at 10x10 0.48 -> 0.34)
    const bool tap = repdl_mfma_exact() && tapdma::applies<MODE_FWD>(d, input, kernel, 64, 1);
    if (!tap && conv_prefers_mm(d, OC, IC * KH * KW, OH * OW))
        return launch_conv_mm<MODE_FWD>(input, kernel, output, d, stream);
    return launch_conv_gemm<MODE_FWD>(input, kernel, output, d, stream);
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
    REPDL_REQUIRE(fits_i32(H + pH + KH) && fits_i32(W + pW + KW) && fits_i32(IC * KH * KW * 4));
    // A 1x1 kernel at a stride, no padding: the positions it reads take the grad-input of the same layer
    // at stride 1 (same chains, same order), every other position an empty chain, +0.  (64 -> 128 at 56x56,
    // stride 2, batch 64: 0.108 -> 0.059 ms; 256 -> 512 at 56x56: 0.65 -> 0.27.)
    if (KH == 1 && KW == 1 && (sH > 1 || sW > 1) && pH == 0 && pW == 0 && OC * OH * OW > 0 &&
        (OH - 1) * sH < H && (OW - 1) * sW < W && repdl_cdiv(total, 256) <= REPDL_I32_MAX)
    {
        hipStream_t s = repdl_stream(stream);
        repdl_route_note(REPDL_ROUTE_DGRAD_POINT_SCATTER);
        const int64_t count = N * IC * OH * OW;
        float *gs = nullptr;
        hipError_t e = repdl_ws_acquire(reinterpret_cast<void **>(&gs), (size_t)count * sizeof(float), s);
        if (e != hipSuccess)
            return (int)e;
        int rc = repdl_hip_conv2d_grad_input(grad_output, kernel, gs, N, OC, OH, OW, IC, 1, 1, OH, OW, 1, 1, 0, 0, stream);
        if (rc == REPDL_OK)
        {
            if (total < (1LL << 31))
                REPDL_LAUNCH(conv_upsample_kernel<uint32_t>, dim3((unsigned)repdl_cdiv(total, 256)), dim3(256), 0, s, gs, grad_input,
                                   total, (int)H, (int)W, (int)OH, (int)OW, (int)sH, (int)sW);
            else
                REPDL_LAUNCH(conv_upsample_kernel<int64_t>, dim3((unsigned)repdl_cdiv(total, 256)), dim3(256), 0, s, gs, grad_input,
                                   total, (int)H, (int)W, (int)OH, (int)OW, (int)sH, (int)sW);
            rc = repdl_launch_status();
        }
        e = repdl_ws_release(gs, s);
        return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
    }
    // Strides, and enough work to pay for a dozen launches (3 GFLOP of products that count): residue by residue,
    // see conv_phase_taps_kernel.  Batch 64, 3x3 at stride 2, before -> after: 64 -> 128 at 56x56 0.366 -> 0.275 ms,
    // 128 -> 256 at 28x28 0.377 -> 0.392, 256 -> 512 at 14x14 0.52 -> 0.35, 512 -> 1024 at 14x14 1.45 -> 0.87; the 7x7
    // stem 3 -> 64 at 224x224 11.2 -> 3.3; batch 16 of the first layer (1.8 GFLOP) 0.148 -> 0.176: not taken there.
    if ((sH > 1 || sW > 1) && OC * OH * OW > 0 && sH <= 8 && sW <= 8 && fits_i32(OC * IC * KH * KW) &&
        repdl_cdiv(N * IC * ((H - 1 + pH) / sH + 1) * ((W - 1 + pW) / sW + 1), 256) <= REPDL_I32_MAX &&
        2.0 * (double)total * (double)(OC * KH * KW) / (double)(sH * sW) >= 3e9)
    {
        hipStream_t s = repdl_stream(stream);
        repdl_route_note(REPDL_ROUTE_DGRAD_RESIDUES);
        const int64_t HPmax = (H - 1 + pH) / sH + 1, WPmax = (W - 1 + pW) / sW + 1;
        const int64_t Amax = (KH + sH - 1) / sH, Bmax = (KW + sW - 1) / sW;
        const size_t ws_k = ((size_t)(OC * IC * Amax * Bmax) * sizeof(float) + 255) / 256 * 256;
        const size_t ws_g = (size_t)(N * IC * HPmax * WPmax) * sizeof(float);
        char *ws = nullptr;
        hipError_t e = repdl_ws_acquire(reinterpret_cast<void **>(&ws), ws_k + ws_g, s);
        if (e != hipSuccess)
            return (int)e;
        float *Ws = reinterpret_cast<float *>(ws), *Gp = reinterpret_cast<float *>(ws + ws_k);
        int rc = REPDL_OK;
        for (int64_t rh = 0; rh < sH && rc == REPDL_OK; rh++)
            for (int64_t rw = 0; rw < sW && rc == REPDL_OK; rw++)
            {
                // h = sH * h' + rh - pH for h' = 0 .. HP - 1 (the first of them may lie above the image)
                if (H - 1 + pH - rh < 0 || W - 1 + pW - rw < 0)
                    continue; // no position of this residue
                const int64_t HP = (H - 1 + pH - rh) / sH + 1, WP = (W - 1 + pW - rw) / sW + 1;
                const int64_t A = rh < KH ? (KH - rh + sH - 1) / sH : 0, B = rw < KW ? (KW - rw + sW - 1) / sW : 0;
                const int64_t count = N * IC * HP * WP;
                const float *src = nullptr;
                if (A > 0 && B > 0)
                {
                    const int64_t kt = OC * IC * A * B;
                    REPDL_LAUNCH(conv_phase_taps_kernel, dim3((unsigned)repdl_cdiv(kt, 256)), dim3(256), 0, s, kernel, Ws, (int)kt,
                                       (int)KH, (int)KW, (int)A, (int)B, (int)rh, (int)rw, (int)sH, (int)sW);
                    rc = repdl_launch_status();
                    if (rc == REPDL_OK)
                        rc = repdl_hip_conv2d_grad_input(grad_output, Ws, Gp, N, OC, OH, OW, IC, A, B, HP, WP, 1, 1, 0, 0, stream);
                    src = Gp;
                }
                if (rc == REPDL_OK)
                {
                    REPDL_LAUNCH(conv_phase_scatter_kernel, dim3((unsigned)repdl_cdiv(count, 256)), dim3(256), 0, s, src, grad_input,
                                       count, (int)HP, (int)WP, (int)H, (int)W, (int)sH, (int)sW, (int)(rh - pH), (int)(rw - pW));
                    rc = repdl_launch_status();
                }
            }
        e = repdl_ws_release(ws, s);
        return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
    }
    ConvDims d{(int)N, (int)IC, (int)H, (int)W, (int)OC, (int)KH, (int)KW, (int)OH,
               (int)OW, (int)sH, (int)sW, (int)pH, (int)pW, 1};
    const bool tap = repdl_mfma_exact() && OC * OH * OW > 0 && tapdma::applies<MODE_DGRAD>(d, grad_output, kernel, 64, 1);
    if (!tap && OC * OH * OW > 0 && conv_prefers_mm(d, IC, OC * KH * KW, H * W))
        return launch_conv_mm<MODE_DGRAD>(grad_output, kernel, grad_input, d, stream);
    return launch_conv_gemm<MODE_DGRAD>(grad_output, kernel, grad_input, d, stream);
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
    ConvDims d{(int)N, (int)IC, (int)H, (int)W, (int)OC, (int)KH, (int)KW, (int)OH,
               (int)OW, (int)sH, (int)sW, (int)pH, (int)pW, 1};
    hipStream_t s = repdl_stream(stream);

    // A 1x1 kernel at a stride, no padding: the input positions it reads, gathered, are the input of the
    // same layer at stride 1 -- same chains, same order, nothing skipped.  (The chain kernel on the
    // strided rows took 47 clocks per step: 64 -> 128 at 56x56, batch 64, 0.99 ms; gathered 0.2x.)
    if (KH == 1 && KW == 1 && (sH > 1 || sW > 1) && pH == 0 && pW == 0 && N * IC * OH * OW > 0 &&
        (OH - 1) * sH < H && (OW - 1) * sW < W && repdl_cdiv(N * IC * OH * OW, 256) <= REPDL_I32_MAX)
    {
        const int64_t count = N * IC * OH * OW;
        repdl_route_note(REPDL_ROUTE_WGRAD_POINT_GATHER);
        float *xs = nullptr;
        hipError_t e = repdl_ws_acquire(reinterpret_cast<void **>(&xs), (size_t)count * sizeof(float), s);
        if (e != hipSuccess)
            return (int)e;
        if (N * IC * H * W < (1LL << 31))
            REPDL_LAUNCH(conv_subsample_kernel<uint32_t>, dim3((unsigned)repdl_cdiv(count, 256)), dim3(256), 0, s, input, xs, count,
                               (int)H, (int)W, (int)OH, (int)OW, (int)sH, (int)sW);
        else
            REPDL_LAUNCH(conv_subsample_kernel<int64_t>, dim3((unsigned)repdl_cdiv(count, 256)), dim3(256), 0, s, input, xs, count,
                               (int)H, (int)W, (int)OH, (int)OW, (int)sH, (int)sW);
        int rc = repdl_launch_status();
        if (rc == REPDL_OK)
            rc = repdl_hip_conv2d_grad_kernel(grad_output, xs, grad_kernel, N, IC, OH, OW, OC, OH, OW, 1, 1, 1, 1, 0, 0, stream);
        e = repdl_ws_release(xs, s);
        return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
    }

    // Many short chains: one matrix product (see wgrad_col_kernel).
    {
        const int64_t NC = IC * KH * KW, K = N * OH * OW;
        if (repdl_mfma_exact() && K > 0 && fits_i32(K) && fits_i32(NC) && K * NC < (1LL << 31) && K * OC < (1LL << 31) &&
            wgrad_prefers_gemm(OC, NC, K, sW, OW, KH * KW))
        {
            const bool skips = pH > 0 || pW > 0;
            repdl_route_note(REPDL_ROUTE_WGRAD_PRODUCT);
            const size_t got_bytes = ((size_t)(K * OC) * sizeof(float) + 255) / 256 * 256;
            const size_t col_bytes = (size_t)(K * NC) * sizeof(float);
            char *ws = nullptr;
            hipError_t e = repdl_ws_acquire(reinterpret_cast<void **>(&ws), GUARD_BYTES + got_bytes + col_bytes, s);
            if (e != hipSuccess)
                return (int)e;
            unsigned *guard = reinterpret_cast<unsigned *>(ws);
            float *GOt = reinterpret_cast<float *>(ws + GUARD_BYTES);
            float *col = reinterpret_cast<float *>(ws + GUARD_BYTES + got_bytes);
            if (skips)
            {
                int ca = 0, cb = 0;
                launch_guard_scan(grad_output, N * OC * OH * OW, input, N * IC * H * W, guard, s, ca, cb);
                launch_guard_final(guard, ca, cb, s);
            }
            REPDL_LAUNCH(wgrad_got_kernel, dim3((unsigned)repdl_cdiv(K * OC, 256)), dim3(256), 0, s, grad_output, GOt,
                               K * OC, (int)OC, (int)(OH * OW));
            REPDL_LAUNCH(wgrad_col_kernel, dim3((unsigned)repdl_cdiv(K * NC, 256)), dim3(256), 0, s, input, col, K * NC,
                               d, (int)NC);
            int rc = repdl_launch_status();
            if (rc == REPDL_OK)
                rc = repdl_hip_mm(GOt, col, grad_kernel, OC, NC, K, 1, 0, stream);
            if (rc == REPDL_OK && skips)
            {
                REPDL_LAUNCH(wgrad_fixup_kernel, dim3((unsigned)repdl_cdiv(total, 256)), dim3(256), 0, s, grad_output,
                                   input, grad_kernel, d, total, guard);
                rc = repdl_launch_status();
            }
            e = repdl_ws_release(ws, s);
            return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
        }
    }

    // Matrix-instruction kernel: geometry of a chunk (see conv_wgrad_mfma_kernel).
    if (repdl_mfma_exact() && sW <= 16 && aligned16(grad_output) && aligned16(input) && OW > 0)
    {
        const int64_t KHW = KH * KW, NC = IC * KHW;
        // instructions per piece: the largest candidate that divides a row of OWr / 4 instructions
        // (OWr: the output width, rounded up to a multiple of 4 in a zero-padded copy of grad_output)
        const int64_t OWr = (OW + 3) / 4 * 4;
        const bool gpad = OWr != OW;
        const int64_t nqr = OWr / 4;
        int64_t QP = 0, NP = 0;
        for (int64_t qp : {16, 14, 7, 4, 2, 1})
            if (QP == 0 && nqr % qp == 0)
            {
                QP = qp;
                NP = nqr / qp;
            }
        const int64_t OWp = 4 * QP * NP;
        int64_t Wp = pW + (W + 3) / 4 * 4;
        const int64_t reach = (OWp - 1) * sW + KW; // the taps of the padded steps must be staged zeros
        if (reach > Wp)
            Wp = reach;
        // A 1x1 kernel without padding: the 16 columns of a block are 16 channels, and lane l reads word
        // CP * (l % 16) + l / 16 of the staged input -- every bank once with CP = 4 mod 32, like
        // grad_output -- so the rows can sit on 16-byte boundaries and be stored four words at a time
        // (the staging waves set the pace of these layers: 256 -> 64 at 56x56, batch 64, 0.97 -> ... ms).
        const bool xv = KHW == 1 && pW == 0 && sW == 1;
        while (xv ? Wp % 4 != 0 : Wp % 32 != KW % 32)
            Wp++;
        const int64_t span = (15 + KHW - 1) / KHW + 1; // channels a 16-column block can span
        const int64_t nic_max = span < IC ? span : IC;
        const int64_t nw4 = (W + 3) / 4;
        // grad_output slots per staging thread: 32 let a chunk of a 3x3 layer at stride 1 be twice as long
        // (64 -> 64 at 56x56, batch 64: 0.955 -> 0.90 ms); where the input slots or LDS set the length
        // of a chunk anyway, 16 (twice the slots repeat the loads and stores: 1x1, 0.97 -> 1.44 ms)
        const int64_t gs_max = sW == 1 && !xv ? MW_GS : 16;
        int64_t R = 0, hrows = 0, GP = 0, CP = 0;
        for (int64_t r = OH; r >= 1 && QP > 0; r--)
        {
            if (OH % r != 0)
                continue; // whole chunks only
            const int64_t hr = (r - 1) * sH + KH;
            int64_t gp = r * OWp;
            while (gp % 32 != 4)
                gp++;
            int64_t cp = hr * Wp;
            while (cp % 32 != (xv ? 4 : KHW % 32))
                cp++;
            if (MW_OC * r * OWp <= 4 * MW_ST * gs_max && nic_max * hr * nw4 <= MW_ST * MW_XS &&
                2 * (64 + MW_OC * gp + nic_max * cp + sH * Wp + 64 + 3) * 4 <= 150 * 1024)
            {
                R = r;
                hrows = hr;
                GP = gp;
                CP = cp;
                break;
            }
        }
        const int64_t xW = (W + 3) / 4 * 4; // input row pitch the staging waves read
        const bool xpad = xW != W;
        if (R > 0 && N * (OH / R) <= REPDL_I32_MAX && fits_i32(IC * H * xW) && fits_i32(OC * OH * OWp * 4) &&
            fits_i32(repdl_cdiv(NC, 16)) &&
            repdl_cdiv(OC, MW_OC) <= 65535)
        {
            repdl_route_note(REPDL_ROUTE_WGRAD_CHAIN);
            // workspace: the guard words, then the operands with rows rounded up to whole
            // instructions (grad_output) / whole float4 (input), when they are not
            const size_t xbytes = xpad ? ((size_t)(N * IC * H * xW) * sizeof(float) + 255) / 256 * 256 : 0;
            const size_t gbytes = gpad ? (size_t)(N * OC * OH * OWp) * sizeof(float) : 0;
            char *ws = nullptr;
            hipError_t e = repdl_ws_acquire(reinterpret_cast<void **>(&ws), GUARD_BYTES + xbytes + gbytes, s);
            if (e != hipSuccess)
                return (int)e;
            unsigned *guard = reinterpret_cast<unsigned *>(ws);
            float *xws = reinterpret_cast<float *>(ws + GUARD_BYTES);
            float *gws = reinterpret_cast<float *>(ws + GUARD_BYTES + xbytes);
            // the reference skips taps only into the padding; rows rounded up add zero steps
            const bool skips = pH > 0 || pW > 0 || gpad;
            int ca = 0, cb = 0;
            if (skips)
                launch_guard_scan(gpad ? nullptr : grad_output, N * OC * OH * OW, xpad ? nullptr : input, N * IC * H * W, guard,
                                  s, ca, cb);
            if (xpad)
            {
                cb = (int)pad_blocks(N * IC);
                REPDL_LAUNCH(conv_pad_kernel, dim3((unsigned)cb), dim3(256), 0, s, input, xws, N * IC, (int)H, (int)W,
                                   (int)H, (int)xW, 0, 0, 1, 1, guard_parts(guard, 1));
            }
            const float *xsrc = xpad ? xws : input;
            if (gpad)
            {
                ca = (int)pad_blocks(N * OC);
                REPDL_LAUNCH(conv_pad_kernel, dim3((unsigned)ca), dim3(256), 0, s, grad_output, gws, N * OC, (int)OH,
                                   (int)OW, (int)OH, (int)OWp, 0, 0, 1, 1, guard_parts(guard, 0));
            }
            if (skips)
                launch_guard_final(guard, ca, cb, s);
            else
                guard = nullptr;
            const float *gsrc = gpad ? gws : grad_output;
            const int64_t xoff = 64 + MW_OC * GP; // 64 zero words, then the grad_output rows, then the input rows
            // (+ a row of slack: the read behind the last piece of a chunk overshoots by one staged row)
            const int64_t bufsz = (xoff + nic_max * CP + sH * Wp + 64 + 3) / 4 * 4; // multiple of 4: float4 stores
            const int64_t gx = repdl_cdiv(NC, 16), gy = repdl_cdiv(OC, MW_OC);
            size_t shmem = (size_t)(2 * bufsz * 4);
            if (shmem < 84 * 1024)
                shmem = 84 * 1024; // one workgroup per CU: every wave has a SIMD to itself
            const bool few = nic_max * hrows * nw4 <= 2 * MW_ST; // input slots per staging thread: 2 or MW_XS
            const bool wide = MW_OC * R * OWp > 4 * MW_ST * 16;  // grad_output slots per staging thread: MW_GS or 16
#define REPDL_WGRAD_MFMA(Q, U, X, G, V)                                                                                 \
    do                                                                                                              \
    {                                                                                                               \
        hipError_t e_ = REPDL_FUNC_SET_ATTRIBUTE(reinterpret_cast<const void *>(&conv_wgrad_mfma_kernel<Q, U, X, G, V>),       \
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);                \
        if (e_ != hipSuccess)                                                                                       \
        {                                                                                                           \
            (void)repdl_ws_release(ws, s);                                                                              \
            return (int)e_;                                                                                         \
        }                                                                                                           \
        REPDL_LAUNCH((conv_wgrad_mfma_kernel<Q, U, X, G, V>), dim3((unsigned)gx, (unsigned)gy), dim3(256), shmem, s, \
                           gsrc, xsrc, grad_output, input, grad_kernel, d, (int)R, (int)NP, (int)GP, (int)Wp,       \
                           (int)CP, (int)hrows, (int)xoff, (int)bufsz, (int)xW, guard);                             \
    } while (0)
#define REPDL_WGRAD_MFMA_Q(Q)                     \
    do                                            \
    {                                             \
        if (xv && few)                                  \
            REPDL_WGRAD_MFMA(Q, 1, 2, 16, true);            \
        else if (xv)                                    \
            REPDL_WGRAD_MFMA(Q, 1, MW_XS, 16, true);        \
        else if (sW == 1 && few && wide)                \
            REPDL_WGRAD_MFMA(Q, 1, 2, MW_GS, false);        \
        else if (sW == 1 && wide)                       \
            REPDL_WGRAD_MFMA(Q, 1, MW_XS, MW_GS, false);    \
        else if (sW == 1 && few)                        \
            REPDL_WGRAD_MFMA(Q, 1, 2, 16, false);           \
        else if (sW == 1)                               \
            REPDL_WGRAD_MFMA(Q, 1, MW_XS, 16, false);       \
        else if (sW == 2 && few)                        \
            REPDL_WGRAD_MFMA(Q, 2, 2, 16, false);           \
        else if (sW == 2)                               \
            REPDL_WGRAD_MFMA(Q, 2, MW_XS, 16, false);       \
        else if (few)                                   \
            REPDL_WGRAD_MFMA(Q, 0, 2, 16, false);           \
        else                                            \
            REPDL_WGRAD_MFMA(Q, 0, MW_XS, 16, false);       \
    } while (0)
            if (QP == 16)
                REPDL_WGRAD_MFMA_Q(16);
            else if (QP == 14)
                REPDL_WGRAD_MFMA_Q(14);
            else if (QP == 7)
                REPDL_WGRAD_MFMA_Q(7);
            else if (QP == 4)
                REPDL_WGRAD_MFMA_Q(4);
            else if (QP == 2)
                REPDL_WGRAD_MFMA_Q(2);
            else
                REPDL_WGRAD_MFMA_Q(1);
#undef REPDL_WGRAD_MFMA_Q
#undef REPDL_WGRAD_MFMA
            const int rc = repdl_launch_status();
            e = repdl_ws_release(ws, s);
            return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
        }
    }

    // Geometry.  A row of OW outputs is cut into NP pieces of PIECE (16/32/64) steps;
    // steps past the end of the row must read zeros, so the staged row pitch Wp covers
    // what is written (pW + roundup4(W)) and what the taps of NP*PIECE steps reach.
    // Lane l of a wave reads LDS word (ic-ic0)*CP + kh*Wp + kw (+ a wave-uniform offset);
    // with Wp = KW and CP = KH*KW modulo 32 that is l + const modulo 32: two lanes per
    // bank, the minimum for 64 lanes.
    const int64_t KHW = KH * KW, NC = IC * KHW;
    const int piece = OW <= 16 ? 16 : OW <= 32 ? 32 : 64;
    const int64_t NP = repdl_cdiv(OW, piece);
    int64_t Wp = pW + (W + 3) / 4 * 4;
    const int64_t reach = (NP * piece - 1) * sW + KW;
    if (reach > Wp)
        Wp = reach;
    while (Wp % 32 != KW % 32)
        Wp++;
    const int64_t span = (63 + KHW - 1) / KHW + 1; // channels a 64-column block can span
    const int64_t nic_max = span < IC ? span : IC;
    const int64_t nseg = (W + 63) / 64;
    // largest R (output rows per chunk) that fits WG_Q pieces, WG_SLOTS staging slots per
    // thread and 150 KiB of LDS
    int64_t R = 0, hrows = 0;
    for (int64_t r = (OH < WG_Q ? OH : WG_Q); r >= 1; r--)
    {
        const int64_t hr = (r - 1) * sH + KH;
        const int64_t slots = repdl_cdiv(nic_max * hr, 16) * nseg;
        if (r * NP <= WG_Q && slots <= WG_SLOTS && 2 * nic_max * (hr * Wp + 31) * 4 <= 150 * 1024)
        {
            R = r;
            hrows = hr;
            break;
        }
    }
    int64_t CP = hrows * Wp; // channel pitch
    while (CP % 32 != KHW % 32)
        CP++;
    const int64_t bufsz = nic_max * CP;
    const int xvec = aligned16(input) && (W % 4 == 0);
    const int64_t gx = repdl_cdiv(NC, 64), gy = repdl_cdiv(OC, 4);
    REPDL_REQUIRE(fits_i32(gx) && gy <= 65535);
    const dim3 grid((unsigned)gx, (unsigned)gy);
    repdl_route_note(REPDL_ROUTE_WGRAD_FMA);
    unsigned *guard = nullptr;
    hipError_t ge = repdl_ws_acquire(reinterpret_cast<void **>(&guard), GUARD_BYTES, s);
    if (ge != hipSuccess)
        return (int)ge;
    int ca = 0, cb = 0;
    launch_guard_scan(grad_output, N * OC * OH * OW, input, N * IC * H * W, guard, s, ca, cb);
    launch_guard_final(guard, ca, cb, s);
    // More than half of a CU's 160 KiB of LDS: one workgroup per CU, so that each of its
    // four waves has a SIMD to itself (the chains are latency-bound, not throughput-bound).
    size_t shmem = (size_t)(2 * bufsz * 4);
    if (shmem < 84 * 1024)
        shmem = 84 * 1024;
#define REPDL_WGRAD(P)                                                                                          \
    do                                                                                                         \
    {                                                                                                          \
        hipError_t e_ = REPDL_FUNC_SET_ATTRIBUTE(reinterpret_cast<const void *>(&conv_wgrad_kernel<P>),             \
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);           \
        if (e_ != hipSuccess)                                                                                  \
        {                                                                                                      \
            (void)repdl_ws_release(guard, s);                                                                      \
            return (int)e_;                                                                                    \
        }                                                                                                      \
        REPDL_LAUNCH((conv_wgrad_kernel<P>), grid, dim3(256), shmem, s, grad_output, input, grad_kernel, \
                           d, (int)R, (int)NP, (int)Wp, (int)CP, (int)hrows, (int)bufsz, xvec, guard);         \
    } while (0)
    if (piece == 16)
        REPDL_WGRAD(16);
    else if (piece == 32)
        REPDL_WGRAD(32);
    else
        REPDL_WGRAD(64);
#undef REPDL_WGRAD
    const int rc = repdl_launch_status();
    ge = repdl_ws_release(guard, s);
    return rc != REPDL_OK ? rc : (ge == hipSuccess ? REPDL_OK : (int)ge);
}

// ---------------------------------------------------------------------------------------------
// The three convolutions with the caller's workspace.  The *_ws entry point installs the buffer
// and runs the plain one under it (every scratch request of the call, nested calls included, is a
// piece of that buffer); the size query runs the same host logic with the launches switched off,
// so the two cannot disagree about the route.  Operand pointers not given to a query are tried on
// and off a 16-byte boundary, the matrix path both ways; the largest need counts.
// ---------------------------------------------------------------------------------------------
namespace
{
template <typename F>
size_t conv_ws_query(const float *a, const float *b, F call)
{
    size_t need = 0;
    for (int ia = 0; ia < 2; ia++)
        for (int ib = 0; ib < 2; ib++)
        {
            if ((a != nullptr && ia == 1) || (b != nullptr && ib == 1))
                continue;
            const float *pa = a != nullptr ? a : repdl_ws_fake_pointer(ia == 0);
            const float *pb = b != nullptr ? b : repdl_ws_fake_pointer(ib == 0);
            const size_t n = repdl_ws_query([&]() { return call(pa, pb); });
            need = n > need ? n : need;
        }
    return need;
}
float *conv_ws_fake_output() { return const_cast<float *>(repdl_ws_fake_pointer(true)); }
} // namespace

REPDL_API size_t repdl_hip_conv2d_workspace_bytes(const float *input, const float *kernel, int64_t N, int64_t IC, int64_t H,
                                                  int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t sH, int64_t sW,
                                                  int64_t pH, int64_t pW, int64_t groups)
{
    return conv_ws_query(input, kernel, [&](const float *x, const float *k) {
        return repdl_hip_conv2d_bias(x, k, nullptr, conv_ws_fake_output(), N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, groups, nullptr);
    });
}

REPDL_API int repdl_hip_conv2d_ws(const float *input, const float *kernel, const float *bias, float *output, int64_t N,
                                  int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t sH,
                                  int64_t sW, int64_t pH, int64_t pW, int64_t groups, void *workspace,
                                  size_t workspace_bytes, void *stream)
{
    RepdlWorkspace ws(workspace, workspace_bytes);
    return repdl_hip_conv2d_bias(input, kernel, bias, output, N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, groups, stream);
}

REPDL_API size_t repdl_hip_conv2d_grad_input_workspace_bytes(const float *grad_output, const float *kernel, int64_t N,
                                                             int64_t OC, int64_t OH, int64_t OW, int64_t IC, int64_t KH,
                                                             int64_t KW, int64_t H, int64_t W, int64_t sH, int64_t sW,
                                                             int64_t pH, int64_t pW)
{
    return conv_ws_query(grad_output, kernel, [&](const float *g, const float *k) {
        return repdl_hip_conv2d_grad_input(g, k, conv_ws_fake_output(), N, OC, OH, OW, IC, KH, KW, H, W, sH, sW, pH, pW, nullptr);
    });
}

REPDL_API int repdl_hip_conv2d_grad_input_ws(const float *grad_output, const float *kernel, float *grad_input, int64_t N,
                                             int64_t OC, int64_t OH, int64_t OW, int64_t IC, int64_t KH, int64_t KW,
                                             int64_t H, int64_t W, int64_t sH, int64_t sW, int64_t pH, int64_t pW,
                                             void *workspace, size_t workspace_bytes, void *stream)
{
    RepdlWorkspace ws(workspace, workspace_bytes);
    return repdl_hip_conv2d_grad_input(grad_output, kernel, grad_input, N, OC, OH, OW, IC, KH, KW, H, W, sH, sW, pH, pW, stream);
}

REPDL_API size_t repdl_hip_conv2d_grad_kernel_workspace_bytes(const float *grad_output, const float *input, int64_t N,
                                                              int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t OH,
                                                              int64_t OW, int64_t KH, int64_t KW, int64_t sH, int64_t sW,
                                                              int64_t pH, int64_t pW)
{
    return conv_ws_query(grad_output, input, [&](const float *g, const float *x) {
        return repdl_hip_conv2d_grad_kernel(g, x, conv_ws_fake_output(), N, IC, H, W, OC, OH, OW, KH, KW, sH, sW, pH, pW, nullptr);
    });
}

REPDL_API int repdl_hip_conv2d_grad_kernel_ws(const float *grad_output, const float *input, float *grad_kernel, int64_t N,
                                              int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t OH, int64_t OW,
                                              int64_t KH, int64_t KW, int64_t sH, int64_t sW, int64_t pH, int64_t pW,
                                              void *workspace, size_t workspace_bytes, void *stream)
{
    RepdlWorkspace ws(workspace, workspace_bytes);
    return repdl_hip_conv2d_grad_kernel(grad_output, input, grad_kernel, N, IC, H, W, OC, OH, OW, KH, KW, sH, sW, pH, pW, stream);
}
