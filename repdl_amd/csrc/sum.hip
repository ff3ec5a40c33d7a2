// Sequential-order fp32 sums for gfx950.
//
// Contract (RepDL backend/cpu/summation.cpp:12-78): each output is ONE chain
//   s = +0.0f; for each element in index order: s = s + x   (binary32, RN)
// followed by one multiply by (float)(average ? 1.0/count : 1.0).  The chain is
// inherently serial per output, so parallelism comes only from independent
// outputs (rows, columns, channels); memory is made coalesced by staging tiles
// through LDS and letting one lane walk one chain.
#include "common.h"

namespace
{
// ---------------------------------------------------------------------------
// Row chains: out[r] = chain over j of in[seg(j)] where the elements of chain r
// are `nseg` contiguous segments of `seglen` floats; segment s of chain r starts
// at in + s*seg_stride + r*row_stride.
//   sum2d_dim1  [M,N]:      rows=M, nseg=1, seglen=N,   row_stride=N
//   sum4d_dim023 [N,C,H,W]: rows=C, nseg=N, seglen=H*W, row_stride=H*W, seg_stride=C*H*W
//   sum1d:                  rows=1, nseg=1, seglen=n
// A workgroup of RW waves owns 64 chains.  All waves load TILE_R x TILE_C tiles
// (coalesced along the segment) into LDS; wave 0 then walks the 64 chains, lane
// l adding row l's TILE_C values in order.  Rows are padded by one float so the
// 64 lanes of the walking wave hit 64 different... banks (stride 65 mod 32 = 1).
// ---------------------------------------------------------------------------
constexpr int ROWS = 64;   // chains per workgroup
constexpr int TC = 64;     // tile columns
constexpr int LDT = TC + 1;
constexpr int RT = 256;    // threads per workgroup

__global__ __launch_bounds__(RT) void rowchain_kernel(const float *__restrict__ in,
                                                      float *__restrict__ out, int64_t rows,
                                                      int64_t nseg, int64_t seglen,
                                                      int64_t row_stride, int64_t seg_stride,
                                                      float factor)
{
    __shared__ float tile[2][ROWS * LDT];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int64_t r0 = (int64_t)blockIdx.x * ROWS;
    const int64_t tiles_per_seg = (seglen + TC - 1) / TC;
    const int64_t ntiles = nseg * tiles_per_seg;

    float acc = 0.0f;
    float stage[ROWS / 4];

    auto load = [&](int64_t t) {
        const int64_t s = t / tiles_per_seg, c0 = (t - s * tiles_per_seg) * TC;
        const float *base = in + s * seg_stride + c0;
#pragma unroll
        for (int i = 0; i < ROWS / 4; i++)
        {
            const int64_t r = r0 + wave + 4 * i;
            float v = 0.0f;
            if (r < rows && c0 + lane < seglen)
                v = base[r * row_stride + lane];
            stage[i] = v;
        }
    };
    auto store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < ROWS / 4; i++)
            tile[buf][(wave + 4 * i) * LDT + lane] = stage[i];
    };

    if (ntiles > 0)
    {
        load(0);
        store(0);
    }
    __syncthreads();
    for (int64_t t = 0; t < ntiles; t++)
    {
        const int cur = (int)(t & 1);
        const bool more = t + 1 < ntiles;
        if (more)
            load(t + 1);
        if (wave == 0)
        {
            const int64_t s = t / tiles_per_seg, c0 = (t - s * tiles_per_seg) * TC;
            const int64_t rem = seglen - c0;
            const float *row = &tile[cur][lane * LDT];
            if (rem >= TC)
            {
#pragma unroll
                for (int c = 0; c < TC; c++)
                    acc = acc + row[c];
            }
            else
            {
                for (int c = 0; c < (int)rem; c++)
                    acc = acc + row[c];
            }
        }
        if (more)
            store(cur ^ 1);
        __syncthreads();
    }
    if (wave == 0 && r0 + lane < rows)
        out[r0 + lane] = factor * acc;
}

// ---------------------------------------------------------------------------
// Column chains: out[j] = chain over i of in[i*N + j] (sum2d_dim0).  One lane
// per column, rows consumed in order; loads are issued UNROLL rows ahead.
// ---------------------------------------------------------------------------
constexpr int CU_UNROLL = 16;

__global__ __launch_bounds__(64) void colchain_kernel(const float *__restrict__ in,
                                                      float *__restrict__ out, int64_t M, int64_t N,
                                                      float factor)
{
    const int64_t j = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (j >= N)
        return;
    const float *p = in + j;
    float acc = 0.0f;
    int64_t i = 0;
    for (; i + CU_UNROLL <= M; i += CU_UNROLL)
    {
        float v[CU_UNROLL];
#pragma unroll
        for (int u = 0; u < CU_UNROLL; u++)
            v[u] = p[(i + u) * N];
#pragma unroll
        for (int u = 0; u < CU_UNROLL; u++)
            acc = acc + v[u];
    }
    for (; i < M; i++)
        acc = acc + p[i * N];
    out[j] = factor * acc;
}
} // namespace

static int launch_rowchain(const float *in, float *out, int64_t rows, int64_t nseg, int64_t seglen,
                           int64_t row_stride, int64_t seg_stride, float factor, void *stream)
{
    if (rows == 0)
        return REPDL_OK;
    const int64_t grid = repdl_cdiv(rows, ROWS);
    REPDL_REQUIRE(grid <= REPDL_I32_MAX);
    hipLaunchKernelGGL(rowchain_kernel, dim3((unsigned)grid), dim3(RT), 0, repdl_stream(stream), in, out,
                       rows, nseg, seglen, row_stride, seg_stride, factor);
    return repdl_launch_status();
}

REPDL_API int repdl_hip_sum1d(const float *in, float *out, int64_t n, int average, void *stream)
{
    REPDL_REQUIRE(n >= 0 && out != nullptr && (n == 0 || in != nullptr));
    return launch_rowchain(in, out, 1, 1, n, n, 0, repdl_sum_factor(average, n), stream);
}

REPDL_API int repdl_hip_sum2d_dim1(const float *in, float *out, int64_t M, int64_t N, int average,
                                   void *stream)
{
    REPDL_REQUIRE(M >= 0 && N >= 0 && (M == 0 || out != nullptr) && (M * N == 0 || in != nullptr));
    return launch_rowchain(in, out, M, 1, N, N, 0, repdl_sum_factor(average, N), stream);
}

REPDL_API int repdl_hip_sum4d_dim023(const float *in, float *out, int64_t N, int64_t C, int64_t H,
                                     int64_t W, int average, void *stream)
{
    REPDL_REQUIRE(N >= 0 && C >= 0 && H >= 0 && W >= 0 && (C == 0 || out != nullptr));
    REPDL_REQUIRE(N * C * H * W == 0 || in != nullptr);
    return launch_rowchain(in, out, C, N, H * W, H * W, C * H * W, repdl_sum_factor(average, N * H * W),
                           stream);
}

REPDL_API int repdl_hip_sum2d_dim0(const float *in, float *out, int64_t M, int64_t N, int average,
                                   void *stream)
{
    REPDL_REQUIRE(M >= 0 && N >= 0 && (N == 0 || out != nullptr) && (M * N == 0 || in != nullptr));
    if (N == 0)
        return REPDL_OK;
    const int64_t grid = repdl_cdiv(N, 64);
    REPDL_REQUIRE(grid <= REPDL_I32_MAX);
    hipLaunchKernelGGL(colchain_kernel, dim3((unsigned)grid), dim3(64), 0, repdl_stream(stream), in, out, M,
                       N, repdl_sum_factor(average, M));
    return repdl_launch_status();
}
