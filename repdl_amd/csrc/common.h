// Shared host-side helpers for the gfx950 kernels: argument checks, launch
// checks and the bit casts used by the device code.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/repdl_hip.h"

#define REPDL_API extern "C" __attribute__((visibility("default")))

#define REPDL_REQUIRE(cond)     \
    do                          \
    {                           \
        if (!(cond))            \
            return REPDL_E_ARG; \
    } while (0)

// Inputs at least this long take the parallel evaluation of the sequential sum.
#define REPDL_SUM1D_MIN_PARALLEL 32768

// Row and channel sums take the parallel evaluation when the chains are at least this long and
// at most REPDL_SUM_ROWS_MAX_PARALLEL in number (few long chains are bound by the latency of one
// chain; many chains keep the memory system busy with one lane per chain).
#define REPDL_SUM_ROWS_MIN_PARALLEL 49152
#define REPDL_SUM_ROWS_MAX_PARALLEL 512

// Largest extent a kernel indexes with 32-bit arithmetic.
#define REPDL_I32_MAX 2147483647LL

static inline int repdl_launch_status()
{
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? REPDL_OK : (int)e;
}

static inline hipStream_t repdl_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

static inline int64_t repdl_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Scratch memory for the duration of a call, ordered on stream s (workspace.hip): in place of
// hipMallocAsync / hipFreeAsync, which hold the host until the work in between has run.
hipError_t repdl_ws_acquire(void **p, size_t bytes, hipStream_t s);
hipError_t repdl_ws_release(void *p, hipStream_t s);

// sum1d.hip: the exact parallel evaluation of sequential sums, for `rows` chains at once
// (chain r: nseg segments of seglen contiguous floats, segment s at in + r*row_stride + s*seg_stride;
// nseg > 1 needs seglen % 16 == 0 and nseg*seglen < 2^31); out[r] = factor * sum.
size_t repdl_sum_chains_workspace_bytes(int64_t rows, int64_t n);
int repdl_sum_chains(const float *in, float *out, int64_t rows, int64_t nseg, int64_t seglen, int64_t row_stride,
                     int64_t seg_stride, float factor, void *workspace, size_t workspace_bytes, void *stream);

// True when the binary32 matrix instructions of the current device were checked (or forced,
// see repdl_hip_set_matrix_path) to evaluate k-ascending chains of single-rounding FMAs;
// the GEMM-shaped operators then use them, otherwise their v_fma_f32 kernels.
bool repdl_mfma_exact();

// mm.hip: a batch of `nbatch` products C_b[M][N] = op(A_b)[M][K] . op(B_b)[K][N] on the kernel that moves
// operands from global memory straight into LDS; operand b lies `stride` elements behind operand b-1
// (0: one operand shared by all).  row_bias[M], if not null, is added to every column of C after the
// chains.  REPDL_E_UNSUPPORTED, and nothing launched, where that kernel cannot take the operands
// (rows off 16-byte boundaries, the matrix path switched off).
int repdl_mm_batched(const float *A, const float *B, float *C, const float *row_bias, int64_t M, int64_t N, int64_t K,
                     int transA, int transB, int64_t nbatch, int64_t strideA, int64_t strideB, int64_t strideC,
                     hipStream_t stream);

__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }

// (float)(average ? 1.0 / count : 1.0): the factor of the reference's sums and
// means, computed in double on the host and rounded once.
static inline float repdl_sum_factor(int average, int64_t count)
{
    return average ? (float)(1.0 / (double)count) : 1.0f;
}
