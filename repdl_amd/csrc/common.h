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

// Largest extent a kernel indexes with 32-bit arithmetic.
#define REPDL_I32_MAX 2147483647LL

static inline int repdl_launch_status()
{
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? REPDL_OK : (int)e;
}

static inline hipStream_t repdl_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

static inline int64_t repdl_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// True when the binary32 matrix instructions of the current device were checked (or forced,
// see repdl_hip_set_matrix_path) to evaluate k-ascending chains of single-rounding FMAs;
// the GEMM-shaped operators then use them, otherwise their v_fma_f32 kernels.
bool repdl_mfma_exact();

__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }

// (float)(average ? 1.0 / count : 1.0): the factor of the reference's sums and
// means, computed in double on the host and rounded once.
static inline float repdl_sum_factor(int average, int64_t count)
{
    return average ? (float)(1.0 / (double)count) : 1.0f;
}
