// The matrix-core contract, checked on the device itself.
//
// The GEMM-shaped kernels of this library need, for every output element, one
// accumulator that receives exactly one single-rounding binary32 fused
// multiply-add per k, k ascending (RepDL backend/cpu/matrix_multiplication.cpp:22-34).
// On gfx950 the binary32 matrix instructions v_mfma_f32_32x32x2_f32 and
// v_mfma_f32_16x16x4_f32 do exactly that: D = fma(a_{K-1}, b_{K-1}, ... fma(a_0, b_0, C)),
// with round-to-nearest-even, subnormal operands and results kept, signed zeros
// and infinities as IEEE 754 prescribes.  This is an observed property of the
// silicon, not a documented one, so the library does not assume it: the kernels
// below compare both instructions with __fmaf_rn chains on operands drawn from
// seven classes (ordinary, any finite, products in the subnormal range, short
// significands that produce exact ties, overflow, exact cancellation, and a mix
// of +-0, +-inf, subnormals and extremes).  repdl_hip_init() -- or, failing that, the
// first use of a matrix kernel on a device -- runs a short version of the check on a
// stream of its own; if a single result differs, every GEMM-shaped operator stays on
// its v_fma_f32 kernel, and no setting overrides that.  repdl_hip_mfma_selftest runs a
// check of any length on request.
#include <mutex>

#include "common.h"

namespace
{
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
constexpr int NCLASS = 7;

__device__ __forceinline__ uint64_t mix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

__device__ __forceinline__ float make_f32(uint32_t sign, uint32_t biased_exp, uint32_t man)
{
    return __uint_as_float((sign << 31) | (biased_exp << 23) | (man & 0x7fffffu));
}

// operand of class cls; factor: a multiplicand (true) or the accumulator input (false)
__device__ float operand(uint64_t r, int cls, bool factor)
{
    const uint32_t lo = (uint32_t)r, hi = (uint32_t)(r >> 32), sg = lo >> 31;
    switch (cls)
    {
    case 0: // ordinary magnitudes
        return make_f32(sg, 107 + (hi % 41), lo);
    case 1: // any finite number
        return make_f32(sg, hi % 255, lo);
    case 2: // products at or below the subnormal range, subnormal accumulators
        return factor ? make_f32(sg, 40 + (hi % 50), lo) : make_f32(sg, hi % 12, lo);
    case 3: // short significands: exact products, frequent ties in the sum
        if (factor)
            return make_f32(sg, 120 + (hi % 15), lo & 0x7ff000u);
        return make_f32(sg, 100 + (hi % 60), lo & (((hi >> 8) & 1) ? 0x7fffffu : 0x7ff800u));
    case 4: // overflow region
        return factor ? make_f32(sg, 180 + (hi % 20), lo) : make_f32(sg, 230 + (hi % 25), lo);
    case 5: // accumulator replaced below by -rn(a*b): exact cancellation
        return make_f32(sg, 107 + (hi % 41), lo);
    default: // zeros, infinities, subnormals, extremes, +-1 among ordinary numbers
    {
        const uint32_t sel = (hi >> 4) % 10;
        if (sel < 3)
            return make_f32(sg, 0, 0);
        if (sel == 3)
            return make_f32(sg, 255, 0);
        if (sel == 4)
            return make_f32(sg, 0, lo);
        if (sel == 5)
            return make_f32(sg, 254, lo | 0x7ffff0u);
        if (sel == 6)
            return make_f32(sg, 127, 0);
        return make_f32(sg, 117 + (hi % 21), lo);
    }
    }
}

__device__ __forceinline__ bool same_result(float want, float got)
{
    return __float_as_uint(want) == __float_as_uint(got) || (want != want && got != got);
}

// One wave per workgroup.  counts[0] += mismatches of the 32x32x2 instruction,
// counts[1] += mismatches of the 16x16x4 instruction.
__global__ __launch_bounds__(64) void mfma_check_kernel(unsigned long long *counts, int trials, uint64_t seed)
{
    __shared__ float A[4][32], B[4][32], C[32][33];
    const int l = threadIdx.x;
    unsigned long long bad32 = 0, bad16 = 0;
    for (int t = 0; t < trials; t++)
    {
        const uint64_t trial = (uint64_t)blockIdx.x * (uint64_t)trials + (uint64_t)t;
        const int cls = (int)(trial % NCLASS);
        const uint64_t base = mix64(seed + trial * 0x1000ULL);
        A[l >> 5][l & 31] = operand(mix64(base + l), cls, true);
        A[2 + (l >> 5)][l & 31] = operand(mix64(base + 64 + l), cls, true);
        B[l >> 5][l & 31] = operand(mix64(base + 128 + l), cls, true);
        B[2 + (l >> 5)][l & 31] = operand(mix64(base + 192 + l), cls, true);
        for (int q = 0; q < 16; q++)
        {
            const int idx = q * 64 + l;
            C[idx >> 5][idx & 31] = operand(mix64(base + 256 + idx), cls, false);
        }
        __syncthreads();
        if (cls == 5)
        {
            for (int q = 0; q < 16; q++)
            {
                const int idx = q * 64 + l, i = idx >> 5, j = idx & 31, k = (i + j) & 1;
                C[i][j] = -(A[k][i] * B[k][j]);
            }
            __syncthreads();
        }
        // 32x32x2: lane l holds A[i = l%32][k = l/32] and B[k = l/32][j = l%32]; register r of
        // the result is row 8*(r/4) + 4*(l/32) + r%4, column l%32.
        {
            f16v c;
#pragma unroll
            for (int r = 0; r < 16; r++)
                c[r] = C[8 * (r >> 2) + 4 * (l >> 5) + (r & 3)][l & 31];
            const f16v d = __builtin_amdgcn_mfma_f32_32x32x2f32(A[l >> 5][l & 31], B[l >> 5][l & 31], c, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; r++)
            {
                const int i = 8 * (r >> 2) + 4 * (l >> 5) + (r & 3), j = l & 31;
                const float want = __fmaf_rn(A[1][i], B[1][j], __fmaf_rn(A[0][i], B[0][j], C[i][j]));
                bad32 += same_result(want, d[r]) ? 0 : 1;
            }
        }
        // 16x16x4 on the top-left 16x16 corner with all four k: lane l holds A[i = l%16][k = l/16];
        // register r of the result is row 4*(l/16) + r, column l%16.
        {
            f4v c;
#pragma unroll
            for (int r = 0; r < 4; r++)
                c[r] = C[4 * (l >> 4) + r][l & 15];
            const f4v d = __builtin_amdgcn_mfma_f32_16x16x4f32(A[l >> 4][l & 15], B[l >> 4][l & 15], c, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; r++)
            {
                const int i = 4 * (l >> 4) + r, j = l & 15;
                float want = C[i][j];
#pragma unroll
                for (int k = 0; k < 4; k++)
                    want = __fmaf_rn(A[k][i], B[k][j], want);
                bad16 += same_result(want, d[r]) ? 0 : 1;
            }
        }
        __syncthreads();
    }
    if (bad32)
        atomicAdd(&counts[0], bad32);
    if (bad16)
        atomicAdd(&counts[1], bad16);
}

// Runs the comparison on a stream of its own (non-blocking: it neither waits for nor holds up
// the null stream or the caller's stream), with memory from the stream-ordered allocator, and
// waits for that stream only.
int run_check(int64_t blocks, int64_t trials, uint64_t seed, unsigned long long out[2])
{
    hipStream_t st = nullptr;
    hipError_t e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking);
    if (e != hipSuccess)
        return (int)e;
    unsigned long long *d = nullptr;
    e = hipMallocAsync(reinterpret_cast<void **>(&d), 2 * sizeof(unsigned long long), st);
    if (e == hipSuccess)
    {
        e = hipMemsetAsync(d, 0, 2 * sizeof(unsigned long long), st);
        if (e == hipSuccess)
        {
            hipLaunchKernelGGL(mfma_check_kernel, dim3((unsigned)blocks), dim3(64), 0, st, d, (int)trials, seed);
            e = hipGetLastError();
        }
        if (e == hipSuccess)
            e = hipMemcpyAsync(out, d, 2 * sizeof(unsigned long long), hipMemcpyDeviceToHost, st);
        const hipError_t e2 = hipFreeAsync(d, st);
        if (e == hipSuccess)
            e = e2;
        const hipError_t e3 = hipStreamSynchronize(st);
        if (e == hipSuccess)
            e = e3;
    }
    (void)hipStreamDestroy(st);
    return e == hipSuccess ? REPDL_OK : (int)e;
}

constexpr int MAX_DEVICES = 64;
std::mutex g_lock;
int g_mode = -1;                 // -1 = the matrix kernels where the check passed, 0 = never, 1 = as -1 (see set_matrix_path)
int g_verdict[MAX_DEVICES] = {}; // 0 = not checked yet, 1 = exact, 2 = not exact

// Verdict of the current device, running the check if it has not run there yet (g_lock held).
// A check that could not run (no device, or a runtime error such as a stream capture in
// progress on this thread) leaves the verdict open: the caller then takes the v_fma_f32
// kernels for this call and the check is tried again at the next one.
int device_verdict(int *rc_out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES)
    {
        if (rc_out)
            *rc_out = e != hipSuccess ? (int)e : REPDL_E_UNSUPPORTED;
        return 0;
    }
    if (g_verdict[dev] == 0)
    {
        unsigned long long bad[2] = {1, 1};
        // 512 waves x 28 trials x (1024 + 256) results: four trials of every class per wave
        const int rc = run_check(512, 4 * NCLASS, 0x52657044 /* any fixed seed */, bad);
        if (rc_out)
            *rc_out = rc;
        if (rc != REPDL_OK)
        {
            (void)hipGetLastError(); // the failed check must not surface in the caller's next launch check
            return 0;
        }
        g_verdict[dev] = (bad[0] == 0 && bad[1] == 0) ? 1 : 2;
    }
    else if (rc_out)
        *rc_out = REPDL_OK;
    return g_verdict[dev];
}
} // namespace

// Whether the GEMM-shaped operators may use the matrix instructions on the current device.
bool repdl_mfma_exact()
{
    // (a workspace-size query asks about both settings without touching the device)
    const int dry = repdl_ws_dry_matrix_path();
    if (dry >= 0)
        return dry == 1;
    std::lock_guard<std::mutex> guard(g_lock);
    if (g_mode == 0)
        return false;
    return device_verdict(nullptr) == 1;
}

REPDL_API int repdl_hip_init(void)
{
    std::lock_guard<std::mutex> guard(g_lock);
    int rc = REPDL_OK;
    (void)device_verdict(&rc);
    return rc;
}

REPDL_API int repdl_hip_mfma_selftest(int64_t waves, int64_t trials, uint64_t seed, uint64_t *mismatches)
{
    REPDL_REQUIRE(mismatches != nullptr && waves > 0 && waves <= REPDL_I32_MAX && trials > 0 && trials <= REPDL_I32_MAX);
    unsigned long long bad[2] = {0, 0};
    const int rc = run_check(waves, trials, seed, bad);
    mismatches[0] = bad[0];
    mismatches[1] = bad[1];
    return rc;
}

REPDL_API int repdl_hip_set_matrix_path(int mode)
{
    REPDL_REQUIRE(mode >= -1 && mode <= 1);
    std::lock_guard<std::mutex> guard(g_lock);
    if (mode == 1)
    {
        // asking for the matrix kernels never bypasses the check: refused where it did not pass
        int rc = REPDL_OK;
        const int v = device_verdict(&rc);
        if (v != 1)
            return rc != REPDL_OK ? rc : REPDL_E_UNSUPPORTED;
    }
    g_mode = mode;
    return REPDL_OK;
}

REPDL_API int repdl_hip_matrix_path(void) { return repdl_mfma_exact() ? 1 : 0; }
