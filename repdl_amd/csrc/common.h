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

// Inputs at least this long (three blocks) take the parallel evaluation of the sequential sum.  The serial kernel
// takes 3.3 us per 1000 elements whatever they are; the two launches of the parallel evaluation of one short
// chain 0.02-0.04 ms up to 16384 elements and 0.03-0.09 up to 32767 (the more the sum hovers near zero), so the
// two meet at 4096-6000 elements on sums that drift and at 8192-12288 on zero-mean ones.
#define REPDL_SUM1D_MIN_PARALLEL 12288

// Row and channel sums take the parallel evaluation when the chains are at least this long and
// at most REPDL_SUM_ROWS_MAX_PARALLEL in number (few long chains are bound by the latency of one
// chain; many chains keep the memory system busy with one lane per chain).
#define REPDL_SUM_ROWS_MIN_PARALLEL 49152
#define REPDL_SUM_ROWS_MAX_PARALLEL 512

// Largest extent a kernel indexes with 32-bit arithmetic.
#define REPDL_I32_MAX 2147483647LL

// True while a workspace-size query runs an entry point's host logic on the calling thread: scratch
// requests are added up, nothing is launched and the device is not touched (workspace.hip).
bool repdl_ws_dry();

static inline int repdl_launch_status()
{
    if (repdl_ws_dry())
        return REPDL_OK;
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? REPDL_OK : (int)e;
}

// Every kernel launch of an entry point that takes scratch memory goes through this (nothing is
// launched during a workspace-size query), and so do its function attributes.
#define REPDL_LAUNCH(...)                    \
    do                                       \
    {                                        \
        if (!repdl_ws_dry())                 \
            hipLaunchKernelGGL(__VA_ARGS__); \
    } while (0)
#define REPDL_FUNC_SET_ATTRIBUTE(fn, attr, value) (repdl_ws_dry() ? hipSuccess : hipFuncSetAttribute(fn, attr, value))

static inline hipStream_t repdl_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

static inline int64_t repdl_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Scratch memory for the duration of a call, ordered on stream s (workspace.hip): in place of
// hipMallocAsync / hipFreeAsync, which hold the host until the work in between has run.  From the
// caller's workspace while the calling thread has one installed (RepdlWorkspace, the *_ws entry
// points), otherwise from the library's cache per device and stream.  Pieces are 256-byte aligned;
// a thread releases its pieces in the reverse order of their acquisition.
hipError_t repdl_ws_acquire(void **p, size_t bytes, hipStream_t s);
hipError_t repdl_ws_release(void *p, hipStream_t s);

// Installs a caller's workspace on the calling thread for the lifetime of the object: every
// repdl_ws_acquire of the entry points called meanwhile (nested ones included) carves from it and
// fails with REPDL_E_WORKSPACE when it does not fit.  With `dry` set nothing is carved or launched:
// the object only records the peak need of the host logic that runs under it, with the matrix
// path taken as `matrix_path` says (workspace-size queries).
class RepdlWorkspace
{
  public:
    RepdlWorkspace(void *base, size_t bytes, bool dry = false, bool matrix_path = false);
    ~RepdlWorkspace();
    RepdlWorkspace(const RepdlWorkspace &) = delete;
    RepdlWorkspace &operator=(const RepdlWorkspace &) = delete;
    size_t peak() const; // bytes of a workspace that the calls made so far would have fitted in
    struct State;

  private:
    State *state_;
    State *previous_;
};
// The matrix path of a workspace-size query in progress on this thread: 1 / 0, or -1 when none is.
int repdl_ws_dry_matrix_path();

// What a workspace-size query reports: `body()` runs an entry point's host logic under a dry
// RepdlWorkspace, once for each setting of the matrix path; the larger peak counts.
template <typename F>
static inline size_t repdl_ws_query(F body)
{
    size_t need = 0;
    for (int mp = 0; mp < 2; mp++)
    {
        RepdlWorkspace dry(nullptr, 0, true, mp != 0);
        if (body() != REPDL_OK)
            return 0; // (the call itself will fail the same way, before it asks for scratch)
        need = dry.peak() > need ? dry.peak() : need;
    }
    return need;
}
// Stand-ins for operand pointers a size query was not given: never dereferenced, one on a 16-byte
// boundary and one off it (the routes look at the alignment of their operands).
static inline const float *repdl_ws_fake_pointer(bool aligned) { return reinterpret_cast<const float *>(aligned ? 0x10000 : 0x10004); }

// Which kernel family a call took.  Every route of the operators that choose among several (by shape,
// alignment, the matrix path, a cost model) notes itself in a process-wide mask when it launches;
// repdl_hip_routes_taken reads it.  For tests: a route that no case reaches any more shows up there.
enum RepdlRoute
{
    // mm: tiles of the kernel that moves operands straight into LDS (16-byte DMA lanes), its 4-byte-lane forms, the v_fma_f32 kernel
    REPDL_ROUTE_MM_128 = 0,          // 128x128, eight waves
    REPDL_ROUTE_MM_128_TALL,         // 128x128, four waves of 64x64 (TN with chains much longer than C is wide)
    REPDL_ROUTE_MM_64_FOUR_BUFFERS,  // 64x64, eight waves, four buffers, four moving waves
    REPDL_ROUTE_MM_64_THREE_BUFFERS, // 64x64, eight waves, three buffers
    REPDL_ROUTE_MM_64_MOVERS,        // 64x64, eight waves, three buffers, four moving waves
    REPDL_ROUTE_MM_64_WIDE_K,        // one 64x64 tile per CU, 513-1024 terms: k-tiles of 64, three buffers, +4
    REPDL_ROUTE_MM_64_DEEP,          // one 64x64 tile per CU, longer chains: k-tiles of 64, four buffers, operands three quads ahead, +4
    REPDL_ROUTE_MM_64_QUAD,          // 64x64, four waves of 32x32
    REPDL_ROUTE_MM_32,               // 32x32
    REPDL_ROUTE_MM_64X32,            // 64x32
    REPDL_ROUTE_MM_UNALIGNED_128,
    REPDL_ROUTE_MM_UNALIGNED_64_MOVERS,
    REPDL_ROUTE_MM_UNALIGNED_64,
    REPDL_ROUTE_MM_UNALIGNED_QUAD,
    REPDL_ROUTE_MM_UNALIGNED_32,
    REPDL_ROUTE_MM_FMA,
    // conv2d / conv2d_grad_input
    REPDL_ROUTE_CONV_PATCH_16,   // 3x3 at stride 1 from an input patch in LDS, 16-byte DMA lanes, tiles of 64 pixels
    REPDL_ROUTE_CONV_PATCH_4,    // the same with 4-byte lanes
    REPDL_ROUTE_CONV_PATCH_16_WIDE, // tiles of 128 pixels
    REPDL_ROUTE_CONV_PATCH_4_WIDE,
    REPDL_ROUTE_CONV_POINT,      // 1x1 at stride 1: both operands streamed
    REPDL_ROUTE_CONV_POINT_MM,   // 1x1 at stride 1: a batch of matrix products per image
    REPDL_ROUTE_CONV_PADDED_64_HALF, // padded copy of the gathered operand, 64-row tiles of 64 pixels
    REPDL_ROUTE_CONV_PADDED_64,
    REPDL_ROUTE_CONV_PADDED_128,
    REPDL_ROUTE_CONV_GATHER_64,  // gather kernel (matrix instructions or v_fma_f32), 64-row tiles
    REPDL_ROUTE_CONV_GATHER_128,
    REPDL_ROUTE_CONV_IM2COL,     // small images: im2col and one matrix product
    REPDL_ROUTE_DGRAD_POINT_SCATTER, // grad-input of a 1x1 kernel at a stride: the stride-1 layer, scattered
    REPDL_ROUTE_DGRAD_RESIDUES,      // grad-input at a stride, residue by residue
    // conv2d_grad_kernel
    REPDL_ROUTE_WGRAD_POINT_GATHER,  // 1x1 at a stride: the input gathered, then the stride-1 layer
    REPDL_ROUTE_WGRAD_PRODUCT,       // many short chains: one matrix product over an im2col
    REPDL_ROUTE_WGRAD_CHAIN,         // dependent matrix instructions with staging waves
    REPDL_ROUTE_WGRAD_FMA,
    // sums
    REPDL_ROUTE_SUM_ROW_WALK,    // one lane per chain
    REPDL_ROUTE_SUM_CHAINS,      // the exact parallel evaluation, all chains at once
    REPDL_ROUTE_SUM_CHAINS_ROUNDS, // ... with speculative rounds
    REPDL_ROUTE_SUM_COLUMN_WALK,
    REPDL_ROUTE_SUM_SERIAL,      // sum1d below the parallel threshold
    // softmax / cross_entropy
    REPDL_ROUTE_LOSS_ONCHIP,     // rows held on chip by a workgroup
    REPDL_ROUTE_LOSS_ROW_PER_WAVE,
    REPDL_ROUTE_COUNT
};
void repdl_route_note(int route); // (nothing during a workspace-size query)

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
