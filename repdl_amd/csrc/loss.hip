// softmax and cross_entropy for gfx950.
//
// Semantics: RepDL backend/cpu/softmax.cpp:15-21 and cross_entropy.cpp:15-24 --
// compositions of a row maximum, exp, the SERIAL row sum, log / division and (for
// the loss) a serial mean over the rows.  One wave owns one row: the maximum is a
// wave reduction (max is exact, so its order is free), exp / division are done
// lane-parallel, and the row sum is a strict j = 0..N-1 chain that every lane
// evaluates redundantly from LDS broadcasts, so all lanes hold the same sum.
// With many rows a wave per row is the wrong shape (every chain step is an LDS broadcast and
// an addition issued for one row, and the SIMDs saturate on those): see "rows held on chip".
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
        int c = 0;
        for (; c + 16 <= cnt; c += 16)
        {
            float b[16]; // sixteen broadcast reads in flight, then their additions in order
#pragma unroll
            for (int u = 0; u < 16; u++)
                b[u] = stage[c + u];
#pragma unroll
            for (int u = 0; u < 16; u++)
                acc = acc + b[u];
        }
        for (; c < cnt; c++)
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
// ---- rows held on chip ------------------------------------------------------------------
// A workgroup of 256 threads owns R rows of at most 64 * (256 / R) columns.  TPR = 256 / R
// threads share a row; thread j of them holds the 16-byte granules j, j + TPR, j + 2 TPR, ...
// of the row in registers (VPT values), so the row is read from memory once, coalesced.
// The maximum is a reduction over registers and the TPR lanes; the exponentials stay in
// the registers and are also laid into LDS (onchip_stride floats per row); after a barrier lane
// l of wave 0 walks row l % R of that image in order, one addition per column for all R rows
// at once, thirty-two values read ahead with ds_read_b128.  The quotients are then
// taken of the register copy and written once: 8 bytes per element in all (4 for the
// loss).  Used for many rows (rows_onchip_wanted), where a wave per row saturates the SIMDs
// with the per-row chain steps, and up to 4096 columns.
constexpr int64_t ROWS_ONCHIP_MIN = 4096;
constexpr int64_t ROWS_ONCHIP_MAX_N = 4096;

// measured: the two shapes are level below about a thousand rows (both bound by one row's
// chain); a wave per row is ahead for short rows (2048x256: 10 against 14 us), the workgroups
// with rows on chip from about two million elements on (4095x1000: 27 against 35 us)
inline bool rows_onchip_wanted(int64_t M, int64_t N)
{
    if (N > ROWS_ONCHIP_MAX_N)
        return false;
    return M >= ROWS_ONCHIP_MIN || (M >= 1024 && M * N >= (1 << 21));
}

typedef float v4f __attribute__((ext_vector_type(4)));

// LDS row of the image: whole 16-byte granules (the chain is walked with ds_read_b128), one more at
// least, an odd number of them in all -- sixteen consecutive rows then start in sixteen different
// groups of four banks, and the walking lanes' reads do not collide
// (rows of 128 columns and fewer, 32 or 64 of them per workgroup, keep N + 1 floats and 4-byte accesses:
// the wider layout made cross_entropy on 65536 x 64 slower, 0.054 -> 0.061 ms)
__host__ __device__ inline int onchip_stride(int N, int R) { return R >= 32 ? N + 1 : 4 * (((N + 3) / 4 + 1) | 1); }

__device__ __forceinline__ float nan_max(float m, float v) { return (v != v) ? v : ((m != m) ? m : (v > m ? v : m)); }

// SOFTMAX: out = softmax rows.  Otherwise: loss[row] = log(sum_j exp(x_j - m)) - (x_target - m).
template <int R, int VPT, bool SOFTMAX>
__global__ __launch_bounds__(256) void rows_onchip_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                          const int64_t *__restrict__ target, float *__restrict__ loss,
                                                          int64_t M, int N, int vec_ok)
{
    constexpr int TPR = 256 / R; // threads per row
    constexpr int G = VPT / 4;   // granules per thread
    __shared__ uint64_t exp_tab[256];
    __shared__ double log_hi[SOFTMAX ? 1 : 128];
    __shared__ float log_invc[SOFTMAX ? 1 : 128], log_lo[SOFTMAX ? 1 : 128];
    __shared__ float rmax[R], rsum[R];
    extern __shared__ __attribute__((aligned(16))) float image[]; // R rows of onchip_stride(N, R) floats
    const int tid = threadIdx.x;
    exp_tab[tid] = g_exp_tab2[tid];
    if (!SOFTMAX && tid < 128)
    {
        log_hi[tid] = g_log_hi2[tid];
        log_invc[tid] = g_log_invc2[tid];
        log_lo[tid] = g_log_lo2[tid];
    }
    const int r = tid / TPR, j = tid % TPR;
    const int64_t row0 = (int64_t)blockIdx.x * R;
    const bool live = row0 + r < M;
    const int64_t row = live ? row0 + r : M - 1; // rows past the end repeat the last one and store nothing
    const float *x = in + row * N;
    constexpr bool VROW = R < 32; // rows as whole 16-byte granules
    const int stride = onchip_stride(N, R);

    // the row, once
    float v[VPT];
#pragma unroll
    for (int i = 0; i < G; i++)
    {
        const int c = (i * TPR + j) * 4;
        if (vec_ok && c + 4 <= N)
        {
            const v4f t = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(x + c));
            v[4 * i + 0] = t.x;
            v[4 * i + 1] = t.y;
            v[4 * i + 2] = t.z;
            v[4 * i + 3] = t.w;
        }
        else
        {
#pragma unroll
            for (int k = 0; k < 4; k++)
                v[4 * i + k] = c + k < N ? x[c + k] : -__builtin_inff(); // exp(-inf - m) = +0: neutral
        }
    }
    float m = -__builtin_inff();
#pragma unroll
    for (int k = 0; k < VPT; k++)
        m = nan_max(m, v[k]);
#pragma unroll
    for (int off = 1; off < TPR; off <<= 1)
        m = nan_max(m, __shfl_xor(m, off, 64));
    if (j == 0)
        rmax[r] = m;
    __syncthreads(); // tables

    // exponentials: whole granule rounds are skipped with a uniform branch, everything inside is
    // computed without branches so that the independent evaluations interleave (columns past N hold
    // -inf and give values that are never stored)
    float *img = image + r * stride;
#pragma unroll
    for (int i = 0; i < G; i++)
    {
        if (i * TPR * 4 < N)
        {
            const int c = (i * TPR + j) * 4;
#pragma unroll
            for (int k = 0; k < 4; k++)
                v[4 * i + k] = crm_exp(v[4 * i + k] - m, exp_tab);
            if (VROW)
            {
                if (c < N) // (columns past N inside the last granule hold exp(-inf) = +0 and are never walked)
                    *reinterpret_cast<v4f *>(img + c) = (v4f){v[4 * i + 0], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]};
            }
            else
            {
#pragma unroll
                for (int k = 0; k < 4; k++)
                    if (c + k < N)
                        img[c + k] = v[4 * i + k];
            }
        }
    }
    __syncthreads();
    // (Which wave walks makes no difference: rotating it with the workgroup id, so that the workgroups of a
    // CU walk on different SIMDs, measured the same 0.160 / 0.180 ms on 65536 x 1000.)
    const int wl = tid;
    if (tid < 64)
    {
        // the chain of row `wl` (lanes R and up of the wave walk the first rows again: a chain of dependent
        // v_add_f32 issues every 6.7 clocks in a full wave, every 8.6 with most lanes off, and masked walks
        // on one CU slow each other to 20): sixteen values ahead in registers while sixteen are added
        const float *wr = image + (wl % R) * stride;
        float acc = 0.0f;
        int whole = 0;
        if (VROW)
        {
            constexpr int WB = 8; // granules per batch: 32 values ahead in registers while 32 are added
            v4f cur[WB], nxt[WB];
            whole = N & ~(4 * WB - 1);
            const v4f *wq = reinterpret_cast<const v4f *>(wr);
            if (whole > 0)
            {
#pragma unroll
                for (int u = 0; u < WB; u++)
                    cur[u] = wq[u];
            }
            for (int k = 0; k < whole; k += 4 * WB)
            {
                if (k + 4 * WB < whole)
                {
#pragma unroll
                    for (int u = 0; u < WB; u++)
                        nxt[u] = wq[(k + 4 * WB) / 4 + u];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < WB; u++)
                {
                    acc = acc + cur[u].x;
                    acc = acc + cur[u].y;
                    acc = acc + cur[u].z;
                    acc = acc + cur[u].w;
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < WB; u++)
                    cur[u] = nxt[u];
            }
        }
        else
        {
            float cur[16], nxt[16]; // sixteen values ahead in registers while sixteen are added
            whole = N & ~15;
            if (whole > 0)
            {
#pragma unroll
                for (int u = 0; u < 16; u++)
                    cur[u] = wr[u];
            }
            for (int k = 0; k < whole; k += 16)
            {
                if (k + 16 < whole)
                {
#pragma unroll
                    for (int u = 0; u < 16; u++)
                        nxt[u] = wr[k + 16 + u];
                }
#pragma unroll
                for (int u = 0; u < 16; u++)
                    acc = acc + cur[u];
#pragma unroll
                for (int u = 0; u < 16; u++)
                    cur[u] = nxt[u];
            }
        }
        for (int k = whole; k < N; k++)
            acc = acc + wr[k];
        if (wl < R)
            rsum[wl] = acc;
    }
    __syncthreads();

    if (SOFTMAX)
    {
        if (!live)
            return;
        const crm_divisor d = crm_divisor_make(rsum[r]);
        float *o = out + row * N;
#pragma unroll
        for (int i = 0; i < G; i++)
        {
            if (i * TPR * 4 < N)
            {
                const int c = (i * TPR + j) * 4;
                v4f t;
                t.x = crm_div_by(v[4 * i + 0], d);
                t.y = crm_div_by(v[4 * i + 1], d);
                t.z = crm_div_by(v[4 * i + 2], d);
                t.w = crm_div_by(v[4 * i + 3], d);
                if (vec_ok && c + 4 <= N)
                    __builtin_nontemporal_store(t, reinterpret_cast<v4f *>(o + c));
                else
                {
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        if (c + k < N)
                            o[c + k] = t[k];
                }
            }
        }
    }
    else if (tid < R && row0 + tid < M)
    {
        crm_log_tables lt;
        lt.invc = log_invc;
        lt.logc_hi = log_hi;
        lt.logc_lo = log_lo;
        const float l = crm_log(rsum[tid], lt);
        const int64_t tg = target[row0 + tid];
        const float shifted = (tg >= 0 && tg < N) ? in[(row0 + tid) * N + tg] - rmax[tid] : __builtin_nanf("");
        loss[row0 + tid] = l - shifted;
    }
}

template <int R, int VPT, bool SOFTMAX>
int launch_rows_onchip(const float *in, float *out, const int64_t *target, float *loss, int64_t M, int64_t N, int vec_ok,
                       hipStream_t s)
{
    auto kern = &rows_onchip_kernel<R, VPT, SOFTMAX>;
    repdl_route_note(REPDL_ROUTE_LOSS_ONCHIP);
    const size_t shmem = (size_t)R * onchip_stride((int)N, R) * sizeof(float);
    if (shmem > 40 * 1024)
    {
        hipError_t e = REPDL_FUNC_SET_ATTRIBUTE(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)shmem);
        if (e != hipSuccess)
            return (int)e;
    }
    REPDL_LAUNCH(kern, dim3((unsigned)repdl_cdiv(M, R)), dim3(256), shmem, s, in, out, target, loss, M, (int)N, vec_ok);
    return repdl_launch_status();
}

// rows per workgroup by row length: the registers of the row's threads must hold it
template <bool SOFTMAX>
int rows_onchip(const float *in, float *out, const int64_t *target, float *loss, int64_t M, int64_t N, hipStream_t s)
{
    const bool aligned = (reinterpret_cast<uintptr_t>(in) & 15) == 0 && (!SOFTMAX || (reinterpret_cast<uintptr_t>(out) & 15) == 0);
    const int vec_ok = N % 4 == 0 && aligned;
    // at most 8192 elements (32 KiB of LDS image, 32 values per thread) per workgroup up to 2048
    // columns, so that four workgroups share a CU and one's loads overlap another's chain
    if (N <= 16)
        return launch_rows_onchip<64, 4, SOFTMAX>(in, out, target, loss, M, N, vec_ok, s);
    if (N <= 32)
        return launch_rows_onchip<64, 8, SOFTMAX>(in, out, target, loss, M, N, vec_ok, s);
    if (N <= 64)
        return launch_rows_onchip<64, 16, SOFTMAX>(in, out, target, loss, M, N, vec_ok, s);
    if (N <= 128)
        return launch_rows_onchip<64, 32, SOFTMAX>(in, out, target, loss, M, N, vec_ok, s);
    if (N <= 256)
        return launch_rows_onchip<32, 32, SOFTMAX>(in, out, target, loss, M, N, vec_ok, s);
    if (N <= 512)
        return launch_rows_onchip<16, 32, SOFTMAX>(in, out, target, loss, M, N, vec_ok, s);
    if (N <= 1024)
        return launch_rows_onchip<8, 32, SOFTMAX>(in, out, target, loss, M, N, vec_ok, s);
    if (N <= 2048)
        return launch_rows_onchip<4, 32, SOFTMAX>(in, out, target, loss, M, N, vec_ok, s);
    return launch_rows_onchip<4, 64, SOFTMAX>(in, out, target, loss, M, N, vec_ok, s);
}
} // namespace

REPDL_API int repdl_hip_softmax(const float *in, float *out, int64_t M, int64_t N, void *stream)
{
    REPDL_REQUIRE(M >= 0 && N >= 0);
    if (M == 0 || N == 0)
        return REPDL_OK;
    REPDL_REQUIRE(in != nullptr && out != nullptr && M <= REPDL_I32_MAX);
    if (rows_onchip_wanted(M, N))
        return rows_onchip<true>(in, out, nullptr, nullptr, M, N, repdl_stream(stream));
    repdl_route_note(REPDL_ROUTE_LOSS_ROW_PER_WAVE);
    REPDL_LAUNCH(softmax_kernel, dim3((unsigned)M), dim3(64), 0, repdl_stream(stream), in, out, M, N);
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
        int rc;
        if (rows_onchip_wanted(M, N))
            rc = rows_onchip<false>(in, nullptr, target, workspace, M, N, repdl_stream(stream));
        else
        {
            repdl_route_note(REPDL_ROUTE_LOSS_ROW_PER_WAVE);
            REPDL_LAUNCH(cross_entropy_rows_kernel, dim3((unsigned)M), dim3(64), 0, repdl_stream(stream),
                               in, target, workspace, M, N);
            rc = repdl_launch_status();
        }
        if (rc != REPDL_OK)
            return rc;
    }
    return repdl_hip_sum1d(workspace, out, M, 1, stream);
}

// cross_entropy with one caller's workspace for the row losses and for the scratch of their mean
REPDL_API size_t repdl_hip_cross_entropy_workspace_bytes(int64_t M, int64_t N)
{
    if (M <= 0 || N <= 0)
        return 0;
    const float *fake = repdl_ws_fake_pointer(true);
    return repdl_ws_query([&]() {
        return repdl_hip_cross_entropy_ws(fake, reinterpret_cast<const int64_t *>(fake), const_cast<float *>(fake), M, N, nullptr, 0, nullptr);
    });
}

REPDL_API int repdl_hip_cross_entropy_ws(const float *in, const int64_t *target, float *out, int64_t M, int64_t N,
                                         void *workspace, size_t workspace_bytes, void *stream)
{
    REPDL_REQUIRE(M >= 0);
    // (a size query calls this with its own dry workspace installed: the caller's buffer only otherwise)
    const bool dry = repdl_ws_dry();
    RepdlWorkspace *ws = dry ? nullptr : new RepdlWorkspace(workspace, workspace_bytes);
    float *rows = nullptr;
    hipError_t e = repdl_ws_acquire(reinterpret_cast<void **>(&rows), (size_t)M * sizeof(float), repdl_stream(stream)); // (nothing for M = 0)
    int rc = e == hipSuccess ? repdl_hip_cross_entropy(in, target, out, M, N, rows, stream) : (int)e;
    if (e == hipSuccess)
        e = repdl_ws_release(rows, repdl_stream(stream));
    delete ws;
    return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
}
