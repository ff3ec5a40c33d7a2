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
// A workgroup of RT threads owns RR chains (4 to 64, chosen from the number of
// rows) and moves through them in tiles of RR x RC floats = 32 KiB.  All its
// waves stream the NEXT tile from global memory into registers with 16-byte
// non-temporal loads (each wave reads contiguous pieces of one row at a time)
// while one wave walks the CURRENT tile in LDS: lane l adds row l's RC values in
// order, reading them back with ds_read_b128.  One LDS buffer (33 KiB) lets four
// workgroups share a CU, which keeps up to 128 KiB of loads in flight per CU --
// what it takes to cover loaded HBM latency.  The walking wave rotates with the
// workgroup index to spread the walks over the SIMDs; a walk costs one dependent
// v_add_f32 per element and chain, well below the memory time of the tile as
// long as enough lanes walk (hence more chains per workgroup when rows abound).
// ---------------------------------------------------------------------------
constexpr int RTILE = 8192;    // floats per tile

typedef float v4f __attribute__((ext_vector_type(4)));

// MULTI: short segments (sum4d_dim023 on small images) -- a tile row holds `spt` whole
// segments of its chain back to back instead of a piece of one, so that a tile is still
// thousands of additions long and its walk covers the latency of the next tile's loads
// (with one 196-element segment per tile, 64 chains of 12 544 took 158 us; so: 35 us).
template <int RR, int RT, bool VEC, bool MULTI>
__global__ __launch_bounds__(RT) void rowchain_kernel(const float *__restrict__ in,
                                                      float *__restrict__ out, int64_t rows,
                                                      int64_t nseg, int64_t seglen,
                                                      int64_t row_stride, int64_t seg_stride,
                                                      float factor, int spt)
{
    constexpr int RC = RTILE / RR; // tile columns
    constexpr int RLD = RC + 4;    // padded LDS row: keeps 16-byte alignment, shifts banks by 4
    constexpr int C4 = RC / 4;     // float4 per tile row
    constexpr int RV = RTILE / 4 / RT; // float4 per thread and tile
    __shared__ __attribute__((aligned(16))) float tile[RR * RLD + 64]; // + 64: the walk reads ahead past the last row
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    // The workgroups that share a CU have ids 256 apart (the same id % 4), and the hardware starts each
    // one's waves on the next SIMD (wave 0 of four co-resident workgroups was seen on SIMDs 1, 3, 0, 2):
    // the same wave index in each puts their walks on different SIMDs.
    const int walker = blockIdx.x % (RT / 64);
    const int64_t r0 = (int64_t)blockIdx.x * RR;
    const int64_t tiles_per_seg = (seglen + RC - 1) / RC;
    const int64_t ntiles = MULTI ? (nseg + spt - 1) / spt : nseg * tiles_per_seg;
    const int slen = (int)seglen; // MULTI: seglen <= RC / 2

    float acc = 0.0f;
    v4f stage[RV];

    auto load_multi = [&](int64_t t) {
        const int64_t s0 = t * spt;
        const int ns = nseg - s0 < spt ? (int)(nseg - s0) : spt;
        const int valid = ns * slen;
#pragma unroll
        for (int i = 0; i < RV; i++)
        {
            const int idx = tid + RT * i;
            const int64_t r = r0 + idx / C4;
            const int c = (idx % C4) << 2;
            v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (r < rows && c < valid)
            {
                const float *rowp = in + s0 * seg_stride + r * row_stride;
                const int sg = c / slen, off = c - sg * slen;
                if (VEC && (slen & 3) == 0) // the four elements lie in one segment, 16-byte aligned
                    v = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(rowp + sg * seg_stride + off));
                else
                {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                    {
                        const int ce = c + e, sge = ce / slen;
                        if (ce < valid)
                            v[e] = rowp[sge * seg_stride + (ce - sge * slen)];
                    }
                }
            }
            stage[i] = v;
        }
    };
    auto load = [&](int64_t t) {
        if (MULTI)
        {
            load_multi(t);
            return;
        }
        const int64_t sgm = t / tiles_per_seg, c0 = (t - sgm * tiles_per_seg) * RC;
        const float *base = in + sgm * seg_stride + c0;
#pragma unroll
        for (int i = 0; i < RV; i++)
        {
            const int idx = tid + RT * i;
            const int64_t r = r0 + idx / C4;
            const int c = (idx % C4) << 2;
            v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (r < rows)
            {
                const float *p = base + r * row_stride + c;
                if (VEC && c0 + c + 3 < seglen)
                    v = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
                else
                {
                    if (c0 + c + 0 < seglen) v.x = p[0];
                    if (c0 + c + 1 < seglen) v.y = p[1];
                    if (c0 + c + 2 < seglen) v.z = p[2];
                    if (c0 + c + 3 < seglen) v.w = p[3];
                }
            }
            stage[i] = v;
        }
    };
    auto store = [&]() {
#pragma unroll
        for (int i = 0; i < RV; i++)
        {
            const int idx = tid + RT * i;
            *reinterpret_cast<v4f *>(&tile[(idx / C4) * RLD + ((idx % C4) << 2)]) = stage[i];
        }
    };

    if (ntiles > 0)
    {
        load(0);
        store();
    }
    __syncthreads();
    for (int64_t t = 0; t < ntiles; t++)
    {
        const bool more = t + 1 < ntiles;
        if (more)
            load(t + 1);
        if (wave == walker)
        {
            // every lane walks (lanes RR and up repeat the first chains): a chain of dependent v_add_f32
            // issues every 8.6 clocks in a wave with 32 or fewer active lanes, every 6.7 with 48 or more
            const int64_t sgm = t / tiles_per_seg, c0 = (t - sgm * tiles_per_seg) * RC;
            const int64_t rem = MULTI ? (nseg - t * spt < spt ? nseg - t * spt : spt) * seglen : seglen - c0;
            const float *row = &tile[(lane % RR) * RLD];
            // 8*WB elements per step, the next ones read from LDS before the adds of the current
            // ones: with few chains per workgroup the walk is the critical path, and it should
            // cost one dependent v_add_f32 per element and little else.  Elements past the end
            // of a short tile are walked one by one (they must not be added at all: -0 + 0 = +0).
            constexpr int WB = RC < 64 ? RC / 8 : 8; // float4 per half step
            const int here = rem >= RC ? RC : (int)rem;
            const int nfull = here - here % (8 * WB);
            if (nfull > 0)
            {
                v4f va[WB], vb[WB];
#pragma unroll
                for (int u = 0; u < WB; u++)
                    va[u] = *reinterpret_cast<const v4f *>(&row[4 * u]);
                for (int c = 0; c < nfull; c += 8 * WB)
                {
                    // (the barriers keep the scheduler from gathering all reads in one place, which
                    // would leave the adds waiting for reads issued just before them)
#pragma unroll
                    for (int u = 0; u < WB; u++)
                        vb[u] = *reinterpret_cast<const v4f *>(&row[c + 4 * WB + 4 * u]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int u = 0; u < WB; u++)
                    {
                        acc = acc + va[u].x;
                        acc = acc + va[u].y;
                        acc = acc + va[u].z;
                        acc = acc + va[u].w;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    // the last step reads 4*WB floats past the row: inside the tile or its pad
#pragma unroll
                    for (int u = 0; u < WB; u++)
                        va[u] = *reinterpret_cast<const v4f *>(&row[c + 8 * WB + 4 * u]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int u = 0; u < WB; u++)
                    {
                        acc = acc + vb[u].x;
                        acc = acc + vb[u].y;
                        acc = acc + vb[u].z;
                        acc = acc + vb[u].w;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            for (int c = nfull; c < here; c++)
                acc = acc + row[c];
        }
        __syncthreads(); // the walk of tile t is over: the buffer may be overwritten
        if (more)
            store();
        __syncthreads();
    }
    if (wave == walker && lane < RR && r0 + lane < rows)
        out[r0 + lane] = factor * acc;
}

// ---------------------------------------------------------------------------
// Column chains: out[j] = chain over i of in[i*N + j] (sum2d_dim0).  Same scheme
// as the row chains, turned: a workgroup owns CW adjacent columns (64, 32 or 16,
// fewer when columns are scarce so that the CUs still get several workgroups each)
// and moves down in tiles of (RTILE / CW) rows x CW columns = 32 KiB.  All waves
// stream the next tile into registers (16-byte non-temporal loads; a row of the
// tile is CW*4 contiguous bytes) and store it transposed, [column][row], while one wave
// walks the current tile in LDS, lane = column, one ds_read_b128 and four dependent
// v_add_f32 per four rows (a ds_read_b32 per row cost 14 clocks per row, this 9).
// ---------------------------------------------------------------------------
// NB = 2 (used when the workgroups are so few that each one's walk is the critical path): half-size
// tiles in two LDS buffers, so that the walk never waits for the movers' stores -- one barrier per
// tile, and the walking wave goes from one tile straight into the next.
template <int CW, bool VEC, int NB>
__global__ __launch_bounds__(320) void coltile_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                      int64_t M, int64_t N, float factor)
{
    constexpr int TFLOATS = RTILE / NB;  // floats per tile
    constexpr int TR = TFLOATS / CW;     // rows per tile
    constexpr int C4 = CW / 4;           // float4 per tile row
    constexpr int RV = TFLOATS / 4 / 256; // float4 per thread and tile
    constexpr int TRP = TR + 4;          // LDS words per column (the pad spreads the walk's 16-byte reads over the banks)
    __shared__ __attribute__((aligned(16))) float tile[NB][CW * TRP]; // [column][row]: the walk reads four rows at once
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    constexpr int walker = 4; // waves 0-3 move the tiles, wave 4 only walks (as a mover too it walked 12.6 clocks per row)
    // Which columns?  With 16 columns a row of the tile is half a 128-byte line, and the
    // workgroup that takes the other half should sit behind the same L2 or the line comes
    // from memory twice.  Workgroups go to the 8 XCDs round-robin by id, so inside every whole
    // group of 16 ids, ids b and b + 8 (same XCD, dispatched back to back) take the two halves
    // of one line; the loads then keep the default cache policy instead of the streaming one.
    constexpr bool HALF_LINE = CW == 16;
    int64_t cg = blockIdx.x;
    if (HALF_LINE && (cg | 15) < (int64_t)gridDim.x)
        cg = (cg & ~(int64_t)15) + ((cg & 7) << 1) + ((cg >> 3) & 1);
    const int64_t col0 = cg * CW;
    const int64_t ntiles = (M + TR - 1) / TR;

    float acc = 0.0f;
    // NB = 2: PD tiles on their way from memory at any time, each in its own set of registers.  One is
    // enough: 65536 x 4096 (256 workgroups, a tile row = half a 128-byte line) takes 0.262 ms with 1, 2, 4
    // or 6, and also with the walk all but switched off -- a CU's movers bring in 16 GB/s of such half
    // lines and no more, whatever is in flight.
    constexpr int PD = 1;
    v4f stages[PD][RV];
    auto load = [&](int64_t t, v4f(&stage)[RV]) {
#pragma unroll
        for (int i = 0; i < RV; i++)
        {
            const int idx = tid + 256 * i;
            const int64_t r = t * TR + idx / C4;
            const int64_t c = col0 + ((idx % C4) << 2);
            v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (r < M)
            {
                const float *p = in + r * N + c;
                if (VEC && c + 3 < N)
                    v = HALF_LINE ? *reinterpret_cast<const v4f *>(p)
                                  : __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
                else
                {
                    if (c + 0 < N) v.x = p[0];
                    if (c + 1 < N) v.y = p[1];
                    if (c + 2 < N) v.z = p[2];
                    if (c + 3 < N) v.w = p[3];
                }
            }
            stage[i] = v;
        }
    };
    auto store = [&](int buf, const v4f(&stage)[RV]) {
#pragma unroll
        for (int i = 0; i < RV; i++)
        {
            const int idx = tid + 256 * i;
            float *q = &tile[buf][((idx % C4) << 2) * TRP + idx / C4]; // transposed on the way in
            q[0 * TRP] = stage[i].x;
            q[1 * TRP] = stage[i].y;
            q[2 * TRP] = stage[i].z;
            q[3 * TRP] = stage[i].w;
        }
    };
    auto walk = [&](int64_t t, int buf) {
        const int64_t rem = M - t * TR; // rows of this tile that exist; the rest must not be added
        // every lane walks (lanes CW and up repeat the first columns): a chain of dependent v_add_f32 in a
        // wave with 32 or fewer active lanes issues every 8.6 clocks, with 48 or more every 6.7 (measured)
        const float *colp = &tile[buf][(lane % CW) * TRP];
        if (rem >= TR)
        {
            // batches of NRW reads = 4 NRW rows, two register sets: the reads of the next batch are
            // issued, then the adds of this one run under their latency (pinned: left to itself
            // the compiler interleaves them and every add then waits for a read)
            // (few workgroups, NB = 2: batches of 64 rows, 100000 x 1000 0.38 -> 0.34 ms; with many workgroups
            // the registers of long batches cost more than they gain: 16 rows)
            constexpr int NRW = NB == 2 ? (TR / 8 < 16 ? TR / 8 : 16) : 4;
            static_assert(TR % (8 * NRW) == 0, "a tile is whole pairs of batches");
            const v4f *cp = reinterpret_cast<const v4f *>(colp);
            v4f va[NRW], vb[NRW];
#pragma unroll
            for (int u = 0; u < NRW; u++)
                va[u] = cp[u];
            for (int r = 0; r < TR; r += 8 * NRW)
            {
#pragma unroll
                for (int u = 0; u < NRW; u++)
                    vb[u] = cp[(r + 4 * NRW) / 4 + u];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < NRW; u++)
                {
                    acc = acc + va[u].x;
                    acc = acc + va[u].y;
                    acc = acc + va[u].z;
                    acc = acc + va[u].w;
                }
                __builtin_amdgcn_sched_barrier(0);
                if (r + 8 * NRW < TR)
                {
#pragma unroll
                    for (int u = 0; u < NRW; u++)
                        va[u] = cp[(r + 8 * NRW) / 4 + u];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < NRW; u++)
                {
                    acc = acc + vb[u].x;
                    acc = acc + vb[u].y;
                    acc = acc + vb[u].z;
                    acc = acc + vb[u].w;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        else
        {
            for (int r = 0; r < (int)rem; r++)
                acc = acc + colp[r];
        }
    };

    const bool mover = wave < 4;
    if (NB == 2)
    {
        // set (t % PD) holds tile t from its request until it is stored
        if (ntiles > 0 && mover)
        {
            load(0, stages[0]);
            store(0, stages[0]);
#pragma unroll
            for (int u = 1; u <= PD; u++)
                if (u < ntiles)
                    load(u, stages[u % PD]);
        }
        __syncthreads();
        for (int64_t t0 = 0; t0 < ntiles; t0 += PD)
        {
#pragma unroll
            for (int u = 0; u < PD; u++)
            {
                const int64_t t = t0 + u;
                if (t >= ntiles)
                    break;
                // tile t + 1 (requested PD tiles ago) into the other buffer, tile t + 1 + PD requested into its registers
                if (mover && t + 1 < ntiles)
                    store((int)((t + 1) & 1), stages[(u + 1) % PD]);
                if (mover && t + 1 + PD < ntiles)
                    load(t + 1 + PD, stages[(u + 1) % PD]);
                if (wave == walker)
                    walk(t, (int)(t & 1));
                __syncthreads(); // tile t + 1 is complete, the walk of tile t is over
            }
        }
    }
    else
    {
        if (ntiles > 0 && mover)
        {
            load(0, stages[0]);
            store(0, stages[0]);
        }
        __syncthreads();
        for (int64_t t = 0; t < ntiles; t++)
        {
            const bool more = t + 1 < ntiles;
            if (more && mover)
                load(t + 1, stages[0]);
            if (wave == walker)
                walk(t, 0);
            __syncthreads(); // the walk of tile t is over: the buffer may be overwritten
            if (more && mover)
                store(0, stages[0]);
            __syncthreads();
        }
    }
    if (wave == walker && lane < CW && col0 + lane < N)
        out[col0 + lane] = factor * acc;
}
} // namespace

static int launch_rowchain(const float *in, float *out, int64_t rows, int64_t nseg, int64_t seglen,
                           int64_t row_stride, int64_t seg_stride, float factor, void *stream)
{
    if (rows == 0)
        return REPDL_OK;
    // Few long chains: one lane per chain would be bound by the latency of a chain (8 to 10 clocks
    // per element whatever the data).  The parallel evaluation of sum1d.hip, all chains at once.
    const int64_t len = nseg * seglen;
    // (At most 64 chains: from half that length on.  There the walks of zero-mean chains take what one lane per
    // chain takes -- 25088 elements 0.103 ms either way, 48000 0.161 -> 0.141 -- and chains that drift a third of it:
    // 0.103 -> 0.041, 0.161 -> 0.039.  More chains of that length, or shorter ones, lose up to 75 % on zero-mean data.)
    const bool long_enough = len >= REPDL_SUM_ROWS_MIN_PARALLEL || (rows <= 64 && len >= REPDL_SUM_ROWS_MIN_PARALLEL / 2);
    if (rows <= REPDL_SUM_ROWS_MAX_PARALLEL && long_enough &&
        (nseg == 1 || (seglen % 16 == 0 && len <= REPDL_I32_MAX)))
    {
        const size_t bytes = repdl_sum_chains_workspace_bytes(rows, len);
        void *ws = nullptr;
        hipError_t e = repdl_ws_acquire(&ws, bytes, repdl_stream(stream));
        if (e != hipSuccess)
            return (int)e;
        const int rc = repdl_sum_chains(in, out, rows, nseg, seglen, row_stride, seg_stride, factor, ws, bytes, stream);
        e = repdl_ws_release(ws, repdl_stream(stream));
        return rc != REPDL_OK ? rc : (e == hipSuccess ? REPDL_OK : (int)e);
    }
    // Chains per workgroup: enough workgroups to fill 256 CUs two to four times
    // over, all resident at once, and as many walking lanes as that allows.
    const bool vec = (reinterpret_cast<uintptr_t>(in) & 15) == 0 && row_stride % 4 == 0 && seg_stride % 4 == 0;
    repdl_route_note(REPDL_ROUTE_SUM_ROW_WALK);
    const int rr = rows >= 49152 ? 64 : rows >= 12288 ? 32 : rows >= 6144 ? 16 : 4;
    const int64_t grid = repdl_cdiv(rows, rr);
    REPDL_REQUIRE(grid <= REPDL_I32_MAX);
    const dim3 g((unsigned)grid);
    hipStream_t st = repdl_stream(stream);
    // short segments: whole segments per tile row (see MULTI)
    const int64_t rc = RTILE / rr;
    const bool multi = nseg > 1 && seglen > 0 && 2 * seglen <= rc;
    const int spt = multi ? (int)(rc / seglen) : 1;
    // Few workgroups (each walk is then the critical path): ask for LDS the kernel does not use,
    // so that a workgroup has its CU to itself.  81 KiB in all: neither a second one of these nor
    // a grad-kernel workgroup (84 KiB) of a launch running beside this one on another stream fits
    // next to it -- a walk that shares its SIMD with matrix instructions ran 1.85 times longer.
    const size_t lds_pad = grid <= 256 ? 48 * 1024 : 0;
#define REPDL_ROWCHAIN_M(RRv, RTv, V, MU)                                                                           \
    do                                                                                                             \
    {                                                                                                              \
        if (lds_pad != 0)                                                                                          \
        {                                                                                                          \
            hipError_t e_ = REPDL_FUNC_SET_ATTRIBUTE(reinterpret_cast<const void *>(&rowchain_kernel<RRv, RTv, V, MU>), \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_pad);         \
            if (e_ != hipSuccess)                                                                                  \
                return (int)e_;                                                                                    \
        }                                                                                                          \
        REPDL_LAUNCH((rowchain_kernel<RRv, RTv, V, MU>), g, dim3(RTv), lds_pad, st, in, out, rows, nseg,     \
                           seglen, row_stride, seg_stride, factor, spt);                                           \
    } while (0)
#define REPDL_ROWCHAIN_V(RRv, RTv, V)              \
    do                                             \
    {                                              \
        if (multi)                                 \
            REPDL_ROWCHAIN_M(RRv, RTv, V, true);   \
        else                                       \
            REPDL_ROWCHAIN_M(RRv, RTv, V, false);  \
    } while (0)
#define REPDL_ROWCHAIN(RRv, RTv)              \
    do                                        \
    {                                         \
        if (vec)                              \
            REPDL_ROWCHAIN_V(RRv, RTv, true); \
        else                                  \
            REPDL_ROWCHAIN_V(RRv, RTv, false);\
    } while (0)
    if (rr == 64)
        REPDL_ROWCHAIN(64, 256);
    else if (rr == 32)
        REPDL_ROWCHAIN(32, 128);
    else if (rr == 16)
        REPDL_ROWCHAIN(16, 256);
    else
        REPDL_ROWCHAIN(4, 256);
#undef REPDL_ROWCHAIN
#undef REPDL_ROWCHAIN_V
#undef REPDL_ROWCHAIN_M
    return repdl_launch_status();
}

// The single serial chain (one lane walks): used for short inputs; long ones take the
// parallel evaluation of sum1d.hip.
int repdl_sum1d_serial(const float *in, float *out, int64_t n, int average, void *stream)
{
    REPDL_REQUIRE(n >= 0 && out != nullptr && (n == 0 || in != nullptr));
    repdl_route_note(REPDL_ROUTE_SUM_SERIAL);
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

// The same two with the caller's workspace (see RepdlWorkspace): the size query runs the host logic
// above with the launches switched off.
REPDL_API size_t repdl_hip_sum2d_dim1_workspace_bytes(int64_t M, int64_t N)
{
    float *fake = const_cast<float *>(repdl_ws_fake_pointer(true));
    return repdl_ws_query([&]() { return repdl_hip_sum2d_dim1(fake, fake, M, N, 0, nullptr); });
}

REPDL_API int repdl_hip_sum2d_dim1_ws(const float *in, float *out, int64_t M, int64_t N, int average, void *workspace,
                                      size_t workspace_bytes, void *stream)
{
    RepdlWorkspace ws(workspace, workspace_bytes);
    return repdl_hip_sum2d_dim1(in, out, M, N, average, stream);
}

REPDL_API size_t repdl_hip_sum4d_dim023_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W)
{
    float *fake = const_cast<float *>(repdl_ws_fake_pointer(true));
    return repdl_ws_query([&]() { return repdl_hip_sum4d_dim023(fake, fake, N, C, H, W, 0, nullptr); });
}

REPDL_API int repdl_hip_sum4d_dim023_ws(const float *in, float *out, int64_t N, int64_t C, int64_t H, int64_t W, int average,
                                        void *workspace, size_t workspace_bytes, void *stream)
{
    RepdlWorkspace ws(workspace, workspace_bytes);
    return repdl_hip_sum4d_dim023(in, out, N, C, H, W, average, stream);
}

REPDL_API int repdl_hip_sum2d_dim0(const float *in, float *out, int64_t M, int64_t N, int average,
                                   void *stream)
{
    REPDL_REQUIRE(M >= 0 && N >= 0 && (N == 0 || out != nullptr) && (M * N == 0 || in != nullptr));
    if (N == 0)
        return REPDL_OK;
    const bool vec = (reinterpret_cast<uintptr_t>(in) & 15) == 0 && N % 4 == 0;
    const int cw = N >= 65536 ? 64 : N >= 8192 ? 32 : 16; // 32 columns = one 128-byte line per row
    const int64_t grid = repdl_cdiv(N, cw);
    REPDL_REQUIRE(grid <= REPDL_I32_MAX);
    const dim3 g((unsigned)grid);
    hipStream_t st = repdl_stream(stream);
    const float factor = repdl_sum_factor(average, M);
    repdl_route_note(REPDL_ROUTE_SUM_COLUMN_WALK);
    // few workgroups, long columns: the walk of each is the critical path -- two LDS buffers
    const bool two = grid <= 512 && M >= 4096;
#define REPDL_COLTILE(CWv, NBv)                                                                               \
    do                                                                                                       \
    {                                                                                                        \
        if (vec)                                                                                             \
            REPDL_LAUNCH((coltile_kernel<CWv, true, NBv>), g, dim3(320), 0, st, in, out, M, N, factor); \
        else                                                                                                 \
            REPDL_LAUNCH((coltile_kernel<CWv, false, NBv>), g, dim3(320), 0, st, in, out, M, N, factor); \
    } while (0)
    if (cw == 64)
        REPDL_COLTILE(64, 1);
    else if (cw == 32)
        REPDL_COLTILE(32, 1);
    else if (two)
        REPDL_COLTILE(16, 2);
    else
        REPDL_COLTILE(16, 1);
#undef REPDL_COLTILE
    return repdl_launch_status();
}
