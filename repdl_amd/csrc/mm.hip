// Reproducible fp32 matrix multiplication for gfx950.
//
// Contract (RepDL backend/cpu/matrix_multiplication.cpp:22-34): every output
// element owns one accumulator that starts at +0.0f and receives exactly one
// fused multiply-add per k, k ascending.  Tiling over M and N and the way the
// operands are staged are free; the order along K is not, so K is never split
// across threads.
//
// Two families of kernels implement it.  mm_dma_kernel feeds v_mfma_f32_16x16x4_f32 from operand
// tiles moved from global memory straight into LDS; on gfx950 the instruction evaluates exactly such
// a chain (four k per instruction, ascending; checked on the device before first use, see
// mfma_check.hip).  mm_kernel is the same computation with one v_fma_f32 per term; it runs when
// that check fails, when the matrix path is switched off, or when an operand tile spans more than
// 32 bits of byte offsets.
//
// mm_kernel layout: a workgroup of 256 threads computes a 128x128 tile of C; each thread
// an 8x8 micro-tile held in registers (rows ty*4+{0..3} and 64+ty*4+{0..3},
// columns tx*4+{0..3} and 64+tx*4+{0..3}).  Both operands are staged through LDS
// k-major (As[k][m], Bs[k][n]) so the inner loop reads its 8+8 operands with
// four ds_read_b128 and issues 64 v_fma_f32.  Global loads for tile t+1 are
// issued before the FMAs of tile t (register prefetch, two LDS buffers).
#include "common.h"

namespace
{
constexpr int BM = 128, BN = 128, BK = 16, NT = 256;
constexpr int LDA = BM + 4; // padded row of the transposing store path
constexpr int LDB = BN + 4;
constexpr int GROUP_M = 8; // tile-rows walked together (see the tile order in the kernel)

struct Frag
{
    float4 v[2];
};

// One operand tile = 128 "r" positions (rows of C for A, columns of C for B) by
// BK steps of k.  KC: element (r,k) at X[r*ld + k] (k contiguous in memory);
// otherwise element (r,k) at X[k*ld + r] (r contiguous).
template <bool KC>
__device__ __forceinline__ void load_tile(const float *__restrict__ X, int64_t ld, int64_t R,
                                          int64_t K, int64_t r0, int64_t k0, bool vec_ok, int tid,
                                          Frag &f)
{
#pragma unroll
    for (int i = 0; i < 2; i++)
    {
        int idx = tid + NT * i;
        int64_t r, k;
        if (KC)
        {
            r = r0 + (idx >> 2);
            k = k0 + ((idx & 3) << 2);
        }
        else
        {
            k = k0 + (idx >> 5);
            r = r0 + ((idx & 31) << 2);
        }
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (KC)
        {
            if (r < R)
            {
                const float *p = X + r * ld + k;
                if (vec_ok && k + 3 < K)
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
            if (k < K)
            {
                const float *p = X + k * ld + r;
                if (vec_ok && r + 3 < R)
                    v = *reinterpret_cast<const float4 *>(p);
                else
                {
                    if (r + 0 < R) v.x = p[0];
                    if (r + 1 < R) v.y = p[1];
                    if (r + 2 < R) v.z = p[2];
                    if (r + 3 < R) v.w = p[3];
                }
            }
        }
        f.v[i] = v;
    }
}

template <bool KC, int LD>
__device__ __forceinline__ void store_tile(float *__restrict__ S, int tid, const Frag &f)
{
#pragma unroll
    for (int i = 0; i < 2; i++)
    {
        int idx = tid + NT * i;
        if (KC)
        {
            int r = idx >> 2, k = (idx & 3) << 2;
            S[(k + 0) * LD + r] = f.v[i].x;
            S[(k + 1) * LD + r] = f.v[i].y;
            S[(k + 2) * LD + r] = f.v[i].z;
            S[(k + 3) * LD + r] = f.v[i].w;
        }
        else
        {
            int k = idx >> 5, r = (idx & 31) << 2;
            *reinterpret_cast<float4 *>(&S[k * LD + r]) = f.v[i];
        }
    }
}

__device__ __forceinline__ void fma_step(const float *__restrict__ As, const float *__restrict__ Bs,
                                         int kk, int ty, int tx, float (&acc)[8][8])
{
    float4 a0 = *reinterpret_cast<const float4 *>(&As[kk * LDA + ty * 4]);
    float4 a1 = *reinterpret_cast<const float4 *>(&As[kk * LDA + 64 + ty * 4]);
    float4 b0 = *reinterpret_cast<const float4 *>(&Bs[kk * LDB + tx * 4]);
    float4 b1 = *reinterpret_cast<const float4 *>(&Bs[kk * LDB + 64 + tx * 4]);
    float a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
    float b[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++)
            acc[i][j] = __fmaf_rn(a[i], b[j], acc[i][j]);
}

// TA: A is stored [K,M]; TB: B is stored [N,K].
template <bool TA, bool TB>
__global__ __launch_bounds__(NT) void mm_kernel(const float *__restrict__ A,
                                                const float *__restrict__ B, float *__restrict__ C,
                                                const float *__restrict__ bias, int64_t M, int64_t N,
                                                int64_t K, int avec, int bvec, int cvec, int64_t gx, int64_t gy,
                                                int64_t ntiles8)
{
    constexpr bool A_KC = !TA; // A[m*K + k]
    constexpr bool B_KC = TB;  // B[n*K + k]
    __shared__ __attribute__((aligned(16))) float As[2][BK * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    // Tile order.  Workgroups are handed to the 8 XCDs round-robin by linear id, and
    // each XCD has its own L2: give every XCD one contiguous band of tile ids, and walk
    // the tiles of a band in groups of GROUP_M tile-rows, column by column, so that the
    // tiles resident on one XCD at a time share A row panels and B column panels.
    int64_t tile = blockIdx.x;
    if (tile < ntiles8)
        tile = (tile & 7) * (ntiles8 >> 3) + (tile >> 3);
    const int64_t group_sz = (int64_t)GROUP_M * gx;
    const int64_t group = tile / group_sz;
    const int64_t first_row = group * GROUP_M;
    const int64_t rows_here = (gy - first_row < GROUP_M) ? gy - first_row : GROUP_M;
    const int64_t in_group = tile - group * group_sz;
    const int64_t trow = first_row + in_group % rows_here, tcol = in_group / rows_here;
    const int64_t m0 = trow * BM, n0 = tcol * BN;
    const int64_t lda = TA ? M : K, ldb = TB ? K : N;

    float acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++)
            acc[i][j] = 0.0f;

    const int64_t nkt = (K + BK - 1) / BK;
    Frag fa, fb;
    if (nkt > 0)
    {
        load_tile<A_KC>(A, lda, M, K, m0, 0, avec, tid, fa);
        load_tile<B_KC>(B, ldb, N, K, n0, 0, bvec, tid, fb);
        store_tile<A_KC, LDA>(As[0], tid, fa);
        store_tile<B_KC, LDB>(Bs[0], tid, fb);
    }
    __syncthreads();

    for (int64_t kt = 0; kt < nkt; kt++)
    {
        const int cur = (int)(kt & 1);
        const bool more = kt + 1 < nkt;
        if (more)
        {
            load_tile<A_KC>(A, lda, M, K, m0, (kt + 1) * BK, avec, tid, fa);
            load_tile<B_KC>(B, ldb, N, K, n0, (kt + 1) * BK, bvec, tid, fb);
        }
        const int64_t krem = K - kt * BK;
        if (krem >= BK)
        {
#pragma unroll
            for (int kk = 0; kk < BK; kk++)
                fma_step(As[cur], Bs[cur], kk, ty, tx, acc);
        }
        else
        {
            for (int kk = 0; kk < (int)krem; kk++)
                fma_step(As[cur], Bs[cur], kk, ty, tx, acc);
        }
        if (more)
        {
            store_tile<A_KC, LDA>(As[cur ^ 1], tid, fa);
            store_tile<B_KC, LDB>(Bs[cur ^ 1], tid, fb);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 8; i++)
    {
        int64_t m = m0 + ty * 4 + (i & 3) + (i >> 2) * 64;
        if (m >= M)
            continue;
#pragma unroll
        for (int jh = 0; jh < 2; jh++)
        {
            int64_t n = n0 + tx * 4 + jh * 64;
            float *p = C + m * N + n;
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; j++)
            {
                v[j] = acc[i][jh * 4 + j];
                if (bias != nullptr && n + j < N)
                    v[j] = v[j] + bias[n + j]; // one rounded add after the chain
            }
            if (cvec && n + 3 < N)
                *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
            else
            {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (n + j < N)
                        p[j] = v[j];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// mm_dma_kernel: operands whose rows start on 16-byte boundaries, any M, N, K; a batch of products.
//
// The operands never pass through registers on their way to LDS: global_load_lds_dwordx4 moves 16
// bytes per lane from global memory straight into LDS, at consecutive lanes' consecutive 16-byte
// slots from an LDS base in M0.  So the layout of a k-tile in LDS is whatever order the lanes are
// given, and both operand orientations have an order that the matrix instruction can read without
// bank conflicts.  The instruction is v_mfma_f32_16x16x4_f32: lane l supplies row (column) l%16 of
// its 16-row block at k = 4q + l/16 and the instruction adds k = 4q .. 4q+3 in ascending order.  A
// k-tile is NQ such quads.  With T = rows of C (A operand) or columns of C (B operand) per tile:
//
//   k contiguous in memory (A of NN/NT, B of NT/TT): lane -> (row r, quad q), 16 bytes = 4 consecutive
//     k of one row; LDS word q*4T + 4r + k%4.  A lane of the matrix instruction reads word
//     q*4T + 4r + l/16: 64 lanes, 64 banks.
//   r contiguous in memory (A of TN/TT, B of NN/TN): lane -> (k%4, group of 4 rows), 16 bytes = 4
//     consecutive rows at one k; LDS word q*4T + 16(r/4) + 4(k%4) + r%4, again one bank per lane.
//
// NB >= 3 LDS buffers per operand.  Quad by quad a wave reads its operands D quads ahead of the
// matrix instructions that use them (a ring of D+1 register sets); the one barrier per k-tile sits
// D quads before the tile's end, where the next tile's first reads begin, and is followed by the
// DMA of the tile NB-1 ahead into the buffer whose reads ended a whole tile ago -- so nobody waits
// on LDS reads at the barrier, and a DMA has NB-2 tiles of matrix work to land in (small tiles need
// several: a 64x64x32 tile is 0.4 us of matrix work, less than one trip to HBM).  The loop holds no
// vector ALU instruction at all.
//
// Edges.  A tile that hangs over the lower or right edge of C loads, for the rows it does not have,
// the operand's last rows again (the lane's address is clamped once, before the loop) and never
// stores what it computes from them.  A last k-tile of fewer than NQ quads is loaded with the lanes
// of the missing quads switched off and runs that many quads.  The up to three k past the last
// whole quad are added afterwards with one v_fma_f32 per term and output, operands read straight
// from global memory: the same chain step as the matrix instruction's.  So nothing is padded and
// no accumulator that is -0 is touched.
//
// DW > 0: the workgroup has DW more waves that issue all the DMA and do nothing else; they meet the
// computing waves at the same barriers (one before the loop, one per whole k-tile) and leave after
// the last one, when every load has landed.
//
// Batch: blockIdx.y selects one of several products with the same shapes, operand b at X + b * stride
// (stride 0: shared by all).  `cbias` is added per column, `rbias` per row (one rounded addition after
// the chain, whichever is given; at most one is).
__device__ __forceinline__ void dma16(const void *base, uint32_t voff, uint32_t lds_byte)
{
    // M0 = LDS byte address of lane 0's slot
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(base), "s"(lds_byte)
                 : "memory", "m0");
}

__device__ __forceinline__ void dma4(const void *base, uint32_t voff, uint32_t lds_byte)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(voff), "s"(base), "s"(lds_byte)
                 : "memory", "m0");
}

struct MmBatch
{
    int64_t a, b, c; // elements between consecutive products' operands and results
};

template <bool TA, bool TB, int FM, int FN, int WGM, int WGN, int NQ, int D, int NB, int DW, int VEC>
__global__ __launch_bounds__(64 * (WGM * WGN + DW)) void mm_dma_kernel(const float *__restrict__ A, const float *__restrict__ B,
                                                               float *__restrict__ C, const float *__restrict__ cbias,
                                                               const float *__restrict__ rbias, int64_t M, int64_t N,
                                                               int64_t K, int64_t gx, int64_t gy, int64_t ntiles8, MmBatch batch)
{
    constexpr int NW = WGM * WGN;
    constexpr int TM = 16 * FM * WGM, TN = 16 * FN * WGN;
    constexpr bool A_KC = !TA, B_KC = TB;
    constexpr int QSA = 4 * TM, QSB = 4 * TN;     // LDS words per quad
    constexpr int OPA = NQ * QSA, OPB = NQ * QSB; // LDS words per k-tile
    constexpr int R = D + 1;                      // register sets in the ring
    static_assert(NQ % R == 0 && D >= 1 && D < NQ, "ring must divide the k-tile");
    static_assert(NB >= 3, "a buffer being read, one landed or landing, one being filled");
    static_assert(VEC == 4 || VEC == 1, "16-byte or 4-byte DMA lanes");
    static_assert((TM * NQ) % 64 == 0 && (TN * NQ) % 64 == 0, "a DMA instruction fills 64 slots");
    constexpr int SPW = 4 / VEC;                                      // slots per 16 bytes of the LDS image
    constexpr int NIA = TM * NQ * SPW / 64, NIB = TN * NQ * SPW / 64; // DMA instructions per k-tile
    constexpr int NI = DW > 0 ? DW : NW;                  // waves that issue them: DW waves that do nothing else, or all
    constexpr int CA = (NIA + NI - 1) / NI, CB = (NIB + NI - 1) / NI;
    static_assert(NB == 3 || (NIA % NI == 0 && NIB % NI == 0), "every wave must issue the same number of loads per tile");
    constexpr int INFLIGHT = (NB - 3) * (CA + CB); // loads of later tiles that may still be under way at a barrier
    static_assert(INFLIGHT < 64, "vmcnt is a 6-bit counter");
    typedef float v4f __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) float smem[]; // [NB][OPA] then [NB][OPB]

    // where the dynamic LDS starts: DMA destinations are LDS byte addresses
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)smem;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int l16 = lane & 15, g = lane >> 4;
    const bool mover = DW > 0 && wave >= NW;              // a wave that only moves operands
    const int wi = DW > 0 ? (mover ? wave - NW : 0) : wave; // index among the issuing waves

    int64_t tile = blockIdx.x;
    if (tile < ntiles8)
        tile = (tile & 7) * (ntiles8 >> 3) + (tile >> 3);
    const int64_t group_sz = (int64_t)GROUP_M * gx;
    const int64_t group = tile / group_sz;
    const int64_t first_row = group * GROUP_M;
    const int64_t rows_here = (gy - first_row < GROUP_M) ? gy - first_row : GROUP_M;
    const int64_t in_group = tile - group * group_sz;
    const int64_t trow = first_row + in_group % rows_here, tcol = in_group / rows_here;
    const int64_t m0 = trow * TM, n0 = tcol * TN;
    const int64_t lda = TA ? M : K, ldb = TB ? K : N;
    A += (int64_t)blockIdx.y * batch.a;
    B += (int64_t)blockIdx.y * batch.b;
    C += (int64_t)blockIdx.y * batch.c;

    // DMA instruction e of an operand with T rows: 64 consecutive slots (16 bytes, or 4 when rows do not
    // start on 16-byte boundaries) of the tile's LDS image.  In 16-byte slots: slot s = quad (s / T),
    // position w = s % T in the quad -- a row's four k where k is contiguous, else four consecutive rows
    // at k = w % 4.  A 4-byte slot x is word x % 4 of the 16-byte slot x / 4.
    // Rows past the operand's last are clamped to rows it has.
    uint32_t va[CA], vb[CB];
    uint32_t la[CA], lb[CB];
    const int64_t am = M - m0, bn = N - n0; // rows (columns) of C this tile really has, if fewer than the tile's
#pragma unroll
    for (int t = 0; t < CA; t++)
    {
        const int e = wi + NI * t, x = 64 * e + lane, s = x / SPW, sub = x % SPW, q = s / TM, w = s % TM;
        if (A_KC)
        {
            const int64_t r = w < am ? w : am - 1;
            va[t] = (uint32_t)((r * lda + 4 * q + sub) * 4);
        }
        else if (VEC == 4)
        {
            const int64_t r = (w & ~3) + 3 < am ? (w & ~3) : am - 4;
            va[t] = (uint32_t)(((int64_t)(4 * q + (w & 3)) * lda + r) * 4);
        }
        else
        {
            const int64_t r = (w & ~3) + sub < am ? (w & ~3) + sub : am - 1;
            va[t] = (uint32_t)(((int64_t)(4 * q + (w & 3)) * lda + r) * 4);
        }
        la[t] = __builtin_amdgcn_readfirstlane(lds0 + 64 * e * 4 * VEC);
    }
#pragma unroll
    for (int t = 0; t < CB; t++)
    {
        const int e = wi + NI * t, x = 64 * e + lane, s = x / SPW, sub = x % SPW, q = s / TN, w = s % TN;
        if (B_KC)
        {
            const int64_t r = w < bn ? w : bn - 1;
            vb[t] = (uint32_t)((r * ldb + 4 * q + sub) * 4);
        }
        else if (VEC == 4)
        {
            const int64_t r = (w & ~3) + 3 < bn ? (w & ~3) : bn - 4;
            vb[t] = (uint32_t)(((int64_t)(4 * q + (w & 3)) * ldb + r) * 4);
        }
        else
        {
            const int64_t r = (w & ~3) + sub < bn ? (w & ~3) + sub : bn - 1;
            vb[t] = (uint32_t)(((int64_t)(4 * q + (w & 3)) * ldb + r) * 4);
        }
        lb[t] = __builtin_amdgcn_readfirstlane(lds0 + NB * OPA * 4 + 64 * e * 4 * VEC);
    }
    const char *a_base = reinterpret_cast<const char *>(A_KC ? A + m0 * lda : A + m0);
    const char *b_base = reinterpret_cast<const char *>(B_KC ? B + n0 * ldb : B + n0);
    const int64_t a_step = (A_KC ? (int64_t)(4 * NQ) : (int64_t)(4 * NQ) * lda) * 4;
    const int64_t b_step = (B_KC ? (int64_t)(4 * NQ) : (int64_t)(4 * NQ) * ldb) * 4;
    // k-tiles: nkt whole ones, then one of tq < NQ whole quads (if any), whose DMA is predicated
    // by quad -- the quads it lacks lie past the end of the operands
    const int64_t nkt = K / (4 * NQ);
    const int tq = (int)((K / 4) % NQ);
    const int64_t ntile = nkt + (tq > 0 ? 1 : 0);
    auto move = [&](const char *base, uint32_t voff, uint32_t lds_byte) {
        if (VEC == 4)
            dma16(base, voff, lds_byte);
        else
            dma4(base, voff, lds_byte);
    };
    auto issue = [&](int buf, bool tail) {
#pragma unroll
        for (int t = 0; t < CA; t++)
            if (NIA % NI == 0 || wi + NI * t < NIA)
            {
                if (!tail)
                    move(a_base, va[t], la[t] + buf * OPA * 4);
                else if ((64 * (wi + NI * t) + lane) / (SPW * TM) < tq)
                    move(a_base, va[t], la[t] + buf * OPA * 4);
            }
#pragma unroll
        for (int t = 0; t < CB; t++)
            if (NIB % NI == 0 || wi + NI * t < NIB)
            {
                if (!tail)
                    move(b_base, vb[t], lb[t] + buf * OPB * 4);
                else if ((64 * (wi + NI * t) + lane) / (SPW * TN) < tq)
                    move(b_base, vb[t], lb[t] + buf * OPB * 4);
            }
        a_base += a_step;
        b_base += b_step;
    };

    if (mover)
    {
        // the same barriers as the computing waves, one per k-tile: wait for the own share of the
        // next tile, meet, refill the buffer whose reads ended a tile ago
        if (ntile > 0)
        {
#pragma unroll
            for (int u = 0; u < NB - 1; u++)
                if (u < ntile)
                    issue(u, u == nkt);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
        int buf = NB - 1;
        for (int64_t kt = 0; kt < nkt; kt++)
        {
            if (INFLIGHT > 0 && kt + NB - 2 < nkt)
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(INFLIGHT) : "memory");
            else
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (kt + NB - 1 < ntile)
                issue(buf, kt + NB - 1 == nkt);
            buf = buf + 1 == NB ? 0 : buf + 1;
        }
        return;
    }

    v4f acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
            acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

    const int ma = wm * 16 * FM + l16, nb = wn * 16 * FN + l16;
    const float *ra = smem + (A_KC ? 4 * ma + g : 16 * (ma >> 2) + 4 * g + (ma & 3));
    const float *rb = smem + NB * OPA + (B_KC ? 4 * nb + g : 16 * (nb >> 2) + 4 * g + (nb & 3));
    float xa[R][FM], xb[R][FN];
    auto read_q = [&](int buf, int q, float(&a)[FM], float(&b)[FN]) {
#pragma unroll
        for (int i = 0; i < FM; i++)
            a[i] = ra[buf * OPA + q * QSA + 64 * i];
#pragma unroll
        for (int j = 0; j < FN; j++)
            b[j] = rb[buf * OPB + q * QSB + 64 * j];
    };
    auto mfma_q = [&](float(&a)[FM], float(&b)[FN]) {
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int j = 0; j < FN; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[j], acc[i][j], 0, 0, 0);
    };

    if (ntile > 0)
    {
#pragma unroll
        for (int u = 0; u < NB - 1; u++)
            if (DW == 0 && u < ntile)
                issue(u, u == nkt);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
#pragma unroll
        for (int q = 0; q < D; q++)
            read_q(0, q, xa[q], xb[q]);
    }
    for (int64_t kt = 0; kt < nkt; kt += NB)
    {
#pragma unroll
        for (int u = 0; u < NB; u++)
        {
            if (kt + u >= nkt)
                break;
            const bool more1 = kt + u + 1 < ntile, more_dma = kt + u + NB - 1 < ntile;
#pragma unroll
            for (int q = 0; q < NQ; q++)
            {
                if (q == NQ - D)
                {
                    // the next tile (this wave's share) has landed; after the barrier everyone's has,
                    // and every read of the tile before this one has long been consumed
                    if (DW > 0)
                        ;
                    else if (INFLIGHT > 0 && kt + u + NB - 2 < nkt)
                        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(INFLIGHT) : "memory");
                    else
                        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    if (DW == 0 && more_dma)
                        issue((u + NB - 1) % NB, kt + u + NB - 1 == nkt);
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
    if (tq > 0)
    {
        // the last k-tile: its first D quads are in the ring already, it has landed and been
        // published by the barrier of the tile before it (or by the one above)
        const int ub = (int)(nkt % NB);
        const float *rat = ra + ub * OPA, *rbt = rb + ub * OPB;
#pragma unroll
        for (int q = 0; q < NQ - 1; q++)
        {
            if (q >= tq)
                break;
            const int qq = q + D;
            if (qq < NQ)
            {
#pragma unroll
                for (int i = 0; i < FM; i++)
                    xa[qq % R][i] = rat[qq * QSA + 64 * i];
#pragma unroll
                for (int j = 0; j < FN; j++)
                    xb[qq % R][j] = rbt[qq * QSB + 64 * j];
            }
            __builtin_amdgcn_sched_barrier(0);
            mfma_q(xa[q % R], xb[q % R]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    const int64_t mw = m0 + wm * 16 * FM + 4 * g, nw = n0 + wn * 16 * FN + l16; // this lane's first row and column
    // the k past the last whole quad (K not a multiple of 4: neither operand has k contiguous): one
    // fused multiply-add per term, operands from global memory
    for (int64_t k = K & ~(int64_t)3; k < K; k++)
    {
        float bk[FN];
#pragma unroll
        for (int j = 0; j < FN; j++)
        {
            const int64_t nn = nw + 16 * j;
            bk[j] = nn < N ? (B_KC ? B[nn * ldb + k] : B[k * ldb + nn]) : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int r = 0; r < 4; r++)
            {
                const int64_t m = mw + 16 * i + r;
                const float av = m < M ? (A_KC ? A[m * lda + k] : A[k * lda + m]) : 0.0f;
#pragma unroll
                for (int j = 0; j < FN; j++)
                    acc[i][j][r] = __builtin_fmaf(av, bk[j], acc[i][j][r]);
            }
    }

    // bias: one rounded add per output after its chain; a lane owns FN columns and 4 FM rows
    float bv[FN];
#pragma unroll
    for (int j = 0; j < FN; j++)
        bv[j] = cbias != nullptr && nw + 16 * j < N ? cbias[nw + 16 * j] : 0.0f;
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int r = 0; r < 4; r++)
        {
            const int64_t m = mw + 16 * i + r;
            if (m >= M)
                continue;
            const float rv = rbias != nullptr ? rbias[m] : 0.0f;
#pragma unroll
            for (int j = 0; j < FN; j++)
            {
                const int64_t nn = nw + 16 * j;
                float v = acc[i][j][r];
                if (cbias != nullptr)
                    v = v + bv[j];
                if (rbias != nullptr)
                    v = v + rv;
                if (nn < N)
                    __builtin_nontemporal_store(v, &C[m * N + nn]);
            }
        }
}

// Whether mm_dma_kernel with this tile can take the product: lane offsets inside an operand tile
// within 32 bits and, with 16-byte DMA lanes (vec4), at least four rows (columns) where rows are
// contiguous (the edge clamp steps back by four).
template <int FM, int FN, int WGM, int WGN, int NQ>
bool dma_applies(int64_t M, int64_t N, int64_t K, int transA, int transB, bool vec4, int64_t nbatch = 1)
{
    constexpr int TM = 16 * FM * WGM, TN = 16 * FN * WGN, BKQ = 4 * NQ;
    if (M < 1 || N < 1 || K < 1 || nbatch < 1 || nbatch > 65535)
        return false;
    if (vec4 && ((transA && M < 4) || (!transB && N < 4)))
        return false;
    const int64_t lda = transA ? M : K, ldb = transB ? K : N;
    const int64_t ea = transA ? (int64_t)BKQ * lda + TM : (int64_t)TM * lda + BKQ;
    const int64_t eb = transB ? (int64_t)TN * ldb + BKQ : (int64_t)BKQ * ldb + TN;
    return ea * 4 < (1LL << 32) && eb * 4 < (1LL << 32) && repdl_cdiv(M, TM) * repdl_cdiv(N, TN) <= REPDL_I32_MAX;
}

template <bool TA, bool TB, int FM, int FN, int WGM, int WGN, int NQ, int D, int NB, int DW = 0, int VEC = 4>
int launch_dma_t(const float *A, const float *B, float *C, const float *cbias, const float *rbias, int64_t M, int64_t N,
                 int64_t K, int64_t nbatch, MmBatch batch, hipStream_t s)
{
    constexpr int TM = 16 * FM * WGM, TN = 16 * FN * WGN;
    constexpr size_t shmem = (size_t)NB * NQ * 4 * (TM + TN) * sizeof(float);
    static_assert(shmem <= 160 * 1024, "LDS of one CU");
    const int64_t gx = repdl_cdiv(N, TN), gy = repdl_cdiv(M, TM);
    const int64_t ntiles8 = (gx * gy) & ~(int64_t)7;
    auto kern = &mm_dma_kernel<TA, TB, FM, FN, WGM, WGN, NQ, D, NB, DW, VEC>;
    if (shmem > 48 * 1024)
    {
        hipError_t e = REPDL_FUNC_SET_ATTRIBUTE(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)shmem);
        if (e != hipSuccess)
            return (int)e;
    }
    REPDL_LAUNCH(kern, dim3((unsigned)(gx * gy), (unsigned)nbatch), dim3(64 * (WGM * WGN + DW)), shmem, s, A, B, C, cbias, rbias, M,
                       N, K, gx, gy, ntiles8, batch);
    return repdl_launch_status();
}

template <int FM, int FN, int WGM, int WGN, int NQ, int D, int NB, int DW = 0, int VEC = 4>
int launch_dma(const float *A, const float *B, float *C, const float *cbias, const float *rbias, int64_t M, int64_t N, int64_t K,
               int transA, int transB, int64_t nbatch, MmBatch batch, hipStream_t s)
{
    if (!transA && !transB)
        return launch_dma_t<false, false, FM, FN, WGM, WGN, NQ, D, NB, DW, VEC>(A, B, C, cbias, rbias, M, N, K, nbatch, batch, s);
    if (transA && !transB)
        return launch_dma_t<true, false, FM, FN, WGM, WGN, NQ, D, NB, DW, VEC>(A, B, C, cbias, rbias, M, N, K, nbatch, batch, s);
    if (!transA && transB)
        return launch_dma_t<false, true, FM, FN, WGM, WGN, NQ, D, NB, DW, VEC>(A, B, C, cbias, rbias, M, N, K, nbatch, batch, s);
    return launch_dma_t<true, true, FM, FN, WGM, WGN, NQ, D, NB, DW, VEC>(A, B, C, cbias, rbias, M, N, K, nbatch, batch, s);
}

// The tile for a batch of products, and its launch; REPDL_E_UNSUPPORTED if mm_dma_kernel cannot
// take the operands.  Shares of the chip's matrix rate (145 TFLOP/s on the 128x128 tile with many
// tiles per CU) by tiles per CU r, measured on whole-tile shapes with K = 2048 (a CU holds two or
// three workgroups of the first two tiles at once).  "+4" = four more waves that only issue the DMA:
// it pays while a CU holds one workgroup (a lone wave per SIMD issues a DMA instruction about every
// 60 clocks, two matrix instructions' worth of its chain), and costs 10 % on 8192^3.
//   128x128, 8 waves of 64x32, k-tile 16:  r = 1 0.82 (0.88 with +4, 2048^3 119 -> 128 TFLOP/s: what four rounds
//     of 64x64 tiles reach, which is what the cost picks there), 2 0.94, 3 0.88, 4 0.95, 5 0.83, 6 0.95, 7 0.89,
//     more 0.97 (an odd count leaves a last round of one workgroup per CU);
//   64x64: r = 1 0.73, 2 0.84, 3 0.875, 4..7 0.89, more 0.92, on
//     r = 1, 2: 8 waves of 16x32, k-tile 32, four buffers, +4 (1024^2 x 2048: 106 TFLOP/s, against 95 without
//            the four, 81-83 with four waves of 32x32 or with three buffers; 2048 x 1024 x 2048: 122); chains of
//            1024 terms and fewer are over before the fourth buffer pays: three buffers, +4 only at r = 1;
//     r = 1: a CU's one workgroup has the whole LDS, and what it lacks is bytes in flight (16 KB per k-tile of
//            32, two tiles under way, a microsecond from request to LDS: 32 GB/s per CU, two thirds of what the
//            chains could take).  k-tiles of 64: three buffers from 513 to 1024 terms (1024^3 0.0246 -> 0.0237 ms), four
//            and operands read three quads ahead beyond (1024^2 x 2048 -3 %, x 4096 -4 %, x 8192 -7 %; 768 x 1024
//            x 1024 -18 %).  With two or more tiles per CU the same forms are 10-25 % slower than the ones above:
//            their 96-128 KB leave room for one workgroup only.
//     r = 3: 8 waves of 16x32, three buffers (1536 x 2048 x 2048: 127 against 125);
//     r >= 4: 4 waves of 32x32, k-tile 16, six workgroups to a CU (2048^2 x 2048: 128 against 121);
//   32x32, 4 waves of one 16x16 block, k-tile 64, read-ahead 7 quads, five buffers, +4: 0.445 at r = 1, 0.52 beyond;
//   64x32, 8 such waves, +4: 0.60 -- for C with fewer 64x64 tiles than CUs: one or two blocks per SIMD, each
//     a chain of dependent instructions (64 x 4096 x 4096: 58 -> 66 TFLOP/s with the four, 128 x 4096 x 4096:
//     80 -> 91, 256 x 1024 x 8192: 62 -> 72; more buffers changed nothing; 64x16 tiles were slower)
// (8192^3 NT: 145 / 138 TFLOP/s on the first two; 3072 x 4096 x 2048: 106-139 by layout / 132-136;
// 4096 x 2048 x 2048: 136 / 132; 5120 x 4096 x 2048: 121 / 134; 1408^2 x 4096: 57 / 108.)  A tile that hangs
// over an edge costs what a whole one does.
// Operand rows off 16-byte boundaries: the same tiles with 4-byte DMA lanes, four times the DMA
// instructions (8190^3 NT / NN / TN: 120 / 124 / 137 TFLOP/s, against 96 through registers); the
// one-workgroup-per-CU forms then take eight moving waves.
int mm_dma_dispatch(const float *A, const float *B, float *C, const float *cbias, const float *rbias, int64_t M, int64_t N,
                    int64_t K, int transA, int transB, int avec, int bvec, int64_t nbatch, MmBatch batch, hipStream_t s)
{
    auto rounds = [&](int64_t tm, int64_t tn) { return repdl_cdiv(repdl_cdiv(M, tm) * repdl_cdiv(N, tn) * nbatch, 256); };
    const bool vec4 = avec && bvec; // else rows off 16-byte boundaries: 4-byte DMA lanes, four times the DMA instructions
    double best = 1e300;
    int pick = 0;
    if (dma_applies<4, 2, 2, 4, 4>(M, N, K, transA, transB, vec4, nbatch))
    {
        const int64_t r = rounds(128, 128);
        static const double e128[8] = {0.82, 0.94, 0.88, 0.95, 0.83, 0.95, 0.89, 0.97};
        const double c = (double)r * 16384.0 / e128[r < 8 ? r - 1 : 7];
        if (c < best)
            best = c, pick = 1;
    }
    if (dma_applies<1, 2, 4, 2, 8>(M, N, K, transA, transB, vec4, nbatch))
    {
        const int64_t r = rounds(64, 64);
        const double c = (double)r * 4096.0 / (r >= 8 ? 0.92 : r >= 4 ? 0.89 : r == 3 ? 0.875 : r == 2 ? 0.84 : 0.73);
        if (c < best)
        {
            const bool wide_k = r == 1 && K > 512 && dma_applies<1, 2, 4, 2, 16>(M, N, K, transA, transB, vec4, nbatch);
            best = c;
            pick = r >= 4 ? 3 : r == 3 ? 6 : wide_k ? (K > 1024 ? 8 : 9) : K > 1024 ? 2 : r == 1 ? 7 : 6;
        }
    }
    if (dma_applies<1, 1, 2, 2, 16>(M, N, K, transA, transB, vec4, nbatch))
    {
        const int64_t r = rounds(32, 32);
        const double c = (double)r * 1024.0 / (r >= 2 ? 0.52 : 0.445);
        if (c < best)
            best = c, pick = 4;
    }
    if (dma_applies<1, 1, 4, 2, 16>(M, N, K, transA, transB, vec4, nbatch))
    {
        const double c = (double)rounds(64, 32) * 2048.0 / 0.60;
        if (c < best)
            best = c, pick = 5;
    }
    if (!vec4)
        switch (pick)
        {
        case 1:
            repdl_route_note(REPDL_ROUTE_MM_UNALIGNED_128);
            return launch_dma<4, 2, 2, 4, 4, 1, 3, 0, 1>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
        case 2:
        case 6:
        case 7:
        case 8:
        case 9:
            // one 64x64 tile per CU: eight waves that only move (1001^2 x 2049: 54 TFLOP/s on the
            // four-wave form, 87 with four movers, 96 with eight)
            if (rounds(64, 64) == 1)
            {
                repdl_route_note(REPDL_ROUTE_MM_UNALIGNED_64_MOVERS);
                return launch_dma<1, 2, 4, 2, 8, 1, 4, 8, 1>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
            }
            repdl_route_note(REPDL_ROUTE_MM_UNALIGNED_64);
            return launch_dma<1, 2, 4, 2, 8, 1, 3, 0, 1>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
        case 3:
            repdl_route_note(REPDL_ROUTE_MM_UNALIGNED_QUAD);
            return launch_dma<2, 2, 2, 2, 4, 1, 3, 0, 1>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
        case 4:
        case 5:
            repdl_route_note(REPDL_ROUTE_MM_UNALIGNED_32);
            return launch_dma<1, 1, 2, 2, 16, 7, 5, 8, 1>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
        default:
            return REPDL_E_UNSUPPORTED;
        }
    switch (pick)
    {
    case 1:
        // Both operands row-contiguous and chains several times longer than C is wide (a Linear layer's
        // weight gradient, the batch as K): the same tile as four waves of 64x64.  With eight waves
        // 4096^2 x 65536 TN ran at 110-135 TFLOP/s depending on the machine (3.5 TB/s from memory: the tiles
        // of an XCD stop sharing their operand rows as they drift apart along K), with four at 140; on
        // every other shape and layout the eight-wave form is the faster one by 4-6 %.
        if (transA && !transB && K >= 4 * (M > N ? M : N))
        {
            repdl_route_note(REPDL_ROUTE_MM_128_TALL);
            return launch_dma_t<true, false, 4, 4, 2, 2, 4, 1, 3>(A, B, C, cbias, rbias, M, N, K, nbatch, batch, s);
        }
        repdl_route_note(REPDL_ROUTE_MM_128);
        return launch_dma<4, 2, 2, 4, 4, 1, 3>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
    case 2:
        repdl_route_note(REPDL_ROUTE_MM_64_FOUR_BUFFERS);
        return launch_dma<1, 2, 4, 2, 8, 1, 4, 4>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
    case 6:
        repdl_route_note(REPDL_ROUTE_MM_64_THREE_BUFFERS);
        return launch_dma<1, 2, 4, 2, 8, 1, 3>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
    case 3:
        repdl_route_note(REPDL_ROUTE_MM_64_QUAD);
        return launch_dma<2, 2, 2, 2, 4, 1, 3>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
    case 7:
        repdl_route_note(REPDL_ROUTE_MM_64_MOVERS);
        return launch_dma<1, 2, 4, 2, 8, 1, 3, 4>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
    case 9:
        repdl_route_note(REPDL_ROUTE_MM_64_WIDE_K);
        return launch_dma<1, 2, 4, 2, 16, 1, 3, 4>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
    case 8:
        repdl_route_note(REPDL_ROUTE_MM_64_DEEP);
        return launch_dma<1, 2, 4, 2, 16, 3, 4, 4>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
    case 4:
        repdl_route_note(REPDL_ROUTE_MM_32);
        return launch_dma<1, 1, 2, 2, 16, 7, 5, 4>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
    case 5:
        repdl_route_note(REPDL_ROUTE_MM_64X32);
        return launch_dma<1, 1, 4, 2, 16, 7, 5, 4>(A, B, C, cbias, rbias, M, N, K, transA, transB, nbatch, batch, s);
    default:
        return REPDL_E_UNSUPPORTED;
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
} // namespace


int repdl_mm_batched(const float *A, const float *B, float *C, const float *row_bias, int64_t M, int64_t N, int64_t K,
                     int transA, int transB, int64_t nbatch, int64_t strideA, int64_t strideB, int64_t strideC,
                     hipStream_t stream)
{
    if (!repdl_mfma_exact() || M < 1 || N < 1 || K < 1 || nbatch < 1)
        return REPDL_E_UNSUPPORTED;
    const int64_t lda = transA ? M : K, ldb = transB ? K : N;
    const int avec = aligned16(A) && lda % 4 == 0 && strideA % 4 == 0;
    const int bvec = aligned16(B) && ldb % 4 == 0 && strideB % 4 == 0;
    if (!avec || !bvec)
        return REPDL_E_UNSUPPORTED;
    return mm_dma_dispatch(A, B, C, nullptr, row_bias, M, N, K, transA, transB, avec, bvec, nbatch,
                           MmBatch{strideA, strideB, strideC}, stream);
}

REPDL_API int repdl_hip_mm(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                           int transA, int transB, void *stream)
{
    return repdl_hip_mm_bias(A, B, nullptr, C, M, N, K, transA, transB, stream);
}

REPDL_API int repdl_hip_mm_bias(const float *A, const float *B, const float *bias, float *C, int64_t M, int64_t N,
                                int64_t K, int transA, int transB, void *stream)
{
    REPDL_REQUIRE(M >= 0 && N >= 0 && K >= 0);
    if (M == 0 || N == 0)
        return REPDL_OK;
    REPDL_REQUIRE(C != nullptr);
    REPDL_REQUIRE(K == 0 || (A != nullptr && B != nullptr));
    const int64_t lda = transA ? M : K, ldb = transB ? K : N;
    const int avec = aligned16(A) && (lda % 4 == 0);
    const int bvec = aligned16(B) && (ldb % 4 == 0);
    hipStream_t s = repdl_stream(stream);
    if (repdl_mfma_exact())
    {
        // the kernel that moves operands straight into LDS, in 16-byte pieces where rows start on
        // 16-byte boundaries, else in 4-byte pieces; it declines operands whose tiles span more than
        // 32 bits of byte offsets (rows of tens of millions of elements), which take the kernel below
        const int rc = mm_dma_dispatch(A, B, C, bias, nullptr, M, N, K, transA, transB, avec, bvec, 1, MmBatch{0, 0, 0}, s);
        if (rc != REPDL_E_UNSUPPORTED)
            return rc;
    }
    const int64_t gx = repdl_cdiv(N, BN), gy = repdl_cdiv(M, BM);
    REPDL_REQUIRE(gx * gy <= REPDL_I32_MAX);
    const int64_t ntiles8 = (gx * gy) & ~(int64_t)7; // tiles covered by whole rounds over the 8 XCDs
    const int cvec = aligned16(C) && (N % 4 == 0);
    dim3 grid((unsigned)(gx * gy)), block(NT);
    repdl_route_note(REPDL_ROUTE_MM_FMA);
    if (!transA && !transB)
        REPDL_LAUNCH((mm_kernel<false, false>), grid, block, 0, s, A, B, C, bias, M, N, K, avec, bvec, cvec, gx, gy,
                           ntiles8);
    else if (transA && !transB)
        REPDL_LAUNCH((mm_kernel<true, false>), grid, block, 0, s, A, B, C, bias, M, N, K, avec, bvec, cvec, gx, gy,
                           ntiles8);
    else if (!transA && transB)
        REPDL_LAUNCH((mm_kernel<false, true>), grid, block, 0, s, A, B, C, bias, M, N, K, avec, bvec, cvec, gx, gy,
                           ntiles8);
    else
        REPDL_LAUNCH((mm_kernel<true, true>), grid, block, 0, s, A, B, C, bias, M, N, K, avec, bvec, cvec, gx, gy,
                           ntiles8);
    return repdl_launch_status();
}
