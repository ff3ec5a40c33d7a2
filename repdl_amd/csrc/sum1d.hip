// sum1d: the strictly sequential binary32 sum  s = +0; for i: s = RN(s + x[i])
// (RepDL backend/cpu/summation.cpp:12-20), evaluated exactly but mostly in
// parallel.
//
// Idea.  While the running sum stays inside one binade [2^E, 2^(E+1)) with one sign,
// it is an integer S in [2^23, 2^24) times the quantum q = 2^(E-23), and adding x is
//     S  ->  S + a[S & 1],   a[p] = X + [r > 1/2] + [r == 1/2] * ((p + X) & 1)
// where sign*x/q = X + r, X integer, 0 <= r < 1 (round to nearest, ties to even: only
// a tie looks at S, and only at its parity).  Such maps compose associatively:
//     (a then b)[p] = a[p] + b[(p + a[p]) & 1]
// so the map of a whole chunk is again one pair of integers, computable in any
// grouping.  Carrying, per starting parity, the minimum of the exact sums before
// rounding and the maximum of the rounded sums over all prefixes tells, once the real
// incoming S is known, whether the sum really stayed inside the binade (the map is
// valid) -- in O(1).
//
// Pipeline (n >= SUM1D_MIN_PARALLEL; shorter inputs take the serial kernel of sum.hip):
//   1. block sums in binary64 over blocks of 4096 elements        (parallel, reads x once)
//   2. exclusive prefix of the block sums                          (one workgroup)
//      (1 and 2 run twice: the second time each element counts for what it is worth on
//      the grid of the state predicted the first time, see quantum_of)
//   3. per chunk of 64 elements: the binade/sign HYPOTHESIS is read off the binary64
//      prefix at the chunk start; tuple (a0,a1,lo0,hi0,lo1,hi1) of the chunk under that
//      hypothesis; tuples of groups of 8 chunks and of the block (64 chunks) wherever
//      the hypotheses agree                                        (parallel, reads x again)
//      (3b: tuples of super-blocks of 64 blocks, same rule)
//   4. one wave walks the super-blocks in order with the true state: a node whose
//      hypothesis matches the state and whose tuple is valid for it is applied in O(1);
//      otherwise its children are tried -- the 64 blocks of a super-block, the 8 groups
//      of a block, the 8 chunks of a group -- and a chunk that fails is replayed with 64
//      real binary32 additions.
// The hypotheses come from an approximation, but they only decide how much is replayed:
// every applied map is checked against the true state, so the result is the sequential
// sum bit for bit for every input (NaN, infinities, zeros and subnormal states simply
// fall through to the replay).
#include <mutex>

#include "common.h"

namespace
{
constexpr int CH = 64;            // elements per chunk
constexpr int BLK = 4096;         // elements per block (64 chunks)
constexpr int GROUPS = 8;         // groups of 8 chunks per block
constexpr int HYP_NONE = -1;      // no usable hypothesis: replay
constexpr int HYP_ANY = 0x200;    // every element is +-0: the identity for any state
constexpr int BIG = 1 << 26;      // "leaves the binade for sure"
constexpr int SAT = 1 << 28;      // saturation bound of all tuple fields

struct __attribute__((aligned(16))) Tup
{
    int t0, t1;   // S -> S + t[p] for starting parity p
    int lo0, hi0; // over all prefixes: min of (offset + X) before rounding, max of offset after
    int lo1, hi1;
    int hyp;      // (sign << 8) | biased exponent of the state this tuple assumes, or HYP_*
    int pad;
};

__device__ __forceinline__ int clampi(int v) { return v < -SAT ? -SAT : (v > SAT ? SAT : v); }

__device__ __forceinline__ Tup tup_identity(int hyp)
{
    Tup t;
    t.t0 = t.t1 = t.lo0 = t.hi0 = t.lo1 = t.hi1 = 0;
    t.hyp = hyp;
    t.pad = 0;
    return t;
}

// a then b (same hypothesis)
__device__ __forceinline__ Tup tup_compose(const Tup &a, const Tup &b)
{
    Tup c;
    const bool p0 = (a.t0 & 1) != 0;       // parity after a, starting even
    const bool p1 = ((1 + a.t1) & 1) != 0; // parity after a, starting odd
    const int bt0 = p0 ? b.t1 : b.t0, blo0 = p0 ? b.lo1 : b.lo0, bhi0 = p0 ? b.hi1 : b.hi0;
    const int bt1 = p1 ? b.t1 : b.t0, blo1 = p1 ? b.lo1 : b.lo0, bhi1 = p1 ? b.hi1 : b.hi0;
    c.t0 = clampi(a.t0 + bt0);
    c.t1 = clampi(a.t1 + bt1);
    c.lo0 = clampi(min(a.lo0, a.t0 + blo0));
    c.hi0 = clampi(max(a.hi0, a.t0 + bhi0));
    c.lo1 = clampi(min(a.lo1, a.t1 + blo1));
    c.hi1 = clampi(max(a.hi1, a.t1 + bhi1));
    c.hyp = a.hyp;
    c.pad = 0;
    return c;
}

// append element x (bit pattern ux, finite) to tuple t under hypothesis (sg, e)
__device__ __forceinline__ void tup_append(Tup &t, uint32_t ux, int sg, int e)
{
    int ex = (int)((ux >> 23) & 0xFFu);
    int m = (int)(ux & 0x7FFFFFu);
    if (ex == 0)
        ex = 1; // subnormal: same scale as the smallest normal, no implicit bit
    else
        m |= 0x800000;
    if (m == 0)
        return; // +-0 changes nothing
    const bool neg = (int)(ux >> 31) != sg; // the element pulls the magnitude down
    const int d = e - ex;
    int X, a0, a1;
    if (d < 0)
    {
        X = a0 = a1 = neg ? -BIG : BIG; // |x| >= 2^(E+1): out of the binade whatever S is
    }
    else if (d > 25)
    {
        X = neg ? -1 : 0; // |x| < q/4: rounds away, but a negative one dips below S first
        a0 = a1 = 0;
    }
    else
    {
        const int v = neg ? -m : m;
        X = v >> d; // floor
        const int rem = v & ((1 << d) - 1);
        const int half = d == 0 ? 0 : (1 << (d - 1));
        const int gt = (d != 0 && rem > half) ? 1 : 0;
        const int tie = (d != 0 && rem == half) ? 1 : 0;
        a0 = X + gt + (tie & (X & 1));       // S even: S + X has the parity of X
        a1 = X + gt + (tie & ((X + 1) & 1)); // S odd
    }
    // compose (t then this element)
    const bool p0 = (t.t0 & 1) != 0, p1 = ((1 + t.t1) & 1) != 0;
    const int ea0 = p0 ? a1 : a0, ea1 = p1 ? a1 : a0;
    t.lo0 = clampi(min(t.lo0, t.t0 + X));
    t.lo1 = clampi(min(t.lo1, t.t1 + X));
    t.t0 = clampi(t.t0 + ea0);
    t.t1 = clampi(t.t1 + ea1);
    t.hi0 = max(t.hi0, t.t0);
    t.hi1 = max(t.hi1, t.t1);
}

__device__ __forceinline__ Tup tup_shfl_down(const Tup &t, int delta)
{
    Tup r;
    r.t0 = __shfl_down(t.t0, delta, 64);
    r.t1 = __shfl_down(t.t1, delta, 64);
    r.lo0 = __shfl_down(t.lo0, delta, 64);
    r.hi0 = __shfl_down(t.hi0, delta, 64);
    r.lo1 = __shfl_down(t.lo1, delta, 64);
    r.hi1 = __shfl_down(t.hi1, delta, 64);
    r.hyp = __shfl_down(t.hyp, delta, 64);
    r.pad = 0;
    return r;
}

// hypotheses merge: ANY is a wildcard, NONE (or a disagreement) poisons
__device__ __forceinline__ int hyp_merge(int a, int b)
{
    if (a == HYP_ANY)
        return b;
    if (b == HYP_ANY)
        return a;
    return a == b ? a : HYP_NONE;
}

__device__ __forceinline__ Tup tup_join(const Tup &a, const Tup &b)
{
    const int h = hyp_merge(a.hyp, b.hyp);
    Tup c = tup_compose(a, b);
    c.hyp = h;
    return c;
}

// ---- the chains ------------------------------------------------------------------------------
// The same pipeline runs on `rows` independent chains at once (row sums of a matrix with few,
// long rows; the channel sums of an NCHW tensor): row r is blockIdx.y (blockIdx.x in the
// one-dimensional launches), its element i sits at
//     x + r*row_stride + (i / seglen)*seg_stride + i % seglen
// (sum1d and row sums: one segment, seglen = n; channel sums: a segment per image, seglen = H*W,
// which must then be a multiple of 16 so that the 16 elements of a thread and the float4 of the
// walk never straddle two segments, and n < 2^31 so that the division is a 32-bit one).  Every
// per-row array (block sums, prefixes, tuples) holds the rows back to back.
struct Chains
{
    int64_t n, row_stride, seg_stride, nblk, nsup;
    int seglen;    // (unused unless segmented)
    int segmented; // more than one segment
};

__device__ __forceinline__ const float *chain_ptr(const float *__restrict__ xr, const Chains &c, int64_t i)
{
    if (!c.segmented)
        return xr + i;
    const uint32_t sg = (uint32_t)i / (uint32_t)c.seglen;
    return xr + (int64_t)sg * c.seg_stride + ((uint32_t)i - sg * (uint32_t)c.seglen);
}

// ---- step 1: binary64 block sums -------------------------------------------------------
// 16 consecutive elements from i0 (a multiple of 16) of the chain at xr
__device__ __forceinline__ void load16(const float *__restrict__ xr, const Chains &c, int64_t i0, bool vec, float (&v)[16])
{
    const int64_t n = c.n;
    if (vec && i0 + 15 < n)
    {
        const float *x = chain_ptr(xr, c, i0) - i0;
#pragma unroll
        for (int q = 0; q < 4; q++)
        {
            const float4 f = reinterpret_cast<const float4 *>(x + i0)[q];
            v[4 * q + 0] = f.x;
            v[4 * q + 1] = f.y;
            v[4 * q + 2] = f.z;
            v[4 * q + 3] = f.w;
        }
    }
    else
    {
#pragma unroll
        for (int q = 0; q < 16; q++)
            v[q] = (i0 + q < n) ? *chain_ptr(xr, c, i0 + q) : 0.0f;
    }
}

__device__ __forceinline__ double wave_sum(double v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        v += __shfl_xor(v, off, 64);
    return v;
}

// The running sum moves by what an element is worth ON THE GRID of the binade the sum is in:
// S + x rounds to a multiple of the quantum q of S, so the step is x rounded to a multiple of
// q (ties aside).  Summing the elements exactly instead predicts the wrong state wherever
// that differs systematically -- a sum of 2^28 values from [0, 1) stops growing at 2^24, where
// every element is below q/2, while the exact sum goes on to 2^27 and every hypothesis after
// that point is wrong.  So the prediction is refined: a second pass rounds each element to
// the grid of the state the first pass predicted for its block, which models exactly that.
struct Quantum
{
    double q, inv_q; // q == 0: leave the element as it is
};

__device__ __forceinline__ Quantum quantum_of(double state)
{
    const uint32_t u = __float_as_uint((float)state);
    int e = (int)((u >> 23) & 0xFFu);
    Quantum r;
    if (e == 255 || state != state)
    {
        r.q = r.inv_q = 0.0;
        return r;
    }
    e = e < 1 ? 1 : e; // subnormal states share the smallest normal binade's grid, 2^-149
    r.q = __longlong_as_double((long long)(e - 150 + 1023) << 52);
    r.inv_q = __longlong_as_double((long long)(150 - e + 1023) << 52);
    return r;
}

__device__ __forceinline__ double quantise(float x, const Quantum &g)
{
    return g.q == 0.0 ? (double)x : rint((double)x * g.inv_q) * g.q;
}

// prev == nullptr: exact sums; else: sums of the elements rounded to the grid of the state
// prev[block] predicted by the previous pass.
__global__ __launch_bounds__(256) void sum1d_blocksum_kernel(const float *__restrict__ x, Chains c,
                                                             const double *__restrict__ prev,
                                                             double *__restrict__ bsum, int vec)
{
    __shared__ double part[4];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.y;
    x += row * c.row_stride;
    bsum += row * c.nblk;
    float v[16];
    load16(x, c, (int64_t)blockIdx.x * BLK + tid * 16, vec, v);
    Quantum g;
    g.q = g.inv_q = 0.0;
    if (prev != nullptr)
        g = quantum_of(prev[row * c.nblk + blockIdx.x]);
    double d = 0.0;
#pragma unroll
    for (int q = 0; q < 16; q++)
        d += quantise(v[q], g);
    d = wave_sum(d);
    if ((tid & 63) == 0)
        part[tid >> 6] = d;
    __syncthreads();
    if (tid == 0)
        bsum[blockIdx.x] = (part[0] + part[1]) + (part[2] + part[3]);
}

// ---- step 2: exclusive prefix of the block sums (one workgroup) ---------------------------
__global__ __launch_bounds__(256) void sum1d_prefix_kernel(const double *__restrict__ bsum,
                                                           double *__restrict__ prefix, int64_t nblk)
{
    __shared__ double seg[256];
    const int tid = threadIdx.x;
    bsum += (int64_t)blockIdx.x * nblk; // one workgroup per row
    prefix += (int64_t)blockIdx.x * nblk;
    const int64_t per = (nblk + 255) / 256;
    const int64_t b0 = tid * per, b1 = (b0 + per < nblk) ? b0 + per : nblk;
    double s = 0.0;
    for (int64_t b = b0; b < b1; b++)
        s += bsum[b];
    seg[tid] = s;
    __syncthreads();
    if (tid == 0)
    {
        double run = 0.0;
        for (int t = 0; t < 256; t++)
        {
            const double v = seg[t];
            seg[t] = run;
            run += v;
        }
    }
    __syncthreads();
    double run = seg[tid];
    for (int64_t b = b0; b < b1; b++)
    {
        prefix[b] = run;
        run += bsum[b];
    }
}

// ---- step 3: chunk and block tuples --------------------------------------------------------
__global__ __launch_bounds__(256) void sum1d_tuple_kernel(const float *__restrict__ x, Chains c,
                                                          const double *__restrict__ prefix,
                                                          Tup *__restrict__ T1, Tup *__restrict__ TG,
                                                          Tup *__restrict__ T2, int vec)
{
    __shared__ double wtot[4];
    __shared__ Tup wt[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t blk = blockIdx.x, row = blockIdx.y;
    x += row * c.row_stride;
    prefix += row * c.nblk;
    T1 += row * c.nblk * (BLK / CH);
    TG += row * c.nblk * GROUPS;
    T2 += row * c.nblk;
    float v[16];
    load16(x, c, blk * BLK + tid * 16, vec, v);

    // binary64 exclusive prefix over the threads of the block (elements on the grid of the
    // state predicted for the block start, as in the refined block sums)
    const Quantum g = quantum_of(prefix[blk]);
    double d = 0.0;
    bool finite = true, allzero = true;
#pragma unroll
    for (int q = 0; q < 16; q++)
    {
        d += quantise(v[q], g);
        const uint32_t a = __float_as_uint(v[q]) & 0x7FFFFFFFu;
        finite = finite && a < 0x7F800000u;
        allzero = allzero && a == 0u;
    }
    double inc = d;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1)
    {
        const double o = __shfl_up(inc, off, 64);
        if (lane >= off)
            inc += o;
    }
    if (lane == 63)
        wtot[wave] = inc;
    __syncthreads();
    double base = prefix[blk];
    for (int w = 0; w < wave; w++)
        base += wtot[w];
    const double excl = base + (inc - d);
    // the chunk (4 consecutive lanes) takes its hypothesis from the prefix at its first lane
    const double cstart = __shfl(excl, lane & ~3, 64);
    const bool cfinite = ((__ballot(finite) >> (lane & ~3)) & 0xFull) == 0xFull;
    const bool czero = ((__ballot(allzero) >> (lane & ~3)) & 0xFull) == 0xFull;
    const uint32_t us = __float_as_uint((float)cstart);
    const int eh = (int)((us >> 23) & 0xFFu);
    int hyp = (eh >= 1 && eh <= 254) ? (int)(us >> 23) : HYP_NONE;
    if (!cfinite)
        hyp = HYP_NONE;
    if (czero)
        hyp = HYP_ANY;

    Tup t = tup_identity(hyp);
    if (hyp >= 0 && hyp != HYP_ANY)
    {
        const int sg = hyp >> 8, e = hyp & 0xFF;
#pragma unroll
        for (int q = 0; q < 16; q++)
            tup_append(t, __float_as_uint(v[q]), sg, e);
    }
    // ordered reduction: 4 lanes -> chunk
    t = tup_compose(t, tup_shfl_down(t, 1));
    t = tup_compose(t, tup_shfl_down(t, 2));
    if ((lane & 3) == 0)
        T1[blk * (BLK / CH) + (tid >> 2)] = t;
    // 8 chunks -> group, 2 groups -> wave, 4 waves -> block (hypotheses merged on the way)
    t = tup_join(t, tup_shfl_down(t, 4));
    t = tup_join(t, tup_shfl_down(t, 8));
    t = tup_join(t, tup_shfl_down(t, 16));
    if ((lane & 31) == 0)
        TG[blk * GROUPS + wave * 2 + (lane >> 5)] = t;
    t = tup_join(t, tup_shfl_down(t, 32));
    if (lane == 0)
        wt[wave] = t;
    __syncthreads();
    if (tid == 0)
        T2[blk] = tup_join(tup_join(wt[0], wt[1]), tup_join(wt[2], wt[3]));
}

// ---- step 4: the walk -----------------------------------------------------------------------
// The state s (a binary32 bit pattern) lives in scalar registers: it is identical in every
// lane.  A tuple with hypothesis h applies to s iff (s >> 23) == h and need_lo <= S0 <= need_hi
// for the parity of S0 = (s & 0x7FFFFF) | 0x800000; both tests together are one interval test
// on s itself, smin[p] <= s <= smax[p] (unsigned), and applying the tuple is s += t[p] (the sum
// stays inside the binade, so nothing carries into the exponent).  The tuples of up to 64
// consecutive nodes sit one per lane in that form; stepping to node i broadcasts lane i's six
// words with v_readlane_b32 (independent of s, so they run ahead of the dependency chain).
struct LaneTup
{
    uint32_t smin0, smax0, smin1, smax1;
    int t0, t1;
};

__device__ __forceinline__ LaneTup lane_tup(const Tup &t)
{
    LaneTup l;
    l.t0 = t.t0;
    l.t1 = t.t1;
    if (t.hyp == HYP_ANY)
    {
        l.smin0 = l.smin1 = 0u;
        l.smax0 = l.smax1 = 0xFFFFFFFFu;
        l.t0 = l.t1 = 0;
    }
    else
    {
        const uint32_t top = (uint32_t)t.hyp << 23;
        // S0 + lo >= 2^23  <=>  frac >= -lo ;  S0 + hi <= 2^24 - 1  <=>  frac <= 0x7FFFFF - hi
        const int a0 = -t.lo0, b0 = 0x7FFFFF - t.hi0, a1 = -t.lo1, b1 = 0x7FFFFF - t.hi1;
        const bool ok0 = t.hyp >= 0 && a0 <= 0x7FFFFF && b0 >= 0 && a0 <= b0;
        const bool ok1 = t.hyp >= 0 && a1 <= 0x7FFFFF && b1 >= 0 && a1 <= b1;
        l.smin0 = ok0 ? top + (uint32_t)a0 : 0xFFFFFFFFu; // empty interval: nothing applies
        l.smax0 = ok0 ? top + (uint32_t)b0 : 0u;
        l.smin1 = ok1 ? top + (uint32_t)a1 : 0xFFFFFFFFu;
        l.smax1 = ok1 ? top + (uint32_t)b1 : 0u;
    }
    return l;
}

// Try node i (wave-uniform) of those held in l; false if it does not apply to state s.
__device__ __forceinline__ bool lane_tup_apply(uint32_t &s, const LaneTup &l, int i)
{
    const uint32_t smin0 = __builtin_amdgcn_readlane(l.smin0, i), smax0 = __builtin_amdgcn_readlane(l.smax0, i);
    const uint32_t smin1 = __builtin_amdgcn_readlane(l.smin1, i), smax1 = __builtin_amdgcn_readlane(l.smax1, i);
    const int t0 = __builtin_amdgcn_readlane(l.t0, i), t1 = __builtin_amdgcn_readlane(l.t1, i);
    const bool odd = (s & 1u) != 0u;
    const uint32_t smin = odd ? smin1 : smin0, smax = odd ? smax1 : smax0;
    const int tt = odd ? t1 : t0;
    const bool ok = s >= smin && s <= smax;
    s = ok ? s + (uint32_t)tt : s;
    return ok;
}

// ---- step 3b: tuples of super-blocks (64 blocks) --------------------------------------------
constexpr int SUP = 64; // blocks per super-block

__global__ __launch_bounds__(256) void sum1d_super_kernel(const Tup *__restrict__ T2, Tup *__restrict__ T3, int64_t nblk,
                                                          int64_t nsup)
{
    const int lane = threadIdx.x & 63;
    const int64_t sb = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (sb >= nsup)
        return;
    T2 += (int64_t)blockIdx.y * nblk; // row
    T3 += (int64_t)blockIdx.y * nsup;
    const int64_t b = sb * SUP + lane;
    Tup t = b < nblk ? T2[b] : tup_identity(HYP_ANY);
#pragma unroll
    for (int off = 1; off < 64; off <<= 1)
        t = tup_join(t, tup_shfl_down(t, off)); // lane 0: the 64 blocks in order
    if (lane == 0)
        T3[sb] = t;
}

// What the walk needs of a block that does not apply as a whole: its data and its group and
// chunk tuples, one slice per lane.
struct BlockRegs
{
    float4 f[BLK / 256];
    Tup tgr, tch;
};

// (x: the row's base; T1, TG: the row's tuples)
__device__ __forceinline__ void load_block(BlockRegs &r, const float *__restrict__ x, const Chains &c,
                                           const Tup *__restrict__ T1, const Tup *__restrict__ TG, int64_t blk, int lane,
                                           int vec)
{
    const int64_t n = c.n;
    r.tgr = TG[blk * GROUPS + (lane & (GROUPS - 1))];
    r.tch = T1[blk * (BLK / CH) + lane];
    const int64_t e0 = blk * BLK;
    if (vec && e0 + BLK <= n)
    {
        if (!c.segmented)
        {
#pragma unroll
            for (int q = 0; q < BLK / 256; q++)
                r.f[q] = reinterpret_cast<const float4 *>(x + e0)[q * 64 + lane];
        }
        else
        {
            // this lane's float4 q starts at element e0 + 4*lane + 256*q: one division for q = 0,
            // then steps of 256 with the segment wrapped by subtraction (a float4 never straddles
            // two segments: their length is a multiple of 16)
            const uint32_t i0 = (uint32_t)(e0 + 4 * lane);
            uint32_t sg = i0 / (uint32_t)c.seglen;
            uint32_t off = i0 - sg * (uint32_t)c.seglen;
#pragma unroll
            for (int q = 0; q < BLK / 256; q++)
            {
                r.f[q] = *reinterpret_cast<const float4 *>(x + (int64_t)sg * c.seg_stride + off);
                off += 256;
                while (off >= (uint32_t)c.seglen)
                {
                    off -= (uint32_t)c.seglen;
                    sg++;
                }
            }
        }
    }
    else
    {
#pragma unroll
        for (int q = 0; q < BLK / 256; q++)
        {
            const int64_t idx = e0 + (int64_t)(q * 64 + lane) * 4;
            r.f[q].x = (idx + 0 < n) ? *chain_ptr(x, c, idx + 0) : 0.0f; // elements past n: s + 0 = s
            r.f[q].y = (idx + 1 < n) ? *chain_ptr(x, c, idx + 1) : 0.0f;
            r.f[q].z = (idx + 2 < n) ? *chain_ptr(x, c, idx + 2) : 0.0f;
            r.f[q].w = (idx + 3 < n) ? *chain_ptr(x, c, idx + 3) : 0.0f;
        }
    }
}

typedef float f4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void read_chunk(const float *__restrict__ xd, int j, f4v (&v)[CH / 4])
{
    const f4v *p = reinterpret_cast<const f4v *>(xd + j * CH);
#pragma unroll
    for (int k = 0; k < CH / 4; k++)
        v[k] = p[k];
}

// 64 real additions
__device__ __forceinline__ uint32_t replay_chunk(uint32_t s, const f4v (&v)[CH / 4])
{
    float acc = __uint_as_float(s);
#pragma unroll
    for (int k = 0; k < CH / 4; k++)
    {
        acc = acc + v[k].x;
        acc = acc + v[k].y;
        acc = acc + v[k].z;
        acc = acc + v[k].w;
    }
    return __builtin_amdgcn_readfirstlane(__float_as_uint(acc));
}

// One wave.  Super-blocks are tried first (far from binade boundaries a whole run of blocks
// is one step), then the blocks of a failing super-block.  Failures cluster (they happen
// where the sum moves along a binade boundary), so when a block fails the next block's data
// and tuples are requested at once, and inside a failing group the LDS reads of a chunk are
// issued one chunk ahead of the additions.
__global__ __launch_bounds__(64) void sum1d_walk_kernel(const float *__restrict__ x, Chains c,
                                                        const Tup *__restrict__ T1,
                                                        const Tup *__restrict__ TG,
                                                        const Tup *__restrict__ T2,
                                                        const Tup *__restrict__ T3, float factor,
                                                        float *__restrict__ out, int vec)
{
    __shared__ __attribute__((aligned(16))) float xd[BLK + 2 * CH]; // + what the read-ahead overshoots
    const int lane = threadIdx.x;
    const int64_t row = blockIdx.x, nblk = c.nblk, nsup = c.nsup;
    x += row * c.row_stride;
    T1 += row * nblk * (BLK / CH);
    TG += row * nblk * GROUPS;
    T2 += row * nblk;
    T3 += row * nsup;
    out += row;
    uint32_t s = 0u; // +0.0f; wave-uniform throughout
    BlockRegs pf;    // the block requested ahead
    int64_t pf_blk = -1;
    load_block(pf, x, c, T1, TG, 0, lane, vec); // (any valid block: the registers are then defined)
    pf_blk = 0;
    Tup nsup_t = (lane < nsup) ? T3[lane] : tup_identity(HYP_ANY);
    // block tuples of the super-block being tried, and of the next one
    Tup blk_next = (lane < nblk) ? T2[lane] : tup_identity(HYP_ANY);
    for (int64_t g0 = 0; g0 < nsup; g0 += 64)
    {
        const LaneTup ls = lane_tup(nsup_t);
        if (g0 + 64 < nsup) // the next 64 super-block tuples, loaded while these are walked
            nsup_t = (g0 + 64 + lane < nsup) ? T3[g0 + 64 + lane] : tup_identity(HYP_ANY);
        const int cnt = (nsup - g0 < 64) ? (int)(nsup - g0) : 64;
        for (int i = 0; i < cnt; i++)
        {
            const int64_t sb = g0 + i;
            const Tup blk_cur = blk_next;
            {
                const int64_t b = (sb + 1) * SUP + lane; // always requested: 32 bytes per block
                blk_next = b < nblk ? T2[b] : tup_identity(HYP_ANY);
            }
            if (lane_tup_apply(s, ls, i))
                continue;
            const LaneTup lb = lane_tup(blk_cur);
            for (int bi = 0; bi < SUP; bi++)
            {
                if (lane_tup_apply(s, lb, bi)) // blocks past the end are identities
                    continue;
                // The block as a whole does not apply.
                const int64_t blk = sb * SUP + bi;
                if (pf_blk != blk)
                    load_block(pf, x, c, T1, TG, blk, lane, vec);
                __syncthreads();
#pragma unroll
                for (int q = 0; q < BLK / 256; q++)
                    *reinterpret_cast<float4 *>(&xd[(q * 64 + lane) * 4]) = pf.f[q];
                const LaneTup lg = lane_tup(pf.tgr), lc = lane_tup(pf.tch);
                __syncthreads();
                {
                    const int64_t nb = blk + 1 < nblk ? blk + 1 : blk;
                    load_block(pf, x, c, T1, TG, nb, lane, vec);
                    pf_blk = nb;
                }
                for (int gr = 0; gr < GROUPS; gr++)
                {
                    if (lane_tup_apply(s, lg, gr))
                        continue;
                    constexpr int CG = BLK / CH / GROUPS; // 8 chunks, reads one chunk ahead
                    const int j0 = gr * CG;
                    f4v va[CH / 4], vb[CH / 4];
                    read_chunk(xd, j0, va);
#pragma unroll
                    for (int j = 0; j < CG; j += 2)
                    {
                        read_chunk(xd, j0 + j + 1, vb);
                        if (!lane_tup_apply(s, lc, j0 + j))
                            s = replay_chunk(s, va);
                        read_chunk(xd, j0 + j + 2, va);
                        if (!lane_tup_apply(s, lc, j0 + j + 1))
                            s = replay_chunk(s, vb);
                    }
                }
            }
        }
    }
    if (lane == 0)
        out[0] = factor * __uint_as_float(s);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline size_t round256(size_t v) { return (v + 255) & ~(size_t)255; }
} // namespace

// serial single-chain kernel of sum.hip
int repdl_sum1d_serial(const float *in, float *out, int64_t n, int average, void *stream);

// Scratch for `rows` chains of n elements.
size_t repdl_sum_chains_workspace_bytes(int64_t rows, int64_t n)
{
    const size_t nblk = (size_t)repdl_cdiv(n, BLK) * (size_t)rows;
    const size_t nsup = (size_t)repdl_cdiv(repdl_cdiv(n, BLK), SUP) * (size_t)rows;
    return round256(nblk * sizeof(double)) * 2 + round256(nsup * sizeof(Tup)) + round256(nblk * sizeof(Tup)) +
           round256(nblk * GROUPS * sizeof(Tup)) + round256(nblk * (BLK / CH) * sizeof(Tup));
}

// out[r] = factor * (the sequential sum of chain r), r < rows, by the parallel evaluation.
// Chain r: nseg segments of seglen contiguous floats, segment s at in + r*row_stride +
// s*seg_stride.  The caller has checked: n = nseg*seglen >= 1, rows in [1, 65535], and for
// nseg > 1 that seglen is a multiple of 16 and n < 2^31.
int repdl_sum_chains(const float *in, float *out, int64_t rows, int64_t nseg, int64_t seglen, int64_t row_stride,
                     int64_t seg_stride, float factor, void *workspace, size_t workspace_bytes, void *stream)
{
    const int64_t n = nseg * seglen;
    REPDL_REQUIRE(rows >= 1 && rows <= 65535 && n >= 1 && in != nullptr && out != nullptr);
    REPDL_REQUIRE(nseg == 1 || (seglen % 16 == 0 && n <= REPDL_I32_MAX));
    if (workspace == nullptr || workspace_bytes < repdl_sum_chains_workspace_bytes(rows, n) ||
        (reinterpret_cast<uintptr_t>(workspace) & 15) != 0)
        return REPDL_E_WORKSPACE;
    const int64_t nblk = repdl_cdiv(n, BLK), nsup = repdl_cdiv(nblk, SUP);
    REPDL_REQUIRE(nblk <= REPDL_I32_MAX);
    Chains c;
    c.n = n;
    c.row_stride = row_stride;
    c.seg_stride = nseg > 1 ? seg_stride : 0;
    c.nblk = nblk;
    c.nsup = nsup;
    c.seglen = nseg > 1 ? (int)seglen : 0;
    c.segmented = nseg > 1;
    char *w = static_cast<char *>(workspace);
    double *bsum = reinterpret_cast<double *>(w);
    w += round256(rows * nblk * sizeof(double));
    double *prefix = reinterpret_cast<double *>(w);
    w += round256(rows * nblk * sizeof(double));
    Tup *T3 = reinterpret_cast<Tup *>(w);
    w += round256(rows * nsup * sizeof(Tup));
    Tup *T2 = reinterpret_cast<Tup *>(w);
    w += round256(rows * nblk * sizeof(Tup));
    Tup *TG = reinterpret_cast<Tup *>(w);
    w += round256(rows * nblk * GROUPS * sizeof(Tup));
    Tup *T1 = reinterpret_cast<Tup *>(w);
    hipStream_t s = repdl_stream(stream);
    // 16-byte loads: every row and segment starts on a 16-byte boundary
    const int vec = aligned16(in) && (rows == 1 || row_stride % 4 == 0) && (nseg == 1 || seg_stride % 4 == 0);
    const dim3 g2((unsigned)nblk, (unsigned)rows);
    hipLaunchKernelGGL(sum1d_blocksum_kernel, g2, dim3(256), 0, s, in, c, static_cast<const double *>(nullptr), bsum, vec);
    hipLaunchKernelGGL(sum1d_prefix_kernel, dim3((unsigned)rows), dim3(256), 0, s, bsum, prefix, nblk);
    // one refinement of the prediction (see quantum_of)
    hipLaunchKernelGGL(sum1d_blocksum_kernel, g2, dim3(256), 0, s, in, c, static_cast<const double *>(prefix), bsum, vec);
    hipLaunchKernelGGL(sum1d_prefix_kernel, dim3((unsigned)rows), dim3(256), 0, s, bsum, prefix, nblk);
    hipLaunchKernelGGL(sum1d_tuple_kernel, g2, dim3(256), 0, s, in, c, prefix, T1, TG, T2, vec);
    hipLaunchKernelGGL(sum1d_super_kernel, dim3((unsigned)repdl_cdiv(nsup, 4), (unsigned)rows), dim3(256), 0, s, T2, T3, nblk,
                       nsup);
    hipLaunchKernelGGL(sum1d_walk_kernel, dim3((unsigned)rows), dim3(64), 0, s, in, c, T1, TG, T2, T3, factor, out, vec);
    return repdl_launch_status();
}

REPDL_API size_t repdl_hip_sum1d_workspace_bytes(int64_t n)
{
    if (n < REPDL_SUM1D_MIN_PARALLEL)
        return 0;
    return repdl_sum_chains_workspace_bytes(1, n);
}

REPDL_API int repdl_hip_sum1d_ws(const float *in, float *out, int64_t n, int average, void *workspace,
                                 size_t workspace_bytes, void *stream)
{
    REPDL_REQUIRE(n >= 0 && out != nullptr && (n == 0 || in != nullptr));
    if (n < REPDL_SUM1D_MIN_PARALLEL)
        return repdl_sum1d_serial(in, out, n, average, stream);
    return repdl_sum_chains(in, out, 1, 1, n, 0, 0, repdl_sum_factor(average, n), workspace, workspace_bytes, stream);
}

REPDL_API int repdl_hip_sum1d(const float *in, float *out, int64_t n, int average, void *stream)
{
    REPDL_REQUIRE(n >= 0 && out != nullptr && (n == 0 || in != nullptr));
    if (n < REPDL_SUM1D_MIN_PARALLEL)
        return repdl_sum1d_serial(in, out, n, average, stream);
    // no workspace given: take it from the stream-ordered allocator for the duration of the call
    const size_t bytes = repdl_hip_sum1d_workspace_bytes(n);
    void *ws = nullptr;
    hipError_t e = hipMallocAsync(&ws, bytes, repdl_stream(stream));
    if (e != hipSuccess)
        return (int)e;
    const int rc = repdl_hip_sum1d_ws(in, out, n, average, ws, bytes, stream);
    e = hipFreeAsync(ws, repdl_stream(stream));
    if (rc != REPDL_OK)
        return rc;
    return e == hipSuccess ? REPDL_OK : (int)e;
}

// ---- sum1d for callers that cannot allocate ---------------------------------------------------
// The scratch memory of the parallel evaluation in a file-scope device array instead of an
// allocation: every device the library runs on holds its own copy of the array until the process
// ends.  In host code the array's name is only a handle for hipGetSymbolAddress; the address
// the kernels get is looked up once per device, with that device current.
namespace
{
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)8 << 20;
__device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
constexpr int STATIC_MAX_DEVICES = 64;
std::mutex g_static_lock;
void *g_static_ptr[STATIC_MAX_DEVICES] = {};

// largest n whose scratch fits (the need grows monotonically with n)
int64_t static_max_n()
{
    int64_t lo = REPDL_SUM1D_MIN_PARALLEL, hi = (int64_t)STATIC_SCRATCH_BYTES * 8;
    while (lo < hi)
    {
        const int64_t mid = lo + (hi - lo + 1) / 2;
        if (repdl_sum_chains_workspace_bytes(1, mid) <= STATIC_SCRATCH_BYTES)
            lo = mid;
        else
            hi = mid - 1;
    }
    return lo;
}
} // namespace

REPDL_API int64_t repdl_hip_sum1d_static_max_n(void)
{
    static const int64_t n = static_max_n();
    return n;
}

REPDL_API int repdl_hip_sum1d_static(const float *in, float *out, int64_t n, int average, void *stream)
{
    REPDL_REQUIRE(n >= 0 && out != nullptr && (n == 0 || in != nullptr));
    if (n < REPDL_SUM1D_MIN_PARALLEL)
        return repdl_sum1d_serial(in, out, n, average, stream); // uses no scratch memory
    if (n > repdl_hip_sum1d_static_max_n())
        return REPDL_E_TOO_LARGE;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return (int)e;
    REPDL_REQUIRE(dev >= 0 && dev < STATIC_MAX_DEVICES);
    void *ptr = nullptr;
    {
        std::lock_guard<std::mutex> guard(g_static_lock);
        if (g_static_ptr[dev] == nullptr)
        {
            e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess)
                return (int)e;
            g_static_ptr[dev] = ptr;
        }
        ptr = g_static_ptr[dev];
    }
    return repdl_hip_sum1d_ws(in, out, n, average, ptr, STATIC_SCRATCH_BYTES, stream);
}
