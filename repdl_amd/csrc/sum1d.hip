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
//
// Long single chains: step 4 alone is one wave, and on data whose sum wanders across binade
// boundaries (zero-mean steps) it replays tens of thousands of chunks one after the other.
// So it is preceded by SPECULATIVE ROUNDS that do the same walk for many candidate states at
// once, everywhere in parallel:
//   4a. a NODE is 4 blocks.  One workgroup per node walks it exactly as step 4 would, but
//       for 256 candidate entry states at once, one per lane: 256 consecutive binary32
//       bit patterns around the node's predicted entry state.  A map is applied when it is
//       valid for every lane of a wave, a chunk is replayed with real additions otherwise
//       (the chunk's elements broadcast from LDS), so every lane ends with the exact exit
//       state of ITS entry state: a table  candidate -> exit state.
//   4b. the sixteen node tables of a super-block are composed: exact where each exit state is
//       again a candidate of the next node, and otherwise an approximate offset (nearest
//       candidate, the excess carried along).
//   4c. one workgroup runs the true state through the super-block tables, staged through
//       LDS, for as long as it finds the state among the candidates (every such step is
//       exact).  At the first miss it keeps the exact state and position reached (the
//       FRONT) and goes on with the approximate offsets: they predict the entry state of
//       every later super-block far better than step 2 could, because they come from real
//       trajectories that start next to the true one.  The next round builds its tables
//       around those predictions, and so on for a fixed number of rounds (each a no-op once
//       the front has reached the end).  On 2^28 zero-mean values the front reaches the end
//       in four rounds.
// Whatever the rounds leave (nothing, as a rule) step 4 walks from the front.  Only exact
// table entries ever touch the true state, so the result is still the sequential sum for
// every input.
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
constexpr int SUP = 64;           // blocks per super-block
constexpr int NODEB = 4;          // blocks per node (the unit of the speculative rounds)
constexpr int NPS = SUP / NODEB;  // nodes per super-block
constexpr int CAND = 256;         // candidate entry states per node
constexpr int HB = 16;            // super-blocks per hyper-block (the unit the resolver steps through)

struct __attribute__((aligned(16))) Tup
{
    int t0, t1;   // S -> S + t[p] for starting parity p
    int lo0, hi0; // over all prefixes: min of (offset + X) before rounding, max of offset after
    int lo1, hi1;
    int hyp;      // (sign << 8) | biased exponent of the state this tuple assumes, or HYP_*
    int heavy;    // chunks below this node whose map does not even hold for the predicted state (an estimate of the replays)
};

__device__ __forceinline__ int clampi(int v) { return v < -SAT ? -SAT : (v > SAT ? SAT : v); }

__device__ __forceinline__ Tup tup_identity(int hyp)
{
    Tup t;
    t.t0 = t.t1 = t.lo0 = t.hi0 = t.lo1 = t.hi1 = 0;
    t.hyp = hyp;
    t.heavy = 0;
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
    c.heavy = a.heavy + b.heavy;
    return c;
}

// append element x (bit pattern ux, finite) to tuple t under hypothesis (sg, e)
// (the branches stay: on most data a wave takes one of the three cases as a whole, and the same
// arithmetic as straight-line code with selects made the tuple pass 12 % slower)
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
    // (no saturation here: sixteen appends from the identity stay below 2^31 -- each step is at most
    // BIG + 1 = 2^26 + 1 in magnitude -- and tup_saturate follows them; a field that would have
    // saturated on the way belongs to a map that holds for no state, with or without the clamp,
    // since the prefix bounds only ever widen)
    t.lo0 = min(t.lo0, t.t0 + X);
    t.lo1 = min(t.lo1, t.t1 + X);
    t.t0 = t.t0 + ea0;
    t.t1 = t.t1 + ea1;
    t.hi0 = max(t.hi0, t.t0);
    t.hi1 = max(t.hi1, t.t1);
}

__device__ __forceinline__ void tup_saturate(Tup &t)
{
    t.t0 = clampi(t.t0);
    t.t1 = clampi(t.t1);
    t.lo0 = clampi(t.lo0);
    t.hi0 = clampi(t.hi0);
    t.lo1 = clampi(t.lo1);
    t.hi1 = clampi(t.hi1);
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
    r.heavy = __shfl_down(t.heavy, delta, 64);
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

// prev == nullptr: exact sums, and the sums of the magnitudes in babs; else: sums of the elements
// rounded to the grid of the state prev[block] predicted by the previous pass -- unless that pass
// found the refinement pointless for this row (refine[row] == 0: nothing is read, bsum stays).
// The first pass clears refine[row] for the prefix launch that follows it.
__global__ __launch_bounds__(256) void sum1d_blocksum_kernel(const float *__restrict__ x, Chains c,
                                                             const double *__restrict__ prev,
                                                             double *__restrict__ bsum, double *__restrict__ babs,
                                                             int *__restrict__ refine, int vec)
{
    __shared__ double part[2][4];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.y;
    if (prev != nullptr && refine[row] == 0)
        return;
    if (prev == nullptr && blockIdx.x == 0 && tid == 0)
        refine[row] = 0;
    x += row * c.row_stride;
    bsum += row * c.nblk;
    float v[16];
    load16(x, c, (int64_t)blockIdx.x * BLK + tid * 16, vec, v);
    Quantum g;
    g.q = g.inv_q = 0.0;
    if (prev != nullptr)
        g = quantum_of(prev[row * c.nblk + blockIdx.x]);
    double d = 0.0, a = 0.0;
#pragma unroll
    for (int q = 0; q < 16; q++)
    {
        d += quantise(v[q], g);
        a += (double)__builtin_fabsf(v[q]);
    }
    d = wave_sum(d);
    if (prev == nullptr)
        a = wave_sum(a);
    if ((tid & 63) == 0)
    {
        part[0][tid >> 6] = d;
        part[1][tid >> 6] = a;
    }
    __syncthreads();
    if (tid == 0)
    {
        bsum[blockIdx.x] = (part[0][0] + part[0][1]) + (part[0][2] + part[0][3]);
        if (prev == nullptr)
            babs[row * c.nblk + blockIdx.x] = (part[1][0] + part[1][1]) + (part[1][2] + part[1][3]);
    }
}

// ---- step 2: exclusive prefix of the block sums -----------------------------------------------
// grid (tiles of 4096 sums, rows).  A workgroup first adds up everything before its tile (a plain
// reduction, every read coalesced; the order is fixed, so the prediction is the same on every run),
// then scans the tile: a thread owns four consecutive sums, the workgroup scans the thread totals.
// Memory is touched in rows of 64 consecutive sums per wave (512 contiguous bytes per instruction) and
// the rows are turned into four-per-thread through LDS, each wave in its own 2 KiB: a thread that
// loaded and stored its own sums directly made every instruction touch 64 separate lines, and one
// workgroup walking all the tiles of a chain of 2^28 elements one after the other took 80 us.
// First pass (babs given): also decides whether the refinement pass is worth its read of the input,
// refine[row] = 1 (it was cleared by the block-sum launch before) if some block enters at a state
// whose grid is within 2^5 of the block's mean magnitude -- where elements lose bits that matter, or
// vanish, the chain drifts away from the exact sum systematically (a sum of 2^28 values in [0,1) stalls
// at 2^24) and only the refined prediction follows it; where the grid is far finer than the elements the
// rounding errors have no direction and the rounds re-centre the windows anyway.  Either answer gives
// the same result: the prediction only places the candidate windows.  Second pass (babs null): nothing
// to do if refine[row] == 0.
constexpr int PREFIX_TILE = 4096;

__global__ __launch_bounds__(1024) void sum1d_prefix_kernel(const double *__restrict__ bsum,
                                                            double *__restrict__ prefix, int64_t nblk,
                                                            const double *__restrict__ babs, int *__restrict__ refine, int64_t n)
{
    constexpr int PER = PREFIX_TILE / 1024;
    __shared__ __attribute__((aligned(16))) double stage[16][64 * PER];
    __shared__ double wsum[2][16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t row = blockIdx.y, base = (int64_t)blockIdx.x * PREFIX_TILE;
    if (babs == nullptr && refine[row] == 0)
        return;
    bsum += row * nblk;
    prefix += row * nblk;
    if (babs != nullptr)
        babs += row * nblk;
    double *const mine = stage[wave];
    // this tile, requested before the reduction below
    double rv[PER], ra[PER];
#pragma unroll
    for (int r = 0; r < PER; r++)
    {
        const int64_t i = base + wave * (64 * PER) + r * 64 + lane;
        rv[r] = i < nblk ? bsum[i] : 0.0;
        ra[r] = babs != nullptr && i < nblk ? babs[i] : 0.0;
    }
    // everything before the tile
    double part = 0.0;
    for (int64_t i = tid; i < base; i += 1024)
        part += bsum[i];
    part = wave_sum(part);
    if (lane == 0)
        wsum[0][wave] = part;
    // rows of 64 (register r: the wave's sum r * 64 + lane) to four consecutive per thread
    auto to_consecutive = [&](const double(&rows)[PER], double(&own)[PER]) {
#pragma unroll
        for (int r = 0; r < PER; r++)
            mine[r * 64 + lane] = rows[r];
        __syncthreads();
#pragma unroll
        for (int d = 0; d < PER; d++)
            own[d] = mine[lane * PER + d];
        __syncthreads();
    };
    const int64_t i0 = base + (int64_t)tid * PER;
    double v[PER], ab[PER];
    to_consecutive(rv, v); // (its barriers also publish wsum[0])
    if (babs != nullptr)   // (uniform)
        to_consecutive(ra, ab);
    double carry = 0.0;
#pragma unroll
    for (int w = 0; w < 16; w++)
        carry += wsum[0][w];
    double tot = 0.0;
#pragma unroll
    for (int d = 0; d < PER; d++)
        tot += v[d];
    double inc = tot;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1)
    {
        const double o = __shfl_up(inc, off, 64);
        if (lane >= off)
            inc += o;
    }
    if (lane == 63)
        wsum[1][wave] = inc;
    __syncthreads();
    double before = 0.0;
#pragma unroll
    for (int w = 0; w < 16; w++)
        before += w < wave ? wsum[1][w] : 0.0;
    double run = carry + before + (inc - tot);
    bool want = false;
#pragma unroll
    for (int d = 0; d < PER; d++)
    {
        mine[lane * PER + d] = run;
        if (babs != nullptr && i0 + d < nblk)
        {
            const int64_t left = n - (i0 + d) * BLK; // elements of this block (the last one may be short)
            want = want || quantum_of(run).q * 32.0 * (double)(left < BLK ? left : BLK) >= ab[d];
        }
        run += v[d];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < PER; r++)
    {
        const int64_t i = base + wave * (64 * PER) + r * 64 + lane;
        if (i < nblk)
            prefix[i] = mine[r * 64 + lane];
    }
    if (babs != nullptr && want)
        refine[row] = 1; // (same value from every writer, in this workgroup and the others)
}

// ---- step 3: chunk and block tuples --------------------------------------------------------
__global__ __launch_bounds__(256) void sum1d_tuple_kernel(const float *__restrict__ x, Chains c,
                                                          const double *__restrict__ prefix,
                                                          Tup *__restrict__ T1, Tup *__restrict__ TG,
                                                          Tup *__restrict__ T2, int vec, int self_prefix)
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

    // The state predicted at the block start.  self_prefix (one short unsegmented chain): the block
    // adds up everything before it in binary64 itself -- at most 63 blocks, from the cache -- which
    // saves the four launches of steps 1 and 2 where a launch is longer than its work.  (Any fixed
    // order serves: the value only predicts.)
    double pstart;
    if (self_prefix)
    {
        const int64_t e0 = blk * BLK;
        double p = 0.0;
        if (vec)
        {
            // (e0 is a multiple of 4096: four loads in flight per thread, four partial sums)
            double p4[4] = {0.0, 0.0, 0.0, 0.0};
            for (int64_t i = (int64_t)tid * 4; i < e0; i += 4096)
            {
                float4 f[4];
#pragma unroll
                for (int u = 0; u < 4; u++)
                    f[u] = *reinterpret_cast<const float4 *>(x + i + 1024 * u);
#pragma unroll
                for (int u = 0; u < 4; u++)
                    p4[u] += ((double)f[u].x + (double)f[u].y) + ((double)f[u].z + (double)f[u].w);
            }
            p = (p4[0] + p4[1]) + (p4[2] + p4[3]);
        }
        else
        {
            for (int64_t i = tid; i < e0; i += 256)
                p += (double)x[i];
        }
        p = wave_sum(p);
        if (lane == 0)
            wtot[wave] = p;
        __syncthreads();
        pstart = (wtot[0] + wtot[1]) + (wtot[2] + wtot[3]);
        __syncthreads(); // (wtot is used again below)
    }
    else
        pstart = prefix[blk];

    // binary64 exclusive prefix over the threads of the block (elements on the grid of the
    // state predicted for the block start, as in the refined block sums)
    const Quantum g = quantum_of(pstart);
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
    double base = pstart;
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
        tup_saturate(t);
    }
    // ordered reduction: 4 lanes -> chunk
    t = tup_compose(t, tup_shfl_down(t, 1));
    t = tup_compose(t, tup_shfl_down(t, 2));
    {
        // does the chunk's map hold for the state predicted at its start?  (counted up the tree:
        // the speculative rounds walk the nodes with the most such chunks first)
        const uint32_t S0 = (us & 0x7FFFFFu) | 0x800000u;
        const int lo = (S0 & 1u) ? t.lo1 : t.lo0, hi = (S0 & 1u) ? t.hi1 : t.hi0;
        const bool holds = hyp == HYP_ANY || (hyp >= 0 && (int)S0 + lo >= 0x800000 && (int)S0 + hi <= 0xFFFFFF);
        t.heavy = holds ? 0 : 1;
    }
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

// The same tuples laid out for the single walking wave, whose cost is its instruction count (a lone
// wave issues an instruction about every 8 clocks whatever it is): node i of 64 sits in lane
// 2 (i % 32) + parity of register set i / 32, as the start and the LENGTH of the interval of states of
// that parity to which the map applies, so that a test is (s - smin) < len on the scalar unit after
// three v_readlane_b32 -- about ten instructions against nineteen for lane_tup_apply.
// (An interval of all 2^32 states is stored with length 2^32 - 1: the state 0xFFFFFFFF then fails
// the test and takes the slower way down to real additions, which is always right.)
struct WalkHalf
{
    uint32_t smin, len;
    int t;
};
struct WalkTup
{
    WalkHalf A, B; // nodes 0..31 and 32..63
};

__device__ __forceinline__ WalkTup walk_tup(const LaneTup &l)
{
    const int lane = threadIdx.x & 63, node = lane >> 1;
    const bool odd = (lane & 1) != 0;
    WalkTup w;
    auto pick = [&](int nd, WalkHalf &h) {
        const uint32_t lo0 = (uint32_t)__shfl((int)l.smin0, nd, 64), hi0 = (uint32_t)__shfl((int)l.smax0, nd, 64);
        const uint32_t lo1 = (uint32_t)__shfl((int)l.smin1, nd, 64), hi1 = (uint32_t)__shfl((int)l.smax1, nd, 64);
        const int t0 = __shfl(l.t0, nd, 64), t1 = __shfl(l.t1, nd, 64);
        const uint32_t lo = odd ? lo1 : lo0, hi = odd ? hi1 : hi0;
        h.smin = lo;
        h.len = hi < lo ? 0u : (hi - lo == 0xFFFFFFFFu ? 0xFFFFFFFFu : hi - lo + 1u);
        h.t = odd ? t1 : t0;
    };
    pick(node, w.A);
    pick(node + 32, w.B);
    return w;
}

// Try node i5 (wave-uniform, 0..31) of those held in h; false if it does not apply to state s.
__device__ __forceinline__ bool walk_apply(uint32_t &s, const WalkHalf &h, int i5)
{
    const int idx = 2 * i5 + (int)(s & 1u);
    const uint32_t smin = __builtin_amdgcn_readlane(h.smin, idx), len = __builtin_amdgcn_readlane(h.len, idx);
    const int tt = __builtin_amdgcn_readlane(h.t, idx);
    const bool ok = s - smin < len;
    s = ok ? s + (uint32_t)tt : s;
    return ok;
}

// ---- step 3b: tuples of nodes (16 blocks) and super-blocks (64 blocks) -------------------------
// Per row: where the true state is known exactly so far (a super-block index and the state
// there); nsup once the whole chain is resolved.
struct Ctl
{
    int front;
    uint32_t s;
};

// Per round of the speculative stage: the list of nodes that have to be walked.  The plan kernel
// puts the nodes that promise long walks at the front (`count` of them, filled upwards from entry
// 0) and the others at the back (`light`, filled downwards from the last entry); walkers take
// the front ones first, so that the longest walks start first.  `next`: entries handed out.
constexpr int MAX_ROUNDS = 12;
constexpr int HEAVY_CHUNKS = 24; // predicted replays from which a node counts as a long walk
struct Work
{
    int count;
    int light;
    int next;
    int unused;
};

__global__ __launch_bounds__(256) void sum1d_super_kernel(const Tup *__restrict__ T2, Tup *__restrict__ TN, Tup *__restrict__ T3,
                                                          Ctl *__restrict__ ctl, Work *__restrict__ work, int64_t nblk, int64_t nnode,
                                                          int64_t nsup)
{
    const int lane = threadIdx.x & 63;
    const int64_t sb = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (blockIdx.x == 0 && threadIdx.x == 0)
    {
        ctl[blockIdx.y].front = 0; // nothing resolved yet; the chain starts at +0.0f
        ctl[blockIdx.y].s = 0u;
    }
    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x < MAX_ROUNDS)
    {
        work[threadIdx.x].count = 0; // the lists of walks of all rounds start empty
        work[threadIdx.x].light = 0;
        work[threadIdx.x].next = 0;
    }
    if (sb >= nsup)
        return;
    T2 += (int64_t)blockIdx.y * nblk; // row
    TN += (int64_t)blockIdx.y * nnode;
    T3 += (int64_t)blockIdx.y * nsup;
    const int64_t b = sb * SUP + lane;
    Tup t = b < nblk ? T2[b] : tup_identity(HYP_ANY);
#pragma unroll
    for (int off = 1; off < NODEB; off <<= 1)
        t = tup_join(t, tup_shfl_down(t, off)); // lanes 0, 4, 8, ...: the blocks of a node in order
    if ((lane & (NODEB - 1)) == 0 && sb * NPS + lane / NODEB < nnode)
        TN[sb * NPS + lane / NODEB] = t;
#pragma unroll
    for (int off = NODEB; off < 64; off <<= 1)
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
                                                        const Tup *__restrict__ T3,
                                                        const Ctl *__restrict__ ctl, float factor,
                                                        float *__restrict__ out, int vec, int inline_super)
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
    // Where the speculative rounds got to (super-block `first`, state there); 0 and +0.0f
    // without rounds; nothing to do if they resolved the whole chain.
    // inline_super (a chain of one super-block, walked from its start at +0.0f): T3 and ctl have not been
    // written -- the launch of step 3b is saved -- and the super-block's tuple is joined here.
    const int64_t first = inline_super ? 0 : __builtin_amdgcn_readfirstlane(ctl[row].front);
    if (first >= nsup)
        return;
    uint32_t s = inline_super ? 0u : __builtin_amdgcn_readfirstlane(ctl[row].s); // wave-uniform throughout
    BlockRegs pf;                                            // the block requested ahead
    int64_t pf_blk = -1;
    load_block(pf, x, c, T1, TG, 0, lane, vec); // (any valid block: the registers are then defined)
    pf_blk = 0;
    const int64_t gfirst = first & ~(int64_t)63;
    Tup nsup_t = tup_identity(HYP_ANY);
    if (inline_super)
    {
        Tup t = lane < nblk ? T2[lane] : tup_identity(HYP_ANY);
#pragma unroll
        for (int off = 1; off < 64; off <<= 1)
            t = tup_join(t, tup_shfl_down(t, off)); // lane 0: the blocks in order
        if (lane == 0)
            nsup_t = t;
    }
    else if (gfirst + lane < nsup)
        nsup_t = T3[gfirst + lane];
    // block tuples of the super-block being tried, and of the next one
    Tup blk_next = (first * SUP + lane < nblk) ? T2[first * SUP + lane] : tup_identity(HYP_ANY);
    for (int64_t g0 = gfirst; g0 < nsup; g0 += 64)
    {
        const WalkTup ls = walk_tup(lane_tup(nsup_t));
        if (g0 + 64 < nsup) // the next 64 super-block tuples, loaded while these are walked
            nsup_t = (g0 + 64 + lane < nsup) ? T3[g0 + 64 + lane] : tup_identity(HYP_ANY);
        const int cnt = (nsup - g0 < 64) ? (int)(nsup - g0) : 64;
        const int i_first = g0 == gfirst ? (int)(first - gfirst) : 0;
        for (int hs = i_first >> 5; hs < 2 && 32 * hs < cnt; hs++)
        {
        const WalkHalf lsh = hs ? ls.B : ls.A;
        const int i_end = cnt < 32 * hs + 32 ? cnt : 32 * hs + 32;
        for (int i = i_first > 32 * hs ? i_first : 32 * hs; i < i_end; i++)
        {
            const int64_t sb = g0 + i;
            const Tup blk_cur = blk_next;
            {
                const int64_t b = (sb + 1) * SUP + lane; // always requested: 32 bytes per block
                blk_next = b < nblk ? T2[b] : tup_identity(HYP_ANY);
            }
            if (walk_apply(s, lsh, i & 31))
                continue;
            const WalkTup lb = walk_tup(lane_tup(blk_cur));
            // blocks of this super-block with a chunk whose map does not even hold for the predicted state:
            // the ones that will most likely fail as wholes, and so the ones to request ahead
            const unsigned long long expect_fail = __ballot(blk_cur.heavy > 0);
            for (int hb = 0; hb < SUP / 32; hb++)
            {
            const WalkHalf lbh = hb ? lb.B : lb.A;
            for (int b5 = 0; b5 < 32; b5++)
            {
                if (walk_apply(s, lbh, b5)) // blocks past the end are identities
                    continue;
                // The block as a whole does not apply.
                const int64_t blk = sb * SUP + 32 * hb + b5;
                if (pf_blk != blk)
                    load_block(pf, x, c, T1, TG, blk, lane, vec);
                __syncthreads();
#pragma unroll
                for (int q = 0; q < BLK / 256; q++)
                    *reinterpret_cast<float4 *>(&xd[(q * 64 + lane) * 4]) = pf.f[q];
                const WalkTup lg = walk_tup(lane_tup(pf.tgr)), lc = walk_tup(lane_tup(pf.tch));
                __syncthreads();
                {
                    const int bi = 32 * hb + b5;
                    const unsigned long long later = bi < 63 ? expect_fail >> (bi + 1) : 0ull;
                    int64_t nb = later != 0ull ? blk + 1 + __builtin_ctzll(later) : blk + 1;
                    nb = nb < nblk ? nb : blk;
                    load_block(pf, x, c, T1, TG, nb, lane, vec);
                    pf_blk = nb;
                }
                for (int gr = 0; gr < GROUPS; gr++)
                {
                    if (walk_apply(s, lg.A, gr))
                        continue;
                    constexpr int CG = BLK / CH / GROUPS; // 8 chunks, reads one chunk ahead
                    static_assert(GROUPS <= 32 && (32 % CG) == 0, "a group's chunks lie in one half");
                    const int j0 = gr * CG;
                    const WalkHalf lch = j0 < 32 ? lc.A : lc.B;
                    f4v va[CH / 4], vb[CH / 4];
                    read_chunk(xd, j0, va);
#pragma unroll
                    for (int j = 0; j < CG; j += 2)
                    {
                        read_chunk(xd, j0 + j + 1, vb);
                        if (!walk_apply(s, lch, (j0 + j) & 31))
                            s = replay_chunk(s, va);
                        read_chunk(xd, j0 + j + 2, va);
                        if (!walk_apply(s, lch, (j0 + j + 1) & 31))
                            s = replay_chunk(s, vb);
                    }
                }
            }
            }
        }
        }
    }
    if (lane == 0)
        out[0] = factor * __uint_as_float(s);
}

// ---- step 4a: a node walked for 256 candidate entry states ------------------------------------
// A state is a binary32 bit pattern; candidate k of a node is base + k (any 32-bit pattern is a
// state, and the walk below is exact for every one of them).

// nearest candidate of the state whose bits are yb, for a window that starts at base
__device__ __forceinline__ uint32_t nearest_candidate(uint32_t yb, uint32_t base, bool &hit)
{
    const uint32_t d = yb - base;
    hit = d < (uint32_t)CAND;
    return hit ? d : (d < 0x80000000u ? (uint32_t)(CAND - 1) : 0u);
}

// The window of candidates for a predicted state: CAND consecutive bit patterns around it, moved
// where necessary to stay inside its binade (same sign and exponent).  The maps of a chunk assume
// one binade, so candidates beyond its edge would be replayed element by element all the way --
// for nothing when the sum sits exactly on the edge, as a sum of positive numbers does once it
// has stopped growing at a power of two.  A true state on the far side of the edge is a miss, and
// the next round's window lies there.
__device__ __forceinline__ uint32_t window_base(uint32_t centre)
{
    const uint32_t lo = centre & 0xFF800000u, hi = centre | 0x007FFFFFu;
    // The window starts on a multiple of WGRID states (lo is one), the centre 96 to 159 states in: a
    // centre that moves by a few states from one round to the next keeps its window, and the node its
    // table (2^28 zero-mean values: 2.47 -> 2.40 ms).
    constexpr uint32_t WGRID = 64;
    uint32_t base = centre - lo < (uint32_t)(CAND / 2) ? lo : (centre - (uint32_t)(CAND / 2) + WGRID / 2) & ~(WGRID - 1);
    if (hi - base < (uint32_t)(CAND - 1))
        base = hi - (uint32_t)(CAND - 1);
    return base;
}

// One approximate step: the state sa (binary64, so that it can carry an excess over the
// candidate it is snapped to) through a table.
__device__ __forceinline__ double approx_step(double sa, uint32_t base, const uint32_t *__restrict__ tab)
{
    bool hit;
    const uint32_t idx = nearest_candidate(__float_as_uint((float)sa), base, hit);
    const double e = sa - (double)__uint_as_float(base + idx);
    const double t = (double)__uint_as_float(tab[idx]);
    return (e == e && e - e == 0.0) ? t + e : t; // a non-finite excess is dropped
}

// The test of lane_tup_apply for a whole wave of different states: the map (wave-uniform) is
// applied if it is valid for every lane's state.
__device__ __forceinline__ bool apply_all(uint32_t &s, const LaneTup &l)
{
    const bool odd = (s & 1u) != 0u;
    const uint32_t smin = odd ? l.smin1 : l.smin0, smax = odd ? l.smax1 : l.smax0;
    const bool ok = s >= smin && s <= smax;
    if (!__all(ok))
        return false;
    s += (uint32_t)(odd ? l.t1 : l.t0);
    return true;
}

// half a chunk (32 elements) from LDS, the same for every lane
__device__ __forceinline__ void read_half(const float *__restrict__ xg, int h, f4v (&v)[CH / 8])
{
    const f4v *p = reinterpret_cast<const f4v *>(xg + h * (CH / 2));
#pragma unroll
    for (int k = 0; k < CH / 8; k++)
        v[k] = p[k];
}

// 32 real additions, each lane on its own state
__device__ __forceinline__ uint32_t add_half(uint32_t s, const f4v (&v)[CH / 8])
{
    float acc = __uint_as_float(s);
#pragma unroll
    for (int k = 0; k < CH / 8; k++)
    {
        acc = acc + v[k].x;
        acc = acc + v[k].y;
        acc = acc + v[k].z;
        acc = acc + v[k].w;
    }
    return __float_as_uint(acc);
}

struct NodeRegs
{
    float4 f[BLK / 1024]; // this thread's 16 elements of the block
    LaneTup lt;           // threads 0..63: a chunk map, 64..71: a group map, 72: the block map
};

// Thread tid's share of block blk (blocks past the end of the chain: -0.0f, which changes no state,
// and identity maps).
__device__ __forceinline__ void load_node_block(NodeRegs &r, const float *__restrict__ x, const Chains &c,
                                                const Tup *__restrict__ T1, const Tup *__restrict__ TG,
                                                const Tup *__restrict__ T2, int64_t blk, int tid, int vec)
{
    const int64_t n = c.n;
    Tup t = tup_identity(HYP_ANY);
    if (blk < c.nblk)
    {
        if (tid < BLK / CH)
            t = T1[blk * (BLK / CH) + tid];
        else if (tid < BLK / CH + GROUPS)
            t = TG[blk * GROUPS + (tid - BLK / CH)];
        else if (tid == BLK / CH + GROUPS)
            t = T2[blk];
    }
    r.lt = lane_tup(t);
    const int64_t e0 = blk * BLK;
#pragma unroll
    for (int q = 0; q < BLK / 1024; q++)
    {
        const int64_t idx = e0 + (int64_t)(q * 256 + tid) * 4;
        if (vec && idx + 3 < n)
            r.f[q] = *reinterpret_cast<const float4 *>(chain_ptr(x, c, idx)); // (segments are multiples of 16 long)
        else
        {
            r.f[q].x = (idx + 0 < n) ? *chain_ptr(x, c, idx + 0) : -0.0f;
            r.f[q].y = (idx + 1 < n) ? *chain_ptr(x, c, idx + 1) : -0.0f;
            r.f[q].z = (idx + 2 < n) ? *chain_ptr(x, c, idx + 2) : -0.0f;
            r.f[q].w = (idx + 3 < n) ? *chain_ptr(x, c, idx + 3) : -0.0f;
        }
    }
}

// Plan of a round: one wave per super-block that is not resolved yet.
//   - the window of each of its nodes: round 0 centres it on the binary64 prediction of step 2,
//     later rounds on the super-block centre the resolver left in sc[], taken through the previous
//     round's tables node by node;
//   - a node whose window has not moved keeps its table; a node whose own map holds for all its
//     candidates gets its table from that map; every other node goes on the list of walks.
// tab_*: [rows][nnode][CAND] exit states, nbase_*: [rows][nnode] first candidate of each window.
__global__ __launch_bounds__(64) void sum1d_plan_kernel(const double *__restrict__ prefix, const Tup *__restrict__ TN,
                                                        const Ctl *__restrict__ ctl, const float *__restrict__ sc,
                                                        const float *__restrict__ hc, const float *__restrict__ SA,
                                                        const uint32_t *__restrict__ sbase,
                                                        const uint32_t *__restrict__ nbase_old, const uint32_t *__restrict__ tab_old,
                                                        uint32_t *__restrict__ nbase_new, uint32_t *__restrict__ tab_new,
                                                        int *__restrict__ worklist, Work *__restrict__ work, int64_t nblk,
                                                        int64_t nnode, int64_t nsup, int round)
{
    const int lane = threadIdx.x;
    const int64_t row = blockIdx.y, sb = blockIdx.x;
    const int cap = (int)(nnode * gridDim.y); // entries of the list
    const int64_t front = ctl[row].front;
    if (front >= nsup || sb < front)
        return; // resolved already
    prefix += row * nblk;
    TN += row * nnode;
    sc += row * nsup;
    hc += row * ((nsup + HB - 1) / HB);
    SA += row * nsup * CAND;
    sbase += row * nsup;
    nbase_old += row * nnode;
    nbase_new += row * nnode;
    tab_old += row * nnode * CAND;
    tab_new += row * nnode * CAND;
    const int64_t n0 = sb * NPS;
    const int cnt = nnode - n0 < NPS ? (int)(nnode - n0) : NPS;
    float centre = 0.0f; // lane i: node n0 + i
    // Later rounds chain through tables -- the approximate offsets of the super-blocks before this one in
    // its hyper-block, then the previous round's tables of its own nodes.  All of them come into LDS first,
    // in one round trip: read where they lie, every step of the chain was a trip to memory of its own.
    __shared__ __attribute__((aligned(16))) float lsa[HB - 1][CAND];
    __shared__ __attribute__((aligned(16))) uint32_t ltab[NPS][CAND];
    __shared__ uint32_t lsb[HB], lnb[NPS];
    if (round == 0)
    {
        if (lane < cnt)
            centre = (float)prefix[(n0 + lane) * NODEB];
    }
    else
    {
        const bool near_front = sb / HB == front / HB;
        const int64_t jh = sb / HB * HB;
        const int before = near_front ? 0 : (int)(sb - jh);
#pragma unroll
        for (int j = 0; j < HB - 1; j++)
            if (j < before)
                reinterpret_cast<uint4 *>(lsa[j])[lane] = reinterpret_cast<const uint4 *>(SA + (jh + j) * CAND)[lane];
#pragma unroll
        for (int i = 0; i < NPS; i++)
            if (i < cnt)
                reinterpret_cast<uint4 *>(ltab[i])[lane] = reinterpret_cast<const uint4 *>(tab_old + (n0 + i) * CAND)[lane];
        if (lane < before)
            lsb[lane] = sbase[jh + lane];
        if (lane < cnt)
            lnb[lane] = nbase_old[n0 + lane];
        // (wave-uniform chain)  The resolver left a centre for every super-block of the hyper-block
        // the front lies in, and for the first super-block of every later hyper-block; from
        // there the centre goes through the approximate offsets of the super-blocks before this one.
        double sa = near_front ? (double)sc[sb] : (double)hc[sb / HB];
        __syncthreads();
        for (int j = 0; j < before; j++)
        {
            bool hit;
            const uint32_t idx = nearest_candidate(__float_as_uint((float)sa), lsb[j], hit);
            sa += (double)lsa[j][idx];
        }
        for (int i = 0; i < cnt; i++)
        {
            centre = lane == i ? (float)sa : centre;
            sa = approx_step(sa, lnb[i], ltab[i]);
        }
    }
    int kind = -1; // 0: keep the old table, 1: the node's own map, 2: walk
    uint32_t base = 0u;
    int t0 = 0, t1 = 0;
    if (lane < cnt)
    {
        base = window_base(__float_as_uint(centre));
        nbase_new[n0 + lane] = base;
        const LaneTup ln = lane_tup(TN[n0 + lane]);
        t0 = ln.t0;
        t1 = ln.t1;
        // candidates base .. base + CAND - 1: the even ones and the odd ones each inside their interval
        const uint32_t e0 = base + (base & 1u), e1 = base + CAND - 2 + (base & 1u);
        const uint32_t o0 = base + 1 - (base & 1u), o1 = base + CAND - 1 - (base & 1u);
        const bool whole = e0 >= ln.smin0 && e1 <= ln.smax0 && o0 >= ln.smin1 && o1 <= ln.smax1 && e1 >= e0 && o1 >= o0;
        kind = (round != 0 && lnb[lane] == base) ? 0 : (whole ? 1 : 2);
        if (kind == 2)
        {
            const int gn = (int)(row * nnode + n0 + lane);
            if (TN[n0 + lane].heavy >= HEAVY_CHUNKS)
                worklist[atomicAdd(&work[round].count, 1)] = gn;
            else
                worklist[cap - 1 - atomicAdd(&work[round].light, 1)] = gn;
        }
    }
    for (int i = 0; i < cnt; i++)
    {
        const int k = __shfl(kind, i, 64);
        if (k == 2)
            continue;
        const uint32_t b = (uint32_t)__shfl((int)base, i, 64);
        const int a0 = __shfl(t0, i, 64), a1 = __shfl(t1, i, 64);
#pragma unroll
        for (int q = 0; q < CAND / 64; q++)
        {
            const int c = q * 64 + lane;
            const uint32_t st = b + (uint32_t)c;
            tab_new[(n0 + i) * CAND + c] = k == 0 ? ltab[i][c] : st + (uint32_t)((st & 1u) ? a1 : a0);
        }
    }
}


// The walks of a round: workgroups of 256 threads take nodes off the list until it is empty
// (every workgroup leaves the loop: the list's length is fixed before the launch).  Thread t
// carries candidate t of the node's window.
__global__ __launch_bounds__(256) void sum1d_cand_walk_kernel(
    const float *__restrict__ x, Chains c, const Tup *__restrict__ T1, const Tup *__restrict__ TG,
    const Tup *__restrict__ T2, const uint32_t *__restrict__ nbase, uint32_t *__restrict__ tab,
    const int *__restrict__ worklist, Work *__restrict__ work, int64_t nnode, int cap, int round, int vec)
{
    __shared__ __attribute__((aligned(16))) float xd[2][BLK];
    __shared__ __attribute__((aligned(16))) LaneTup lmap[2][BLK / CH + GROUPS + 1];
    __shared__ int item_s;
    const int tid = threadIdx.x;
    const int front_count = work[round].count, count = front_count + work[round].light;
    // A workgroup's first node is the one of its own index, the later ones come off a counter: a round
    // with nothing (or little) left to walk costs the idle workgroups no atomic -- a thousand of them on
    // one address were 12 us of every such round.
    for (bool first = true;; first = false)
    {
        if (first && (int)blockIdx.x >= count) // (uniform)
            break;
        if (!first && tid == 0)
            item_s = (int)gridDim.x + atomicAdd(&work[round].next, 1);
        __syncthreads();
        const int item = first ? (int)blockIdx.x : item_s;
        __syncthreads(); // (everyone has read item_s, and has finished with the LDS of the previous node)
        if (item >= count)
            break;
        const int64_t gn = worklist[item < front_count ? item : cap - 1 - (item - front_count)], row = gn / nnode,
                      nd = gn - row * nnode;
        const float *xr = x + row * c.row_stride;
        const Tup *T1r = T1 + row * c.nblk * (BLK / CH), *TGr = TG + row * c.nblk * GROUPS, *T2r = T2 + row * c.nblk;
        uint32_t s = nbase[gn] + (uint32_t)tid;
        NodeRegs r;
        load_node_block(r, xr, c, T1r, TGr, T2r, nd * NODEB, tid, vec);
        for (int b = 0; b < NODEB; b++)
        {
            const int buf = b & 1;
#pragma unroll
            for (int q = 0; q < BLK / 1024; q++)
                *reinterpret_cast<float4 *>(&xd[buf][(q * 256 + tid) * 4]) = r.f[q];
            if (tid <= BLK / CH + GROUPS)
                lmap[buf][tid] = r.lt;
            // One barrier per block is enough: a wave that stores block b + 1 into the other buffer
            // has passed this barrier, so every wave has finished walking block b - 1 in it.
            __syncthreads();
            if (b + 1 < NODEB)
                load_node_block(r, xr, c, T1r, TGr, T2r, nd * NODEB + b + 1, tid, vec);
            if (apply_all(s, lmap[buf][BLK / CH + GROUPS]))
                continue;
            // Where the sum is small against its elements nothing applies, block after block; a
            // test costs a quarter of a replay there, and a replay is always right.  So after two
            // failures in a row the rest of the unit (the groups of a block, the chunks of a group)
            // is taken without testing.
            int gfail = 0;
            for (int gr = 0; gr < GROUPS; gr++)
            {
                if (gfail < 2 && apply_all(s, lmap[buf][BLK / CH + gr]))
                {
                    gfail = 0;
                    continue;
                }
                gfail++;
                constexpr int CG = BLK / CH / GROUPS; // 8 chunks; their data is read half a chunk ahead of the additions
                const float *xg = &xd[buf][gr * CG * CH];
                f4v ha[CH / 8], hb[CH / 8];
                int cfail = 0;
                read_half(xg, 0, ha);
#pragma unroll
                for (int j = 0; j < CG; j++)
                {
                    read_half(xg, 2 * j + 1, hb);
                    const bool replay = cfail >= 2 || !apply_all(s, lmap[buf][gr * CG + j]);
                    if (replay)
                    {
                        s = add_half(s, ha);
                    }
                    if (j + 1 < CG)
                        read_half(xg, 2 * j + 2, ha);
                    if (replay)
                        s = add_half(s, hb);
                    cfail = replay ? cfail + 1 : 0;
                }
            }
        }
        tab[gn * CAND + tid] = s;
    }
}

// ---- step 4b: the node tables of a super-block composed ----------------------------------------
// grid (super-blocks, rows), 256 threads: thread k takes candidate k of the super-block's first
// node through the tables of its nodes.  SE[k]: the exit state, exact if bit k of SOK is set
// (every intermediate state was a candidate of the next node); SA[k]: exit minus entry as a
// binary32 offset, approximate where a state had to be snapped to the nearest candidate.
__global__ __launch_bounds__(256) void sum1d_compose_kernel(const uint32_t *__restrict__ nbase, const uint32_t *__restrict__ tab,
                                                            const Ctl *__restrict__ ctl, uint32_t *__restrict__ SE,
                                                            float *__restrict__ SA, uint32_t *__restrict__ SOK,
                                                            uint32_t *__restrict__ sbase, int64_t nnode, int64_t nsup)
{
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.y, sb = blockIdx.x;
    const int64_t front = ctl[row].front;
    if (front >= nsup || sb < front)
        return;
    nbase += row * nnode;
    tab += row * nnode * CAND;
    SE += (row * nsup + sb) * CAND;
    SA += (row * nsup + sb) * CAND;
    SOK += (row * nsup + sb) * (CAND / 32);
    const int64_t n0 = sb * NPS;
    const int cnt = nnode - n0 < NPS ? (int)(nnode - n0) : NPS;
    // the tables of the super-block's nodes, brought into LDS together: the chain below is then sixteen
    // LDS reads in a row instead of sixteen round trips to memory
    __shared__ uint32_t ltab[NPS][CAND];
    __shared__ uint32_t lbase[NPS];
#pragma unroll
    for (int i = 0; i < NPS; i++)
        if (i < cnt)
            ltab[i][tid] = tab[(n0 + i) * CAND + tid];
    if (tid < cnt)
        lbase[tid] = nbase[n0 + tid];
    __syncthreads();
    const uint32_t base0 = lbase[0];
    uint32_t y = base0 + (uint32_t)tid; // exact while ok
    bool ok = true;
    double sa = 0.0; // the approximate state once a window was missed
    for (int i = 0; i < cnt; i++)
    {
        const uint32_t b = lbase[i];
        const uint32_t *t = ltab[i];
        if (ok)
        {
            const uint32_t d = y - b;
            if (d < (uint32_t)CAND)
            {
                y = t[d];
                continue;
            }
            ok = false;
            sa = (double)__uint_as_float(y);
        }
        sa = approx_step(sa, b, t);
    }
    const double entry = (double)__uint_as_float(base0 + (uint32_t)tid);
    SE[tid] = y;
    SA[tid] = (float)((ok ? (double)__uint_as_float(y) : sa) - entry);
    const unsigned long long m = __ballot(ok);
    if ((tid & 63) == 0)
    {
        SOK[(tid >> 6) * 2] = (uint32_t)m;
        SOK[(tid >> 6) * 2 + 1] = (uint32_t)(m >> 32);
    }
    if (tid == 0)
        sbase[row * nsup + sb] = base0;
}

// ---- step 4b': the super-block tables of a hyper-block composed ----------------------------------
// The same composition one level up: grid (hyper-blocks, rows), 256 threads; thread k takes candidate
// k of the hyper-block's first unresolved super-block through its super-blocks.  HE / HOK / HA as
// SE / SOK / SA.
__global__ __launch_bounds__(256) void sum1d_compose2_kernel(const uint32_t *__restrict__ SE, const float *__restrict__ SA,
                                                             const uint32_t *__restrict__ SOK, const uint32_t *__restrict__ sbase,
                                                             const Ctl *__restrict__ ctl, uint32_t *__restrict__ HE,
                                                             float *__restrict__ HA, uint32_t *__restrict__ HOK,
                                                             uint32_t *__restrict__ hbase, int64_t nsup, int64_t nhyp)
{
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.y, h = blockIdx.x;
    const int64_t front = ctl[row].front;
    if (front >= nsup || h < front / HB)
        return;
    SE += row * nsup * CAND;
    SA += row * nsup * CAND;
    SOK += row * nsup * (CAND / 32);
    sbase += row * nsup;
    HE += (row * nhyp + h) * CAND;
    HA += (row * nhyp + h) * CAND;
    HOK += (row * nhyp + h) * (CAND / 32);
    const int64_t j0 = h * HB > front ? h * HB : front, j1 = (h + 1) * HB < nsup ? (h + 1) * HB : nsup;
    const int cnt = (int)(j1 - j0);
    // the tables of the hyper-block's super-blocks in LDS (as in sum1d_compose_kernel)
    __shared__ uint32_t lse[HB][CAND];
    __shared__ float lsa[HB][CAND];
    __shared__ uint32_t lok[HB][CAND / 32];
    __shared__ uint32_t lbase[HB];
#pragma unroll
    for (int i = 0; i < HB; i++)
        if (i < cnt)
        {
            lse[i][tid] = SE[(j0 + i) * CAND + tid];
            lsa[i][tid] = SA[(j0 + i) * CAND + tid];
        }
    if (tid < cnt * (CAND / 32))
        lok[tid / (CAND / 32)][tid % (CAND / 32)] = SOK[j0 * (CAND / 32) + tid];
    else if (tid >= 128 && tid < 128 + cnt)
        lbase[tid - 128] = sbase[j0 + tid - 128];
    __syncthreads();
    const uint32_t base0 = lbase[0];
    uint32_t y = base0 + (uint32_t)tid; // exact while ok
    bool ok = true;
    double sa = 0.0;
    for (int i = 0; i < cnt; i++)
    {
        const uint32_t b = lbase[i];
        if (ok)
        {
            const uint32_t d = y - b;
            if (d < (uint32_t)CAND && ((lok[i][d >> 5] >> (d & 31u)) & 1u) != 0u)
            {
                y = lse[i][d];
                continue;
            }
            ok = false;
            sa = (double)__uint_as_float(y);
        }
        bool hit;
        const uint32_t idx = nearest_candidate(__float_as_uint((float)sa), b, hit);
        sa += (double)lsa[i][idx];
    }
    const double entry = (double)__uint_as_float(base0 + (uint32_t)tid);
    HE[tid] = y;
    HA[tid] = (float)((ok ? (double)__uint_as_float(y) : sa) - entry);
    const unsigned long long m = __ballot(ok);
    if ((tid & 63) == 0)
    {
        HOK[(tid >> 6) * 2] = (uint32_t)m;
        HOK[(tid >> 6) * 2 + 1] = (uint32_t)(m >> 32);
    }
    if (tid == 0)
        hbase[row * nhyp + h] = base0;
}

// ---- step 4c: the true state through the tables --------------------------------------------------
// One workgroup of 256 threads per row; every thread runs the same chain (all reads are LDS
// broadcasts), so that the workgroup can stage tables together wherever the chain needs them.
// The state steps through the hyper-block tables (RB at a time in LDS, requested RD batches
// ahead) while it finds itself among the candidates and the entry is exact.  At the first miss
// the sixteen super-block tables of that hyper-block come into LDS and the state steps through
// those up to the super-block that misses: the new front.  From there the chain is approximate
// (nearest candidate, the excess kept in binary64) and leaves the predictions of the next round:
// sc[] for the rest of this hyper-block, hc[] for every later hyper-block.
constexpr int RB = 4; // hyper-blocks per batch
constexpr int RD = 4; // batches in flight

__global__ __launch_bounds__(256) void sum1d_resolve_kernel(
    const uint32_t *__restrict__ HE, const float *__restrict__ HA, const uint32_t *__restrict__ HOK,
    const uint32_t *__restrict__ hbase, const uint32_t *__restrict__ SE, const float *__restrict__ SA,
    const uint32_t *__restrict__ SOK, const uint32_t *__restrict__ sbase, float *__restrict__ sc, float *__restrict__ hc,
    Ctl *__restrict__ ctl, float factor, float *__restrict__ out, int64_t nsup, int64_t nhyp)
{
    __shared__ __attribute__((aligned(16))) uint32_t lhe[2][RB][CAND];
    __shared__ __attribute__((aligned(16))) float lha[2][RB][CAND];
    __shared__ uint32_t lhok[2][RB][CAND / 32];
    __shared__ uint32_t lhbase[2][RB];
    __shared__ __attribute__((aligned(16))) uint32_t dse[HB][CAND];
    __shared__ __attribute__((aligned(16))) float dsa[HB][CAND];
    __shared__ uint32_t dok[HB][CAND / 32];
    __shared__ uint32_t dbase[HB];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int64_t front = ctl[row].front;
    if (front >= nsup)
        return;
    HE += row * nhyp * CAND;
    HA += row * nhyp * CAND;
    HOK += row * nhyp * (CAND / 32);
    hbase += row * nhyp;
    SE += row * nsup * CAND;
    SA += row * nsup * CAND;
    SOK += row * nsup * (CAND / 32);
    sbase += row * nsup;
    sc += row * nsup;
    hc += row * nhyp;
    const int64_t h0 = front / HB;
    const int64_t nbatch = (nhyp - h0 + RB - 1) / RB;
    // this thread's part of a batch: 16 bytes of each hyper-block's exact and approximate table
    // (tid: hyper-block tid / 64, piece tid % 64), one word of the masks / bases
    const int wh = tid >> 6, wq = tid & 63;
    uint4 pfe[RD], pfa[RD];
    uint32_t pfw[RD];
    auto request = [&](int64_t bt, uint4 &ve, uint4 &va, uint32_t &word) {
        ve = va = make_uint4(0u, 0u, 0u, 0u);
        word = 0u;
        if (bt >= nbatch)
            return;
        const int64_t h = h0 + bt * RB + wh;
        if (h < nhyp)
        {
            ve = reinterpret_cast<const uint4 *>(HE + h * CAND)[wq];
            va = reinterpret_cast<const uint4 *>(HA + h * CAND)[wq];
        }
        if (tid < RB * (CAND / 32))
        {
            const int64_t hh = h0 + bt * RB + tid / (CAND / 32);
            word = hh < nhyp ? HOK[hh * (CAND / 32) + tid % (CAND / 32)] : 0u;
        }
        else if (tid < RB * (CAND / 32) + RB)
        {
            const int64_t hh = h0 + bt * RB + (tid - RB * (CAND / 32));
            word = hh < nhyp ? hbase[hh] : 0u;
        }
    };
#pragma unroll
    for (int d = 0; d < RD; d++)
        request(d, pfe[d], pfa[d], pfw[d]);
    uint32_t s = ctl[row].s;
    bool exact = true;
    double sa = 0.0;
    int64_t new_front = nsup;
    uint32_t s_front = 0u;
    for (int64_t bt0 = 0; bt0 < nbatch; bt0 += RD)
    {
#pragma unroll
        for (int d = 0; d < RD; d++)
        {
            const int64_t bt = bt0 + d;
            if (bt >= nbatch) // (uniform)
                break;
            const int buf = d & 1; // RD is even
            reinterpret_cast<uint4 *>(&lhe[buf][wh][0])[wq] = pfe[d];
            reinterpret_cast<uint4 *>(&lha[buf][wh][0])[wq] = pfa[d];
            if (tid < RB * (CAND / 32))
                lhok[buf][tid / (CAND / 32)][tid % (CAND / 32)] = pfw[d];
            else if (tid < RB * (CAND / 32) + RB)
                lhbase[buf][tid - RB * (CAND / 32)] = pfw[d];
            // (this batch's buffer was last read two batches ago, and a barrier lies in between)
            __syncthreads();
            request(bt + RD, pfe[d], pfa[d], pfw[d]);
            for (int i = 0; i < RB; i++)
            {
                const int64_t h = h0 + bt * RB + i;
                if (h >= nhyp)
                    break;
                const uint32_t base = lhbase[buf][i];
                if (exact)
                {
                    const uint32_t dd = s - base;
                    const uint32_t k = dd < (uint32_t)CAND ? dd : 0u;
                    const uint32_t nxt = lhe[buf][i][k];
                    const uint32_t okw = lhok[buf][i][k >> 5];
                    if (dd < (uint32_t)CAND && ((okw >> (k & 31u)) & 1u) != 0u)
                    {
                        s = nxt; // an exact step over a whole hyper-block
                        continue;
                    }
                    // somewhere inside this hyper-block the state is not among the candidates:
                    // its super-block tables, together
                    const int64_t j0 = h * HB > front ? h * HB : front, j1 = (h + 1) * HB < nsup ? (h + 1) * HB : nsup;
                    const int cnt = (int)(j1 - j0);
                    __syncthreads(); // (whoever still reads the tables of an earlier descent)
                    for (int q = tid; q < cnt * (CAND / 4); q += 256)
                    {
                        const int jj = q / (CAND / 4), pc = q % (CAND / 4);
                        reinterpret_cast<uint4 *>(&dse[jj][0])[pc] = reinterpret_cast<const uint4 *>(SE + (j0 + jj) * CAND)[pc];
                        reinterpret_cast<uint4 *>(&dsa[jj][0])[pc] = reinterpret_cast<const uint4 *>(SA + (j0 + jj) * CAND)[pc];
                    }
                    if (tid < cnt * (CAND / 32))
                        dok[tid / (CAND / 32)][tid % (CAND / 32)] = SOK[(j0 + tid / (CAND / 32)) * (CAND / 32) + tid % (CAND / 32)];
                    else if (tid >= 128 && tid < 128 + cnt)
                        dbase[tid - 128] = sbase[j0 + tid - 128];
                    __syncthreads();
                    int jj = 0;
                    for (; jj < cnt; jj++)
                    {
                        const uint32_t d2 = s - dbase[jj];
                        const uint32_t k2 = d2 < (uint32_t)CAND ? d2 : 0u;
                        if (!(d2 < (uint32_t)CAND && ((dok[jj][k2 >> 5] >> (k2 & 31u)) & 1u) != 0u))
                            break;
                        s = dse[jj][k2];
                    }
                    if (jj == cnt)
                        continue; // (every super-block hit after all)
                    exact = false;
                    new_front = j0 + jj;
                    s_front = s;
                    sa = (double)__uint_as_float(s);
                    for (; jj < cnt; jj++)
                    {
                        const float f = (float)sa;
                        if (tid == 0)
                            sc[j0 + jj] = f;
                        bool hit;
                        const uint32_t idx = nearest_candidate(__float_as_uint(f), dbase[jj], hit);
                        sa += (double)dsa[jj][idx];
                    }
                    continue;
                }
                // approximate from here on: predictions for the next round
                const float f = (float)sa;
                if (tid == 0)
                    hc[h] = f;
                bool hit;
                const uint32_t idx = nearest_candidate(__float_as_uint(f), base, hit);
                sa += (double)lha[buf][i][idx];
            }
        }
    }
    if (tid == 0)
    {
        if (exact)
        {
            ctl[row].front = (int)nsup;
            ctl[row].s = s;
            out[row] = factor * __uint_as_float(s);
        }
        else
        {
            ctl[row].front = (int)new_front;
            ctl[row].s = s_front;
        }
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline size_t round256(size_t v) { return (v + 255) & ~(size_t)255; }
} // namespace

// serial single-chain kernel of sum.hip
int repdl_sum1d_serial(const float *in, float *out, int64_t n, int average, void *stream);

// Number of speculative rounds for `rows` chains of n elements (0: step 4 alone).
static int spec_rounds(int64_t rows, int64_t n)
{
    // Chains that come in rows: three rounds when the chains are very long and their nodes few enough
    // for one pass of the walkers.  Zero-mean chains gain (16 x 802816: 1.27 -> 0.42 ms, 8 x 2^20: 1.07 ->
    // 0.37), chains that drift lose the rounds' fifteen launches (0.09 -> 0.14 ms).  At 200704 elements
    // (64 channels of 64 images of 56x56) gain and loss are the same 0.1 ms (0.50 -> 0.33 against 0.08 ->
    // 0.18) and a residual block with BatchNorm got 3 % slower with the rounds: not there.  256 x 262144
    // (4096 nodes) got slower either way; 64 x 802816 (3136 nodes: the first BatchNorm of a ResNet at batch 64)
    // 1.37 -> 0.69 ms zero-mean, 0.21 -> 0.33 drifting.  (Rounds from 2^17 elements made a ResNet-18 training step at
    // batch 64 five milliseconds slower, 49 -> 54.7, and still one millisecond slower, 38.8 -> 39.9, once the host no
    // longer waited for every workspace: they fill the chip that the other streams' kernels would use.)
    if (rows > 1)
        return (n >= ((int64_t)1 << 19) && rows * repdl_cdiv(repdl_cdiv(n, BLK), NODEB) <= 3200) ? 3 : 0;
    // A single chain: two rounds from 2^18 elements on.  The lone walk of step 4 on zero-mean data takes
    // 0.54 / 0.62 / 0.81 / 1.07 ms at 2^18 / 2^19 / 2^20 / 2^21 elements (it grows with the length, and 2^22
    // with four rounds takes 0.36); after two rounds it is 0.20 / 0.21 / 0.21 / 0.22 ms.  Chains that drift
    // pay the rounds' ten launches: 0.044 / 0.056 / 0.062 / 0.070 -> 0.09 / 0.08 / 0.085 / 0.09 ms.  (At 2^17
    // elements: 0.27 -> 0.20 against 0.04 -> 0.07, and the mean of a cross_entropy over that many rows is of
    // the drifting kind: not there.  Three rounds instead of two: 0.01 ms slower both ways.)
    if (n < ((int64_t)1 << 18))
        return 0;
    if (n < ((int64_t)1 << 22))
        return 2;
    return n < ((int64_t)1 << 24) ? 4 : (n < ((int64_t)1 << 26) ? 8 : MAX_ROUNDS);
}

namespace
{
struct Layout
{
    size_t bsum, babs, refine, prefix, T3, TN, T2, TG, T1, ctl, work, sc, nbase[2], tab[2], worklist, SE, SA, SOK, sbase, HE, HA, HOK, hbase, hc, total;
};

Layout layout(int64_t rows, int64_t n)
{
    const size_t nblk = (size_t)repdl_cdiv(n, BLK), nnode = (size_t)repdl_cdiv((int64_t)nblk, NODEB),
                 nsup = (size_t)repdl_cdiv((int64_t)nblk, SUP), r = (size_t)rows;
    Layout l;
    size_t at = 0;
    auto take = [&](size_t bytes) {
        const size_t here = at;
        at += round256(bytes);
        return here;
    };
    l.bsum = take(r * nblk * sizeof(double));
    l.babs = take(r * nblk * sizeof(double));
    l.refine = take(r * sizeof(int));
    l.prefix = take(r * nblk * sizeof(double));
    l.T3 = take(r * nsup * sizeof(Tup));
    l.TN = take(r * nnode * sizeof(Tup));
    l.T2 = take(r * nblk * sizeof(Tup));
    l.TG = take(r * nblk * GROUPS * sizeof(Tup));
    l.T1 = take(r * nblk * (BLK / CH) * sizeof(Tup));
    l.ctl = take(r * sizeof(Ctl));
    l.work = take(MAX_ROUNDS * sizeof(Work));
    const bool spec = spec_rounds(rows, n) > 0;
    l.sc = take(spec ? r * nsup * sizeof(float) : 0);
    for (int i = 0; i < 2; i++)
        l.nbase[i] = take(spec ? r * nnode * sizeof(uint32_t) : 0);
    for (int i = 0; i < 2; i++)
        l.tab[i] = take(spec ? r * nnode * CAND * sizeof(uint32_t) : 0);
    l.worklist = take(spec ? r * nnode * sizeof(int) : 0);
    l.SE = take(spec ? r * nsup * CAND * sizeof(uint32_t) : 0);
    l.SA = take(spec ? r * nsup * CAND * sizeof(float) : 0);
    l.SOK = take(spec ? r * nsup * (CAND / 32) * sizeof(uint32_t) : 0);
    l.sbase = take(spec ? r * nsup * sizeof(uint32_t) : 0);
    const size_t nhyp = (nsup + HB - 1) / HB;
    l.HE = take(spec ? r * nhyp * CAND * sizeof(uint32_t) : 0);
    l.HA = take(spec ? r * nhyp * CAND * sizeof(float) : 0);
    l.HOK = take(spec ? r * nhyp * (CAND / 32) * sizeof(uint32_t) : 0);
    l.hbase = take(spec ? r * nhyp * sizeof(uint32_t) : 0);
    l.hc = take(spec ? r * nhyp * sizeof(float) : 0);
    l.total = at;
    return l;
}
} // namespace

// Scratch for `rows` chains of n elements.
size_t repdl_sum_chains_workspace_bytes(int64_t rows, int64_t n) { return layout(rows, n).total; }

// out[r] = factor * (the sequential sum of chain r), r < rows, by the parallel evaluation.
// Chain r: nseg segments of seglen contiguous floats, segment s at in + r*row_stride +
// s*seg_stride.  The caller has checked: n = nseg*seglen >= 1, rows in [1, 65535], and for
// nseg > 1 that seglen is a multiple of 16 and n < 2^31.
// Every word of the scratch memory that is read has been written earlier in the same call, so
// it may hold anything on entry.
int repdl_sum_chains(const float *in, float *out, int64_t rows, int64_t nseg, int64_t seglen, int64_t row_stride,
                     int64_t seg_stride, float factor, void *workspace, size_t workspace_bytes, void *stream)
{
    const int64_t n = nseg * seglen;
    REPDL_REQUIRE(rows >= 1 && rows <= 65535 && n >= 1 && in != nullptr && out != nullptr);
    REPDL_REQUIRE(nseg == 1 || (seglen % 16 == 0 && n <= REPDL_I32_MAX));
    const Layout l = layout(rows, n);
    if (workspace == nullptr || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 15) != 0)
        return REPDL_E_WORKSPACE;
    const int64_t nblk = repdl_cdiv(n, BLK), nnode = repdl_cdiv(nblk, NODEB), nsup = repdl_cdiv(nblk, SUP);
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
    double *bsum = reinterpret_cast<double *>(w + l.bsum), *prefix = reinterpret_cast<double *>(w + l.prefix);
    Tup *T3 = reinterpret_cast<Tup *>(w + l.T3), *TN = reinterpret_cast<Tup *>(w + l.TN), *T2 = reinterpret_cast<Tup *>(w + l.T2),
        *TG = reinterpret_cast<Tup *>(w + l.TG), *T1 = reinterpret_cast<Tup *>(w + l.T1);
    Ctl *ctl = reinterpret_cast<Ctl *>(w + l.ctl);
    Work *work = reinterpret_cast<Work *>(w + l.work);
    hipStream_t s = repdl_stream(stream);
    // 16-byte loads: every row and segment starts on a 16-byte boundary
    const int vec = aligned16(in) && (rows == 1 || row_stride % 4 == 0) && (nseg == 1 || seg_stride % 4 == 0);
    const dim3 g2((unsigned)nblk, (unsigned)rows);
    double *babs = reinterpret_cast<double *>(w + l.babs);
    int *refine = reinterpret_cast<int *>(w + l.refine);
    const int rounds = spec_rounds(rows, n);
    // One short chain: two launches instead of seven (the map pass makes its own prediction, the walk joins
    // the one super-block's tuple itself).  65536 elements: 0.040 -> 0.016 ms.
    if (rows == 1 && nseg == 1 && rounds == 0 && nsup == 1)
    {
        repdl_route_note(REPDL_ROUTE_SUM_CHAINS);
        REPDL_LAUNCH(sum1d_tuple_kernel, g2, dim3(256), 0, s, in, c, prefix, T1, TG, T2, vec, 1);
        REPDL_LAUNCH(sum1d_walk_kernel, dim3(1), dim3(64), 0, s, in, c, T1, TG, T2, T3, ctl, factor, out, vec, 1);
        return repdl_launch_status();
    }
    REPDL_LAUNCH(sum1d_blocksum_kernel, g2, dim3(256), 0, s, in, c, static_cast<const double *>(nullptr), bsum, babs, refine, vec);
    REPDL_LAUNCH(sum1d_prefix_kernel, dim3((unsigned)repdl_cdiv(nblk, PREFIX_TILE), (unsigned)rows), dim3(1024), 0, s, bsum, prefix,
                 nblk, static_cast<const double *>(babs), refine, n);
    // Chains of one super-block, walked from their start: four launches instead of seven.  The refinement is for
    // sums that stall -- elements below half a quantum of the state, which takes 2^24 of them -- and the walk joins
    // the one super-block's tuple itself (channel sums of [64,128,28,28]: 0.186 -> 0.181 ms, of its ReLU 0.060 -> 0.055).
    if (rounds == 0 && nsup == 1)
    {
        repdl_route_note(REPDL_ROUTE_SUM_CHAINS);
        REPDL_LAUNCH(sum1d_tuple_kernel, g2, dim3(256), 0, s, in, c, prefix, T1, TG, T2, vec, 0);
        REPDL_LAUNCH(sum1d_walk_kernel, dim3((unsigned)rows), dim3(64), 0, s, in, c, T1, TG, T2, T3, ctl, factor, out, vec, 1);
        return repdl_launch_status();
    }
    // one refinement of the prediction (see quantum_of)
    REPDL_LAUNCH(sum1d_blocksum_kernel, g2, dim3(256), 0, s, in, c, static_cast<const double *>(prefix), bsum, babs, refine, vec);
    REPDL_LAUNCH(sum1d_prefix_kernel, dim3((unsigned)repdl_cdiv(nblk, PREFIX_TILE), (unsigned)rows), dim3(1024), 0, s, bsum, prefix,
                 nblk, static_cast<const double *>(nullptr), refine, n);
    REPDL_LAUNCH(sum1d_tuple_kernel, g2, dim3(256), 0, s, in, c, prefix, T1, TG, T2, vec, 0);
    REPDL_LAUNCH(sum1d_super_kernel, dim3((unsigned)repdl_cdiv(nsup, 4), (unsigned)rows), dim3(256), 0, s, T2, TN, T3, ctl,
                       work, nblk, nnode, nsup);
    repdl_route_note(rounds > 0 ? REPDL_ROUTE_SUM_CHAINS_ROUNDS : REPDL_ROUTE_SUM_CHAINS);
    if (rounds > 0)
    {
        float *sc = reinterpret_cast<float *>(w + l.sc);
        uint32_t *nbase[2] = {reinterpret_cast<uint32_t *>(w + l.nbase[0]), reinterpret_cast<uint32_t *>(w + l.nbase[1])};
        uint32_t *tab[2] = {reinterpret_cast<uint32_t *>(w + l.tab[0]), reinterpret_cast<uint32_t *>(w + l.tab[1])};
        uint32_t *SE = reinterpret_cast<uint32_t *>(w + l.SE), *SOK = reinterpret_cast<uint32_t *>(w + l.SOK),
                 *sbase = reinterpret_cast<uint32_t *>(w + l.sbase);
        float *SA = reinterpret_cast<float *>(w + l.SA);
        int *worklist = reinterpret_cast<int *>(w + l.worklist);
        const int64_t nhyp = repdl_cdiv(nsup, HB);
        uint32_t *HE = reinterpret_cast<uint32_t *>(w + l.HE), *HOK = reinterpret_cast<uint32_t *>(w + l.HOK),
                 *hbase = reinterpret_cast<uint32_t *>(w + l.hbase);
        float *HA = reinterpret_cast<float *>(w + l.HA), *hc = reinterpret_cast<float *>(w + l.hc);
        for (int r = 0; r < rounds; r++)
        {
            const int cur = r & 1, old = cur ^ 1;
            REPDL_LAUNCH(sum1d_plan_kernel, dim3((unsigned)nsup, (unsigned)rows), dim3(64), 0, s, prefix, TN, ctl, sc, hc, SA, sbase,
                               nbase[old], tab[old], nbase[cur], tab[cur], worklist, work, nblk, nnode, nsup, r);
            const int64_t walkers = nnode * rows < 1024 ? nnode * rows : 1024; // four workgroups per CU
            REPDL_LAUNCH(sum1d_cand_walk_kernel, dim3((unsigned)walkers), dim3(256), 0, s, in, c, T1, TG, T2, nbase[cur], tab[cur],
                               worklist, work, nnode, (int)(nnode * rows), r, vec);
            REPDL_LAUNCH(sum1d_compose_kernel, dim3((unsigned)nsup, (unsigned)rows), dim3(256), 0, s, nbase[cur], tab[cur], ctl,
                               SE, SA, SOK, sbase, nnode, nsup);
            REPDL_LAUNCH(sum1d_compose2_kernel, dim3((unsigned)nhyp, (unsigned)rows), dim3(256), 0, s, SE, SA, SOK, sbase, ctl, HE,
                               HA, HOK, hbase, nsup, nhyp);
            REPDL_LAUNCH(sum1d_resolve_kernel, dim3((unsigned)rows), dim3(256), 0, s, HE, HA, HOK, hbase, SE, SA, SOK, sbase, sc,
                               hc, ctl, factor, out, nsup, nhyp);
        }
    }
    // whatever the rounds left (everything, without rounds), from the front
    REPDL_LAUNCH(sum1d_walk_kernel, dim3((unsigned)rows), dim3(64), 0, s, in, c, T1, TG, T2, T3, ctl, factor, out, vec, 0);
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
    // no workspace given: take it from the scratch cache for the duration of the call
    const size_t bytes = repdl_hip_sum1d_workspace_bytes(n);
    void *ws = nullptr;
    hipError_t e = repdl_ws_acquire(&ws, bytes, repdl_stream(stream));
    if (e != hipSuccess)
        return (int)e;
    const int rc = repdl_hip_sum1d_ws(in, out, n, average, ws, bytes, stream);
    e = repdl_ws_release(ws, repdl_stream(stream));
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

