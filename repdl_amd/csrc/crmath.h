// crmath.h -- correctly rounded binary32 div / sqrt and glibc-compatible
// binary32 exp / log, written with nothing but IEEE binary64 +, -, *, fma,
// conversions and integer operations.  No reciprocal, square-root, exponential
// or logarithm instruction (v_rcp_*, v_rsq_*, v_sqrt_*, v_exp_*, v_log_*) and no
// '/' operator is used, so the same source gives the same bits when compiled for
// the GPU (hipcc) and for a CPU (gcc, for exhaustive checking against libm).
// Must be compiled with floating-point contraction off: every fused operation
// is an explicit crm_fma.
//
//   crm_div(a, b)  = RN32(a / b)                    -- RepDL repdl/ops.py:98-103
//   crm_sqrt(x)    = RN32(RN64(sqrt(x))) = IEEE sqrt -- RepDL repdl/ops.py:122-123
//   crm_exp(x)     = RN32(exp64(x)),  exp64 = glibc's binary64 exp
//   crm_log(x)     = RN32(log64(x)),  log64 = glibc's binary64 log
//                                       -- RepDL backend/cpu/math.cpp:14-17, 32-35
#pragma once

#include <stdint.h>

#include "crmath_tables.h"

#if defined(__HIP_DEVICE_COMPILE__) || defined(__HIPCC__)
#define CRM_FN __device__ __forceinline__
#define CRM_DEVICE 1
#else
#include <math.h>
#include <string.h>
#define CRM_FN static inline
#define CRM_DEVICE 0
#endif

// ---- bit casts and the three primitives that differ between the builds -----
#if CRM_DEVICE
CRM_FN uint64_t crm_d2u(double d) { return (uint64_t)__double_as_longlong(d); }
CRM_FN double crm_u2d(uint64_t u) { return __longlong_as_double((long long)u); }
CRM_FN uint32_t crm_f2u(float f) { return __float_as_uint(f); }
CRM_FN float crm_u2f(uint32_t u) { return __uint_as_float(u); }
CRM_FN double crm_fma(double a, double b, double c) { return __fma_rn(a, b, c); }
CRM_FN float crm_d2f(double d) { return __double2float_rn(d); }
#else
CRM_FN uint64_t crm_d2u(double d) { uint64_t u; memcpy(&u, &d, 8); return u; }
CRM_FN double crm_u2d(uint64_t u) { double d; memcpy(&d, &u, 8); return d; }
CRM_FN uint32_t crm_f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
CRM_FN float crm_u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
CRM_FN double crm_fma(double a, double b, double c) { return fma(a, b, c); }
CRM_FN float crm_d2f(double d) { return (float)d; }
#endif

#define CRM_QNAN_POS 0x7FC00000u
#define CRM_QNAN_NEG 0xFFC00000u

// Given a positive approximation q of a positive real t with |q - t| < ulp(q)
// and the sign of the exact residual (t - q scaled by a positive factor),
// return t rounded to odd in binary64: exact if the residual is zero, else the
// neighbour of t whose last mantissa bit is 1.  Rounding that value to 24 (or
// fewer) bits gives the correctly rounded result (53 >= 24 + 2).
CRM_FN double crm_round_to_odd(double q, double residual)
{
    const uint64_t ur = crm_d2u(residual);
    const uint32_t rhi = (uint32_t)(ur >> 32);
    // the residual is an exact binary64 value that is never subnormal here, so it
    // is non-zero iff its exponent field is; its sign bit says q lies above t
    const uint64_t inexact = (rhi & 0x7FF00000u) != 0u;
    const uint64_t above_t = (uint64_t)(rhi >> 31) & inexact;
    // t in (q, q+ulp): q|1;  t in (q-ulp, q): (q-1)|1;  t == q: q
    return crm_u2d((crm_d2u(q) - above_t) | inexact);
}

// 1 / b for finite positive binary64 b in [2^-149, 2^128), relative error
// below 2^-26: integer seed (error < 12.5 %), then two cubically convergent
// steps y <- y + y*(e + e*e), e = 1 - b*y.
CRM_FN double crm_recip_approx(double b)
{
    double y = crm_u2d(0x7FDE6238502484BAULL - crm_d2u(b));
    double e = crm_fma(-b, y, 1.0);
    y = crm_fma(y, crm_fma(e, e, e), y);
    e = crm_fma(-b, y, 1.0);
    y = crm_fma(y, crm_fma(e, e, e), y);
    e = crm_fma(-b, y, 1.0);
    y = crm_fma(y, crm_fma(e, e, e), y);
    return y;
}

// |a| / |b| for finite non-zero a, b given the approximate reciprocal y of |b|,
// rounded to binary32 (sign not applied).
CRM_FN float crm_div_core(double da, double db, double y)
{
    double q = da * y;
    double r = crm_fma(-q, db, da); // exact
    q = crm_fma(r, y, q);           // within 0.75 ulp of da/db
    r = crm_fma(-q, db, da);        // exact; its sign tells on which side q lies
    return crm_d2f(crm_round_to_odd(q, r));
}

CRM_FN float crm_div_special(uint32_t ua, uint32_t ub, float generic)
{
    const uint32_t aa = ua & 0x7FFFFFFFu, ab = ub & 0x7FFFFFFFu;
    const uint32_t sign = (ua ^ ub) & 0x80000000u;
    uint32_t res = crm_f2u(generic) | sign;
    if (aa == 0u || ab == 0x7F800000u)
        res = sign; // 0 / y, x / inf
    if (ab == 0u || aa == 0x7F800000u)
        res = sign | 0x7F800000u; // x / 0, inf / y
    if ((aa == 0u && ab == 0u) || (aa == 0x7F800000u && ab == 0x7F800000u))
        res = CRM_QNAN_NEG; // invalid: the x86 default NaN
    if (ab > 0x7F800000u)
        res = ub | 0x00400000u; // NaN divisor, quieted
    if (aa > 0x7F800000u)
        res = ua | 0x00400000u; // a NaN dividend wins
    return crm_u2f(res);
}

CRM_FN float crm_div(float a, float b)
{
    const uint32_t ua = crm_f2u(a), ub = crm_f2u(b);
    // |a|, |b| as doubles (exact, subnormals included).  Zero, infinity and NaN
    // run through the arithmetic harmlessly (nothing traps, nothing is indexed
    // by the values) and are overridden afterwards.
    const double da = (double)crm_u2f(ua & 0x7FFFFFFFu);
    const double db = (double)crm_u2f(ub & 0x7FFFFFFFu);
    const float g = crm_div_core(da, db, crm_recip_approx(db));
    return crm_div_special(ua, ub, g);
}

// Division of many dividends by one divisor: the reciprocal is computed once.
typedef struct
{
    const float *invc;
    const double *logc_hi;
    const float *logc_lo;
} crm_log_tables;

// the same tables with invc and logc_lo widened to binary64 (exact), for kernels that fill their
// own copy once per workgroup
typedef struct
{
    const double *invc;
    const double *logc_hi;
    const double *logc_lo;
} crm_log_tables_wide;

typedef struct
{
    double db, y;
    uint32_t ub;
} crm_divisor;

CRM_FN crm_divisor crm_divisor_make(float b)
{
    crm_divisor d;
    d.ub = crm_f2u(b);
    d.db = (double)crm_u2f(d.ub & 0x7FFFFFFFu);
    d.y = crm_recip_approx(d.db);
    return d;
}

CRM_FN float crm_div_by(float a, crm_divisor d)
{
    const uint32_t ua = crm_f2u(a);
    double da = (double)crm_u2f(ua & 0x7FFFFFFFu);
    return crm_div_special(ua, d.ub, crm_div_core(da, d.db, d.y));
}

// sqrt: reciprocal-square-root seed by integer arithmetic on the high word
// (error < 3.5 %), three Newton steps y <- y + y*(1/2 - (x/2)*y*y), then s = x*y
// with one residual correction: s is within 1 ulp64 of sqrt(x).  That is enough
// for a correctly rounded binary32 result: sqrt(x) of a 24-bit x is either
// exactly a 24-bit number (then s, within 1 ulp64 of a binary64 value, rounds to
// it) or farther than 2^-50.5 relative (2.8 ulp64) from every binary32 value and
// midpoint, so s lies on the same side of every rounding boundary.
CRM_FN float crm_sqrt(float x)
{
    const uint32_t ux = crm_f2u(x);
    const double dx = (double)x; // exact; subnormals become normal
    const double hx = 0.5 * dx;
    const uint32_t hi = (uint32_t)(crm_d2u(dx) >> 32);
    double y = crm_u2d((uint64_t)(0x5FE6EB50u - (hi >> 1)) << 32);
    double e = crm_fma(-hx, y * y, 0.5);
    y = crm_fma(y, e, y);
    e = crm_fma(-hx, y * y, 0.5);
    y = crm_fma(y, e, y);
    e = crm_fma(-hx, y * y, 0.5);
    y = crm_fma(y, e, y);
    double s = dx * y;
    const double r = crm_fma(-s, s, dx);
    s = crm_fma(r, 0.5 * y, s);
    const uint32_t gen = crm_f2u(crm_d2f(s));
    // +-0, +inf, negatives, -inf and NaNs ((ux - 1) wraps 0 to the top); written as
    // selects, not branches, so that consecutive elements interleave
    const uint32_t ax = ux & 0x7FFFFFFFu;
    uint32_t sp = CRM_QNAN_POS;                          // negative, -inf (PyTorch CPU convention)
    sp = (ax == 0u || ux == 0x7F800000u) ? ux : sp;      // +-0, +inf
    sp = (ax > 0x7F800000u) ? (ux | 0x00400000u) : sp;   // NaN: sign and payload kept, quieted
    return crm_u2f((ux - 1u >= 0x7F7FFFFFu) ? sp : gen);
}

// ---- exp --------------------------------------------------------------------
// The published algorithm of glibc's binary64 exp (sysdeps/ieee754/dbl-64/e_exp.c,
// N = 128, degree-5 polynomial) in its FMA-contracted form, restricted to the
// binary32 argument range; then one rounding to binary32.
//   k = round(x * N/ln2),  r = x - k*ln2/N,  exp(x) = 2^(k/N) * exp(r)
//   exp(r) ~ 1 + tail + r + r^2 (C2 + r C3) + r^4 (C4 + r C5)
// tab: the 256-word table of crmath_tables.h (CRM_EXP_TAB_INIT).
#define CRM_EXP_INVLN2N 0x1.71547652b82fep+7
#define CRM_EXP_NEGLN2HIN (-0x1.62e42fefa0000p-8)
#define CRM_EXP_NEGLN2LON (-0x1.cf79abc9e3b3ap-47)
#define CRM_EXP_SHIFT 0x1.8p52
#define CRM_EXP_C2 0x1.ffffffffffdbdp-2
#define CRM_EXP_C3 0x1.555555555543cp-3
#define CRM_EXP_C4 0x1.55555cf172b91p-5
#define CRM_EXP_C5 0x1.1111167a4d017p-7

CRM_FN double crm_exp64_core(double x, const uint64_t *tab)
{
    double kd = crm_fma(CRM_EXP_INVLN2N, x, CRM_EXP_SHIFT);
    const uint64_t ki = crm_d2u(kd);
    kd -= CRM_EXP_SHIFT;
    double r = crm_fma(kd, CRM_EXP_NEGLN2HIN, x);
    r = crm_fma(kd, CRM_EXP_NEGLN2LON, r);
    const uint32_t idx = 2u * ((uint32_t)ki & 127u);
    const uint64_t top = ki << (52 - CRM_EXP_TABLE_BITS);
    const double tail = crm_u2d(tab[idx]);
    const uint64_t sbits = tab[idx + 1] + top;
    const double r2 = r * r;
    double tmp = crm_fma(r2, crm_fma(r, CRM_EXP_C3, CRM_EXP_C2), tail + r);
    tmp = crm_fma(r2 * r2, crm_fma(r, CRM_EXP_C5, CRM_EXP_C4), tmp);
    const double scale = crm_u2d(sbits);
    return crm_fma(scale, tmp, scale);
}

CRM_FN float crm_exp(float x, const uint64_t *tab)
{
    const uint32_t ux = crm_f2u(x);
    const uint32_t ax = ux & 0x7FFFFFFFu;
    // |x| > 104 (also inf, NaN): the binary32 result is 0 or +inf whatever the
    // binary64 value is (exp(-104) < 2^-150, exp(89) > 2^128).  Such arguments
    // still run through the core harmlessly: the table index is masked.
    const uint32_t gen = crm_f2u(crm_d2f(crm_exp64_core((double)x, tab)));
    uint32_t sp = (ux >> 31) ? 0u : 0x7F800000u;
    sp = (ax > 0x7F800000u) ? (ux | 0x00400000u) : sp; // NaN + 1.0: sign and payload kept, quieted
    return crm_u2f((ax > 0x42D00000u) ? sp : gen);
}

// ---- log --------------------------------------------------------------------
// x = 2^k z, z in [0.6875, 1.375); r = z*invc - 1 (exact for 24-bit z);
// log(x) = k ln2 + logc + log1p(r), summed as an exact head
// w = k*LN2_HI + logc_hi, a compensated hi + lo, and a degree-9 polynomial.
// Tables (crmath_tables.h): invc[128] binary32, logc_hi[128] binary64, logc_lo[128] binary32.
// (index, exponent and reduced argument of x; the table entry is fetched by the caller)
CRM_FN double crm_log64_reduce(double x, uint32_t *idx, int32_t *kexp)
{
    const uint64_t ix = crm_d2u(x);
    // only the high word takes part in the reduction (the offset has a zero low word)
    const uint32_t hi = (uint32_t)(ix >> 32);
    const uint32_t tmp = hi - 0x3FE60000u;
    *idx = (tmp >> 13) & 127u;
    *kexp = (int32_t)tmp >> 20;
    const uint32_t zhi = hi - (tmp & 0xFFF00000u);
    return crm_u2d(((uint64_t)zhi << 32) | (ix & 0xFFFFFFFFu));
}

CRM_FN double crm_log64_eval(double z, int32_t k, double invc, double logc_hi, double logc_lo)
{
    const double kd = (double)k;
    const double r = crm_fma(z, invc, -1.0);
    const double w = crm_fma(kd, CRM_LN2_HI, logc_hi); // exact
    const double hi_sum = w + r;
    double lo = (w - hi_sum) + r;
    lo += crm_fma(kd, CRM_LN2_LO, logc_lo);
    const double r2 = r * r;
    double p = crm_fma(r, 0x1.c71c71c71c71cp-4, -0.125); // r^9/9 - r^8/8
    p = crm_fma(r, p, 0x1.2492492492492p-3);
    p = crm_fma(r, p, -0x1.5555555555555p-3);
    p = crm_fma(r, p, 0.2);
    p = crm_fma(r, p, -0.25);
    p = crm_fma(r, p, 0x1.5555555555555p-2);
    p = crm_fma(r, p, -0.5);
    return hi_sum + crm_fma(r2, p, lo);
}

CRM_FN double crm_log64_core(double x, crm_log_tables tab)
{
    uint32_t i;
    int32_t k;
    const double z = crm_log64_reduce(x, &i, &k);
    return crm_log64_eval(z, k, (double)tab.invc[i], tab.logc_hi[i], (double)tab.logc_lo[i]);
}

// the same with the two binary32 tables widened beforehand (two conversions less per element)
CRM_FN double crm_log64_core_wide(double x, crm_log_tables_wide tab)
{
    uint32_t i;
    int32_t k;
    const double z = crm_log64_reduce(x, &i, &k);
    return crm_log64_eval(z, k, tab.invc[i], tab.logc_hi[i], tab.logc_lo[i]);
}

// the special inputs of log in three selects: x + x is +inf for +inf and, for a NaN, the same
// NaN quieted (sign and payload kept); a NaN compares false both times
CRM_FN float crm_log_finish(float x, double core)
{
    const uint32_t ux = crm_f2u(x);
    const uint32_t gen = crm_f2u(crm_d2f(core));
    uint32_t sp = crm_f2u(x + x);
    sp = (x < 0.0f) ? CRM_QNAN_NEG : sp;  // log(negative), log(-inf): (x-x)/(x-x) on x86
    sp = (x == 0.0f) ? 0xFF800000u : sp;  // log(+-0) = -inf
    return crm_u2f((ux - 1u >= 0x7F7FFFFFu) ? sp : gen);
}

CRM_FN float crm_log(float x, crm_log_tables tab)
{
    // zeros, negatives, infinities and NaNs run through the core harmlessly (the
    // table index is masked) and are overridden
    return crm_log_finish(x, crm_log64_core((double)x, tab));
}

CRM_FN float crm_log_wide(float x, crm_log_tables_wide tab)
{
    return crm_log_finish(x, crm_log64_core_wide((double)x, tab));
}
