/*
 * crmath_check.c -- CPU build of the device math (repdl_amd/csrc/crmath.h) plus
 * sweep drivers that compare it, bit for bit, with the host's libm / IEEE
 * hardware over ranges of binary32 bit patterns.  Test tool only.
 *
 * Build: gcc -O2 -fopenmp -ffp-contract=off -mfma -shared -fPIC (see
 * tests/crmath_host.py).  -mfma only makes fma() a single instruction; the
 * value is the same single-rounding result either way.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#include "../repdl_amd/csrc/crmath.h"

static const uint64_t EXP_TAB[256] = CRM_EXP_TAB_INIT;
static const float LOG_INVC[128] = CRM_LOG_INVC_INIT;
static const double LOG_HI[128] = CRM_LOG_HI_INIT;
static const float LOG_LO[128] = CRM_LOG_LO_INIT;
static const crm_log_tables LOG_TAB = {LOG_INVC, LOG_HI, LOG_LO};

#define API __attribute__((visibility("default")))

static inline uint32_t fbits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float ffrom(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* ---- host references (what the reference's CPU path computes) ---- */
static inline uint32_t ref_exp(uint32_t u) { return fbits((float)exp((double)ffrom(u))); }
static inline uint32_t ref_log(uint32_t u) { return fbits((float)log((double)ffrom(u))); }
static inline uint32_t ref_sqrt(uint32_t u)
{
    if ((u & 0x7fffffffu) > 0x7f800000u)
        return u | 0x00400000u;
    if ((u >> 31) && (u & 0x7fffffffu))
        return 0x7fc00000u; /* PyTorch CPU: positive quiet NaN */
    return fbits((float)sqrt((double)ffrom(u)));
}
static inline uint32_t ref_div(uint32_t ua, uint32_t ub)
{
    if ((ua & 0x7fffffffu) > 0x7f800000u)
        return ua | 0x00400000u;
    if ((ub & 0x7fffffffu) > 0x7f800000u)
        return ub | 0x00400000u;
    volatile float a = ffrom(ua), b = ffrom(ub);
    volatile float q = a / b;
    if (q != q)
        return 0xffc00000u;
    return fbits(q);
}

/* single-value entry points (for directed tests from Python) */
API uint32_t crmc_exp(uint32_t u) { return fbits(crm_exp(ffrom(u), EXP_TAB)); }
API uint32_t crmc_log(uint32_t u) { return fbits(crm_log(ffrom(u), LOG_TAB)); }
API uint32_t crmc_sqrt(uint32_t u) { return fbits(crm_sqrt(ffrom(u))); }
API uint32_t crmc_div(uint32_t a, uint32_t b) { return fbits(crm_div(ffrom(a), ffrom(b))); }
API uint32_t crmc_ref_exp(uint32_t u) { return ref_exp(u); }
API uint32_t crmc_ref_log(uint32_t u) { return ref_log(u); }
API uint32_t crmc_ref_sqrt(uint32_t u) { return ref_sqrt(u); }
API uint32_t crmc_ref_div(uint32_t a, uint32_t b) { return ref_div(a, b); }

#define RECORD(pat)                               \
    do                                            \
    {                                             \
        _Pragma("omp critical")                   \
        {                                         \
            if (nbad < (uint64_t)maxbad)          \
                bad[nbad] = (pat);                \
            nbad++;                               \
        }                                         \
    } while (0)

/* Sweep bit patterns start, start+stride, ... (count of them); returns the number
 * of mismatches and stores the first maxbad offending patterns. */
#define UNARY_SWEEP(name, mine, ref)                                                              \
    API uint64_t name(uint32_t start, uint64_t count, uint32_t stride, uint32_t *bad, int maxbad) \
    {                                                                                             \
        uint64_t nbad = 0;                                                                        \
        _Pragma("omp parallel for schedule(static)") for (int64_t i = 0; i < (int64_t)count; i++) \
        {                                                                                         \
            uint32_t u = start + (uint32_t)((uint64_t)i * stride);                                \
            if (mine != ref)                                                                      \
                RECORD(u);                                                                        \
        }                                                                                         \
        return nbad;                                                                              \
    }

UNARY_SWEEP(crmc_sweep_exp, fbits(crm_exp(ffrom(u), EXP_TAB)), ref_exp(u))
UNARY_SWEEP(crmc_sweep_log, fbits(crm_log(ffrom(u), LOG_TAB)), ref_log(u))
UNARY_SWEEP(crmc_sweep_sqrt, fbits(crm_sqrt(ffrom(u))), ref_sqrt(u))

/* all dividends (strided) over one divisor, both through crm_div and through the
 * hoisted-reciprocal form used for scalar divisors */
API uint64_t crmc_sweep_div_by(uint32_t ub, uint32_t start, uint64_t count, uint32_t stride,
                               uint32_t *bad, int maxbad)
{
    uint64_t nbad = 0;
    const crm_divisor d = crm_divisor_make(ffrom(ub));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)count; i++)
    {
        uint32_t ua = start + (uint32_t)((uint64_t)i * stride);
        uint32_t want = ref_div(ua, ub);
        if (fbits(crm_div(ffrom(ua), ffrom(ub))) != want || fbits(crm_div_by(ffrom(ua), d)) != want)
            RECORD(ua);
    }
    return nbad;
}

static inline uint64_t splitmix(uint64_t *s)
{
    uint64_t z = (*s += 0x9E3779B97F4A7C15ULL);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

/* random pairs; mode 0: both operands uniform over all bit patterns; mode 1:
 * exponents close together (quotients near 1, many near-tie cases); mode 2:
 * quotient in the subnormal range. bad receives (a,b) pairs. */
API uint64_t crmc_sweep_div_random(uint64_t seed, uint64_t count, int mode, uint32_t *bad, int maxbad)
{
    uint64_t nbad = 0;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)count; i++)
    {
        uint64_t s = seed + 0x632BE59BD9B4E019ULL * (uint64_t)i;
        uint64_t z = splitmix(&s);
        uint32_t ua = (uint32_t)z, ub = (uint32_t)(z >> 32);
        if (mode == 1)
            ub = (ub & 0x807FFFFFu) | (ua & 0x7F800000u);
        else if (mode == 2)
        {
            ua = (ua & 0x807FFFFFu) | ((1u + (uint32_t)(splitmix(&s) % 40u)) << 23);
            ub = (ub & 0x807FFFFFu) | ((127u + (uint32_t)(splitmix(&s) % 60u)) << 23);
        }
        if (fbits(crm_div(ffrom(ua), ffrom(ub))) != ref_div(ua, ub))
        {
#pragma omp critical
            {
                if (nbad < (uint64_t)maxbad)
                {
                    bad[2 * nbad] = ua;
                    bad[2 * nbad + 1] = ub;
                }
                nbad++;
            }
        }
    }
    return nbad;
}
