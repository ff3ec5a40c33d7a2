/*
 * sanitize_crmath.c -- the CPU build of the device math (repdl_amd/csrc/crmath.h through
 * tests/crmath_check.c) under AddressSanitizer and UndefinedBehaviorSanitizer: strided sweeps of
 * exp, log, sqrt and the two divisions over the whole range of bit patterns (table indices, shifts
 * and integer conversions at every exponent), compared with the host's libm on the way.  Test tool
 * only (built and run by tests/test_sanitizers.py); prints "ok" when nothing differed.
 */
#include <stdio.h>

#include "crmath_check.c"

int main(void)
{
    uint32_t bad[8];
    const uint32_t stride = 65521; /* a prime: every exponent, varied significands */
    const uint64_t count = 0x100000000ull / stride;
    uint64_t n = 0;
    n += crmc_sweep_exp(0, count, stride, bad, 8);
    n += crmc_sweep_log(0, count, stride, bad, 8);
    n += crmc_sweep_sqrt(0, count, stride, bad, 8);
    n += crmc_sweep_div_by(0x41200000u /* 10.0f */, 0, count, stride, bad, 8);
    n += crmc_sweep_div_random(1, 200000, 0, bad, 8);
    n += crmc_sweep_div_random(2, 200000, 1, bad, 8);
    if (n != 0)
    {
        printf("%llu mismatches, first 0x%08x\n", (unsigned long long)n, bad[0]);
        return 1;
    }
    puts("ok");
    return 0;
}
