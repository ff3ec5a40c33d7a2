/*
 * sanitize_oracle.c -- the CPU checker (oracle/repdl_oracle.c) under AddressSanitizer and
 * UndefinedBehaviorSanitizer: every operator on small ragged shapes with strides, paddings beyond
 * the kernel's reach, groups, empty extents and special values, from heap buffers of exactly the
 * operands' sizes, so that an index that strays by one element is reported.  Test tool only
 * (built and run by tests/test_sanitizers.py); prints "ok" when nothing was reported.
 */
#include <stdio.h>

#include "../oracle/repdl_oracle.c"

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static float rnd(void)
{
    rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
    uint32_t r = (uint32_t)(rng_state >> 33);
    switch (r & 63)
    {
    case 0:
        return 0.0f;
    case 1:
        return -0.0f;
    case 2:
        return INFINITY;
    case 3:
        return 1e-42f;
    default:
        return ((int32_t)(r >> 6) % 20001 - 10000) * 1e-3f;
    }
}
static float *buf(int64_t n)
{
    float *p = (float *)malloc((size_t)(n > 0 ? n : 0) * sizeof(float) + (n > 0 ? 0 : 1));
    for (int64_t i = 0; i < n; i++)
        p[i] = rnd();
    return p;
}

static void conv_case(int64_t N, int64_t IC, int64_t H, int64_t W, int64_t OC, int64_t KH, int64_t KW, int64_t sH,
                      int64_t sW, int64_t pH, int64_t pW, int64_t g)
{
    int64_t OH = (H + 2 * pH - KH) / sH + 1, OW = (W + 2 * pW - KW) / sW + 1;
    float *x = buf(N * IC * H * W), *w = buf(OC * (IC / g) * KH * KW), *y = buf(N * OC * OH * OW);
    repdl_oracle_conv2d(x, w, y, N, IC, H, W, OC, KH, KW, sH, sW, pH, pW, g);
    if (g == 1)
    {
        float *gi = buf(N * IC * H * W), *gk = buf(OC * IC * KH * KW);
        repdl_oracle_conv2d_grad_input(y, w, gi, N, OC, OH, OW, IC, KH, KW, H, W, sH, sW, pH, pW);
        repdl_oracle_conv2d_grad_kernel(y, x, gk, N, IC, H, W, OC, OH, OW, KH, KW, sH, sW, pH, pW);
        free(gi);
        free(gk);
    }
    free(x);
    free(w);
    free(y);
}

int main(void)
{
    /* mm: every layout, ragged against the blocking (8 x 512 panels), K = 0 */
    static const int64_t mm[][3] = {{1, 1, 1}, {7, 513, 9}, {9, 5, 0}, {17, 1030, 33}, {8, 512, 64}, {3, 2, 1000}};
    for (size_t c = 0; c < sizeof(mm) / sizeof(mm[0]); c++)
        for (int tA = 0; tA < 2; tA++)
            for (int tB = 0; tB < 2; tB++)
            {
                int64_t M = mm[c][0], N = mm[c][1], K = mm[c][2];
                float *a = buf(M * K), *b = buf(K * N), *o = buf(M * N);
                repdl_oracle_mm(a, b, o, M, N, K, tA, tB);
                free(a);
                free(b);
                free(o);
            }
    conv_case(2, 3, 7, 5, 4, 3, 3, 1, 1, 1, 1, 1);
    conv_case(1, 4, 9, 9, 6, 1, 1, 1, 1, 2, 2, 2);  /* padding beyond the kernel's reach, groups */
    conv_case(2, 2, 10, 11, 3, 3, 2, 2, 3, 0, 1, 1); /* strides that leave rows and columns over */
    conv_case(1, 1, 5, 6, 1, 5, 6, 1, 1, 0, 0, 1);   /* one output */
    conv_case(3, 6, 8, 8, 9, 2, 2, 3, 3, 0, 0, 3);   /* stride wider than the kernel */
    conv_case(1, 2, 4, 4, 2, 3, 3, 4, 4, 3, 3, 1);   /* padding as wide as the kernel */
    /* sums: ragged, empty, one element */
    static const int64_t sm[][2] = {{1, 1}, {5, 7}, {0, 4}, {4, 0}, {33, 129}};
    for (size_t c = 0; c < sizeof(sm) / sizeof(sm[0]); c++)
        for (int avg = 0; avg < 2; avg++)
        {
            int64_t M = sm[c][0], N = sm[c][1];
            float *x = buf(M * N), *o0 = buf(N), *o1 = buf(M);
            (void)repdl_oracle_sum1d(x, M * N, avg);
            repdl_oracle_sum2d_dim0(x, o0, M, N, avg);
            repdl_oracle_sum2d_dim1(x, o1, M, N, avg);
            free(x);
            free(o0);
            free(o1);
        }
    {
        float *x = buf(3 * 5 * 2 * 7), *o = buf(5);
        repdl_oracle_sum4d_dim023(x, o, 3, 5, 2, 7, 1);
        free(x);
        free(o);
    }
    /* elementwise, softmax, cross_entropy, the optimizer steps */
    {
        int64_t n = 1001;
        float *a = buf(n), *b = buf(n), *o = buf(n);
        repdl_oracle_exp(a, o, n);
        repdl_oracle_log(a, o, n);
        repdl_oracle_sqrt(a, o, n);
        repdl_oracle_div(a, b, o, n);
        repdl_oracle_div_scalar(a, 10.0f, o, n);
        free(a);
        free(b);
        free(o);
        int64_t M = 13, N = 10;
        float *z = buf(M * N), *s = buf(M * N), *scratch = buf(M);
        int64_t *t = (int64_t *)malloc((size_t)M * sizeof(int64_t));
        for (int64_t i = 0; i < M; i++)
            t[i] = i % N;
        repdl_oracle_softmax(z, s, M, N);
        (void)repdl_oracle_cross_entropy(z, t, M, N, scratch);
        free(z);
        free(s);
        free(scratch);
        free(t);
        float *p = buf(n), *g = buf(n), *m = buf(n), *v = buf(n), *vm = buf(n);
        for (int64_t i = 0; i < n; i++)
            v[i] = fabsf(v[i]), vm[i] = fabsf(vm[i]);
        repdl_oracle_adam_step(p, g, m, v, vm, n, 0.9f, 0.1f, 0.999f, 0.001f, 1e-8f, 0.01f, 0.1f, -0.01f);
        repdl_oracle_adam_step(p, g, m, v, NULL, n, 0.9f, 0.1f, 0.999f, 0.001f, 1e-8f, 0.0f, 0.1f, -0.01f);
        repdl_oracle_sgd_step(p, g, n, 0.01f);
        free(p);
        free(g);
        free(m);
        free(v);
        free(vm);
    }
    puts("ok");
    return 0;
}
