/*
 * Sanitizer run of the CPU checker: drives every function of tab_oracle.c on small seeded inputs with exactly sized
 * heap buffers (AddressSanitizer: any read or write past an operand aborts; UndefinedBehaviorSanitizer: shifts,
 * signed overflow, misaligned access), over the edge shapes the parity tests use: C not a multiple of 64 or 32, one
 * channel, padding wider than the kernel, strides that leave a remainder, 1x1 and even kernels, one output element.
 * TEST INFRASTRUCTURE ONLY (built by `make -C oracle sanitize`, run by tests/test_oracle_sanitize.py).  It checks
 * memory safety and the shape of the results, not values: those are pinned by the other oracle tests.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

int oracle_out_extent(int in, int pad, int k, int stride);
void oracle_quantize_ternary(const float *x, const float *ths, int N, int H, int W, int C, int64_t *q);
void oracle_quantize_binary(const float *x, const float *ths, int N, int H, int W, int C, int64_t *q);
void oracle_quantize_drf(const float *x, const float *ths, int N, int H, int W, int C, int64_t *q);
void oracle_quantize_rtn(const float *x, const float *ths, int N, int H, int W, int C, int64_t *q);
void oracle_btn_weight(const int64_t *qx_ternary, int N, long words_per_item, int32_t *btn);
int oracle_conv2d(const float *x, const int64_t *qw, const float *ths, const int32_t *btn, int type, int p1, int p2, int s1,
                  int s2, int N, int H, int W, int C, int KN, int KH, int KW, float *y);

static uint64_t state = 88172645463325252ull;
static float next_float(void)
{
    state ^= state << 13; state ^= state >> 7; state ^= state << 17;
    return (float)((double)(state >> 11) / 9007199254740992.0 * 4.0 - 2.0);
}

static int words(int type, int C, int weight)
{
    if (type == 5) return (C + 31) / 32;
    const int pc = (C + 63) / 64;
    const int two = type == 4 || (weight ? (type == 0 || type == 2) : type < 2);
    return pc * (two ? 2 : 1);
}

static int run_case(int type, int N, int H, int W, int C, int KN, int KH, int KW, int p1, int p2, int s1, int s2)
{
    const int OH = oracle_out_extent(H, p1, KH, s1), OW = oracle_out_extent(W, p2, KW, s2);
    const size_t nx = (size_t)N * H * W * C, nw = (size_t)KN * KH * KW * C;
    float *x = malloc(sizeof(float) * nx), *w = malloc(sizeof(float) * nw);
    float *xt = malloc(sizeof(float) * N), *wt = malloc(sizeof(float) * KN);
    int64_t *qw = malloc(sizeof(int64_t) * (size_t)KN * KH * KW * words(type, C, 1));
    int32_t *btn = malloc(sizeof(int32_t) * KN);
    if (!x || !w || !xt || !wt || !qw || !btn) return 1;
    for (size_t i = 0; i < nx; i++) x[i] = next_float();
    for (size_t i = 0; i < nw; i++) w[i] = next_float();
    x[0] = NAN; x[nx - 1] = INFINITY; w[0] = -0.0f;   /* the special values go through every compare */
    for (int i = 0; i < N; i++) xt[i] = 0.5f;
    for (int i = 0; i < KN; i++) { wt[i] = 0.4f; btn[i] = 0; }
    switch (type) {
    case 0: case 2:
        oracle_quantize_ternary(w, wt, KN, KH, KW, C, qw);
        oracle_btn_weight(qw, KN, (long)KH * KW * ((C + 63) / 64), btn);
        break;
    case 1: case 3: oracle_quantize_binary(w, wt, KN, KH, KW, C, qw); break;
    case 4: oracle_quantize_drf(w, wt, KN, KH, KW, C, qw); break;
    default: oracle_quantize_rtn(w, wt, KN, KH, KW, C, qw); break;
    }
    int rc = 0;
    if (OH >= 1 && OW >= 1) {
        float *y = malloc(sizeof(float) * (size_t)N * OH * OW * KN);
        if (!y) return 1;
        rc = oracle_conv2d(x, qw, xt, btn, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW, y);
        const int bound = KH * KW * C * (type == 4 ? 9 : 1);
        for (size_t i = 0; rc == 0 && i < (size_t)N * OH * OW * KN; i++)
            if (!(fabsf(y[i]) <= (float)bound) || y[i] != truncf(y[i])) rc = 2;  /* integers within the length of K */
        free(y);
    }
    free(x); free(w); free(xt); free(wt); free(qw); free(btn);
    if (rc) fprintf(stderr, "case type %d N%d %dx%dx%d->%d k%dx%d p%d%d s%d%d: rc %d\n", type, N, H, W, C, KN, KH, KW, p1, p2, s1, s2, rc);
    return rc;
}

int main(void)
{
    static const int cases[][11] = {
        /* N, H, W, C, KN, KH, KW, p1, p2, s1, s2 */
        {1, 8, 8, 64, 5, 3, 3, 1, 1, 1, 1},   {2, 9, 6, 70, 5, 3, 3, 1, 0, 1, 2},   {2, 7, 7, 64, 8, 3, 3, 1, 1, 2, 2},
        {1, 6, 5, 200, 7, 2, 3, 2, 1, 1, 1},  {3, 5, 5, 33, 4, 1, 1, 1, 0, 2, 1},   {1, 3, 3, 64, 1, 3, 3, 0, 0, 1, 1},
        {1, 9, 9, 1, 3, 3, 3, 1, 1, 1, 1},    {2, 5, 5, 64, 8, 3, 3, 3, 3, 1, 1},   {2, 13, 13, 128, 8, 3, 3, 1, 1, 4, 4},
        {3, 1, 17, 96, 12, 1, 3, 0, 1, 1, 1}, {2, 4, 4, 1030, 6, 2, 2, 1, 1, 1, 1}, {4, 2, 2, 31, 5, 2, 2, 0, 0, 1, 1},
    };
    int failed = 0, n = 0;
    for (int type = 0; type < 6; type++)
        for (size_t c = 0; c < sizeof(cases) / sizeof(cases[0]); c++, n++) {
            const int *k = cases[c];
            failed += run_case(type, k[0], k[1], k[2], k[3], k[4], k[5], k[6], k[7], k[8], k[9], k[10]) != 0;
        }
    printf("sanitize_check: %d cases, %d failed\n", n, failed);
    return failed != 0;
}
