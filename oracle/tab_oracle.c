/*
 * CPU oracle for the TAB quantize + bitwise-convolution path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the HIP path is
 * compared against (tests/, __graft_entry__.smoke(), bench.py's cpu_baseline
 * leg).  Nothing in the product (tab_amd/, include/) links, loads or calls it.
 *
 * It restates, in plain C, the algorithm of ntuliuteam/TAB:
 *   - quantize/bit-pack          TAB_GEMM.cu:163-247 (encodings, bit order),
 *                                TAB_CPU.cpp:56-87,168-185 (ths[n], strict compares)
 *   - btn popcount               TAB_GEMM.cu:150-160
 *   - zero padding of packed words   TAB_GEMM.cuh:73-89, TAB_CPU.cpp:39,155
 *   - im2row, K order (kh,kw,c)  TAB_GEMM.cuh:92-115, TAB_CPU.h:27-63
 *   - the four popcount GEMMs    TAB_CPU.cpp:242-328 (== TAB_GEMM.cu:25-147)
 *   - the two CPU-only GEMMs     TAB_CPU.cpp:332-383 (type 4 DoReFa 2-bit, type 5 RTN)
 *   - the conv pipeline          TAB_GEMM.cu:325-527, TAB_CPU.cpp:507-614
 *
 * Pinning (what checks each function independently of this file's own formulas):
 *   gemm_*        : bit-exact against the reference's own *GEMM_baseline functions
 *                   compiled from /root/reference (oracle/_ref, golden fixtures);
 *   img2row       : against the reference's Parallel_Img2Row_NHWCB_3x3 (same build);
 *   quantize_*    : brute-force closed form per element incl. ties/NaN/inf/-0.0,
 *                   one-hot bit-order test, the demo notebook's stored words
 *                   (binary word == ~ternary nonzero word), and the reference CPU
 *                   ternarizer compiled from /root/reference on single-image inputs;
 *   btn           : equals the number of nonzero ternary weights per filter;
 *   conv2d        : torch.nn.functional.conv2d on the dequantised {-1,0,+1} tensors
 *                   (padding value 0 for ternary, +1 for binary activations);
 *   gemm_drf/rtn  : bit-exact against DRFGEMM_baseline / RTNGEMM_baseline compiled from
 *                   /root/reference (oracle/_ref, golden fixtures), and against integer dot
 *                   products of the decoded values (levels 0..3; ternary fields);
 *   quantize_drf, quantize_rtn : PARITY UNPINNED.  The reference has no quantizer for these
 *                   two types (TAB_Conv names Parallel_Binarize_NCHW and
 *                   Parallel_Ternarize_RTN, TAB_CPU.cpp:522,527, which no file defines); the
 *                   word layouts follow from the GEMMs, the value rules are this build's
 *                   own and are only checked against brute-force closed forms.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define WORD_BITS 64

/*
 * The shared object is built once and may run on a different x86-64 host than the one
 * that compiled it, so the build uses a conservative baseline (-mpopcnt); each GEMM body
 * is compiled again for AVX2 and for AVX-512 VPOPCNTDQ and chosen at run time by
 * __builtin_cpu_supports.  All variants run the same C loop, so results are identical.
 */
#if defined(__x86_64__) && defined(__GNUC__) && !defined(__clang__)
#define HAVE_ISA_VARIANTS 1
#define TARGET_AVX2 __attribute__((target("avx2,popcnt")))
#define TARGET_AVX512 __attribute__((target("avx512f,avx512bw,avx512dq,avx512vl,avx512vpopcntdq,popcnt")))
static int isa_level(void)
{
    static int level = -1;
    if (level < 0) {
        __builtin_cpu_init();
        if (__builtin_cpu_supports("avx512vpopcntdq") && __builtin_cpu_supports("avx512vl") &&
            __builtin_cpu_supports("avx512bw") && __builtin_cpu_supports("avx512dq"))
            level = 2;
        else if (__builtin_cpu_supports("avx2"))
            level = 1;
        else
            level = 0;
    }
    return level;
}
#else
#define HAVE_ISA_VARIANTS 0
#endif
#define ALWAYS_INLINE static inline __attribute__((always_inline))

static inline int packed_channels(int C) { return (C + WORD_BITS - 1) / WORD_BITS; }

int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Output extent along one axis; integer division as in TAB_GEMM.cu:354-357. */
int oracle_out_extent(int in, int pad, int k, int stride)
{
    return (in + 2 * pad - k + 1) / stride;
}

/*
 * Ternarize + pack (TAB_GEMM.cu:163-208).  x is NHWC fp32, qx is
 * [N*H*W][PC][2] int64 with plane 0 = sign marker, plane 1 = nonzero marker.
 * v >  t  -> (0,1)   (+1)
 * v < -t  -> (1,1)   (-1)   (only tested when the first compare fails)
 * else    -> (0,0)
 * Channel c lands in word c/64, bit c%64 (LSB first, TAB_GEMM.cu:252-258).
 * The threshold of image n is ths[n] (TAB_CPU.cpp:67,72).
 */
void oracle_quantize_ternary(const float *x, const float *ths, int N, int H, int W, int C,
                             int64_t *qx)
{
    const int PC = packed_channels(C);
    const long pix_per_img = (long)H * W;
#pragma omp parallel for schedule(static)
    for (long p = 0; p < (long)N * pix_per_img; p++) {
        const float t = ths[p / pix_per_img];
        const float *src = x + p * C;
        uint64_t *dst = (uint64_t *)qx + p * PC * 2;
        for (int w = 0; w < PC; w++) {
            uint64_t sign = 0, nz = 0;
            const int c_hi = (w + 1) * WORD_BITS < C ? (w + 1) * WORD_BITS : C;
            for (int c = w * WORD_BITS; c < c_hi; c++) {
                const uint64_t bit = (uint64_t)1 << (c - w * WORD_BITS);
                const float v = src[c];
                if (v > t) {
                    nz |= bit;
                } else if (v < -t) {
                    sign |= bit;
                    nz |= bit;
                }
            }
            dst[2 * w + 0] = sign;
            dst[2 * w + 1] = nz;
        }
    }
}

/* Binarize + pack (TAB_GEMM.cu:211-247): bit = 1 iff v < t (value -1). */
void oracle_quantize_binary(const float *x, const float *ths, int N, int H, int W, int C,
                            int64_t *qx)
{
    const int PC = packed_channels(C);
    const long pix_per_img = (long)H * W;
#pragma omp parallel for schedule(static)
    for (long p = 0; p < (long)N * pix_per_img; p++) {
        const float t = ths[p / pix_per_img];
        const float *src = x + p * C;
        uint64_t *dst = (uint64_t *)qx + p * PC;
        for (int w = 0; w < PC; w++) {
            uint64_t neg = 0;
            const int c_hi = (w + 1) * WORD_BITS < C ? (w + 1) * WORD_BITS : C;
            for (int c = w * WORD_BITS; c < c_hi; c++)
                if (src[c] < t) neg |= (uint64_t)1 << (c - w * WORD_BITS);
            dst[w] = neg;
        }
    }
}

/*
 * DoReFa 2-bit levels (type 4).  Word layout from DRFGEMM_baseline (TAB_CPU.cpp:345-354):
 * [pixel][PC][2] with plane 0 the weight-2 bit and plane 1 the weight-1 bit of a level 0..3.
 * Value rule (this build's own, the reference defines none): a uniform quantizer with step
 * t = ths[n], level = (v >= 0.5t) + (v >= 1.5t) + (v >= 2.5t), each bound rounded to fp32;
 * NaN gives level 0.
 */
void oracle_quantize_drf(const float *x, const float *ths, int N, int H, int W, int C,
                         int64_t *qx)
{
    const int PC = packed_channels(C);
    const long pix_per_img = (long)H * W;
#pragma omp parallel for schedule(static)
    for (long p = 0; p < (long)N * pix_per_img; p++) {
        const float t = ths[p / pix_per_img];
        const float b1 = 0.5f * t, b2 = 1.5f * t, b3 = 2.5f * t;
        const float *src = x + p * C;
        uint64_t *dst = (uint64_t *)qx + p * PC * 2;
        for (int w = 0; w < PC; w++) {
            uint64_t hi = 0, lo = 0;
            const int c_hi = (w + 1) * WORD_BITS < C ? (w + 1) * WORD_BITS : C;
            for (int c = w * WORD_BITS; c < c_hi; c++) {
                const float v = src[c];
                const int level = (v >= b1) + (v >= b2) + (v >= b3);
                hi |= (uint64_t)(level >> 1) << (c - w * WORD_BITS);
                lo |= (uint64_t)(level & 1) << (c - w * WORD_BITS);
            }
            dst[2 * w + 0] = hi;
            dst[2 * w + 1] = lo;
        }
    }
}

/*
 * RTN ternary fields (type 5).  Word layout from RTNGEMM_baseline (TAB_CPU.cpp:364-379, mask
 * 0x5555...) and TAB_CPU.cpp:520-521 (32 channels per word): channel c sits in word c/32 as a
 * 2-bit field, bit 2*(c%32) = nonzero marker, bit 2*(c%32)+1 = sign marker.  Value rule: the
 * ternarizer's (v > t -> +1, else v < -t -> -1, TAB_GEMM.cu:184-192), this build's choice.
 */
void oracle_quantize_rtn(const float *x, const float *ths, int N, int H, int W, int C,
                         int64_t *qx)
{
    const int PC = (C + 31) / 32;
    const long pix_per_img = (long)H * W;
#pragma omp parallel for schedule(static)
    for (long p = 0; p < (long)N * pix_per_img; p++) {
        const float t = ths[p / pix_per_img];
        const float *src = x + p * C;
        uint64_t *dst = (uint64_t *)qx + p * PC;
        for (int w = 0; w < PC; w++) {
            uint64_t word = 0;
            const int c_hi = (w + 1) * 32 < C ? (w + 1) * 32 : C;
            for (int c = w * 32; c < c_hi; c++) {
                const float v = src[c];
                uint64_t field = 0;
                if (v > t) field = 1;
                else if (v < -t) field = 3;
                word |= field << (2 * (c - w * 32));
            }
            dst[w] = word;
        }
    }
}

/*
 * btn[n] = sum of popcounts of the nonzero-plane words of item n
 * (TAB_GEMM.cu:150-160); words_per_item = H*W*PC.  Computed for every n.
 */
void oracle_btn_weight(const int64_t *qx_ternary, int N, long words_per_item, int32_t *btn)
{
    for (int n = 0; n < N; n++) {
        const uint64_t *row = (const uint64_t *)qx_ternary + (long)n * words_per_item * 2;
        int32_t cnt = 0;
        for (long k = 0; k < words_per_item; k++) cnt += __builtin_popcountll(row[2 * k + 1]);
        btn[n] = cnt;
    }
}

/*
 * Spatial zero padding of packed words (TAB_GEMM.cuh:73-89; border bits are zero as in
 * the CPU path's zero-initialised buffer, TAB_CPU.cpp:39,155).
 * a: [N][H][W][D] words, y: [N][H+2*p1][W+2*p2][D] words.
 */
void oracle_pad(const int64_t *a, int N, int H, int W, int D, int p1, int p2, int64_t *y)
{
    const int PH = H + 2 * p1, PW = W + 2 * p2;
    memset(y, 0, sizeof(int64_t) * (size_t)N * PH * PW * D);
#pragma omp parallel for schedule(static)
    for (long nh = 0; nh < (long)N * H; nh++) {
        const long n = nh / H, h = nh % H;
        memcpy(y + ((n * PH + h + p1) * PW + p2) * D, a + nh * W * D,
               sizeof(int64_t) * (size_t)W * D);
    }
}

/*
 * im2row over packed words (TAB_GEMM.cuh:92-115, TAB_CPU.h:27-63).
 * a: [N][PH][PW][D] (already padded), rows: [N*OH*OW][KH*KW*D] with the K axis ordered
 * (kh, kw, d).  OH/OW use the reference's integer-division formula on the padded extent.
 */
void oracle_img2row(const int64_t *a, int N, int PH, int PW, int D, int KH, int KW, int s1,
                    int s2, int64_t *rows)
{
    const int OH = (PH - KH + 1) / s1, OW = (PW - KW + 1) / s2;
    const long row_len = (long)KH * KW * D;
#pragma omp parallel for schedule(static)
    for (long m = 0; m < (long)N * OH * OW; m++) {
        const long n = m / ((long)OH * OW);
        const int oh = (int)((m / OW) % OH), ow = (int)(m % OW);
        int64_t *dst = rows + m * row_len;
        for (int kh = 0; kh < KH; kh++) {
            const int64_t *src = a + ((n * PH + (long)oh * s1 + kh) * PW + (long)ow * s2) * D;
            memcpy(dst + (long)kh * KW * D, src, sizeof(int64_t) * (size_t)KW * D);
        }
    }
}

/*
 * The four popcount GEMMs, TAB_CPU.cpp:242-328.  a is [M][K] (or [M][K][2] when the
 * activation is ternary), b is [N][K] (or [N][K][2] when the weight is ternary),
 * y is [M][N] int32.  Rows of y are split over OpenMP threads as in the reference
 * (TAB_CPU.cpp:246,270,294,315).
 */
ALWAYS_INLINE void body_tnn(const uint64_t *a, const uint64_t *b, long m0, long m1, int N,
                            int K, int32_t *y)
{
    for (long m = m0; m < m1; m++)
        for (int n = 0; n < N; n++) {
            const uint64_t *ra = a + m * K * 2, *rb = b + (long)n * K * 2;
            int32_t nonzero = 0, negative = 0;
            for (int k = 0; k < K; k++) {
                const uint64_t diff = ra[2 * k] ^ rb[2 * k];
                const uint64_t both = ra[2 * k + 1] & rb[2 * k + 1];
                nonzero += __builtin_popcountll(both);
                negative += __builtin_popcountll(diff & both);
            }
            y[m * N + n] = nonzero - 2 * negative;
        }
}

ALWAYS_INLINE void body_tbn(const uint64_t *a, const uint64_t *b, long m0, long m1, int N,
                            int K, int32_t *y)
{
    for (long m = m0; m < m1; m++)
        for (int n = 0; n < N; n++) {
            const uint64_t *ra = a + m * K * 2, *rb = b + (long)n * K;
            int32_t nonzero = 0, negative = 0;
            for (int k = 0; k < K; k++) {
                const uint64_t diff = ra[2 * k] ^ rb[k];
                const uint64_t mask = ra[2 * k + 1];
                nonzero += __builtin_popcountll(mask);
                negative += __builtin_popcountll(diff & mask);
            }
            y[m * N + n] = nonzero - 2 * negative;
        }
}

ALWAYS_INLINE void body_btn(const uint64_t *a, const uint64_t *b, const int32_t *btn, long m0,
                            long m1, int N, int K, int32_t *y)
{
    for (long m = m0; m < m1; m++)
        for (int n = 0; n < N; n++) {
            const uint64_t *ra = a + m * K, *rb = b + (long)n * K * 2;
            int32_t negative = 0;
            for (int k = 0; k < K; k++)
                negative += __builtin_popcountll((ra[k] ^ rb[2 * k]) & rb[2 * k + 1]);
            y[m * N + n] = btn[n] - 2 * negative;
        }
}

ALWAYS_INLINE void body_bnn(const uint64_t *a, const uint64_t *b, long m0, long m1, int N,
                            int K, int NUM, int32_t *y)
{
    for (long m = m0; m < m1; m++)
        for (int n = 0; n < N; n++) {
            const uint64_t *ra = a + m * K, *rb = b + (long)n * K;
            int32_t differ = 0;
            for (int k = 0; k < K; k++) differ += __builtin_popcountll(ra[k] ^ rb[k]);
            y[m * N + n] = NUM - 2 * differ;
        }
}

/* DoReFa 2-bit (TAB_CPU.cpp:332-358): y = sum over k of (2*a0 + a1) * (2*b0 + b1) per bit */
ALWAYS_INLINE void body_drf(const uint64_t *a, const uint64_t *b, long m0, long m1, int N,
                            int K, int32_t *y)
{
    for (long m = m0; m < m1; m++)
        for (int n = 0; n < N; n++) {
            const uint64_t *ra = a + m * K * 2, *rb = b + (long)n * K * 2;
            int32_t hh = 0, cross = 0, ll = 0;
            for (int k = 0; k < K; k++) {
                hh += __builtin_popcountll(ra[2 * k] & rb[2 * k]);
                cross += __builtin_popcountll(ra[2 * k + 1] & rb[2 * k]);
                cross += __builtin_popcountll(ra[2 * k] & rb[2 * k + 1]);
                ll += __builtin_popcountll(ra[2 * k + 1] & rb[2 * k + 1]);
            }
            y[m * N + n] = 4 * hh + 2 * cross + ll;
        }
}

/*
 * RTN (TAB_CPU.cpp:362-383): 2-bit fields, even bit = nonzero, odd bit = sign;
 * y = popcount(both nonzero) - 2 * popcount(both nonzero and signs differ).
 */
ALWAYS_INLINE void body_rtn(const uint64_t *a, const uint64_t *b, long m0, long m1, int N,
                            int K, int32_t *y)
{
    const uint64_t even = 0x5555555555555555ull;
    for (long m = m0; m < m1; m++)
        for (int n = 0; n < N; n++) {
            const uint64_t *ra = a + m * K, *rb = b + (long)n * K;
            int32_t nonzero = 0, negative = 0;
            for (int k = 0; k < K; k++) {
                const uint64_t both = ra[k] & rb[k] & even;
                const uint64_t differ = (ra[k] ^ rb[k]) >> 1;
                nonzero += __builtin_popcountll(both);
                negative += __builtin_popcountll(differ & both);
            }
            y[m * N + n] = nonzero - 2 * negative;
        }
}

/*
 * One exported entry per type.  VARIANTS expands the row-range body once per ISA level;
 * the exported function splits the M rows into contiguous blocks, one per OpenMP thread
 * (the reference's "omp parallel for" over rows), and runs the chosen variant on each.
 */
static void row_block(long M, long *m0, long *m1)
{
#ifdef _OPENMP
    const long nt = omp_get_num_threads(), t = omp_get_thread_num();
#else
    const long nt = 1, t = 0;
#endif
    *m0 = M * t / nt;
    *m1 = M * (t + 1) / nt;
}

#if HAVE_ISA_VARIANTS
#define VARIANTS(name, params, args)                                                          \
    static void name##_base params { body_##name args; }                                      \
    TARGET_AVX2 static void name##_avx2 params { body_##name args; }                          \
    TARGET_AVX512 static void name##_avx512 params { body_##name args; }                      \
    static void run_##name params                                                             \
    {                                                                                         \
        const int lv = isa_level();                                                           \
        if (lv == 2) name##_avx512 args;                                                      \
        else if (lv == 1) name##_avx2 args;                                                   \
        else name##_base args;                                                                \
    }
#else
#define VARIANTS(name, params, args) static void run_##name params { body_##name args; }
#endif

VARIANTS(tnn, (const uint64_t *a, const uint64_t *b, long m0, long m1, int N, int K, int32_t *y),
         (a, b, m0, m1, N, K, y))
VARIANTS(tbn, (const uint64_t *a, const uint64_t *b, long m0, long m1, int N, int K, int32_t *y),
         (a, b, m0, m1, N, K, y))
VARIANTS(btn, (const uint64_t *a, const uint64_t *b, const int32_t *btn, long m0, long m1, int N, int K, int32_t *y),
         (a, b, btn, m0, m1, N, K, y))
VARIANTS(bnn, (const uint64_t *a, const uint64_t *b, long m0, long m1, int N, int K, int NUM, int32_t *y),
         (a, b, m0, m1, N, K, NUM, y))

VARIANTS(drf, (const uint64_t *a, const uint64_t *b, long m0, long m1, int N, int K, int32_t *y),
         (a, b, m0, m1, N, K, y))
VARIANTS(rtn, (const uint64_t *a, const uint64_t *b, long m0, long m1, int N, int K, int32_t *y),
         (a, b, m0, m1, N, K, y))

void oracle_gemm_tnn(const int64_t *a, const int64_t *b, long M, int N, int K, int32_t *y)
{
#pragma omp parallel
    {
        long m0, m1;
        row_block(M, &m0, &m1);
        run_tnn((const uint64_t *)a, (const uint64_t *)b, m0, m1, N, K, y);
    }
}
void oracle_gemm_tbn(const int64_t *a, const int64_t *b, long M, int N, int K, int32_t *y)
{
#pragma omp parallel
    {
        long m0, m1;
        row_block(M, &m0, &m1);
        run_tbn((const uint64_t *)a, (const uint64_t *)b, m0, m1, N, K, y);
    }
}
void oracle_gemm_btn(const int64_t *a, const int64_t *b, const int32_t *btn, long M, int N,
                     int K, int32_t *y)
{
#pragma omp parallel
    {
        long m0, m1;
        row_block(M, &m0, &m1);
        run_btn((const uint64_t *)a, (const uint64_t *)b, btn, m0, m1, N, K, y);
    }
}
void oracle_gemm_bnn(const int64_t *a, const int64_t *b, long M, int N, int K, int NUM,
                     int32_t *y)
{
#pragma omp parallel
    {
        long m0, m1;
        row_block(M, &m0, &m1);
        run_bnn((const uint64_t *)a, (const uint64_t *)b, m0, m1, N, K, NUM, y);
    }
}

void oracle_gemm_drf(const int64_t *a, const int64_t *b, long M, int N, int K, int32_t *y)
{
#pragma omp parallel
    {
        long m0, m1;
        row_block(M, &m0, &m1);
        run_drf((const uint64_t *)a, (const uint64_t *)b, m0, m1, N, K, y);
    }
}
void oracle_gemm_rtn(const int64_t *a, const int64_t *b, long M, int N, int K, int32_t *y)
{
#pragma omp parallel
    {
        long m0, m1;
        row_block(M, &m0, &m1);
        run_rtn((const uint64_t *)a, (const uint64_t *)b, m0, m1, N, K, y);
    }
}

/*
 * Conv2d on an activation that is already packed, all six types of the CPU path
 * (TAB_CPU.cpp:507-614): zero-pad, im2row, GEMM.  Words per pixel D: 2*PC for types 0, 1, 4
 * (two planes), PC for 2, 3 (PC = ceil(C/64)), ceil(C/32) for type 5 (TAB_CPU.cpp:520-521).
 * Padded taps are zero words: value 0 for types 0, 1, 4, 5 and +1 for binary activations.
 */
int oracle_conv2d_packed(const int64_t *qx, const int64_t *qw, const int32_t *btn, int type,
                         int p1, int p2, int s1, int s2, int N, int H, int W, int C, int KN,
                         int KH, int KW, float *y)
{
    if (type < 0 || type > 5 || s1 < 1 || s2 < 1) return -1;
    const int PC = type == 5 ? (C + 31) / 32 : packed_channels(C);
    const int D = (type < 2 || type == 4) ? PC * 2 : PC;
    const int PH = H + 2 * p1, PW = W + 2 * p2;
    const int OH = oracle_out_extent(H, p1, KH, s1), OW = oracle_out_extent(W, p2, KW, s2);
    if (OH < 1 || OW < 1) return -1;
    const long M = (long)N * OH * OW;
    const int K = KH * KW * PC;

    int64_t *padded = malloc(sizeof(int64_t) * (size_t)N * PH * PW * D);
    int64_t *rows = malloc(sizeof(int64_t) * (size_t)M * KH * KW * D);
    int32_t *acc = malloc(sizeof(int32_t) * (size_t)M * KN);
    int rc = -1;
    if (padded && rows && acc) {
        oracle_pad(qx, N, H, W, D, p1, p2, padded);
        oracle_img2row(padded, N, PH, PW, D, KH, KW, s1, s2, rows);
        switch (type) {
        case 0: oracle_gemm_tnn(rows, qw, M, KN, K, acc); break;
        case 1: oracle_gemm_tbn(rows, qw, M, KN, K, acc); break;
        case 2: oracle_gemm_btn(rows, qw, btn, M, KN, K, acc); break;
        case 3: oracle_gemm_bnn(rows, qw, M, KN, K, KH * KW * C, acc); break;
        case 4: oracle_gemm_drf(rows, qw, M, KN, K, acc); break;
        default: oracle_gemm_rtn(rows, qw, M, KN, K, acc); break;
        }
#pragma omp parallel for schedule(static)
        for (long i = 0; i < M * KN; i++) y[i] = (float)acc[i];
        rc = 0;
    }
    free(padded); free(rows); free(acc);
    return rc;
}

/*
 * Whole Conv2d call (TAB_GEMM.cu:325-527): quantize the activation by type (ternary for
 * 0/1, binary for 2/3; 419-426; for the CPU-only types, levels for 4 and ternary fields for
 * 5), then the packed pipeline above with M=N*OH*OW, K=KH*KW*PC, NUM=KH*KW*C (509).  y holds
 * the int result converted to fp32 at y[m*KN + kn], i.e. (n,oh,ow,kn) memory order
 * (TAB_GEMM.cu:53,526).  Returns 0, or -1 on a bad type / empty output / allocation failure.
 */
int oracle_conv2d(const float *x, const int64_t *qw, const float *ths, const int32_t *btn,
                  int type, int p1, int p2, int s1, int s2, int N, int H, int W, int C, int KN,
                  int KH, int KW, float *y)
{
    if (type < 0 || type > 5) return -1;
    const int PC = type == 5 ? (C + 31) / 32 : packed_channels(C);
    const int D = (type < 2 || type == 4) ? PC * 2 : PC; /* activation words per pixel */
    int64_t *q = malloc(sizeof(int64_t) * (size_t)N * H * W * D);
    if (!q) return -1;
    switch (type) {
    case 0: case 1: oracle_quantize_ternary(x, ths, N, H, W, C, q); break;
    case 2: case 3: oracle_quantize_binary(x, ths, N, H, W, C, q); break;
    case 4: oracle_quantize_drf(x, ths, N, H, W, C, q); break;
    default: oracle_quantize_rtn(x, ths, N, H, W, C, q); break;
    }
    const int rc = oracle_conv2d_packed(q, qw, btn, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW, y);
    free(q);
    return rc;
}
