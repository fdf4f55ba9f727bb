// Matrix-core microbenchmark for the conv roofline: (1) checks that the FP4 (E2M1) encodings the conv
// kernel builds from packed bit planes multiply to exact integers in v_mfma_f32_32x32x64_f8f6f4 for
// all four operand combinations, (2) measures the instruction's issue rate alone and with the
// per-tile expansion work of each conv type in front of it, for the tiles per wave and workgroups per CU the conv
// kernel runs (2x2 at up to four workgroups, 4x2 / 2x4 at two), (3) measures how many independent vector
// instructions fit in an MFMA's shadow, (4) compares the two orders of a step of the conv kernel's loop: all
// expansions, then the MFMAs (serial), against the next step's expansions spread dword by dword over the MFMAs of
// this step, into a second set of operand registers (pipelined), with the expansion constants in registers as in
// the kernel, and reports the shader clock each run held (s_memtime over s_memrealtime).
// Register-resident: no memory traffic in the timed loops.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
#include <cstdlib>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); return 1; } } while (0)
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
#define M0 0x11111111u
#define M1 0x22222222u
#define M2 0x44444444u
#define M3 0x88888888u
// E2M1 nibble: bit3 sign, bits 2:1 exponent, bit0 mantissa: 0001=0.5 0010=1 0100=2
// BNN: A-side weights per nibble bit j: (0.5, 1, 2, 2); B-side: (2, 1, 0.5, 0.5).  A ternary operand is +-2 or 0 in
// every position, its binary partner +-0.5; two ternary operands give four times the sum.
__device__ __forceinline__ v8i bin_a(uint32_t w)   // value (bit ? -1 : +1) * weight
{
    v8i r = {0, 0, 0, 0, 0, 0, 0, 0};
    r[0] = (int)(((w << 3) & M3) | M0); r[1] = (int)(((w << 2) & M3) | M1); r[2] = (int)(((w << 1) & M3) | M2); r[3] = (int)((w & M3) | M2);
    return r;
}
__device__ __forceinline__ v8i bin_b(uint32_t w)
{
    v8i r = {0, 0, 0, 0, 0, 0, 0, 0};
    r[0] = (int)(((w << 3) & M3) | M2); r[1] = (int)(((w << 2) & M3) | M1); r[2] = (int)(((w << 1) & M3) | M0); r[3] = (int)((w & M3) | M0);
    return r;
}
__device__ __forceinline__ v8i bin_half(uint32_t w)   // (bit ? -1 : +1) * 0.5
{
    v8i r = {0, 0, 0, 0, 0, 0, 0, 0};
    r[0] = (int)(((w << 3) & M3) | M0); r[1] = (int)(((w << 2) & M3) | M0); r[2] = (int)(((w << 1) & M3) | M0); r[3] = (int)((w & M3) | M0);
    return r;
}
// nz * (sign ? -2 : +2): pair words of the even and of the odd positions, (nonzero, sign) adjacent, then the pairs
// as the top two bits of each nibble
__device__ __forceinline__ v8i ter(uint32_t s, uint32_t z)
{
    v8i r = {0, 0, 0, 0, 0, 0, 0, 0};
    const uint32_t a = (z & 0x55555555u) | ((s << 1) & 0xAAAAAAAAu), b = (s & 0xAAAAAAAAu) | ((z >> 1) & 0x55555555u);
    r[0] = (int)((a << 2) & 0xCCCCCCCCu); r[1] = (int)((b << 2) & 0xCCCCCCCCu); r[2] = (int)(a & 0xCCCCCCCCu); r[3] = (int)(b & 0xCCCCCCCCu);
    return r;
}
__device__ __forceinline__ v16f mfma(v8i a, v8i b, v16f c) { return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 4, 4, 0, 0, 0, 0); }
// A: [32 rows][2 dwords] planes s,z ; B: [32 cols][2 dwords]; mode bit0: A ternary, bit1: B ternary
__global__ void k_check(const uint32_t *As, const uint32_t *Az, const uint32_t *Bs, const uint32_t *Bz, float *C, int mode)
{
    const int lane = threadIdx.x, r = lane & 31, kb = lane >> 5;
    v8i a = (mode & 1) ? ter(As[r * 2 + kb], Az[r * 2 + kb]) : (mode & 2) ? bin_half(As[r * 2 + kb]) : bin_a(As[r * 2 + kb]);
    v8i b = (mode & 2) ? ter(Bs[r * 2 + kb], Bz[r * 2 + kb]) : (mode & 1) ? bin_half(Bs[r * 2 + kb]) : bin_b(Bs[r * 2 + kb]);
    v16f c = {0};
    c = mfma(a, b, c);
    for (int j = 0; j < 4; j++)
        for (int i = 0; i < 4; i++) C[(8 * j + 4 * kb + i) * 32 + r] = c[4 * j + i];
}
// The conv kernel's expansions with their constants in registers (masks in SGPRs, patterns in VGPRs): 7 vector
// instructions for a binary operand, 10 for a ternary one (a shift and a three-input bit operation per pair word, a
// shift and an AND for dwords 0 and 1, an AND for dwords 2 and 3), dword by dword.
struct ExpandRegs { uint32_t m3, p0, p1, p2, even, odd, pair; };
__device__ __forceinline__ ExpandRegs expand_regs()
{
    ExpandRegs k = {M3, M0, M1, M2, 0x55555555u, 0xAAAAAAAAu, 0xCCCCCCCCu};
    asm volatile("" : "+s"(k.m3), "+s"(k.even), "+s"(k.odd), "+s"(k.pair));
    asm volatile("" : "+v"(k.p0), "+v"(k.p1), "+v"(k.p2));
    return k;
}
__device__ __forceinline__ int bin_dword(uint32_t w, int d, const ExpandRegs &k)
{
    return (int)(((w << (3 - d)) & k.m3) | (d == 0 ? k.p0 : d == 1 ? k.p1 : k.p2));
}
__device__ __forceinline__ int ter_dword(uint32_t s, uint32_t z, int d, uint32_t (&pw)[2], const ExpandRegs &k)
{
    if (d == 0) {
        const uint32_t s1 = s << 1;
        uint32_t a = ((z ^ s1) & k.even) ^ s1;
        asm("" : "+v"(a));  // opaque, or the optimiser re-derives every dword from s and z
        pw[0] = a;
        return (int)((a << 2) & k.pair);
    }
    if (d == 1) {
        const uint32_t z1 = z >> 1;
        uint32_t b = ((s ^ z1) & k.odd) ^ z1;
        asm("" : "+v"(b));
        pw[1] = b;
        return (int)((b << 2) & k.pair);
    }
    return (int)(pw[d - 2] & k.pair);
}
__device__ __forceinline__ v8i ter_op(uint32_t s, uint32_t z, const ExpandRegs &k)
{
    v8i r = {0, 0, 0, 0, 0, 0, 0, 0};
    uint32_t pw[2];
#pragma unroll
    for (int d = 0; d < 4; d++) r[d] = ter_dword(s, z, d, pw, k);
    return r;
}
__device__ __forceinline__ v8i bin_op(uint32_t w, const ExpandRegs &k)
{
    v8i r = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int d = 0; d < 4; d++) r[d] = bin_dword(w, d, k);
    return r;
}
__device__ __forceinline__ v8i half_op(uint32_t w, const ExpandRegs &k)
{
    v8i r = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int d = 0; d < 4; d++) r[d] = (int)(((w << (3 - d)) & k.m3) | k.p0);
    return r;
}
// MODE 0: mfma only; 1: BNN expansions; 2: TNN expansions; 3: TBN.  TM x TN MFMA tiles per wave, one expansion per
// operand tile and step as in the conv kernel: 2x2 (the 128x128 workgroup tile), 4x2 and 2x4 (256x128 / 128x256).
template <int MODE, int TM, int TN>
__global__ __launch_bounds__(256) void k_tput(float *out, int iters, uint32_t seed)
{
    v16f c[TM][TN];
    for (int i = 0; i < TM; i++) for (int j = 0; j < TN; j++) for (int e = 0; e < 16; e++) c[i][j][e] = 0;
    uint32_t w[2 * (TM + TN)];
    for (int i = 0; i < 2 * (TM + TN); i++) w[i] = seed * (threadIdx.x + 1) * (2 * i + 1);
    const ExpandRegs k = expand_regs();
    v8i a[TM], b[TN];
    for (int i = 0; i < TM; i++) a[i] = bin_a(w[i]);
    for (int i = 0; i < TN; i++) b[i] = bin_b(w[TM + i]);
    for (int it = 0; it < iters; it++) {
        if (MODE != 0) {
            for (int i = 0; i < TM; i++) a[i] = (MODE == 1) ? bin_op(w[i], k) : ter_op(w[i], w[TM + TN + i], k);
            for (int i = 0; i < TN; i++) b[i] = (MODE == 2) ? ter_op(w[TM + i], w[2 * TM + TN + i], k) : (MODE == 3) ? half_op(w[TM + i], k) : bin_op(w[TM + i], k);
            w[0] += 0x9e3779b9u; for (int i = 1; i < 2 * (TM + TN); i++) w[i] ^= w[i - 1];
        }
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) c[i][j] = mfma(a[i], b[j], c[i][j]);
    }
    float s = 0;
    for (int i = 0; i < TM; i++) for (int j = 0; j < TN; j++) for (int e = 0; e < 16; e++) s += c[i][j][e];
    if (s == 12345.678f) out[threadIdx.x] = s;
}
template <int MODE, int TM, int TN> int tput(const char *name, int bpc)
{
    float *out; CK(hipMalloc(&out, 4096));
    const int iters = 4000, blocks = 256 * bpc;
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    k_tput<MODE, TM, TN><<<blocks, 256>>>(out, 10, 3); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0)); k_tput<MODE, TM, TN><<<blocks, 256>>>(out, iters, 3); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    double macs = (double)blocks * 4 * iters * TM * TN * 32 * 32 * 64;
    printf("%-16s tiles/wave=%dx%d blocks/CU=%d %.3f ms  %.0f binary-equivalent TOP/s; cycles per MFMA per SIMD @2.4GHz = %.1f\n", name, TM, TN,
           bpc, ms, 2 * macs / (ms * 1e-3) / 1e12, ms * 1e-3 * 2.4e9 / ((double)bpc * iters * TM * TN));
    CK(hipFree(out));
    return 0;
}
// What fits in an MFMA's shadow: eight independent MFMAs per round, each followed by NV pairs of vector instructions
// (shift, and-or: the expansion's instructions) on registers the MFMAs do not read.
template <int NV>
__global__ __launch_bounds__(256) void k_shadow(float *out, int iters, uint32_t seed)
{
    v16f c[8];
    for (int i = 0; i < 8; i++) for (int e = 0; e < 16; e++) c[i][e] = 0;
    uint32_t w[8];
    for (int i = 0; i < 8; i++) w[i] = seed * (threadIdx.x + 1) * (2 * i + 1);
    const v8i a = {1, 2, 3, 4, 0, 0, 0, 0}, b = {5, 6, 7, 8, 0, 0, 0, 0};
    uint32_t mask = M3, pat = M1;
    asm volatile("" : "+s"(mask));
    asm volatile("" : "+v"(pat));
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int m = 0; m < 8; m++) {
            c[m] = mfma(a, b, c[m]);
#pragma unroll
            for (int v = 0; v < NV; v++) w[(m * NV + v) & 7] = ((w[(m * NV + v) & 7] << 1) & mask) | pat;
        }
    }
    float s = 0;
    for (int i = 0; i < 8; i++) { for (int e = 0; e < 16; e++) s += c[i][e]; s += (float)w[i]; }
    if (s == 12345.678f) out[threadIdx.x] = s;
}
template <int NV> int shadow(int bpc)
{
    float *out; CK(hipMalloc(&out, 4096));
    const int iters = 2000, blocks = 256 * bpc;
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    k_shadow<NV><<<blocks, 256>>>(out, 10, 3); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0)); k_shadow<NV><<<blocks, 256>>>(out, iters, 3); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    printf("mfma + %2d independent vector instructions each, blocks/CU=%d: cycles per MFMA per SIMD @2.4GHz = %.1f\n", 2 * NV, bpc,
           ms * 1e-3 * 2.4e9 / ((double)bpc * iters * 8));
    CK(hipFree(out));
    return 0;
}

// TER: ternary operands on both sides.  PIPE 0: the TM + TN expansions of a step, then its TM * TN MFMAs; 1: the
// MFMAs of a step with the next step's expansions spread over them dword by dword, into the other operand set.
// Order pinned.
template <int TER, int PIPE, int TM, int TN>
__global__ __launch_bounds__(256) void k_step_order(float *out, long long *clocks, int iters, uint32_t seed)
{
    constexpr int NE = TM + TN, NM = TM * TN;
    constexpr int PER = (4 * NE + NM - 1) / NM;  // dwords after each MFMA
    v16f c[TM][TN];
    for (int i = 0; i < TM; i++) for (int j = 0; j < TN; j++) for (int e = 0; e < 16; e++) c[i][j][e] = 0;
    uint32_t w[2 * NE];
    for (int i = 0; i < 2 * NE; i++) w[i] = seed * (threadIdx.x + 1) * (2 * i + 1);
    const ExpandRegs k = expand_regs();
    v8i op[2][NE];
    uint32_t pw[2];
    auto piece = [&](int q, int set) {
        const int e = q / 4, d = q % 4;
        op[set][e][d] = TER ? ter_dword(w[e], w[NE + e], d, pw, k) : bin_dword(w[e], d, k);
    };
    for (int set = 0; set < 2; set++) for (int e = 0; e < NE; e++) op[set][e] = v8i{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int q = 0; q < 4 * NE; q++) piece(q, 0);
    const long long t0 = clock64(), r0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            if (PIPE == 0) {
#pragma unroll
                for (int q = 0; q < 4 * NE; q++) piece(q, s);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < NM; i++) c[i / TN][i % TN] = mfma(op[s][i / TN], op[s][TM + i % TN], c[i / TN][i % TN]);
                __builtin_amdgcn_sched_barrier(0);
            } else {
#pragma unroll
                for (int i = 0; i < NM; i++) {
                    c[i / TN][i % TN] = mfma(op[s][i / TN], op[s][TM + i % TN], c[i / TN][i % TN]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int q = i * PER; q < (i + 1) * PER; q++)
                        if (q < 4 * NE) piece(q, s ^ 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            w[0] += 0x9e3779b9u; for (int i = 1; i < 2 * NE; i++) w[i] ^= w[i - 1];  // new raw words every step
        }
    }
    const long long t1 = clock64(), r1 = wall_clock64();
    if (blockIdx.x == 0 && threadIdx.x == 0) { clocks[0] = t1 - t0; clocks[1] = r1 - r0; }
    float sum = 0;
    for (int i = 0; i < TM; i++) for (int j = 0; j < TN; j++) for (int e = 0; e < 16; e++) sum += c[i][j][e];
    if (sum == 12345.678f) out[threadIdx.x] = sum;
}
template <int TER, int PIPE, int TM, int TN> int step_order(int bpc)
{
    float *out; long long *clocks, h[2];
    CK(hipMalloc(&out, 4096)); CK(hipMalloc(&clocks, 16));
    const int iters = 2000, blocks = 256 * bpc;
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    k_step_order<TER, PIPE, TM, TN><<<blocks, 256>>>(out, clocks, 10, 3); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0)); k_step_order<TER, PIPE, TM, TN><<<blocks, 256>>>(out, clocks, iters, 3); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    CK(hipMemcpy(h, clocks, 16, hipMemcpyDeviceToHost));
    const double mhz = (double)h[0] / ((double)h[1] / 100.0);  // s_memrealtime ticks at 100 MHz
    const double per_simd = (double)bpc * iters * 2 * TM * TN;
    printf("%s operands, %s step, tiles/wave=%dx%d blocks/CU=%d: %.3f ms, shader clock %.0f MHz, cycles per MFMA per SIMD at that clock = %.1f, %.0f binary-equivalent TOP/s\n",
           TER ? "ternary" : "binary ", PIPE ? "pipelined" : "serial   ", TM, TN, bpc, ms, mhz, ms * 1e-3 * mhz * 1e6 / per_simd,
           2.0 * 256 * 4 * per_simd * 32 * 32 * 64 / (ms * 1e-3) / 1e12);
    CK(hipFree(out)); CK(hipFree(clocks));
    return 0;
}
static int val_t(uint32_t s, uint32_t z, int k) { return ((z >> k) & 1) ? (((s >> k) & 1) ? -1 : 1) : 0; }
static int val_b(uint32_t w, int k) { return ((w >> k) & 1) ? -1 : 1; }
int main()
{
    setvbuf(stdout, NULL, _IONBF, 0);
    uint32_t h[4][64]; float hC[1024];
    srand(7);
    for (int p = 0; p < 4; p++) for (int i = 0; i < 64; i++) h[p][i] = ((uint32_t)rand() << 16) ^ (uint32_t)rand() ^ ((uint32_t)rand() << 31);
    uint32_t *d[4]; float *dC;
    for (int p = 0; p < 4; p++) { CK(hipMalloc(&d[p], 256)); CK(hipMemcpy(d[p], h[p], 256, hipMemcpyHostToDevice)); }
    CK(hipMalloc(&dC, 4096));
    for (int mode = 0; mode < 4; mode++) {
        k_check<<<1, 64>>>(d[0], d[1], d[2], d[3], dC, mode); CK(hipDeviceSynchronize());
        CK(hipMemcpy(hC, dC, 4096, hipMemcpyDeviceToHost));
        int bad = 0;
        for (int m = 0; m < 32; m++) for (int n = 0; n < 32; n++) {
            int s = 0;
            for (int k = 0; k < 64; k++) {
                const int q = k >> 5, kk = k & 31;
                const int av = (mode & 1) ? val_t(h[0][m * 2 + q], h[1][m * 2 + q], kk) : val_b(h[0][m * 2 + q], kk);
                const int bv = (mode & 2) ? val_t(h[2][n * 2 + q], h[3][n * 2 + q], kk) : val_b(h[2][n * 2 + q], kk);
                s += av * bv;
            }
            bad += hC[m * 32 + n] != (float)(mode == 3 ? 4 * s : s);  // ternary x ternary: +-2 x +-2
        }
        printf("check A %s x B %s: %d mismatches of 1024 (C[0][0]=%g)\n", (mode & 1) ? "ternary" : "binary", (mode & 2) ? "ternary" : "binary", bad, hC[0]);
    }
    // 2x2 tiles per wave run up to four workgroups per CU in the conv kernel, eight tiles per wave two
    for (int bpc : {1, 2, 3, 4}) {
        tput<0, 2, 2>("f4 mfma only", bpc); tput<1, 2, 2>("BNN expansions", bpc); tput<3, 2, 2>("TBN expansions", bpc); tput<2, 2, 2>("TNN expansions", bpc);
    }
    for (int bpc : {1, 2}) {
        tput<1, 4, 2>("BNN expansions", bpc); tput<3, 2, 4>("TBN expansions", bpc); tput<2, 4, 2>("TNN expansions", bpc);
    }
    for (int bpc : {2, 4}) { shadow<0>(bpc); shadow<1>(bpc); shadow<2>(bpc); shadow<3>(bpc); shadow<4>(bpc); shadow<6>(bpc); }
    for (int bpc : {1, 2}) { step_order<0, 0, 4, 2>(bpc); step_order<0, 1, 4, 2>(bpc); step_order<1, 0, 4, 2>(bpc); step_order<1, 1, 4, 2>(bpc); }
    step_order<0, 0, 2, 2>(4); step_order<0, 1, 2, 2>(4); step_order<1, 0, 2, 2>(4); step_order<1, 1, 2, 2>(4);
    return 0;
}
