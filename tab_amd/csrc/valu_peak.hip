// Microbenchmark of the issue rate of the VALU instructions the conv kernels are made of
// (v_xor/v_and/v_bitop3 and v_bcnt_u32_b32), in lanes per clock per CU at 2.4 GHz, at 1..8
// workgroups of 4 waves per CU.  Its output is what the conv roofline is priced with.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); return 1; } } while (0)

template <int MODE>
__global__ __launch_bounds__(256) void k(uint32_t *out, int iters, uint32_t seed)
{
    uint32_t a[8], acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) { a[i] = seed * (threadIdx.x + i + 1); acc[i] = i; }
    uint32_t b = seed ^ threadIdx.x, m = ~seed;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int r = 0; r < 8; r++) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if (MODE == 0) {  // xor + bcnt (BNN pair)
                    uint32_t t;
                    asm volatile("v_xor_b32 %0, %1, %2" : "=v"(t) : "v"(a[i]), "v"(b));
                    asm volatile("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc[i]) : "v"(t));
                } else if (MODE == 1) {  // bcnt only
                    asm volatile("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc[i]) : "v"(a[i]));
                } else if (MODE == 2) {  // xor only
                    asm volatile("v_xor_b32 %0, %1, %0" : "+v"(acc[i]) : "v"(a[i]));
                } else if (MODE == 3) {  // bitop3 + bcnt
                    uint32_t t;
                    asm volatile("v_bitop3_b32 %0, %1, %2, %3 bitop3:0x28" : "=v"(t) : "v"(a[i]), "v"(b), "v"(m));
                    asm volatile("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc[i]) : "v"(t));
                } else if (MODE == 4) {  // and,bcnt,bitop3,bcnt (TNN pair)
                    uint32_t t, u;
                    asm volatile("v_and_b32 %0, %1, %2" : "=v"(t) : "v"(a[i]), "v"(m));
                    asm volatile("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc[i]) : "v"(t));
                    asm volatile("v_bitop3_b32 %0, %1, %2, %3 bitop3:0x28" : "=v"(u) : "v"(a[i]), "v"(b), "v"(t));
                    asm volatile("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc[i]) : "v"(u));
                } else if (MODE == 5) {  // add only (v_add_u32)
                    asm volatile("v_add_u32 %0, %1, %0" : "+v"(acc[i]) : "v"(a[i]));
                }
            }
        }
    }
    uint32_t s = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) s += acc[i];
    if (s == 0x12345678) out[threadIdx.x] = s;
}

template <int MODE> int run(const char *name, int ops_per_inner, int blocks_per_cu)
{
    uint32_t *out;
    CK(hipMalloc(&out, 4096));
    const int iters = 2000;
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    const int blocks = 256 * blocks_per_cu;
    k<MODE><<<blocks, 256>>>(out, 10, 3);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    k<MODE><<<blocks, 256>>>(out, iters, 3);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    double laneops = (double)blocks * 256 * iters * 64 * ops_per_inner;
    printf("%-28s blocks/CU=%d  %.3f ms  %.3e lane-ops/s  = %.1f lanes/clk/CU @2.4GHz\n", name, blocks_per_cu, ms,
           laneops / (ms * 1e-3), laneops / (ms * 1e-3) / 256 / 2.4e9);
    CK(hipFree(out));
    return 0;
}

int main()
{
    for (int bpc : {1, 2, 4, 8}) {
        run<0>("xor+bcnt", 2, bpc);
        run<1>("bcnt", 1, bpc);
        run<2>("xor", 1, bpc);
        run<3>("bitop3+bcnt", 2, bpc);
        run<4>("and,bcnt,bitop3,bcnt", 4, bpc);
        run<5>("add_u32", 1, bpc);
    }
    return 0;
}
