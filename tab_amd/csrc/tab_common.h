// Shared declarations of the gfx950 TAB kernels (internal; the public surface is
// include/tab_amd.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tab {

constexpr int kWordBits = 64;  // channels per packed int64 word (CNTBITS, TAB_GEMM.cuh:10)

// Exact x / d for x < 65536 and 1 <= d < 65536 with one multiply-high:
// magic = floor(2^32 / d) + 1 gives floor(x * magic / 2^32) == floor(x / d) whenever
// x * d < 2^32.  d == 1 has no 32-bit magic and is passed through.
struct FastDiv {
    uint32_t magic;
    uint32_t d;
};
inline FastDiv make_fastdiv(uint32_t d)
{
    FastDiv f;
    f.d = d;
    f.magic = d > 1 ? (uint32_t)(0x100000000ull / d) + 1u : 0u;
    return f;
}
__device__ __forceinline__ uint32_t fastdiv(uint32_t x, FastDiv f)
{
    return f.d == 1 ? x : __umulhi(x, f.magic);
}

// Exact x / d for 0 <= x < 2^31 and 1 <= d < 2^31 with one 32x32 -> 64-bit multiply and a shift (a runtime
// divisor otherwise costs some 25 instructions a lane): with s = ceil(log2 d) and mul = floor(2^(31+s) / d) + 1,
// mul * d exceeds 2^(31+s) by at most d <= 2^s, so the quotient's error term x * (mul * d - 2^(31+s)) / (d * 2^(31+s))
// stays below 1 / d for every x < 2^31.
struct Div32 {
    uint32_t mul, shift;
};
inline Div32 make_div32(uint32_t d)
{
    uint32_t s = 0;
    while (((uint64_t)1 << s) < d) s++;
    Div32 f;
    f.shift = 31 + s;
    f.mul = (uint32_t)((((uint64_t)1 << (31 + s)) / d) + 1);
    return f;
}
__host__ __device__ __forceinline__ uint32_t div32(uint32_t x, Div32 f)
{
    return (uint32_t)(((uint64_t)x * f.mul) >> f.shift);
}

// Arguments of the fused pad + im2row + popcount-GEMM kernel.
struct ConvArgs {
    const uint64_t *qx;  // packed activation [N][H][W][PC][APL]; PC = words per pixel and plane
    const uint64_t *qw;  // packed weight     [KN][KH][KW][PC][BPL]
    const int32_t *btn;  // [KN] (BTN only)
    float *y;            // [M][KN]
    // packed output instead of y (matrix-core kernel only): 32-bit halves of [M][ceil(KN/64)][out_bits]
    uint32_t *qy;
    const float *out_ths;  // [N] thresholds applied to the outputs of image n
    int out_bits;          // 1 or 2
    int N, H, W, PC;
    int KN, KH, KW;
    int p1, p2, s1, s2;
    int OH, OW;
    int M;         // N*OH*OW
    int G;         // KH*KW*PC, packed words along K per plane
    int kcw;       // words per K chunk (<= kMaxChunkWords)
    int nchunks;   // ceil(G / kcw)
    int num;       // KH*KW*C (BNN constant)
    int tiles_m;   // ceil(M / BM)
    int tiles_n;   // filter tiles when the workgroups are ordered by rows of Y (LDS-direct kernel, short K), else 0
    Div32 div_tiles_m;  // by tiles_m, or by 8 * tiles_n in that order (set by the launchers)
    int y_cached;       // fp32 output through the caches (1) or with non-temporal stores (0)
    int xcd_share;      // tiles each of the 8 XCDs takes as one contiguous run of rows of Y (0: order not XCD-aware)
    int filter_tiles;   // ceil(KN / BN), with div_filter_tiles, for that order
    Div32 div_filter_tiles;
    int tail_big;       // the mixed launch (conv_mfma_tail): workgroups that take whole 128x128 tiles; the rest take quarters
    int tail_chunks;    // chunks of K of a quarter in that launch
    FastDiv div_pc, div_kw;
    Div32 div_pixels, div_ow;  // by OH*OW and OW: an output row's image and line
};

// Compute units of the current device (256 on MI355X), looked up once; 256 if the lookup fails.
int device_compute_units();

// Launchers (tab_conv.hip / tab_quantize.hip); they enqueue on `stream` and return the
// launch status.
hipError_t launch_conv(int type, const ConvArgs &args, hipStream_t stream);
// Matrix-core (FP4 MFMA) variant; shape picks the workgroup tile.  conv_mfma_exact() says whether K is
// short enough for its fp32 accumulators to hold every partial sum exactly.
bool conv_mfma_exact(const ConvArgs &args);
bool conv_mfma_exact_levels(const ConvArgs &args);  // the same for type 4, whose products reach 9
int conv_mfma_shape(int type, const ConvArgs &args, float *cost_us = nullptr);
hipError_t launch_conv_mfma(int type, const ConvArgs &args, int shape, hipStream_t stream);
hipError_t launch_conv_mfma_tnn(const ConvArgs &args, int shape, hipStream_t stream);
hipError_t launch_conv_mfma_tbn(const ConvArgs &args, int shape, hipStream_t stream);
hipError_t launch_conv_mfma_btn(const ConvArgs &args, int shape, hipStream_t stream);
hipError_t launch_conv_mfma_bnn(const ConvArgs &args, int shape, hipStream_t stream);
hipError_t launch_conv_mfma_drf(const ConvArgs &args, int shape, hipStream_t stream);
hipError_t launch_conv_mfma_rtn(const ConvArgs &args, int shape, hipStream_t stream);
hipError_t launch_quantize(const float *x, const float *ths, int bitwidth, long pixels_per_item,
                           long items, int C, uint64_t *qx, int32_t *btn, hipStream_t stream);

// The same quantizer reading x as [N][C][H*W] (the CPU path's input layout, TAB_CPU.cpp:20-206); output as above.
hipError_t launch_quantize_nchw(const float *x, const float *ths, int bitwidth, int N, int C, long HW, uint64_t *qx,
                                int32_t *btn, hipStream_t stream);

// Packers of the CPU-only conv types: format 4 = DoReFa 2-bit levels, 5 = RTN fields.
hipError_t launch_quantize_format(const float *x, const float *ths, int format, long pixels_per_item, long items, int C,
                                  uint64_t *qx, hipStream_t stream);

// Quantize only the pixels (oh*s1, ow*s2) of every image into a compact [N][OH][OW][PC] activation
// (what a 1x1 convolution with stride and no padding reads).
bool quantize_strided_supported(const float *x, int H, int W, int C, int OH, int OW);
hipError_t launch_quantize_strided(const float *x, const float *ths, int bitwidth, int N, int H, int W, int C, int OH,
                                   int OW, int s1, int s2, uint64_t *qx, hipStream_t stream);

// ths[n] = scale * mean|x[n]| over per_item elements; `partial` holds items * threshold_splits()
// floats of scratch.
int threshold_splits(long items, long per_item);
hipError_t launch_threshold(const float *x, long items, long per_item, float scale, float *ths, float *partial,
                            hipStream_t stream);

// Quantize + 1x1 conv in one launch (tab_conv_fused1x1.hip), for calls that are bound by their launches.
bool conv1x1_fused_supported(int type, const float *x, int C, int KH, int KW, int p1, int p2, long M, int KN);
hipError_t launch_conv1x1_fused(int type, const float *x, const float *ths, const uint64_t *qw, const int32_t *btn, float *y, int N,
                                int H, int W, int C, int KN, int s1, int s2, int OH, int OW, hipStream_t stream);

void force_conv_tile(int tm, int ng);  // tuning hook: 0,0 restores the automatic choice
void set_tail_round(int workgroups);   // test hook of the mixed launch: workgroups counted as one round of the chip (0: the CUs)
int tail_round();
bool conv_kernel_forced();             // true while tab_set_conv_kernel holds a choice other than the automatic one

}  // namespace tab
