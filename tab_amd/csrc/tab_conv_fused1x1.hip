// Quantize + 1x1 convolution in one launch, for calls small enough to be bound by their launches rather than by memory or
// arithmetic (the 1x1 stride-2 layers of a ResNet at a small batch): ConvWithCuda_TAB's quantize, pad, im2row and GEMM
// stages (TAB_GEMM.cu:419-509) without the packed activation ever reaching memory.
//
// A 1x1 convolution without padding reads each input pixel (oh*s1, ow*s2) for one output pixel only, so the activation
// a workgroup multiplies is exactly the activation it quantizes.  A workgroup owns 32 output pixels and 128 filters:
//   * its four waves read the 32 pixels' channels as fp32, one 64-channel word per 16-lane DPP row, 4 rows per wave
//     instruction (the quantizer's lane layout, tab_pack.h), threshold them with the image's threshold
//     (TAB_GEMM.cu:184-192, 231) and leave the packed halves in LDS, [plane][word][half][pixel];
//   * meanwhile every lane has requested its own dwords of the weights: lane (kb, r) of wave w feeds half kb of filter
//     128*y + 32*w + r, all PC words, straight from global memory (tab_conv_mfma_regs.h does the same);
//   * after one barrier each wave multiplies the tile with its 32 filters, PC MFMAs of 32x32x64 FP4 (operands expanded
//     as in tab_conv_mfma.h), and stores its 32x32 block of Y, 128 contiguous bytes of two rows per instruction.
// Filter groups beyond the first quantize the same pixels again (KN / 128 times in all): cheap where this kernel is
// used, and the launcher keeps large launches on the two-kernel path, whose quantizer reads X once.
#include "tab_conv_mfma.h"
#include "tab_pack.h"

namespace tab {
namespace {

struct Fused1x1Args {
    const float *x;       // fp32 [N][H][W][C]
    const float *ths;     // [N]
    const uint64_t *qw;   // packed weight [KN][PC][BPL]
    const int32_t *btn;   // [KN] (BTN only)
    float *y;             // [M][KN]
    int N, H, W, C;
    int KN, s1, s2;
    int OH, OW, M;
    int num;              // C (BNN constant)
    Div32 div_pixels, div_ow;
};

// PC: 64-channel words per pixel (1, 2, 4 or 8).
template <int TYPE, int PC>
__global__ __launch_bounds__(kConvThreads) void conv1x1_fused(const Fused1x1Args p)
{
    static_assert(TYPE >= 0 && TYPE <= 3, "types 0..3");
    constexpr int APL = Planes<TYPE>::A, BPL = Planes<TYPE>::B;
    constexpr int MODE = APL;           // ternary or binary activation
    constexpr int PASSES = 2 * PC;      // workgroup-wide passes over the tile's 32 * PC rows (a wave takes 4 rows of each)

    // packed activation of the tile: dword ((plane * PC + word) * 2 + half) * 32 + pixel
    __shared__ uint32_t act[APL * PC * 2 * 32];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int r = lane & 31, kb = lane >> 5;
    const int sub = lane >> 4, l = lane & 15;
    const int m0 = blockIdx.x * 32;
    const int n0 = blockIdx.y * 128 + wave * 32;
    const int pixels = p.OH * p.OW;
    const ExpandConsts consts;

    // ---- activation: row = pixel * PC + word of the tile; pass i hands this 16-lane row the row 16*i + 4*wave + sub ----
    floatx4 v[PASSES];
    float th[PASSES];
#pragma unroll
    for (int i = 0; i < PASSES; i++) {
        const int row = 16 * i + 4 * wave + sub;
        const int pixel = row / PC, word = row % PC;
        int m = m0 + pixel;
        m = m < p.M ? m : p.M - 1;  // pixels past M read the last pixel again and are never stored
        const int n = (int)div32((uint32_t)m, p.div_pixels);
        const int rem = m - n * pixels;
        const int oh = (int)div32((uint32_t)rem, p.div_ow), ow = rem - oh * p.OW;
        const size_t in_pixel = ((size_t)n * p.H + (size_t)oh * p.s1) * p.W + (size_t)ow * p.s2;
        v[i] = *reinterpret_cast<const floatx4 *>(p.x + in_pixel * p.C + word * 64 + l * 4);
        th[i] = p.ths[n];
    }

    // ---- weights: filter n0 + r, half kb of every word and plane (filters past KN repeat the last one, never stored) ----
    const uint32_t *qw32 = reinterpret_cast<const uint32_t *>(p.qw);
    uint32_t raw[PC][BPL];
    {
        int f = n0 + r;
        f = f < p.KN ? f : p.KN - 1;
#pragma unroll
        for (int w = 0; w < PC; w++)
#pragma unroll
            for (int pl = 0; pl < BPL; pl++) raw[w][pl] = qw32[(((size_t)f * PC + w) * BPL + pl) * 2 + kb];
    }

    // ---- threshold, pack, deposit -----------------------------------------------------------------------------------
#pragma unroll
    for (int i = 0; i < PASSES; i++) {
        const int row = 16 * i + 4 * wave + sub;
        const int pixel = row / PC, word = row % PC;
        uint32_t sign, nz, out[4];
        compare4<MODE>(v[i], th[i], sign, nz);
        pack_row<MODE>(sign, nz, l, out);  // lane 0 of the row holds (plane 0 low, high[, plane 1 low, high])
        if (l == 0) {
#pragma unroll
            for (int pl = 0; pl < APL; pl++)
#pragma unroll
                for (int half = 0; half < 2; half++) act[((pl * PC + word) * 2 + half) * 32 + pixel] = out[2 * pl + half];
        }
    }
    __syncthreads();

    // ---- multiply: accumulator element 4j+i of lane (kb, r) is pixel 8j+4kb+i, filter n0 + r ----------------------------
    f32x16 acc;
    int nonzero = 0;  // BTN: bits set in the nonzero plane of this lane's half of its filter
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.f;
#pragma unroll
    for (int w = 0; w < PC; w++) {
        const uint32_t a0 = act[((0 * PC + w) * 2 + kb) * 32 + r];
        const uint32_t a1 = APL == 2 ? act[((1 * PC + w) * 2 + kb) * 32 + r] : a0;
        const i32x8 af = expand_operand<TYPE, 0>(a0, a1, consts);
        const i32x8 bf = expand_operand<TYPE, 1>(raw[w][0], raw[w][BPL - 1], consts);
        if (TYPE == 2) nonzero += __builtin_popcount(raw[w][BPL - 1]);
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af, bf, acc, 4, 4, 0, 0, 0, 0);
    }
    if (TYPE == 0) acc *= 0.25f;  // both operands are +-2: four times the sums

    // BTN btn[f] - popcount(b1 of f), BNN NUM - 64 per word (TAB_GEMM.cu:116, 144)
    float bias = TYPE == 3 ? (float)(p.num - 64 * PC) : 0.f;
    if (TYPE == 2) {
        const int f = n0 + r;
        bias = (float)((f < p.KN ? p.btn[f] : 0) - (nonzero + __shfl_xor(nonzero, 32, 64)));
    }

    // ---- store: a buffer descriptor that ends with the tile's last live row drops the pixels past M; filters past KN get an
    // offset out of range ----------------------------------------------------------------------------------------------
    const int rows_left = p.M - m0 < 32 ? p.M - m0 : 32;
    const uint32_t row_bytes = (uint32_t)p.KN * 4u;
    const __amdgpu_buffer_rsrc_t out = __builtin_amdgcn_make_buffer_rsrc((void *)(p.y + (size_t)m0 * p.KN), 0,
                                                                         (int)((uint32_t)rows_left * row_bytes), kBufferFlags);
    const bool col_ok = n0 + r < p.KN;
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t off = col_ok ? (uint32_t)(8 * j + 4 * kb + i) * row_bytes + (uint32_t)(n0 + r) * 4u : kNoData;
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc[4 * j + i] + bias), out, off, 0, kStreamingStore);
        }
}

template <int TYPE, int PC>
hipError_t launch_fused_words(const Fused1x1Args &a, hipStream_t stream)
{
    const dim3 grid((unsigned)((a.M + 31) / 32), (unsigned)((a.KN + 127) / 128));
    conv1x1_fused<TYPE, PC><<<grid, dim3(kConvThreads), 0, stream>>>(a);
    return hipGetLastError();
}

template <int TYPE>
hipError_t launch_fused_type(const Fused1x1Args &a, hipStream_t stream)
{
    switch (a.C / kWordBits) {
    case 1: return launch_fused_words<TYPE, 1>(a, stream);
    case 2: return launch_fused_words<TYPE, 2>(a, stream);
    case 4: return launch_fused_words<TYPE, 4>(a, stream);
    case 8: return launch_fused_words<TYPE, 8>(a, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

// True when conv1x1_fused takes the call: a 1x1 kernel without padding on 64, 128, 256 or 512 channels, types 0..3, X
// aligned for 16-byte loads, and a launch of at most kFusedMaxWorkgroups workgroups (beyond that the two-kernel path,
// whose quantizer reads X once and whose conv kernel tiles the filters, is the faster one).
bool conv1x1_fused_supported(int type, const float *x, int C, int KH, int KW, int p1, int p2, long M, int KN)
{
    constexpr long kFusedMaxWorkgroups = 4096;
    const int pc = C / kWordBits;
    return type >= 0 && type <= 3 && KH == 1 && KW == 1 && p1 == 0 && p2 == 0 && C % kWordBits == 0 &&
           (pc == 1 || pc == 2 || pc == 4 || pc == 8) && (uintptr_t)x % 16 == 0 &&
           (M + 31) / 32 * ((KN + 127) / 128) <= kFusedMaxWorkgroups && (KN + 127) / 128 <= 65535;
}

hipError_t launch_conv1x1_fused(int type, const float *x, const float *ths, const uint64_t *qw, const int32_t *btn, float *y, int N,
                                int H, int W, int C, int KN, int s1, int s2, int OH, int OW, hipStream_t stream)
{
    Fused1x1Args a;
    a.x = x; a.ths = ths; a.qw = qw; a.btn = btn; a.y = y;
    a.N = N; a.H = H; a.W = W; a.C = C; a.KN = KN; a.s1 = s1; a.s2 = s2; a.OH = OH; a.OW = OW;
    a.M = N * OH * OW;
    a.num = C;
    a.div_pixels = make_div32((uint32_t)(OH * OW));
    a.div_ow = make_div32((uint32_t)OW);
    switch (type) {
    case 0: return launch_fused_type<0>(a, stream);
    case 1: return launch_fused_type<1>(a, stream);
    case 2: return launch_fused_type<2>(a, stream);
    case 3: return launch_fused_type<3>(a, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace tab
