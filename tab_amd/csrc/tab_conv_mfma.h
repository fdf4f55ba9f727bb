// Matrix-core variant of the fused pad + im2row + bitwise GEMM: the packed bit planes are
// expanded in registers to FP4 (E2M1) operands of v_mfma_f32_32x32x64_f8f6f4.
//
// With a_k = a1*(1 - 2*a0) the decoded ternary value (any bit pattern of the two planes) and
// (1 - 2*a) the value of a binary bit, the four TAB formulas (TAB_GEMM.cu:25-147) are plain
// dot products D over all 64*G packed bit positions:
//   TNN  sum popc(a1&b1) - 2*sum popc((a0^b0)&a1&b1)  = D
//   TBN  sum popc(a1)    - 2*sum popc((a0^b)&a1)      = D
//   BTN  btn[n]          - 2*sum popc((a^b0)&b1)      = D + btn[n] - popc(b1 of filter n)
//   BNN  NUM             - 2*sum popc(a^b)            = D - (64*G - NUM)
// Zero words (padded taps, rows past M) decode to 0 for a ternary and to +1 for a binary
// operand, which is what the reference's padding means (TAB_CPU.cpp:39,155).
//
// E2M1 nibble = sign, 2 exponent bits, 1 mantissa bit: 0001 = 0.5, 0010 = 1, 0100 = 2, and a
// lone sign bit is -0.  Bit j of every nibble of a 32-bit slice goes to operand dword j with
// one AND (plus a shift where the bit has to move): magnitude weights (0.5, 1, 2, 2) on the A
// side meet (2, 1, 0.5, 0.5) on the B side, so every product is exactly +-1 or 0.  The order
// of k inside an operand is irrelevant as long as A and B agree, and they do: both come from
// the same bit of the same slice.  All partial sums are integers below 2^24 in magnitude
// (64*G is bounded by the launcher), hence exact in the fp32 accumulators.
//
// Tiling: 256 threads = WM x WN waves, each wave TM x TN MFMA tiles of 32x32.  In the kernel of this file
// operands are staged in LDS through registers exactly as for the popcount kernel (tab_conv_stage.h), and
// per 64-bit word a lane reads the 32-bit half lane/32 selects of its row (A) or column (B), lane%32; it
// serves chunks of K that cross filter taps and the k-split shape.  Chunks inside one tap take the kernel
// of tab_conv_mfma_direct.h, which shares the expansions and the epilogue defined here.
#pragma once
#include "tab_conv_stage.h"
#include <type_traits>

namespace tab {
namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kBit0 = 0x11111111u, kBit1 = 0x22222222u, kBit2 = 0x44444444u, kBit3 = 0x88888888u;

// The constants of the expansion, made opaque to the optimiser and pinned to register classes:
// this ISA takes no literal in a three-operand VALU instruction and only one scalar register, so
// (x & sign_bits) | pattern becomes a single v_and_or_b32 only when the mask sits in an SGPR and the
// pattern in a VGPR; with literals the compiler emits a v_and and a v_or.  (An inline-asm
// v_and_or_b32 is not an option: the compiler's hazard recogniser does not see registers written by
// inline asm and may then leave too few wait states before the MFMA that reads them.)
struct ExpandConsts {
    uint32_t sign_bits;          // kBit3, SGPR
    uint32_t half, one, two;     // the E2M1 patterns of 0.5, 1, 2 in every nibble, VGPRs
    uint32_t even, odd, pair;    // masks of the ternary expansion, SGPRs
    __device__ __forceinline__ ExpandConsts()
        : sign_bits(kBit3), half(kBit0), one(kBit1), two(kBit2), even(0x55555555u), odd(0xAAAAAAAAu), pair(0xCCCCCCCCu)
    {
        asm volatile("" : "+s"(sign_bits));
        asm volatile("" : "+v"(half), "+v"(one), "+v"(two));
        asm("" : "+s"(even), "+s"(odd), "+s"(pair));
    }
};

// Binary operand of BNN.  SIDE 0 = activation (weights 0.5, 1, 2, 2), SIDE 1 = weight operand (2, 1, 0.5, 0.5): the
// products are +-1 and both sides have the same number of instructions.
template <int SIDE>
__device__ __forceinline__ i32x8 expand_binary(uint32_t w, const ExpandConsts &c)
{
    const uint32_t m0 = SIDE ? c.two : c.half, m2 = SIDE ? c.half : c.two;
    i32x8 r = {0, 0, 0, 0, 0, 0, 0, 0};
    r[0] = (int)(((w << 3) & c.sign_bits) | m0);
    r[1] = (int)(((w << 2) & c.sign_bits) | c.one);
    r[2] = (int)(((w << 1) & c.sign_bits) | m2);
    r[3] = (int)((w & c.sign_bits) | m2);
    return r;
}

// Dword d of the binary partner of a ternary operand (TBN weights, BTN activations): +-0.5 in every dword.
__device__ __forceinline__ int half_binary_dword(uint32_t w, int d, const ExpandConsts &c)
{
    return (int)(((w << (3 - d)) & c.sign_bits) | c.half);
}

// Ternary operand (either side), 10 vector instructions: the (nonzero, sign) bits of the even positions of a slice are
// merged into one word of adjacent pairs and those of the odd positions into another (a shift and one three-input
// v_bitop3_b32 each); a pair is already the two top bits of an E2M1 nibble, sign and the exponent bit of 2, so dwords 2
// and 3 are one AND of a pair word and dwords 0 and 1 a shift and an AND.  Dword d holds the elements 4i + d of the
// slice, as in the binary expansions.  Every ternary element is +-2 or (+-)0; a binary partner is +-0.5 throughout
// (products +-1), and two ternary sides give four times the sum, which the kernels scale back with scale_ternary_sums
// (exact: 4 * 64 * G < 2^24 for every G the library takes).  With separate sign and magnitude masks per dword
// ((s << k) & sign | (z >> j) & bit) the same operand took 12 instructions (activation side) or 14 (weight side).
// d = 0 and d = 1 make the pair words and leave them in pw for d = 2 and d = 3.
__device__ __forceinline__ int ternary_dword(uint32_t s, uint32_t z, int d, uint32_t (&pw)[2], const ExpandConsts &c)
{
    if (d == 0) {
        const uint32_t s1 = s << 1;
        uint32_t a = ((z ^ s1) & c.even) ^ s1;  // bit 2j = z[2j], bit 2j+1 = s[2j]
        asm("" : "+v"(a));  // opaque: the optimiser otherwise re-derives each dword from s and z (14 instructions)
        pw[0] = a;
        return (int)((a << 2) & c.pair);
    }
    if (d == 1) {
        const uint32_t z1 = z >> 1;
        uint32_t b = ((s ^ z1) & c.odd) ^ z1;  // bit 2j = z[2j+1], bit 2j+1 = s[2j+1]
        asm("" : "+v"(b));
        pw[1] = b;
        return (int)((b << 2) & c.pair);
    }
    return (int)(pw[d - 2] & c.pair);
}

__device__ __forceinline__ i32x8 expand_ternary(uint32_t s, uint32_t z, const ExpandConsts &c)
{
    i32x8 r = {0, 0, 0, 0, 0, 0, 0, 0};
    uint32_t pw[2];
#pragma unroll
    for (int d = 0; d < 4; d++) r[d] = ternary_dword(s, z, d, pw, c);
    return r;
}

// TNN: both operands are +-2, the accumulators hold four times the sums
template <int TYPE, int TM, int TN>
__device__ __forceinline__ void scale_ternary_sums(f32x16 (&acc)[TM][TN])
{
    if (TYPE != 0) return;
#pragma unroll
    for (int mt = 0; mt < TM; mt++)
#pragma unroll
        for (int nt = 0; nt < TN; nt++) acc[mt][nt] *= 0.25f;
}

// Type 4 (TAB_CPU.cpp:332-358): planes (hi, lo) of a level 0..3 on both sides; E2M1 holds 1 = 0010,
// 2 = 0100 and 3 = 0101 exactly, so exponent bit 1 = hi, exponent bit 0 = lo & ~hi, mantissa = hi & lo,
// and the products (at most 9) and their sums stay exact integers.
__device__ __forceinline__ i32x8 expand_levels(uint32_t hi, uint32_t lo)
{
    const uint32_t one = lo & ~hi, three = hi & lo;
    i32x8 r = {0, 0, 0, 0, 0, 0, 0, 0};
    r[0] = (int)(((hi & kBit0) << 2) | ((one & kBit0) << 1) | (three & kBit0));
    r[1] = (int)(((hi & kBit1) << 1) | (one & kBit1) | ((three & kBit1) >> 1));
    r[2] = (int)((hi & kBit2) | ((one & kBit2) >> 1) | ((three & kBit2) >> 2));
    r[3] = (int)(((hi & kBit3) >> 1) | ((one & kBit3) >> 2) | ((three & kBit3) >> 3));
    return r;
}

// Type 5 (TAB_CPU.cpp:362-383): a 32-bit slice holds 16 fields (even bit = nonzero, odd bit = sign).
// The fields at even positions of the slice fill one operand dword, those at odd positions the next,
// each as the nibble (sign, 0, nonzero, 0) = +-1 or +-0.  A slice is 16 of the 32 elements a lane
// feeds, so a lane takes both halves of one word per MFMA and the two half-waves take alternate words.
__device__ __forceinline__ i32x8 expand_fields(uint32_t lo, uint32_t hi)
{
    i32x8 r = {0, 0, 0, 0, 0, 0, 0, 0};
    r[0] = (int)(((lo << 1) & kBit1) | ((lo << 2) & kBit3));
    r[1] = (int)(((lo >> 1) & kBit1) | (lo & kBit3));
    r[2] = (int)(((hi << 1) & kBit1) | ((hi << 2) & kBit3));
    r[3] = (int)(((hi >> 1) & kBit1) | (hi & kBit3));
    return r;
}

// The FP4 operand of one MFMA: SIDE 0 = activation, 1 = weight; p0, p1 = the lane's 32-bit slice of
// plane 0 and of the last plane (the same slice for one-plane operands); type 5: the two halves of
// the lane's word.
template <int TYPE, int SIDE>
__device__ __forceinline__ i32x8 expand_operand(uint32_t p0, uint32_t p1, const ExpandConsts &c)
{
    if (TYPE == 4) return expand_levels(p0, p1);
    if (TYPE == 5) return expand_fields(p0, p1);
    constexpr int PL = SIDE ? Planes<TYPE>::B : Planes<TYPE>::A;
    if (PL == 2) return expand_ternary(p0, p1, c);
    if (TYPE == 3) return expand_binary<SIDE>(p0, c);
    i32x8 r = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int d = 0; d < 4; d++) r[d] = half_binary_dword(p0, d, c);
    return r;
}

// Epilogue shared by the matrix-core kernels: accumulator element 4*j + i of lane (kb, r) is
// C[8*j + 4*kb + i][r] of the wave's 32x32 tile (mt, nt).  b_nonzero: BTN, bits set in the nonzero plane of
// the k-positions this lane multiplied, per filter tile; partial: KS * 17 * 64 floats of LDS when the KS
// waves of the workgroup hold partial sums of one tile; padded: words of K the kernel multiplied, K rounded up to whole
// chunks (the words past K are zeros, which add +64 each for binary x binary: the BNN bias counts them).
template <int TYPE, int TM, int TN, int KCH, int KS>
__device__ __forceinline__ void conv_mfma_epilogue(const ConvArgs &p, f32x16 (&acc)[TM][TN], int (&b_nonzero)[TN], int wave_m0,
                                                   int wave_n0, int lane, int ks, float *partial, int padded)
{
    const int r = lane & 31, kb = lane >> 5;
    // btn of this lane's filters (BTN); loaded here rather than before the loop because the registers they would hold
    // through it push the 128x128 shape over its 128-register budget (requesting them early gained nothing)
    int btn_col[TN];
#pragma unroll
    for (int nt = 0; nt < TN; nt++) {
        const int col = wave_n0 + nt * 32 + r;
        btn_col[nt] = (TYPE == 2 && col < p.KN) ? p.btn[col] : 0;
    }
    if (KS > 1) {
        // the KS waves hold partial sums of the same tile: exchange them through LDS; wave ks
        // finishes rows 8*ks .. 8*ks+7
#pragma unroll
        for (int e = 0; e < 16; e++) partial[(ks * 17 + e) * 64 + lane] = acc[0][0][e];
        partial[(ks * 17 + 16) * 64 + lane] = (float)b_nonzero[0];
        __syncthreads();
        float sum[5];
#pragma unroll
        for (int e = 0; e < 5; e++) {
            sum[e] = 0.f;
            const int src = e < 4 ? 4 * ks + e : 16;
#pragma unroll
            for (int k = 0; k < KS; k++) sum[e] += partial[(k * 17 + src) * 64 + lane];
        }
        const int col = wave_n0 + r;
        const bool col_ok = col < p.KN;
        float bias = 0.f;
        if (TYPE == 2) bias = (float)btn_col[0] - (sum[4] + __shfl_xor(sum[4], 32, 64));
        if (TYPE == 3) bias = (float)(p.num - 64 * padded);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int m = wave_m0 + 8 * ks + 4 * kb + i;
            if (col_ok && m < p.M) __builtin_nontemporal_store(sum[i] + bias, &p.y[(size_t)m * p.KN + col]);
        }
        return;
    }
    // Y is written once and read by nobody here: non-temporal stores keep it from pushing the operands out of L2
    // (N=256 28x28x512->512: HBM reads 30-78 MB -> 15-31 MB, 1.1-1.3 x the operands' size, and 2-4 % less time);
    // p.y_cached (set from the size of Y by the host) selects ordinary stores instead.
    // fp32 output through a buffer descriptor over the wave's rows of Y: rows past M lie past its end and
    // columns past KN get an offset past it, so every store is unconditional (a branch per store, which
    // "if (in range) store" compiles to, cost more than the store: the epilogue of a 256x128 tile took 6.5 us)
    const long rows_left = (long)p.M - wave_m0;
    if (rows_left <= 0) return;  // wave-uniform
    const size_t y_bytes = (size_t)(rows_left < 32 * TM ? rows_left : 32 * TM) * p.KN * 4;  // < 2 GiB (launch check)
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.y + (size_t)wave_m0 * p.KN), 0, (int)y_bytes, kBufferFlags);
    const uint32_t row_bytes = (uint32_t)p.KN * 4u;
#pragma unroll
    for (int nt = 0; nt < TN; nt++) {
        const int col = wave_n0 + nt * 32 + r;
        float bias = 0.f;
        if (TYPE == 2) {
            const int nonzero = b_nonzero[nt] + __shfl_xor(b_nonzero[nt], 32, 64);
            bias = (float)(btn_col[nt] - nonzero);
        }
        if (TYPE == 3) bias = (float)(p.num - 64 * padded);
        // kNoFilter + any offset inside the tile stays out of range without wrapping
        const uint32_t lane_off = col < p.KN ? (uint32_t)(4 * kb) * row_bytes + (uint32_t)col * 4u : kNoFilter;
        auto store_tiles = [&](auto policy) {
#pragma unroll
            for (int mt = 0; mt < TM; mt++)
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int row = mt * 32 + 8 * j + i;  // + 4*kb, already in lane_off
                        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc[mt][nt][4 * j + i] + bias), y_rsrc,
                                                              lane_off + (uint32_t)row * row_bytes, 0, decltype(policy)::value);
                    }
        };
        if (p.y_cached) store_tiles(std::integral_constant<int, 0>());  // wave-uniform
        else store_tiles(std::integral_constant<int, kStreamingStore>());
    }
}

// Packed output for a kernel that multiplied with the weights as the FIRST MFMA operand: accumulator element 4j+i of
// lane (kb, r) is then filter 8j+4kb+i of filter tile nt and pixel r of row tile mt, i.e. a lane holds 16 filters of ONE
// pixel.  It thresholds them against that pixel's threshold (a per-lane constant) exactly as the quantizer would
// threshold them as the next layer's NHWC activation (item = image, channel = filter; TAB_GEMM.cu:184-192, 231) into 16
// bits, and the other half-wave's lane of the same pixel supplies the other 16 of the 32-bit half word: no ballot and
// no cross-lane deposit per value (packing by wave ballot, with the activation as the first operand, costs about 13 vector
// instructions per pair of rows, this 2-3 per value).  The per-filter bias of BTN (btn - nonzero weights, known per lane = filter after the loop) is
// handed to the lanes that need it through `exchange`, 32*TN dwords of LDS private to the wave.
template <int TYPE, int TM, int TN, int KCH>
__device__ __forceinline__ void conv_mfma_epilogue_packed(const ConvArgs &p, f32x16 (&acc)[TM][TN], int (&b_nonzero)[TN], int wave_m0,
                                                          int wave_n0, int lane, uint32_t *exchange, int padded)
{
    const int r = lane & 31, kb = lane >> 5;
    const long rows_left = (long)p.M - wave_m0;
    if (rows_left <= 0) return;  // wave-uniform
    const int out_words = (p.KN + 63) >> 6;
    const uint32_t element = p.out_bits == 1 ? 8u : 16u;
    const uint32_t row_bytes = (uint32_t)out_words * element;
    const __amdgpu_buffer_rsrc_t out = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(reinterpret_cast<char *>(p.qy) + (size_t)wave_m0 * row_bytes), 0,
        (int)((uint32_t)(rows_left < 32 * TM ? rows_left : 32 * TM) * row_bytes), kBufferFlags);

    float bias[TN][16];
#pragma unroll
    for (int nt = 0; nt < TN; nt++) {
        if (TYPE == 2) {
            const int col = wave_n0 + nt * 32 + r;
            const int btn = col < p.KN ? p.btn[col] : 0;
            const int nonzero = b_nonzero[nt] + __shfl_xor(b_nonzero[nt], 32, 64);
            exchange[nt * 32 + r] = __float_as_uint((float)(btn - nonzero));  // both half-waves write the same value
        }
    }
    if (TYPE == 2) __builtin_amdgcn_wave_barrier();  // LDS operations of one wave complete in order
#pragma unroll
    for (int nt = 0; nt < TN; nt++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            u32x4 v = {0, 0, 0, 0};
            if (TYPE == 2) v = *reinterpret_cast<const u32x4 *>(exchange + nt * 32 + 8 * j + 4 * kb);
#pragma unroll
            for (int i = 0; i < 4; i++)
                bias[nt][4 * j + i] = TYPE == 2 ? __uint_as_float(v[i]) : (TYPE == 3 ? (float)(p.num - 64 * padded) : 0.f);
        }

    auto pack_rows = [&](auto out_bits_constant) {
        constexpr int OUT_BITS = decltype(out_bits_constant)::value;
#pragma unroll
        for (int mt = 0; mt < TM; mt++) {
            int n = (int)div32((uint32_t)(wave_m0 + mt * 32 + r), p.div_pixels);
            n = n < p.N ? n : p.N - 1;  // rows past M are computed but not stored
            const float th = p.out_ths[n];
            uint32_t sign_half[TN], nz_half[TN];
#pragma unroll
            for (int nt = 0; nt < TN; nt++) {
                uint32_t sg = 0, nz = 0;
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float v = (TYPE == 2 || TYPE == 3) ? acc[mt][nt][4 * j + i] + bias[nt][4 * j + i] : acc[mt][nt][4 * j + i];
                        const uint32_t bit = 1u << (8 * j + i);  // shifted by 4*kb below
                        if (OUT_BITS == 1) {
                            sg |= v < th ? bit : 0u;
                        } else {
                            const bool pos = v > th, neg = !pos && v < -th;
                            sg |= neg ? bit : 0u;
                            nz |= (pos || neg) ? bit : 0u;
                        }
                    }
                const int cols_left = p.KN - (wave_n0 + nt * 32);  // filters of this tile that exist: tail bits stay zero
                const uint32_t live = cols_left >= 32 ? 0xffffffffu : (cols_left <= 0 ? 0u : (1u << cols_left) - 1u);
                sg <<= 4 * kb;
                nz <<= 4 * kb;
                sign_half[nt] = (sg | (uint32_t)__shfl_xor((int)sg, 32, 64)) & live;
                nz_half[nt] = (nz | (uint32_t)__shfl_xor((int)nz, 32, 64)) & live;
            }
            // the lower half-wave stores; a word past the last one and the upper half-wave get an offset out of range
            const uint32_t row_off = (uint32_t)(mt * 32 + r) * row_bytes;
            if constexpr (TN % 2 == 0) {  // wave_n0 is a multiple of 64: tiles 2t, 2t+1 are the halves of one word
#pragma unroll
                for (int t = 0; t < TN / 2; t++) {
                    const int word = (wave_n0 >> 6) + t;
                    const uint32_t off = (kb == 0 && word < out_words) ? row_off + (uint32_t)word * element : kNoData;
                    if (OUT_BITS == 1)
                        __builtin_amdgcn_raw_buffer_store_b64(u32x2{sign_half[2 * t], sign_half[2 * t + 1]}, out, off, 0, 0);
                    else
                        __builtin_amdgcn_raw_buffer_store_b128(u32x4{sign_half[2 * t], sign_half[2 * t + 1], nz_half[2 * t], nz_half[2 * t + 1]}, out, off, 0, 0);
                }
            } else {
#pragma unroll
                for (int nt = 0; nt < TN; nt++) {
                    const int col0 = wave_n0 + nt * 32, word = col0 >> 6, half = (col0 >> 5) & 1;
                    const uint32_t off = (kb == 0 && word < out_words) ? row_off + (uint32_t)word * element + (uint32_t)half * 4u : kNoData;
                    __builtin_amdgcn_raw_buffer_store_b32(sign_half[nt], out, off, 0, 0);
                    if (OUT_BITS == 2) __builtin_amdgcn_raw_buffer_store_b32(nz_half[nt], out, off == kNoData ? kNoData : off + 8u, 0, 0);
                }
            }
        }
    };
    if (p.out_bits == 1) pack_rows(std::integral_constant<int, 1>());  // wave-uniform
    else pack_rows(std::integral_constant<int, 2>());
}

// Workgroup -> tile.  Small launches: the row tiles of one filter tile first.  From 64 tiles on: each XCD an eighth
// of the tiles, ordered (row tile, filter tile).
// Short K and a large Y (p.tiles_n != 0; the launch is bound by writing Y): groups of eight row tiles walk the
// filter tiles together, so that the workgroups running at one time write whole rows of Y rather than one
// 512-byte column block of many rows (N=256 28x28x512->1024 1x1 BNN: 176 -> 150 us; N=32 56x56x256->1024: 110 -> 78).
// False for the workgroups that pad the last group.
__device__ __forceinline__ bool tile_of_workgroup(const ConvArgs &p, int &tile_m, int &tile_n)
{
    if (p.tiles_n != 0) {
        const int group = (int)div32(blockIdx.x, p.div_tiles_m), in_group = (int)blockIdx.x - group * 8 * p.tiles_n;
        tile_n = in_group >> 3;
        tile_m = group * 8 + (in_group & 7);
        return tile_m < p.tiles_m;
    }
    if (p.xcd_share != 0) {
        // consecutive workgroups go to consecutive XCDs, each with an L2 of its own: XCD x takes tiles
        // x * share .. (x + 1) * share - 1 in the order (row tile, filter tile), i.e. an eighth of the rows of Y with
        // all their filter tiles, so that every XCD fetches its own eighth of the activation and not all of it
        const uint32_t b = blockIdx.x;
        const uint32_t logical = b < 8u * (uint32_t)p.xcd_share ? (b & 7u) * (uint32_t)p.xcd_share + (b >> 3) : b;
        tile_m = (int)div32(logical, p.div_filter_tiles);
        tile_n = (int)logical - tile_m * p.filter_tiles;
        return true;
    }
    tile_n = (int)div32(blockIdx.x, p.div_tiles_m);
    tile_m = (int)blockIdx.x - tile_n * p.tiles_m;
    return true;
}

constexpr long kLargeY = 192L << 20;  // bytes of Y from which a short-K launch orders its workgroups by rows of Y

// Chooses the order (a.tiles_m is set) and returns the number of workgroups.  From a sweep of 1x1 layers (C = 64..1024,
// KN = 256..2048, N = 32..256): up to -30 % where Y is large and K a few words (a two-plane activation turns the gain
// into a loss from 8 words on, a one-plane one from 16), +1-4 % where Y is a few tens of megabytes.
template <int APL>
long order_workgroups(ConvArgs &a, int tiles_n)
{
    const bool by_rows_of_y = tiles_n >= 2 && (long)a.M * a.KN * 4 >= kLargeY && a.G <= (APL == 1 ? 8 : 4);
    a.tiles_n = by_rows_of_y ? tiles_n : 0;
    a.div_tiles_m = make_div32((uint32_t)(by_rows_of_y ? 8 * tiles_n : a.tiles_m));
    a.filter_tiles = tiles_n;
    a.div_filter_tiles = make_div32((uint32_t)tiles_n);
    // XCD-aware order (tile_of_workgroup): HBM reads of N=32 56x56x256->256 16.8 -> 6.0 MB, N=256 28x28x512->512
    // 75 -> 54 MB, durations within -2 .. +3 %
    const long tiles = (long)a.tiles_m * tiles_n;
    a.xcd_share = !by_rows_of_y && tiles >= 64 && tiles / 8 <= 0x0fffffffL ? (int)(tiles / 8) : 0;
    return by_rows_of_y ? (long)((a.tiles_m + 7) / 8) * 8 * tiles_n : (long)a.tiles_m * tiles_n;
}

// LDS of a CU, and the workgroups of four waves (one wave per SIMD each) that a CU holds by it.
constexpr int kLdsBytesPerCu = 160 * 1024;
constexpr int waves_by_lds(int lds_bytes) { return lds_bytes <= 0 ? 8 : (kLdsBytesPerCu / lds_bytes < 1 ? 1 : kLdsBytesPerCu / lds_bytes); }

// Waves per SIMD asked of the register allocation.  The shapes with four MFMA tiles per wave are capped at 128
// registers, i.e. four workgroups per CU (the 128x128 shape otherwise takes 136-152, 64 of them accumulators, and runs
// three, measured 3-7 % slower); 256-row tiles need the state of more staged rows and get 168 (three workgroups), eight
// tiles per wave 256 (two).  Never more than the LDS of the workgroup lets a CU hold: a request beyond that only costs
// registers.
constexpr int mfma_waves_per_eu(int wm, int tm, int tn, int lds_bytes)
{
    const int by_registers = tm * tn > 4 ? 2 : (wm * tm > 4 ? 3 : 4);
    return waves_by_lds(lds_bytes) < by_registers ? waves_by_lds(lds_bytes) : by_registers;
}
template <int TYPE, int WM, int WN, int TM, int TN, int KCH, bool INTAP, int KS>
constexpr int conv_mfma_lds_bytes()
{
    constexpr int BM = 32 * WM * TM, BN = 32 * WN * TN;
    using Stager = typename std::conditional<INTAP, TapStager<TYPE, BM, BN, INTAP ? KCH : 2>, TileStager<TYPE, BM, BN, KCH>>::type;
    return 4 * (2 * (Stager::A_DWORDS + Stager::B_DWORDS) + (KS > 1 ? KS * 17 * 64 : 1));
}

// PACKED: packed output (p.qy): the weights are the first MFMA operand and the epilogue packs inside a lane.
template <int TYPE, int WM, int WN, int TM, int TN, int KCH, bool INTAP, int KS = 1, bool PACKED = false>
__global__ __launch_bounds__(kConvThreads)
__attribute__((amdgpu_waves_per_eu(mfma_waves_per_eu(WM, TM, TN, conv_mfma_lds_bytes<TYPE, WM, WN, TM, TN, KCH, INTAP, KS>())))) void conv_mfma(const ConvArgs p)
{
    static_assert(WM * WN * KS * 64 == kConvThreads, "four waves");
    static_assert(!PACKED || KS == 1, "packed output: whole tiles per wave");
    static_assert(KCH % KS == 0 && (KS == 1 || (TM == 1 && TN == 1)), "k-split waves share one 32x32 tile");
    constexpr int WPW = KCH / KS;  // words of a chunk each wave multiplies
    constexpr int APL = Planes<TYPE>::A, BPL = Planes<TYPE>::B;
    static_assert(TYPE != 5 || WPW % 2 == 0, "type 5 multiplies two words per MFMA");
    constexpr int STEPS = TYPE == 5 ? WPW / 2 : WPW;  // MFMAs per tile pair and chunk
    constexpr int ASL = TYPE == 5 ? 2 : APL, BSL = TYPE == 5 ? 2 : BPL;
    constexpr int BM = 32 * WM * TM, BN = 32 * WN * TN;
    using Stager = typename std::conditional<INTAP, TapStager<TYPE, BM, BN, INTAP ? KCH : 2>, TileStager<TYPE, BM, BN, KCH>>::type;
    constexpr int A_STRIDE = Stager::A_STRIDE, B_STRIDE = Stager::B_STRIDE;
    constexpr int Q = Stager::Q, A_DWORDS = Stager::A_DWORDS, B_DWORDS = Stager::B_DWORDS;

    __shared__ __attribute__((aligned(16))) uint32_t lds[2 * (A_DWORDS + B_DWORDS)];
    __shared__ float partial[KS > 1 ? KS * 17 * 64 : 1];  // k-split: 16 accumulators + the BTN count per lane

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31;   // row of an A tile / column of a B tile
    const int kb = lane >> 5;  // which 32-bit half of the word this lane feeds
    const int ks = wave / (WM * WN);  // which words of every chunk this wave takes
    const int wm = (wave % (WM * WN)) % WM, wn = (wave % (WM * WN)) / WM;
    int tile_m, tile_n;
    if (!tile_of_workgroup(p, tile_m, tile_n)) return;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    Stager st;
    st.init(p, tid, m0, n0);
    const ExpandConsts consts;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int mt = 0; mt < TM; mt++)
#pragma unroll
        for (int nt = 0; nt < TN; nt++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[mt][nt][e] = 0.f;
    int b_nonzero[TN];  // BTN: bits set in the nonzero plane of this lane's half of its filters
#pragma unroll
    for (int nt = 0; nt < TN; nt++) b_nonzero[nt] = 0;

    const int wave_m0 = m0 + wm * (32 * TM), wave_n0 = n0 + wn * (32 * TN);

    st.fetch(p, 0);
    st.stage(lds);
    __syncthreads();

    const int a_off = wm * (32 * TM) + r, b_off = wn * (32 * TN) + r;
    for (int chunk = 0; chunk < p.nchunks; chunk++) {
        const bool more = chunk + 1 < p.nchunks;
        if (more) st.fetch(p, chunk + 1);

        // Every chunk is exactly KCH words: the stager zero-fills words past the end of K, which add
        // nothing for a ternary operand and +64 per word for binary x binary (the BNN bias below
        // counts them).
        const uint32_t *la = lds + (chunk & 1) * (A_DWORDS + B_DWORDS) + a_off, *lb = la - a_off + A_DWORDS + b_off;
        // one step = one MFMA per tile pair; ASL, BSL = the 32-bit slices a lane reads per operand tile and
        // step: its half of the word of every plane, or (type 5) both halves of its own word
        uint32_t a_w[STEPS][ASL][TM], b_w[STEPS][BSL][TN];
        auto read_step = [&](int w) {
#pragma unroll
            for (int sl = 0; sl < ASL; sl++) {
                const int slice = TYPE == 5 ? 2 * (ks + KS * (2 * w + kb)) + sl : sl * Q + 2 * (ks + KS * w) + kb;
#pragma unroll
                for (int mt = 0; mt < TM; mt++) a_w[w][sl][mt] = la[slice * A_STRIDE + mt * 32];
            }
#pragma unroll
            for (int sl = 0; sl < BSL; sl++) {
                const int slice = TYPE == 5 ? 2 * (ks + KS * (2 * w + kb)) + sl : sl * Q + 2 * (ks + KS * w) + kb;
#pragma unroll
                for (int nt = 0; nt < TN; nt++) b_w[w][sl][nt] = lb[slice * B_STRIDE + nt * 32];
            }
        };
        // LDS reads run ahead of the matrix cores: the whole chunk up front when that is few registers
        // (one-plane operands; measured +3 % on BNN, a loss for the two-plane types), else one step ahead
        constexpr bool ALL_AHEAD = (ASL * TM + BSL * TN) * STEPS <= 16;
        if (ALL_AHEAD) {
#pragma unroll
            for (int w = 0; w < STEPS; w++) read_step(w);
            __builtin_amdgcn_sched_barrier(0);
        } else {
            read_step(0);
        }
#pragma unroll
        for (int w = 0; w < STEPS; w++) {
            if (!ALL_AHEAD && w + 1 < STEPS) read_step(w + 1);
            i32x8 af[TM], bf[TN];
#pragma unroll
            for (int mt = 0; mt < TM; mt++) af[mt] = expand_operand<TYPE, 0>(a_w[w][0][mt], a_w[w][ASL - 1][mt], consts);
#pragma unroll
            for (int nt = 0; nt < TN; nt++) {
                bf[nt] = expand_operand<TYPE, 1>(b_w[w][0][nt], b_w[w][BSL - 1][nt], consts);
                if (TYPE == 2) b_nonzero[nt] += __builtin_popcount(b_w[w][BSL - 1][nt]);
            }
#pragma unroll
            for (int mt = 0; mt < TM; mt++)
#pragma unroll
                for (int nt = 0; nt < TN; nt++)
                    acc[mt][nt] = PACKED ? __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[nt], af[mt], acc[mt][nt], 4, 4, 0, 0, 0, 0)
                                         : __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[mt], bf[nt], acc[mt][nt], 4, 4, 0, 0, 0, 0);
        }

        if (more) st.stage(lds + ((chunk + 1) & 1) * (A_DWORDS + B_DWORDS));
        __syncthreads();
    }

    scale_ternary_sums<TYPE>(acc);
    if constexpr (PACKED)  // (the chunk loop ends on a barrier: the operand buffers are free for BTN's exchange of biases)
        conv_mfma_epilogue_packed<TYPE, TM, TN, KCH>(p, acc, b_nonzero, wave_m0, wave_n0, lane, lds + wave * (32 * TN), p.nchunks * KCH);
    else
        conv_mfma_epilogue<TYPE, TM, TN, KCH, KS>(p, acc, b_nonzero, wave_m0, wave_n0, lane, ks, partial, p.nchunks * KCH);
}

// Chunk length for G words: 1..4, the one with the least padded work (a barrier is priced as half a
// word), longer chunks on ties.
inline int mfma_chunk_words(int G)
{
    int best = 4, best_cost = 0x7fffffff;
    for (int k = 4; k >= 1; k--) {
        const int cost = ((G + k - 1) / k) * (2 * k + 1);
        if (cost < best_cost) { best = k; best_cost = cost; }
    }
    return best;
}

template <int TYPE, int WM, int WN, int TM, int TN, int KCH, bool INTAP, int KS = 1>
hipError_t launch_mfma_tile(ConvArgs a, hipStream_t stream)
{
    constexpr int BM = 32 * WM * TM, BN = 32 * WN * TN;
    a.kcw = KCH;
    a.nchunks = (a.G + KCH - 1) / KCH;
    a.tiles_m = (a.M + BM - 1) / BM;
    const long blocks = order_workgroups<Planes<TYPE>::A>(a, (a.KN + BN - 1) / BN);
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    if (a.qy != nullptr) {
        if constexpr (KS == 1)
            conv_mfma<TYPE, WM, WN, TM, TN, KCH, INTAP, KS, true><<<dim3((unsigned)blocks), dim3(kConvThreads), 0, stream>>>(a);
        else
            return hipErrorInvalidValue;  // no packed output from the k-split 32x32 shape
    } else {
        conv_mfma<TYPE, WM, WN, TM, TN, KCH, INTAP, KS><<<dim3((unsigned)blocks), dim3(kConvThreads), 0, stream>>>(a);
    }
    return hipGetLastError();
}

// Chunks of whole word pairs that stay inside a filter tap (PC even) go from global memory straight into LDS
// (tab_conv_mfma_direct.h), measured 2-14 % faster than staging them through registers; the k-split shape keeps the piece stager of the kernel
// above (its chunks are too short to split into pairs of words per wave, and it measured no better).
template <int TYPE, int WM, int WN, int TM, int TN, int KCH, int KS = 1, int ARUN = 0>
hipError_t launch_mfma_direct(ConvArgs a, hipStream_t stream);
template <int TYPE, int WM, int WN, int TM, int TN, int KS, int WORDS>
hipError_t launch_mfma_split(const ConvArgs &a, hipStream_t stream);
template <int TYPE>
hipError_t launch_mfma_tail(ConvArgs a, hipStream_t stream);
template <int TYPE>
hipError_t launch_mfma_tail_wide(ConvArgs a, hipStream_t stream);

template <int TYPE, int WM, int WN, int TM, int TN, int KCH, int KS = 1>
hipError_t launch_mfma_intap(const ConvArgs &a, hipStream_t stream)
{
    if constexpr (KS == 1)
        return launch_mfma_direct<TYPE, WM, WN, TM, TN, KCH>(a, stream);
    else
        return launch_mfma_tile<TYPE, WM, WN, TM, TN, KCH, true, KS>(a, stream);
}

// LONG: the launch is small enough to be latency-bound, so prefer few long chunks (fewer serial
// fetch round trips) over a small LDS footprint.
template <int TYPE, int WM, int WN, int TM, int TN, bool LONG = false>
hipError_t launch_mfma_shape(const ConvArgs &a, hipStream_t stream)
{
    // whole word pairs inside one tap (PC even) load LDS directly
    if constexpr (LONG) {
        if (a.PC % 4 == 0 && a.G % 12 == 0) return launch_mfma_intap<TYPE, WM, WN, TM, TN, 12>(a, stream);
        if (a.PC % 8 == 0) return launch_mfma_intap<TYPE, WM, WN, TM, TN, 8>(a, stream);
    }
    if (a.PC % 4 == 0) return launch_mfma_intap<TYPE, WM, WN, TM, TN, 4>(a, stream);
    // PC = 2, 6, 10 ...: chunks of six words across taps rather than one pair of words per barrier (+5-13 %),
    // unless two two-plane operands would push the big tiles' LDS past four workgroups per CU
    if constexpr (LONG || Planes<TYPE>::A + Planes<TYPE>::B <= 3)
        if (a.PC % 2 == 0 && a.G % 6 == 0) return launch_mfma_intap<TYPE, WM, WN, TM, TN, 6>(a, stream);
    if constexpr (LONG && TYPE != 5)
        if (a.G % 9 == 0) return launch_mfma_tile<TYPE, WM, WN, TM, TN, 9, false>(a, stream);
    if (a.PC % 2 == 0) return launch_mfma_intap<TYPE, WM, WN, TM, TN, 2>(a, stream);
    if constexpr (TYPE == 5) {  // whole pairs of words per chunk
        if ((a.G + 1) / 2 % 2 == 0) return launch_mfma_tile<TYPE, WM, WN, TM, TN, 4, false>(a, stream);
        return launch_mfma_tile<TYPE, WM, WN, TM, TN, 2, false>(a, stream);
    } else {
        switch (mfma_chunk_words(a.G)) {
        case 1: return launch_mfma_tile<TYPE, WM, WN, TM, TN, 1, false>(a, stream);
        case 2: return launch_mfma_tile<TYPE, WM, WN, TM, TN, 2, false>(a, stream);
        case 3: return launch_mfma_tile<TYPE, WM, WN, TM, TN, 3, false>(a, stream);
        default: return launch_mfma_tile<TYPE, WM, WN, TM, TN, 4, false>(a, stream);
        }
    }
}

// The short-K kernel with the weights resident in registers (tab_conv_mfma_regs.h), types 0..3.
template <int TYPE>
hipError_t launch_mfma_regs(const ConvArgs &a, hipStream_t stream);

// shape: 0 = 128x128, 1 = 128x64, 2 = 64x64 (rows x filters per workgroup), 3 = 32x32 with the four
// waves splitting every chunk of four words between them, 4 = 256x64, 5 = 256x128 and 6 = 128x256
// (eight MFMA tiles per wave: fewer operand expansions per MFMA, half the occupancy), 7 = the register-resident
// short-K kernel (K of at most nine words; longer K falls back to the shape picked from the launch),
// 8 = 64x64 with K split over the four waves (each wave 2x2 MFMA tiles over a quarter of every chunk), 9 = 128x128 with K
// split over two pairs of waves (each wave 2x4 MFMA tiles over half of every chunk); both need an even number of words per
// pixel and otherwise run as shapes 2 and 0, 10 = 128x128 tiles for the whole rounds of the chip and 64x64 split-K quarters for
// the rest of the last round (an even number of words per pixel; otherwise shape 0), 11 = the same with whole tiles of 128x256
// (words per pixel in fours; otherwise shape 6)
template <int TYPE>
hipError_t launch_mfma_type(const ConvArgs &a, int shape, hipStream_t stream)
{
    if (shape == 7) {
        if constexpr (TYPE <= 3)
            if (a.G <= 9) return launch_mfma_regs<TYPE>(a, stream);
        shape = conv_mfma_shape(TYPE, a);
        if (shape == 7) return hipErrorInvalidValue;
    }
    if (shape == 11) {
        if (a.PC % 4 == 0) return launch_mfma_tail_wide<TYPE>(a, stream);
        shape = 6;
    }
    if (shape == 10) {
        if (a.PC % 2 == 0) return launch_mfma_tail<TYPE>(a, stream);
        shape = 0;
    }
    if (shape == 8 && a.PC % 2 != 0) shape = 2;
    if (shape == 9 && a.PC % 2 != 0) shape = 0;
    switch (shape) {
    case 8: return launch_mfma_split<TYPE, 1, 1, 2, 2, 4, 2>(a, stream);
    case 9: return launch_mfma_split<TYPE, 2, 1, 2, 4, 2, 2>(a, stream);
    case 0: return launch_mfma_shape<TYPE, 2, 2, 2, 2>(a, stream);
    case 1: return launch_mfma_shape<TYPE, 4, 1, 1, 2>(a, stream);
    case 2: return launch_mfma_shape<TYPE, 2, 2, 1, 1, true>(a, stream);
    case 4: return launch_mfma_shape<TYPE, 4, 1, 2, 2>(a, stream);
    case 5: return launch_mfma_shape<TYPE, 2, 2, 4, 2>(a, stream);
    case 6: return launch_mfma_shape<TYPE, 2, 2, 2, 4>(a, stream);
    case 3:
        // these launches are latency-bound: few long chunks (three or six words per wave) beat many short ones
        if constexpr (TYPE != 5) {
            if (a.G % 24 == 0) return launch_mfma_tile<TYPE, 1, 1, 1, 1, 24, false, 4>(a, stream);
            if (a.G % 12 == 0) return launch_mfma_tile<TYPE, 1, 1, 1, 1, 12, false, 4>(a, stream);
        }
        if (a.PC % 8 == 0) return launch_mfma_intap<TYPE, 1, 1, 1, 1, 8, 4>(a, stream);
        if constexpr (TYPE == 5) {  // two words per wave and chunk at least
            return launch_mfma_tile<TYPE, 1, 1, 1, 1, 8, false, 4>(a, stream);
        } else {
            if (a.PC % 4 == 0) return launch_mfma_intap<TYPE, 1, 1, 1, 1, 4, 4>(a, stream);
            if (a.G > 4) return launch_mfma_tile<TYPE, 1, 1, 1, 1, 12, false, 4>(a, stream);
            return launch_mfma_tile<TYPE, 1, 1, 1, 1, 4, false, 4>(a, stream);
        }
    default: return hipErrorInvalidValue;
    }
}

}  // namespace
}  // namespace tab
