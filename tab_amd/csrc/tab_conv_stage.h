// Operand staging shared by the conv kernels: global memory -> registers -> LDS.
//
// A workgroup of 256 threads owns a BM x BN tile of Y.  K is walked in chunks of at most KCH
// packed 64-bit words; per chunk every thread fetches a few (row, word) elements of A - the
// im2row view of the packed activation, padding and stride in the address math, out-of-range
// taps as all-zero words (TAB_GEMM.cuh:73-115, TAB_CPU.cpp:39,155) - and of B (the packed
// weights), splits them into 32-bit halves and stores them k-major in LDS:
// dword index ((plane * Q + q) * ROWS + row), q = 2 * word + half, Q = 2 * KCH.
#pragma once
#include "tab_common.h"

namespace tab {

constexpr int kConvThreads = 256;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Types 4 (DoReFa 2-bit levels, two planes on both sides) and 5 (RTN, 2-bit fields interleaved in one
// plane on both sides) are the CPU-only ones of the reference (TAB_CPU.cpp:332-383).
template <int TYPE> struct Planes {
    static constexpr int A = (TYPE == 0 || TYPE == 1 || TYPE == 4) ? 2 : 1;  // activation planes (TAB_GEMM.cu:367-372)
    static constexpr int B = (TYPE == 0 || TYPE == 2 || TYPE == 4) ? 2 : 1;  // weight planes (TAB_GEMM.cu:374-379)
};

// One packed word (all planes) of one row of an operand, held in registers between the
// global load and the LDS store.  Memory order is [plane][half] as 64-bit words.
template <int PL> struct Item {
    uint32_t d[2 * PL];
};

// Buffer descriptor word 3 for untyped 32-bit data on this ISA generation.
constexpr int kBufferFlags = 0x00020000;

// Loads through a buffer descriptor: an offset at or past the descriptor's size returns zeros, so
// "this tap is padding", "this row is past M" and "this word is past the end of K" all become one
// offset select instead of a branch around the load.
template <int PL>
__device__ __forceinline__ Item<PL> load_item(__amdgpu_buffer_rsrc_t rsrc, uint32_t offset)
{
    Item<PL> it;
    if (PL == 2) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, offset, 0, 0);
        it.d[0] = v[0]; it.d[1] = v[1]; it.d[2] = v[2]; it.d[3] = v[3];
    } else {
        const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, offset, 0, 0);
        it.d[0] = v[0]; it.d[1] = v[1];
    }
    return it;
}

template <int PL, int ROWS, int Q>
__device__ __forceinline__ void store_item(uint32_t *lds, const Item<PL> &it, int word, int row)
{
#pragma unroll
    for (int pl = 0; pl < PL; pl++)
#pragma unroll
        for (int half = 0; half < 2; half++)
            lds[((pl * Q) + 2 * word + half) * ROWS + row] = it.d[pl * 2 + half];
}

constexpr int kStreamingStore = 2;  // cache policy of a buffer store: non-temporal (the nt bit)
constexpr uint32_t kNoData = 0xffffffffu;     // activation offset that is always out of range
constexpr uint32_t kNoFilter = 0x80000000u;   // weight offsets stay below this; adding it leaves the range

template <int TYPE, int BM, int BN, int KCH>
struct TileStager {
    static constexpr int APL = Planes<TYPE>::A, BPL = Planes<TYPE>::B;
    static constexpr int Q = 2 * KCH;  // 32-bit k-slices per chunk
    static constexpr int A_STRIDE = BM, B_STRIDE = BN;  // dwords between consecutive k-slices
    static constexpr int A_DWORDS = APL * Q * BM, B_DWORDS = BPL * Q * BN;
    static constexpr int A_STEP = kConvThreads / BM, B_STEP = kConvThreads / BN;  // words per pass over the rows
    static constexpr int A_ITEMS = (KCH + A_STEP - 1) / A_STEP, B_ITEMS = (KCH + B_STEP - 1) / B_STEP;
    static_assert(kConvThreads % BM == 0 && kConvThreads % BN == 0, "tile rows must divide the workgroup");

    // A: this thread fetches words (a_w0 + i*A_STEP) of output pixel m0 + a_row.  a_base is the
    // byte offset of input pixel (ih0, iw0) from the first image the tile touches, in wrapping
    // 32-bit arithmetic (the pixel itself may lie in the padding).
    __amdgpu_buffer_rsrc_t a_rsrc, b_rsrc;
    int a_row, a_w0, ih0, iw0;
    uint32_t a_base;
    // B: this thread fetches words (b_w0 + i*B_STEP) of filter n0 + b_row
    int b_row, b_w0;
    uint32_t b_base;
    Item<APL> a_reg[A_ITEMS];
    Item<BPL> b_reg[B_ITEMS];

    __device__ __forceinline__ void init(const ConvArgs &p, int tid, int m0, int n0)
    {
        a_row = tid % BM;
        // a wave shares its word index when the tile has at least 64 rows: the tap decode stays scalar
        a_w0 = BM >= 64 ? __builtin_amdgcn_readfirstlane(tid / BM) : tid / BM;
        const int pixels = p.OH * p.OW;
        const int n_first = (int)div32((uint32_t)m0, p.div_pixels);  // uniform
        const size_t image_words = (size_t)p.H * p.W * p.PC * APL;
        const size_t a_bytes = (size_t)(p.N - n_first) * image_words * 8;
        a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.qx + (size_t)n_first * image_words), 0,
                                                   a_bytes > 0xffffffffull ? (int)0xffffffffu : (int)a_bytes, kBufferFlags);
        const int a_m = m0 + a_row;
        const bool a_live = a_m < p.M;
        const int mm = a_live ? a_m : m0;
        const int n = (int)div32((uint32_t)mm, p.div_pixels);
        const int r = mm - n * pixels;
        const int oh = (int)div32((uint32_t)r, p.div_ow), ow = r - oh * p.OW;
        ih0 = a_live ? oh * p.s1 - p.p1 : -(1 << 30);  // a dead row fails every bounds check
        iw0 = ow * p.s2 - p.p2;
        a_base = (uint32_t)((((n - n_first) * p.H + (oh * p.s1 - p.p1)) * p.W + iw0) * p.PC) * (uint32_t)(APL * 8);

        b_row = tid % BN;
        b_w0 = BN >= 64 ? __builtin_amdgcn_readfirstlane(tid / BN) : tid / BN;
        const size_t filter_bytes = (size_t)p.G * BPL * 8;
        const size_t b_bytes = (size_t)(p.KN - n0) * filter_bytes;
        b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.qw + (size_t)n0 * p.G * BPL), 0,
                                                   b_bytes > kNoFilter ? (int)kNoFilter : (int)b_bytes, kBufferFlags);
        b_base = (n0 + b_row) < p.KN ? (uint32_t)b_row * (uint32_t)filter_bytes : kNoFilter;
    }

    // issue the global loads of one chunk into registers
    __device__ __forceinline__ void fetch(const ConvArgs &p, int chunk)
    {
        const int g0 = chunk * p.kcw;
#pragma unroll
        for (int i = 0; i < A_ITEMS; i++) {
            const int w = a_w0 + i * A_STEP;
            const int g = g0 + w;
            const uint32_t tap = fastdiv((uint32_t)g, p.div_pc);
            const int pc = g - (int)tap * p.PC;
            uint32_t kh = fastdiv(tap, p.div_kw);
            const int kw = (int)tap - (int)kh * p.KW;
            if (w >= p.kcw || g >= p.G) kh = 1u << 29;  // past the chunk or past K: no row is in range
            const uint32_t tap_off = (uint32_t)(((int)kh * p.W + kw) * p.PC + pc) * (uint32_t)(APL * 8);
            const bool ok = (unsigned)(ih0 + (int)kh) < (unsigned)p.H && (unsigned)(iw0 + kw) < (unsigned)p.W;
            a_reg[i] = load_item<APL>(a_rsrc, ok ? a_base + tap_off : kNoData);
        }
#pragma unroll
        for (int i = 0; i < B_ITEMS; i++) {
            const int w = b_w0 + i * B_STEP;
            const int g = g0 + w;
            // select, not add: two out-of-range markers added together would wrap back into the range
            const bool live = b_base != kNoFilter && w < p.kcw && g < p.G;
            b_reg[i] = load_item<BPL>(b_rsrc, live ? b_base + (uint32_t)g * (uint32_t)(BPL * 8) : kNoFilter);
        }
    }

    // write the fetched chunk to an LDS buffer of A_DWORDS + B_DWORDS dwords
    __device__ __forceinline__ void stage(uint32_t *buf) const
    {
        uint32_t *la = buf, *lb = buf + A_DWORDS;
#pragma unroll
        for (int i = 0; i < A_ITEMS; i++) {
            const int w = a_w0 + i * A_STEP;
            if (w < KCH) store_item<APL, BM, Q>(la, a_reg[i], w, a_row);
        }
#pragma unroll
        for (int i = 0; i < B_ITEMS; i++) {
            const int w = b_w0 + i * B_STEP;
            if (w < KCH) store_item<BPL, BN, Q>(lb, b_reg[i], w, b_row);
        }
    }
};

// Stager for the case where a chunk never leaves a filter tap (PC % KCH == 0, KCH even): the tap
// decode is one scalar computation per chunk, and threads fetch 16-byte pieces (two words of a
// one-plane operand, one word of a two-plane operand) with the pieces of a row on neighbouring
// lanes, so that one load instruction covers whole runs of the row's K-contiguous memory instead
// of 8 bytes from each of 64 rows.  LDS layout as in TileStager, but k-slices are ROWS + 8
// dwords apart so that the pieces of one store instruction fall into different banks.
template <int TYPE, int BM, int BN, int KCH>
struct TapStager {
    static constexpr int APL = Planes<TYPE>::A, BPL = Planes<TYPE>::B;
    static constexpr int Q = 2 * KCH;
    static constexpr int A_STRIDE = BM + 8, B_STRIDE = BN + 8;
    static constexpr int A_DWORDS = APL * Q * A_STRIDE, B_DWORDS = BPL * Q * B_STRIDE;
    static constexpr int PA = KCH * APL / 2, PB = KCH * BPL / 2;  // 16-byte pieces per row and chunk
    static constexpr int A_ITEMS = (BM * PA + kConvThreads - 1) / kConvThreads;
    static constexpr int B_ITEMS = (BN * PB + kConvThreads - 1) / kConvThreads;
    static_assert(KCH % 2 == 0, "pieces pair the words of one-plane operands");

    __amdgpu_buffer_rsrc_t a_rsrc, b_rsrc;
    int ih0[A_ITEMS], iw0[A_ITEMS];
    uint32_t a_base[A_ITEMS], b_base[B_ITEMS];  // byte offsets, piece included
    int a_lds[A_ITEMS], b_lds[B_ITEMS];         // dword index of the piece's first slice; < 0: no piece
    u32x4 a_reg[A_ITEMS], b_reg[B_ITEMS];

    template <int PL, int P, int STRIDE>
    static __device__ __forceinline__ int lds_index(int row, int piece)
    {
        // one-plane: piece = words 2*piece, 2*piece+1 -> slices 4*piece..; two-plane: piece = word
        return (PL == 1 ? 4 * piece : 2 * piece) * STRIDE + row;
    }

    __device__ __forceinline__ void init(const ConvArgs &p, int tid, int m0, int n0)
    {
        const int pixels = p.OH * p.OW;
        const int n_first = (int)div32((uint32_t)m0, p.div_pixels);  // uniform
        const size_t image_words = (size_t)p.H * p.W * p.PC * APL;
        const size_t a_bytes = (size_t)(p.N - n_first) * image_words * 8;
        a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.qx + (size_t)n_first * image_words), 0,
                                                   a_bytes > 0xffffffffull ? (int)0xffffffffu : (int)a_bytes, kBufferFlags);
#pragma unroll
        for (int i = 0; i < A_ITEMS; i++) {
            const int idx = tid + i * kConvThreads;
            const int row = idx / PA, piece = idx % PA;
            const int a_m = m0 + row;
            const bool live = row < BM && a_m < p.M;
            const int mm = live ? a_m : m0;
            const int n = (int)div32((uint32_t)mm, p.div_pixels);
            const int r = mm - n * pixels;
            const int oh = (int)div32((uint32_t)r, p.div_ow), ow = r - oh * p.OW;
            ih0[i] = live ? oh * p.s1 - p.p1 : -(1 << 30);  // a dead row fails every bounds check
            iw0[i] = ow * p.s2 - p.p2;
            a_base[i] = (uint32_t)((((n - n_first) * p.H + (oh * p.s1 - p.p1)) * p.W + iw0[i]) * p.PC) * (uint32_t)(APL * 8) +
                        (uint32_t)piece * 16u;
            a_lds[i] = row < BM ? lds_index<APL, PA, A_STRIDE>(row, piece) : -1;
        }
        const size_t filter_bytes = (size_t)p.G * BPL * 8;
        const size_t b_bytes = (size_t)(p.KN - n0) * filter_bytes;
        b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.qw + (size_t)n0 * p.G * BPL), 0,
                                                   b_bytes > kNoFilter ? (int)kNoFilter : (int)b_bytes, kBufferFlags);
#pragma unroll
        for (int i = 0; i < B_ITEMS; i++) {
            const int idx = tid + i * kConvThreads;
            const int row = idx / PB, piece = idx % PB;
            const bool live = row < BN && (n0 + row) < p.KN;
            b_base[i] = live ? (uint32_t)row * (uint32_t)filter_bytes + (uint32_t)piece * 16u : kNoFilter;
            b_lds[i] = row < BN ? lds_index<BPL, PB, B_STRIDE>(row, piece) : -1;
        }
    }

    __device__ __forceinline__ void fetch(const ConvArgs &p, int chunk)
    {
        const int g0 = chunk * KCH;  // first word of the chunk; the whole chunk lies in one tap
        const uint32_t tap = fastdiv((uint32_t)g0, p.div_pc);
        const int pc = g0 - (int)tap * p.PC;
        const int kh = (int)fastdiv(tap, p.div_kw);
        const int kw = (int)tap - kh * p.KW;
        const uint32_t tap_off = (uint32_t)((kh * p.W + kw) * p.PC + pc) * (uint32_t)(APL * 8);
#pragma unroll
        for (int i = 0; i < A_ITEMS; i++) {
            const bool ok = (unsigned)(ih0[i] + kh) < (unsigned)p.H && (unsigned)(iw0[i] + kw) < (unsigned)p.W;
            a_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, ok ? a_base[i] + tap_off : kNoData, 0, 0);
        }
        const uint32_t word_off = (uint32_t)g0 * (uint32_t)(BPL * 8);
#pragma unroll
        for (int i = 0; i < B_ITEMS; i++)
            b_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, b_base[i] + word_off, 0, 0);
    }

    template <int PL, int STRIDE>
    static __device__ __forceinline__ void store_piece(uint32_t *lds, int index, const u32x4 &v)
    {
        if (index < 0) return;
        if (PL == 1) {  // (word, half) = (0,0) (0,1) (1,0) (1,1): four consecutive slices
#pragma unroll
            for (int j = 0; j < 4; j++) lds[index + j * STRIDE] = v[j];
        } else {        // (plane, half): slices 2w, 2w+1 of plane 0, then of plane 1
#pragma unroll
            for (int j = 0; j < 4; j++) lds[index + ((j >> 1) * Q + (j & 1)) * STRIDE] = v[j];
        }
    }

    __device__ __forceinline__ void stage(uint32_t *buf) const
    {
#pragma unroll
        for (int i = 0; i < A_ITEMS; i++) store_piece<APL, A_STRIDE>(buf, a_lds[i], a_reg[i]);
#pragma unroll
        for (int i = 0; i < B_ITEMS; i++) store_piece<BPL, B_STRIDE>(buf + A_DWORDS, b_lds[i], b_reg[i]);
    }
};

}  // namespace tab
