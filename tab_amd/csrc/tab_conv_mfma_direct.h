// Matrix-core conv kernel whose operands go from global memory straight into LDS
// (buffer_load_dwordx4 ... lds): no staging registers, no LDS store instructions, and the next
// chunk streams in while the matrix cores work on the current one.
//
// A chunk is KCH consecutive words of K (KCH even, G % KCH == 0), moved as 16-byte granules: two words of
// a one-plane operand, one word (sign low/high, nonzero low/high) of a two-plane operand.  The two words
// of a one-plane activation granule must lie in one filter tap, so PC is even; a chunk may span taps
// (each wave instruction decodes the tap of its granules, one scalar computation).
// An LDS-direct load writes lane i's 16 bytes at base + 16*i, and a lane whose offset is out of
// range writes zeros (padding taps, rows past M, filters past KN).  The P granules of a row and chunk are
// taken in runs of RUN = 4, 2 or 1 (see granule_run): granule index = (run * ROWS + row) * RUN +
// column, so RUN neighbouring lanes fetch 16 * RUN contiguous bytes of one row and a wave instruction touches
// 64 / RUN cache lines, and column = (granule of the run + run_swizzle(row)) % RUN spreads the 16-byte reads of one
// granule of 16 consecutive rows over the LDS banks.  A run of an activation row must lie within one filter tap.
//
// Per pair of words p the half-waves take alternate words: lane (kb, r) owns word 2p + kb of row r and
// multiplies its low half in one MFMA and its high half in the next.  A one-plane operand reads its
// 8 bytes of the pair's granule (ds_read_b64), a two-plane operand the granule of its word
// (ds_read_b128); both operands follow the same (word, half) order, so any mix of plane counts agrees
// on k.
#pragma once
#include "tab_conv_mfma.h"

namespace tab {
namespace {

// 16 bytes per lane from a buffer straight into LDS: lane i's data lands at dst + 16*i (dst is
// wave-uniform), an out-of-range offset writes zeros.  In a function of its own because the cast to the
// LDS address space must not appear in the kernel's body, which the host pass also parses.
__device__ __forceinline__ void load16_to_lds(__amdgpu_buffer_rsrc_t rsrc, uint32_t *dst, uint32_t byte_offset)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void *)dst, 16, byte_offset, 0, 0, 0);
}

// Granules of a row and chunk fetched by neighbouring lanes.
// (Pairs of one-plane granules, read 8 bytes a lane, measured no faster than single ones.)
constexpr int granule_run(int per_row, int planes) { return per_row % 4 == 0 ? 4 : (per_row % 2 == 0 && planes == 2 ? 2 : 1); }

// Column rotation of a row (mod 16) in a run layout.  Reads of one granule by 16 consecutive rows must fall into 16
// different 16-byte bank groups, by 8 consecutive rows into 8 different ones: with RUN = 4 the rotation differs
// between rows r, r+4, r+8, r+12 and between the four row pairs of an aligned 8; with RUN = 2 between r and r+4
// within an aligned 8 and between r and r+8.
template <int RUN>
__device__ __forceinline__ int run_swizzle(int row)
{
    return RUN == 4 ? ((row >> 1) + (row >> 3)) & 3 : (RUN == 2 ? ((row >> 2) + (row >> 3)) & 1 : 0);
}

// LDS dwords one wave deposits per 32x32 tile when KS waves exchange partial sums: 16 accumulator elements a lane as four
// 16-byte quads, quad q of lane l at dword q * 256 + 4 * l (consecutive lanes 16 bytes apart: conflict-free 16-byte
// accesses), then one dword a lane for BTN's count of nonzero weight bits.
constexpr int kSplitTileDwords = 16 * 64 + 64;
constexpr int kSplitRoundTiles = 2;  // tiles a wave deposits per exchange round (34 KB of LDS for the four waves)

// PACKED: packed output (p.qy): the weights are the first MFMA operand and the epilogue packs inside a lane.
// KS > 1: K split inside the workgroup.  The workgroup's WM x WN x KS waves form KS groups that share one
// 32*WM*TM x 32*WN*TN tile of Y; all of them fetch every chunk together, wave group ks multiplies the pairs of words
// ks, ks + KS, ... of each chunk, and the partial sums meet in LDS after the loop (exact in any order: they are
// integers below 2^24).  A launch whose grid is a round or two of the chip lasts as long as one tile's serial K loop;
// this quarters (halves) that loop for the same tile, or lets a tile of a quarter (half) the size - four (two) times
// the workgroups to spread over the CUs - keep the large tile's ratio of operand expansions to MFMAs.  K need not be a
// multiple of the chunk: words past it are fetched as zeros (the BNN bias counts them).
// ARUN: granules of an activation row that neighbouring lanes fetch (0: the widest the chunk allows); a run must not
// straddle filter taps, so layers with few words per pixel take a shorter one.
template <int TYPE, int WM, int WN, int TM, int TN, int KCH, int KS>
constexpr int conv_mfma_direct_lds_dwords()
{
    constexpr int APL = Planes<TYPE>::A, BPL = Planes<TYPE>::B;
    constexpr int BM = 32 * WM * TM, BN = 32 * WN * TN;
    constexpr int A_ITEMS = (KCH * APL / 2 * BM + kConvThreads - 1) / kConvThreads, B_ITEMS = (KCH * BPL / 2 * BN + kConvThreads - 1) / kConvThreads;
    constexpr int buffers = 2 * 4 * (A_ITEMS + B_ITEMS) * kConvThreads;  // two chunks of whole wave instructions
    // partial sums of the KS wave groups: kSplitRoundTiles tiles per wave and round, then the packed epilogue's 32 dwords a wave
    constexpr int split = KS > 1 ? (kConvThreads / 64) * (kSplitRoundTiles * kSplitTileDwords + 32) : 0;
    return buffers > split ? buffers : split;
}

// One tile of Y, by the whole workgroup: tile (tile_m, tile_n) of the launch's BM x BN grid, operands through the
// workgroup's LDS `lds` (conv_mfma_direct_lds_dwords<...>() dwords); nchunks = ceil(G / KCH), from the host.
template <int TYPE, int WM, int WN, int TM, int TN, int KCH, bool PACKED, int KS, int ARUN>
__device__ __forceinline__ void conv_mfma_direct_tile(const ConvArgs &p, uint32_t *lds, int tile_m, int tile_n, int nchunks)
{
    static_assert(WM * WN * KS * 64 == kConvThreads && KCH % (2 * KS) == 0, "four waves, whole pairs of words per wave group");
    constexpr int PAIRS = KCH / 2;
    constexpr int PPW = PAIRS / KS;  // pairs of words a wave multiplies per chunk
    constexpr int APL = Planes<TYPE>::A, BPL = Planes<TYPE>::B;
    constexpr int BM = 32 * WM * TM, BN = 32 * WN * TN;
    constexpr int PA = KCH * APL / 2, PB = KCH * BPL / 2;  // granules per row and chunk
    constexpr int A_GRANULES = PA * BM, B_GRANULES = PB * BN;
    constexpr int A_ITEMS = (A_GRANULES + kConvThreads - 1) / kConvThreads, B_ITEMS = (B_GRANULES + kConvThreads - 1) / kConvThreads;
    constexpr int BUF_DWORDS = 4 * (A_ITEMS + B_ITEMS) * kConvThreads;  // whole wave instructions
    constexpr int A_RUN = ARUN ? ARUN : granule_run(PA, APL), B_RUN = granule_run(PB, BPL);
    static_assert(BM % 64 == 0 && BN % 64 == 0, "one wave instruction moves 64 / RUN rows of one run");
    static_assert(PA % A_RUN == 0, "whole runs");

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int r = lane & 31, kb = lane >> 5;
    const int ks = wave / (WM * WN), wsub = wave % (WM * WN);  // wave group along K, wave inside the group
    const int wm = wsub % WM, wn = wsub / WM;
    const int pixels = p.OH * p.OW;
    const size_t image_words = (size_t)p.H * p.W * p.PC * APL;
    const size_t filter_bytes = (size_t)p.G * BPL * 8;

    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // ---- what this lane fetches: granule idx = tid + i * 256 = (run * ROWS + row) * RUN + column ------
    int ih0[A_ITEMS], iw0[A_ITEMS];
    uint32_t a_base[A_ITEMS], b_base[B_ITEMS];
    int b_word[KS > 1 ? B_ITEMS : 1];  // KS > 1: first word of the lane's granule inside a chunk (words past K are zeros)
    const int n_first = (int)div32((uint32_t)m0, p.div_pixels);  // uniform
    const size_t a_bytes = (size_t)(p.N - n_first) * image_words * 8;
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.qx + (size_t)n_first * image_words), 0,
        a_bytes > 0xffffffffull ? (int)0xffffffffu : (int)a_bytes, kBufferFlags);
#pragma unroll
    for (int i = 0; i < A_ITEMS; i++) {
        const int idx = tid + i * kConvThreads;
        const int row = idx / A_RUN % BM;
        const int in_run = (idx % A_RUN - run_swizzle<A_RUN>(row & 15)) & (A_RUN - 1);
        const int granule = idx / A_RUN / BM * A_RUN + in_run;  // of the row's chunk
        const int a_m = m0 + row;
        const bool live = granule < PA && a_m < p.M;
        const int mm = live ? a_m : m0;
        const int n = (int)div32((uint32_t)mm, p.div_pixels);
        const int rem = mm - n * pixels;
        const int oh = (int)div32((uint32_t)rem, p.div_ow), ow = rem - oh * p.OW;
        ih0[i] = live ? oh * p.s1 - p.p1 : -(1 << 30);  // a dead granule fails every bounds check
        iw0[i] = ow * p.s2 - p.p2;
        a_base[i] = (uint32_t)((((n - n_first) * p.H + (oh * p.s1 - p.p1)) * p.W + iw0[i]) * p.PC) * (uint32_t)(APL * 8) +
                    (uint32_t)in_run * 16u;
    }
    const size_t b_bytes = (size_t)(p.KN - n0) * filter_bytes;
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(p.qw + (size_t)n0 * p.G * BPL), 0,
        b_bytes > kNoFilter ? (int)kNoFilter : (int)b_bytes, kBufferFlags);
#pragma unroll
    for (int i = 0; i < B_ITEMS; i++) {
        const int idx = tid + i * kConvThreads;
        const int row = idx / B_RUN % BN;
        const int granule = idx / B_RUN / BN * B_RUN + ((idx % B_RUN - run_swizzle<B_RUN>(row & 15)) & (B_RUN - 1));
        const bool live = granule < PB && (n0 + row) < p.KN;
        b_base[i] = live ? (uint32_t)row * (uint32_t)filter_bytes + (uint32_t)granule * 16u : kNoFilter;
        if (KS > 1) b_word[i] = granule * (BPL == 1 ? 2 : 1);
    }
    // chunk `chunk` into buf; !live_chunk: zeros (every offset out of range)
    auto fetch = [&](int chunk, uint32_t *buf, bool live_chunk) {
        const int g0 = chunk * KCH;  // first word of the chunk
#pragma unroll
        for (int i = 0; i < A_ITEMS; i++) {
            // the first word of the run this wave instruction moves and its tap: the same for all its rows
            const int g = g0 + (i * kConvThreads + wave * 64) / A_RUN / BM * A_RUN * (APL == 1 ? 2 : 1);
            const uint32_t tap = fastdiv((uint32_t)g, p.div_pc);
            const int pc = g - (int)tap * p.PC;
            const int kh = (int)fastdiv(tap, p.div_kw);
            const int kw = (int)tap - kh * p.KW;
            const uint32_t tap_off = (uint32_t)((kh * p.W + kw) * p.PC + pc) * (uint32_t)(APL * 8);
            // (KS > 1: the last chunk may reach past K; a run lies inside a tap, hence on one side of the end of K)
            const bool ok = live_chunk && (KS == 1 || g < p.G) && (unsigned)(ih0[i] + kh) < (unsigned)p.H && (unsigned)(iw0[i] + kw) < (unsigned)p.W;
            load16_to_lds(a_rsrc, buf + 4 * (i * kConvThreads + wave * 64), ok ? a_base[i] + tap_off : kNoData);
        }
        const uint32_t word_off = (uint32_t)g0 * (uint32_t)(BPL * 8);
#pragma unroll
        for (int i = 0; i < B_ITEMS; i++)
            load16_to_lds(b_rsrc, buf + 4 * ((A_ITEMS + i) * kConvThreads + wave * 64),
                          b_base[i] == kNoFilter || !live_chunk || (KS > 1 && g0 + b_word[i % (KS > 1 ? B_ITEMS : 1)] >= p.G)
                              ? kNoFilter : b_base[i] + word_off);
    };

    const ExpandConsts consts;
    f32x16 acc[TM][TN];
    int b_nonzero[TN];

    // dword offset of this lane's part of a pair of words: one-plane: 8 bytes of the pair's granule; two-plane:
    // the granule of its own word, 2 * pair + kb.  Tile and wave offsets are multiples of 32 rows, so the
    // column rotation is that of r.
    const int a_row = wm * (32 * TM) + r, b_row = wn * (32 * TN) + r;
    const int a_sw = run_swizzle<A_RUN>(r & 15), b_sw = run_swizzle<B_RUN>(r & 15);
    auto lane_part = [kb](int planes, int run, int rows, int row, int sw, int pair) {
        const int granule = planes == 1 ? pair : 2 * pair + kb;
        // granule / run and granule % run without dividing by what the compiler cannot see is 0 or 1
        const int group = run == 1 ? granule : (planes == 1 ? pair / run : 2 * pair / run);
        const int in_run = run == 1 ? 0 : (planes == 1 ? pair % run : 2 * pair % run + kb);
        return ((group * rows + row) * run + ((in_run + sw) & (run - 1))) * 4 + (planes == 1 ? 2 * kb : 0);
    };
    constexpr int B_REGION = 4 * A_ITEMS * kConvThreads;

    constexpr int HS = TYPE == 5 ? 1 : 2;  // MFMA steps per pair of words: one per half, type 5 both halves at once
    constexpr int STEPS = PPW * HS;
    // (with one expansion or more per MFMA the vector unit is the limit either way and the pinned order only costs)
    constexpr bool PIPELINED = TYPE != 5 && TM * TN >= 8;
    constexpr int NM = TM * TN, NE = TM + TN;
    uint32_t a_w[2][TM][2 * APL], b_w[2][TN][2 * BPL];  // [low half, high half] of every plane of the lane's word
    // the wave's pair j of a chunk (pair ks + KS * j of the chunk) into register set j & 1
    auto read_pair = [&](const uint32_t *buf, int j) {
        const int pair = KS == 1 ? j : ks + KS * j;
#pragma unroll
        for (int mt = 0; mt < TM; mt++) {
            const uint32_t *src = buf + lane_part(APL, A_RUN, BM, a_row, a_sw, pair) + mt * 32 * A_RUN * 4;
            if (APL == 1) {
                const u32x2 v = *reinterpret_cast<const u32x2 *>(src);
                a_w[j & 1][mt][0] = v[0]; a_w[j & 1][mt][1] = v[1];
            } else {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(src);
#pragma unroll
                for (int e = 0; e < 4; e++) a_w[j & 1][mt][e] = v[e];
            }
        }
#pragma unroll
        for (int nt = 0; nt < TN; nt++) {
            const uint32_t *src = buf + B_REGION + lane_part(BPL, B_RUN, BN, b_row, b_sw, pair) + nt * 32 * B_RUN * 4;
            if (BPL == 1) {
                const u32x2 v = *reinterpret_cast<const u32x2 *>(src);
                b_w[j & 1][nt][0] = v[0]; b_w[j & 1][nt][1] = v[1];
            } else {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(src);
#pragma unroll
                for (int e = 0; e < 4; e++) b_w[j & 1][nt][e] = v[e];
            }
        }
    };
    // Software pipeline over the MFMA steps (PIPELINED): while the matrix cores work on step s the vector unit expands
    // the operands of step s + 1 into the other set of operand registers, a few dwords after each MFMA (a wave issues in
    // order: expansions written in front of their own MFMAs leave the matrix pipe idle meanwhile).  The raw words of a
    // pair are read from LDS a step before their first expansion; those of the next chunk's first pair right after the
    // barrier, which therefore stands before the chunk's last step.  The order is pinned with scheduling barriers: left
    // alone, the scheduler sinks the LDS reads to their first use and the wave waits for LDS in the middle of the MFMAs.
    i32x8 af[2][PIPELINED ? TM : 1], bf[2][PIPELINED ? TN : 1];
    // piece q of a step's expansions: dword q % 4 of operand q / 4, the operands in the order the MFMAs need them:
    // A0, B0 .. B(TN-1), A1 .. A(TM-1).  (Indexing the whole expansion leaves the other three dwords to dead-code
    // elimination.)  Dword-sized pieces spread the vector work evenly over the MFMAs: whole operands of a ternary side
    // (10 instructions) outlast the MFMA they follow.
    // (the ternary expansion goes dword by dword with its pair words kept in between: indexing the whole expansion
    // would compute them once per piece)
    uint32_t pair_words[2];
    auto expand_piece = [&](int q, int pair, int h, int set) {
        const int e = q / 4, d = q % 4;
        if (e == 0 || e > TN) {
            const int mt = e == 0 ? 0 : e - TN;
            const uint32_t *w = a_w[pair & 1][mt];
            if constexpr (TYPE <= 2)
                af[set][mt][d] = APL == 2 ? ternary_dword(w[h], w[2 + h], d, pair_words, consts) : half_binary_dword(w[h], d, consts);
            else
                af[set][mt][d] = expand_operand<TYPE, 0>(w[h], w[2 * (APL - 1) + h], consts)[d];
        } else {
            const int nt = e - 1;
            const uint32_t *w = b_w[pair & 1][nt];
            if constexpr (TYPE <= 2)
                bf[set][nt][d] = BPL == 2 ? ternary_dword(w[h], w[2 + h], d, pair_words, consts) : half_binary_dword(w[h], d, consts);
            else
                bf[set][nt][d] = expand_operand<TYPE, 1>(w[h], w[2 * (BPL - 1) + h], consts)[d];
            if (TYPE == 2 && d == 0) b_nonzero[nt] += __builtin_popcount(w[2 + h]);  // (the zeros past the last chunk add nothing)
        }
    };
    if constexpr (PIPELINED) {
#pragma unroll
        for (int set = 0; set < 2; set++) {
#pragma unroll
            for (int mt = 0; mt < TM; mt++) af[set][mt] = i32x8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int nt = 0; nt < TN; nt++) bf[set][nt] = i32x8{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }

    const int wave_m0 = m0 + wm * (32 * TM), wave_n0 = n0 + wn * (32 * TN);
#pragma unroll
    for (int mt = 0; mt < TM; mt++)
#pragma unroll
        for (int nt = 0; nt < TN; nt++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[mt][nt][e] = 0.f;
#pragma unroll
    for (int nt = 0; nt < TN; nt++) b_nonzero[nt] = 0;
    fetch(0, lds, true);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if constexpr (PIPELINED) {
        read_pair(lds, 0);
#pragma unroll
        for (int q = 0; q < 4 * NE; q++) expand_piece(q, 0, 0, 0);
    }

    for (int chunk = 0; chunk < nchunks; chunk++) {
        const bool more = chunk + 1 < nchunks;
        const uint32_t *buf = lds + (chunk & 1) * BUF_DWORDS;
        uint32_t *next = lds + ((chunk + 1) & 1) * BUF_DWORDS;

        if constexpr (PIPELINED) {
            // past the last chunk: zeros, which the last step expands and nobody uses
            fetch(chunk + 1, next, more);
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                const int pair = s / 2, h = s % 2;
                const bool last = s == STEPS - 1;
                __builtin_amdgcn_sched_barrier(0);
                if (last) {
                    __builtin_amdgcn_s_waitcnt(0);  // this wave's part of the next chunk has landed
                    __syncthreads();
                    read_pair(next, 0);
                } else if (h == 0 && pair + 1 < PPW) {
                    read_pair(buf, pair + 1);
                }
                __builtin_amdgcn_sched_barrier(0);
                // the last step's expansions wait for the reads just issued: two MFMAs go first
                const int delay = last ? 2 : 0;
                const int per = (4 * NE + (NM - delay) - 1) / (NM - delay);  // pieces after each MFMA
                const int npair = last ? 0 : (s + 1) / 2, nh = (s + 1) % 2;
                int done = 0;
#pragma unroll
                for (int i = 0; i < NM; i++) {
                    const int mt = i / TN, nt = i % TN;
                    acc[mt][nt] = PACKED ? __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[s & 1][nt], af[s & 1][mt], acc[mt][nt], 4, 4, 0, 0, 0, 0)
                                         : __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[s & 1][mt], bf[s & 1][nt], acc[mt][nt], 4, 4, 0, 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    const int upto = i < delay ? 0 : ((i + 1 - delay) * per < 4 * NE ? (i + 1 - delay) * per : 4 * NE);
#pragma unroll
                    for (int q = 0; q < 4 * NE; q++)
                        if (q >= done && q < upto) expand_piece(q, npair, nh, (s + 1) & 1);
                    done = upto;
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        } else {
            if (more) fetch(chunk + 1, next, true);
            read_pair(buf, 0);
#pragma unroll
            for (int pair = 0; pair < PPW; pair++) {
                if (pair + 1 < PPW) read_pair(buf, pair + 1);
#pragma unroll
                for (int h = 0; h < HS; h++) {
                    i32x8 a_op[TM], b_op[TN];
#pragma unroll
                    for (int mt = 0; mt < TM; mt++) {
                        const uint32_t *w = a_w[pair & 1][mt];
                        a_op[mt] = TYPE == 5 ? expand_operand<TYPE, 0>(w[0], w[1], consts)
                                             : expand_operand<TYPE, 0>(w[h], w[2 * (APL - 1) + h], consts);
                    }
#pragma unroll
                    for (int nt = 0; nt < TN; nt++) {
                        const uint32_t *w = b_w[pair & 1][nt];
                        b_op[nt] = TYPE == 5 ? expand_operand<TYPE, 1>(w[0], w[1], consts)
                                             : expand_operand<TYPE, 1>(w[h], w[2 * (BPL - 1) + h], consts);
                        if (TYPE == 2) b_nonzero[nt] += __builtin_popcount(w[2 + h]);
                    }
#pragma unroll
                    for (int mt = 0; mt < TM; mt++)
#pragma unroll
                        for (int nt = 0; nt < TN; nt++)
                            acc[mt][nt] = PACKED ? __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b_op[nt], a_op[mt], acc[mt][nt], 4, 4, 0, 0, 0, 0)
                                             : __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a_op[mt], b_op[nt], acc[mt][nt], 4, 4, 0, 0, 0, 0);
                }
            }
            // keep the wait at the end of the chunk's MFMAs (the scheduler would hoist it above them, since
            // only memory operations order it): the next chunk's loads have a whole chunk of work to land in
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0);  // this wave's part of the next chunk has landed
            __syncthreads();
        }
    }
    scale_ternary_sums<TYPE>(acc);
    if constexpr (KS > 1) {
        // The KS groups hold partial sums of the same tiles.  Rounds of kSplitRoundTiles tiles: every wave deposits its
        // part of the round's tiles (and BTN's partial count of nonzero weight bits), the wave group (round's tile) % KS
        // of each wave position adds the KS parts of one tile and finishes it like a wave that owned it alone.
        constexpr int NT = TM * TN, RT = kSplitRoundTiles;
        static_assert(NT % RT == 0, "whole rounds");
        float *parts = reinterpret_cast<float *>(lds);
        uint32_t *exchange = lds + (kConvThreads / 64) * RT * kSplitTileDwords + wave * 32;
        __syncthreads();  // the operand buffers are free: every wave has read its last pair
#pragma unroll
        for (int round = 0; round < NT / RT; round++) {
#pragma unroll
            for (int i = 0; i < RT; i++) {
                const int t = round * RT + i, mt = t / TN, nt = t % TN;
                float *dst = parts + (wave * RT + i) * kSplitTileDwords;
#pragma unroll
                for (int q = 0; q < 4; q++)
                    *reinterpret_cast<f32x4 *>(dst + q * 256 + lane * 4) =
                        f32x4{acc[mt][nt][4 * q], acc[mt][nt][4 * q + 1], acc[mt][nt][4 * q + 2], acc[mt][nt][4 * q + 3]};
                if (TYPE == 2) dst[16 * 64 + lane] = __int_as_float(b_nonzero[nt]);
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < RT; i++) {
                const int t = round * RT + i, mt = t / TN, nt = t % TN;
                if (ks != t % KS) continue;  // wave-uniform
                f32x16 sum[1][1];
                int nonzero[1] = {0};
#pragma unroll
                for (int e = 0; e < 16; e++) sum[0][0][e] = 0.f;
#pragma unroll
                for (int k = 0; k < KS; k++) {
                    const float *src = parts + ((k * (WM * WN) + wsub) * RT + i) * kSplitTileDwords;
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const f32x4 v = *reinterpret_cast<const f32x4 *>(src + q * 256 + lane * 4);
#pragma unroll
                        for (int e = 0; e < 4; e++) sum[0][0][4 * q + e] += v[e];
                    }
                    if (TYPE == 2) nonzero[0] += __float_as_int(src[16 * 64 + lane]);
                }
                if constexpr (PACKED)
                    conv_mfma_epilogue_packed<TYPE, 1, 1, KCH>(p, sum, nonzero, wave_m0 + mt * 32, wave_n0 + nt * 32, lane, exchange, nchunks * KCH);
                else
                    conv_mfma_epilogue<TYPE, 1, 1, KCH, 1>(p, sum, nonzero, wave_m0 + mt * 32, wave_n0 + nt * 32, lane, 0, nullptr, nchunks * KCH);
            }
            if (round + 1 < NT / RT) __syncthreads();  // the parts are read before the next round overwrites them
        }
    } else if constexpr (PACKED) {
        // BTN hands its biases round through LDS: not before every wave has read its last operands (the pipelined
        // loop reads the zeros past the last chunk after the chunk's barrier and counts their nonzero weights)
        if (TYPE == 2) __syncthreads();
        conv_mfma_epilogue_packed<TYPE, TM, TN, KCH>(p, acc, b_nonzero, wave_m0, wave_n0, lane, lds + wave * (32 * TN), nchunks * KCH);
    } else {
        conv_mfma_epilogue<TYPE, TM, TN, KCH, 1>(p, acc, b_nonzero, wave_m0, wave_n0, lane, 0, nullptr, nchunks * KCH);
    }
}

template <int TYPE, int WM, int WN, int TM, int TN, int KCH, bool PACKED, int KS = 1, int ARUN = 0>
__global__ __launch_bounds__(kConvThreads)
__attribute__((amdgpu_waves_per_eu(mfma_waves_per_eu(KS > 1 ? 1 : WM, TM, TN, 4 * conv_mfma_direct_lds_dwords<TYPE, WM, WN, TM, TN, KCH, KS>())))) void conv_mfma_direct(const ConvArgs p)
{
    __shared__ __attribute__((aligned(16))) uint32_t lds[conv_mfma_direct_lds_dwords<TYPE, WM, WN, TM, TN, KCH, KS>()];
    int tile_m, tile_n;
    if (!tile_of_workgroup(p, tile_m, tile_n)) return;
    conv_mfma_direct_tile<TYPE, WM, WN, TM, TN, KCH, PACKED, KS, ARUN>(p, lds, tile_m, tile_n, p.nchunks);
}

// Mixed launch for grids of a few rounds of the chip: a launch lasts as long as its busiest CU, and with T tiles on C CUs that
// is ceil(T / C) tiles although the mean is T / C (392 tiles of 128x128 on 256 CUs: two against 1.53; 784: four against 3.06).
// Here the first floor(T / C) * C workgroups take whole 128x128 tiles (four MFMA tiles a wave, chunks of KCH words as the plain
// 128x128 launch would take them) and the remaining tiles are cut into four 64x64 quarters each, run by the split-K body (the
// large tile's ratio of expansions to MFMAs): the last, partial round is dealt out in quarters, so the busiest CU carries at
// most a quarter tile more than the others.  Workgroups are dispatched in index order, whole tiles first.  Needs an even
// number of words per pixel.
// TNB = 4: the whole tiles are 128x256 (eight MFMA tiles a wave, the pipelined loop, two workgroups a CU) and a remaining tile
// makes eight quarters.
template <int TYPE, int KCH, int ARUN, bool PACKED, int TNB = 2>
__global__ __launch_bounds__(kConvThreads) __attribute__((amdgpu_waves_per_eu(TNB == 4 ? 2 : 4))) void conv_mfma_tail(const ConvArgs p)
{
    constexpr int BIG = conv_mfma_direct_lds_dwords<TYPE, 2, 2, 2, TNB, KCH, 1>(), SMALL = conv_mfma_direct_lds_dwords<TYPE, 1, 1, 2, 2, 8, 4>();
    __shared__ __attribute__((aligned(16))) uint32_t lds[BIG > SMALL ? BIG : SMALL];
    const uint32_t b = blockIdx.x;
    if (b < (uint32_t)p.tail_big) {  // uniform over the workgroup
        // XCD-aware order over the whole tiles, as in tile_of_workgroup
        const uint32_t logical = b < 8u * (uint32_t)p.xcd_share ? (b & 7u) * (uint32_t)p.xcd_share + (b >> 3) : b;
        const int tile_m = (int)div32(logical, p.div_filter_tiles);
        conv_mfma_direct_tile<TYPE, 2, 2, 2, TNB, KCH, PACKED, 1, 0>(p, lds, tile_m, (int)logical - tile_m * p.filter_tiles, p.nchunks);
    } else {
        constexpr uint32_t PIECES = 2 * TNB;  // 64x64 quarters of a whole tile
        const uint32_t j = b - (uint32_t)p.tail_big, t = (uint32_t)p.tail_big + j / PIECES, q = j % PIECES;
        const int big_m = (int)div32(t, p.div_filter_tiles), big_n = (int)t - big_m * p.filter_tiles;
        const int tile_m = 2 * big_m + (int)(q & 1u), tile_n = TNB * big_n + (int)(q >> 1);
        if (tile_m * 64 >= p.M || tile_n * 64 >= p.KN) return;  // a quarter wholly past the edge of Y
        conv_mfma_direct_tile<TYPE, 1, 1, 2, 2, 8, PACKED, 4, ARUN>(p, lds, tile_m, tile_n, p.tail_chunks);
    }
}

template <int TYPE, int KCH, int ARUN, int TNB = 2>
hipError_t launch_mfma_tail_run(ConvArgs a, long blocks, hipStream_t stream)
{
    a.kcw = KCH;
    a.nchunks = a.G / KCH;
    a.tail_chunks = (a.G + 7) / 8;  // the quarters' chunks of eight words, the last one padded with zeros
    if (a.qy != nullptr) {
        conv_mfma_tail<TYPE, KCH, ARUN, true, TNB><<<dim3((unsigned)blocks), dim3(kConvThreads), 0, stream>>>(a);
    } else {
        conv_mfma_tail<TYPE, KCH, ARUN, false, TNB><<<dim3((unsigned)blocks), dim3(kConvThreads), 0, stream>>>(a);
    }
    return hipGetLastError();
}

// False when the layer does not fit the mixed launch (an odd number of words per pixel).
inline bool mfma_tail_supported(const ConvArgs &a) { return a.PC % 2 == 0; }

// Whole tiles of 128x256 (words per pixel in fours).
template <int TYPE>
hipError_t launch_mfma_tail_wide(ConvArgs a, hipStream_t stream)
{
    if (a.PC % 4 != 0) return hipErrorInvalidValue;
    const long filter_tiles = (a.KN + 255) / 256, tiles = (long)((a.M + 127) / 128) * filter_tiles;
    const long round = tail_round();
    const long whole = tiles / round * round;
    const long blocks = whole + 8 * (tiles - whole);
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    a.tiles_m = (a.M + 127) / 128;
    a.tiles_n = 0;
    a.tail_big = (int)whole;
    a.filter_tiles = (int)filter_tiles;
    a.div_filter_tiles = make_div32((uint32_t)filter_tiles);
    a.xcd_share = whole >= 64 ? (int)(whole / 8) : 0;
    if (a.PC * Planes<TYPE>::A / 2 % 4 == 0) return launch_mfma_tail_run<TYPE, 4, 4, 4>(a, blocks, stream);
    return launch_mfma_tail_run<TYPE, 4, 2, 4>(a, blocks, stream);
}

template <int TYPE>
hipError_t launch_mfma_tail(ConvArgs a, hipStream_t stream)
{
    if (!mfma_tail_supported(a)) return hipErrorInvalidValue;
    const long filter_tiles = (a.KN + 127) / 128, tiles = (long)((a.M + 127) / 128) * filter_tiles;
    const long round = tail_round();
    const long whole = tiles / round * round;
    const long blocks = whole + 4 * (tiles - whole);
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    a.tiles_m = (a.M + 127) / 128;
    a.tiles_n = 0;
    a.tail_big = (int)whole;
    a.filter_tiles = (int)filter_tiles;
    a.div_filter_tiles = make_div32((uint32_t)filter_tiles);
    a.xcd_share = whole >= 64 ? (int)(whole / 8) : 0;
    // The whole tiles' chunk as the plain 128x128 launch picks it (launch_mfma_shape): four words inside a tap, else six words
    // across taps for the operand pairs that leave LDS for four workgroups a CU, else two.  The quarters' run of activation
    // granules from the granules of a pixel, as launch_mfma_split picks it.
    constexpr int APL = Planes<TYPE>::A;
    const int granules_per_pixel = a.PC * APL / 2;
    if (a.PC % 4 == 0) {
        if (granules_per_pixel % 4 == 0) return launch_mfma_tail_run<TYPE, 4, 4>(a, blocks, stream);
        return launch_mfma_tail_run<TYPE, 4, 2>(a, blocks, stream);
    }
    if constexpr (APL + Planes<TYPE>::B <= 3) {
        if (a.G % 6 == 0) {
            if constexpr (APL == 2) return launch_mfma_tail_run<TYPE, 6, 2>(a, blocks, stream);
            return launch_mfma_tail_run<TYPE, 6, 1>(a, blocks, stream);
        }
    }
    if constexpr (APL == 2) return launch_mfma_tail_run<TYPE, 2, 2>(a, blocks, stream);
    return launch_mfma_tail_run<TYPE, 2, 1>(a, blocks, stream);
}

template <int TYPE, int WM, int WN, int TM, int TN, int KCH, int KS, int ARUN>
hipError_t launch_mfma_direct(ConvArgs a, hipStream_t stream)
{
    constexpr int BM = 32 * WM * TM, BN = 32 * WN * TN;
    // words of a run of activation granules, which must not straddle filter taps
    constexpr int A_RUN_WORDS = (ARUN ? ARUN : granule_run(KCH * Planes<TYPE>::A / 2, Planes<TYPE>::A)) * (Planes<TYPE>::A == 1 ? 2 : 1);
    if ((KS == 1 && a.G % KCH != 0) || a.PC % A_RUN_WORDS != 0) return hipErrorInvalidValue;
    a.kcw = KCH;
    a.nchunks = (a.G + KCH - 1) / KCH;  // the split-K kernels fetch the words past K as zeros
    a.tiles_m = (a.M + BM - 1) / BM;
    const long blocks = order_workgroups<Planes<TYPE>::A>(a, (a.KN + BN - 1) / BN);
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    if (a.qy != nullptr) {
        conv_mfma_direct<TYPE, WM, WN, TM, TN, KCH, true, KS, ARUN><<<dim3((unsigned)blocks), dim3(kConvThreads), 0, stream>>>(a);
    } else {
        conv_mfma_direct<TYPE, WM, WN, TM, TN, KCH, false, KS, ARUN><<<dim3((unsigned)blocks), dim3(kConvThreads), 0, stream>>>(a);
    }
    return hipGetLastError();
}

// Split-K launch: chunk length and run of activation granules from the layer's words per pixel.  WORDS = words every
// wave group multiplies per chunk.  False (nothing launched) when the layer's words per pixel fit no run.
template <int TYPE, int WM, int WN, int TM, int TN, int KS, int WORDS>
hipError_t launch_mfma_split(const ConvArgs &a, hipStream_t stream)
{
    constexpr int APL = Planes<TYPE>::A;
    constexpr int KCH = KS * WORDS;
    constexpr int PA = KCH * APL / 2;
    // granules of 16 bytes: two words of a one-plane activation, one word of a two-plane one
    const int granules_per_pixel = a.PC * APL / 2;  // PC is even here
    if (a.PC % 2 != 0) return hipErrorInvalidValue;
    if constexpr (PA % 4 == 0)
        if (granules_per_pixel % 4 == 0) return launch_mfma_direct<TYPE, WM, WN, TM, TN, KCH, KS, 4>(a, stream);
    if constexpr (PA % 2 == 0)
        if (granules_per_pixel % 2 == 0) return launch_mfma_direct<TYPE, WM, WN, TM, TN, KCH, KS, 2>(a, stream);
    return launch_mfma_direct<TYPE, WM, WN, TM, TN, KCH, KS, 1>(a, stream);
}

}  // namespace
}  // namespace tab

#include "tab_conv_mfma_regs.h"
