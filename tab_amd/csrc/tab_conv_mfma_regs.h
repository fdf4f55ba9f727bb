// Matrix-core conv kernel for short K (at most nine packed words per plane: 64 channels under 3x3 taps, 1x1 layers
// on up to 512 channels), where the tiled kernels spend as long on a tile's prologue and epilogue as on its MFMAs.
//
// No LDS and no workgroup barrier: every wave works alone.
//   * The weights of the wave's 32*TN filters, all G words of K, are expanded to FP4 once and stay in registers
//     (4*G*TN of them) for the life of the wave.
//   * Lane (kb, r) feeds the 32-bit half kb of output pixel r and loads exactly that dword itself, straight from
//     global memory through a buffer descriptor (padding taps and pixels past M are an offset select that reads
//     zeros).  Consecutive output pixels of a stride-1 layer are consecutive packed pixels, so one wave load covers
//     a contiguous run of the activation.  A two-plane activation is loaded eight bytes a lane (the lower half-wave
//     the sign plane, the upper one the nonzero plane of the same pixels: 512 contiguous bytes an instruction) and
//     one v_permlane32_swap hands each half-wave the halves it multiplies.
//   * fp32 output: activations are the row operand of the MFMA, so accumulator element 4j+i of lane (kb, r) is pixel
//     8j+4kb+i, filter r, and a store instruction writes 128 contiguous bytes of two rows of Y (stores of 16 bytes a
//     lane from the transposed product touch 32 bytes of every row and ran a fifth slower on the same bytes).
//   * Packed output: weights are the row operand, element 4j+i is filter 8j+4kb+i of pixel r, so a lane thresholds
//     16 bits of its own pixel's word per filter tile and one cross-half exchange completes them: no ballot and no
//     lane broadcast per accumulator element.
//   * A wave walks its tiles of 32 output pixels in a loop (tile, tile + waves, ...) and issues the loads of its next
//     tile before the MFMAs of the current one; the stores of a tile drain while the next tile is computed.
//
// Measured on MI355X (N=256, 56x56x64 -> 64, 3x3): packed output 24 us against 38 us for the tiled kernel (BNN; TNN 26
// against 42); fp32 output 37 us against 36 us: both kernels then write Y's 205 MB at 5.5 TB/s, where a plain fill of
// the same bytes reaches 6.8 TB/s, so the launcher uses this kernel for packed output only.
#pragma once
#include "tab_conv_mfma.h"

#include <atomic>

namespace tab {
namespace {

constexpr int kRegsMaxWords = 9;  // longest K (words per plane) the register-resident kernel takes

// What a wave writes.  One kernel per mode, so that the tile loop is straight-line code: a branch inside it whose sides
// issue different numbers of stores makes the compiler's wait for the next tile's loads cover this tile's stores too.
enum RegsOut {
    kOutRows = 0,    // fp32, every filter of the wave's tiles exists
    kOutFloat = 1,   // fp32, ragged KN: filters past KN dropped by an offset select
    kOutBits1 = 2,   // thresholded and packed, one plane (p.qy, p.out_bits == 1)
    kOutBits2 = 3    // thresholded and packed, two planes
};

// G: words of K per plane (runtime p.G <= G; missing words are zero on both sides), TN: 32-filter tiles per wave.
template <int TYPE, int G, int TN, int OUT>
__global__ __launch_bounds__(kConvThreads) __attribute__((amdgpu_waves_per_eu(2, 3))) void conv_mfma_regs(const ConvArgs p)
{
    constexpr int APL = Planes<TYPE>::A, BPL = Planes<TYPE>::B;
    static_assert(TYPE >= 0 && TYPE <= 3, "types 0..3");
    constexpr bool PACKED = OUT == kOutBits1 || OUT == kOutBits2;
    static_assert(!PACKED || TN % 2 == 0, "packed output writes whole 64-filter words");
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 31, kb = lane >> 5;
    const int n0 = blockIdx.y * (32 * TN);
    const ExpandConsts consts;

    // ---- activation addressing ------------------------------------------------------------------------------
    // Offsets are taken from the image's pixel (-p1, -p2), so that the offset of an output pixel's window origin is
    // never negative and the tap offset can ride in the scalar offset of the load, outside the range check; taps in
    // the padding are never issued (their offset is replaced by one that is out of range and reads zeros).
    const int pixels = p.OH * p.OW;
    const uint32_t pixel_bytes = (uint32_t)p.PC * (APL * 8);
    const size_t image_bytes = (size_t)p.H * p.W * pixel_bytes;
    const size_t lead_bytes = ((size_t)p.p1 * p.W + p.p2) * pixel_bytes;
    uint32_t tap_off[G];
    int tap_kh[G], tap_kw[G];
#pragma unroll
    for (int w = 0; w < G; w++) {
        const uint32_t tap = fastdiv((uint32_t)w, p.div_pc);
        const int pc = w - (int)tap * p.PC;
        tap_kh[w] = (int)fastdiv(tap, p.div_kw);
        tap_kw[w] = (int)tap - tap_kh[w] * p.KW;
        tap_off[w] = (uint32_t)((tap_kh[w] * p.W + tap_kw[w]) * p.PC + pc) * (uint32_t)(APL * 8);
        if (w >= p.G) tap_kh[w] = 1 << 29;  // a word past K: no row is in range
    }
    const int tiles = (p.M + 31) >> 5;
    const int waves = (int)gridDim.x * (kConvThreads / 64);

    // two tiles of activation in registers: the one being multiplied and the next one in flight (a second tile in
    // flight measured no faster and cost a wave per SIMD in registers)
    uint32_t buf0[G][APL], buf1[G][APL];
    float th0 = 0.f, th1 = 0.f;  // packed output: threshold of the lane's pixel, requested with the tile's loads
    auto load_tile = [&](int tile_index, uint32_t (&dst)[G][APL], float &th) {
        const int tile = __builtin_amdgcn_readfirstlane(tile_index);  // the same for the whole wave: descriptors stay scalar
        const int m_first = tile < tiles ? tile * 32 : 0;
        const int n_first = (int)div32((uint32_t)m_first, p.div_pixels);  // uniform
        const size_t bytes = (size_t)(p.N - n_first) * image_bytes + lead_bytes;
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(reinterpret_cast<const char *>(p.qx) + (size_t)n_first * image_bytes - lead_bytes), 0,
            bytes > 0xfffffff0ull ? (int)0xfffffff0u : (int)bytes, kBufferFlags);
        const int m = m_first + r;
        const bool live = tile < tiles && m < p.M;
        const int mm = live ? m : m_first;
        const int n = (int)div32((uint32_t)mm, p.div_pixels);
        const int rem = mm - n * pixels;
        const int oh = (int)div32((uint32_t)rem, p.div_ow), ow = rem - oh * p.OW;
        const int ih0 = live ? oh * p.s1 - p.p1 : -(1 << 30);  // a dead pixel fails every range check
        const int iw0 = ow * p.s2 - p.p2;
        // one plane: the lane's half of the word; two planes: all of plane kb, exchanged after the wait (use_tile)
        const uint32_t base = (uint32_t)((((n - n_first) * p.H + oh * p.s1) * p.W + ow * p.s2)) * pixel_bytes + (uint32_t)kb * (APL * 4u);
#pragma unroll
        for (int w = 0; w < G; w++) {
            const bool ok = (unsigned)(ih0 + tap_kh[w]) < (unsigned)p.H && (unsigned)(iw0 + tap_kw[w]) < (unsigned)p.W;
            const uint32_t off = ok ? base : kNoData;
            if (APL == 1) {
                dst[w][0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off, tap_off[w], 0);
            } else {
                const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, off, tap_off[w], 0);
                dst[w][0] = v[0];
                dst[w][APL - 1] = v[1];
            }
        }
        if (PACKED) th = p.out_ths[n];
    };

    // the first tile's activation is requested before the weights, so that both are in flight together
    int tile = (int)blockIdx.x * (kConvThreads / 64) + wave;
    if (tile >= tiles) return;
    load_tile(tile, buf0, th0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- weights: filter n0 + 32*nt + r, half kb of every word, expanded once ---------------------------------
    // one plane: the lane's half of each word; two planes: the lower half-wave fetches the sign plane, the upper one the
    // nonzero plane, and a swap gives every lane (sign half kb, nonzero half kb)
    const uint32_t *qw32 = reinterpret_cast<const uint32_t *>(p.qw);
    int wq[G][TN][4];
    int nonzero[TN];  // BTN: bits set in the nonzero plane of this lane's half of filter r of tile nt
    {
        uint32_t raw[G][TN][BPL];
#pragma unroll
        for (int nt = 0; nt < TN; nt++) {
            int f = n0 + nt * 32 + r;
            f = f < p.KN ? f : p.KN - 1;  // filters past KN repeat the last one and are never stored
#pragma unroll
            for (int w = 0; w < G; w++) {
                const int ww = w < p.G ? w : p.G - 1;  // words past K are read somewhere valid and zeroed below
                const size_t word = ((size_t)f * p.G + ww) * BPL;
                if (BPL == 1) {
                    raw[w][nt][0] = qw32[word * 2 + kb];
                } else {
                    const u32x2 v = *reinterpret_cast<const u32x2 *>(qw32 + (word + kb) * 2);
                    raw[w][nt][0] = v[0];
                    raw[w][nt][BPL - 1] = v[1];
                }
            }
        }
#pragma unroll
        for (int nt = 0; nt < TN; nt++) {
            nonzero[nt] = 0;
#pragma unroll
            for (int w = 0; w < G; w++) {
                uint32_t p0 = raw[w][nt][0], p1 = raw[w][nt][BPL - 1];
                if (BPL == 2) {
                    const u32x2 sw = __builtin_amdgcn_permlane32_swap(p0, p1, false, false);
                    p0 = sw[0];
                    p1 = sw[1];
                }
                if (w >= p.G) p0 = p1 = 0u;
                if (TYPE == 2) nonzero[nt] += __builtin_popcount(p1);
                const i32x8 e = expand_operand<TYPE, 1>(p0, p1, consts);
#pragma unroll
                for (int d = 0; d < 4; d++) wq[w][nt][d] = e[d];
            }
        }
    }
    // What every accumulator starts from: BTN btn[f] - popcount(b1 of f), BNN NUM - 64 per word (TAB_GEMM.cu:116, 144).
    // SWAP (packed output): element 4j+i of tile nt belongs to filter 8j+4kb+i; else to filter r.
    constexpr bool SWAP = PACKED;
    float bias[TN][SWAP ? 16 : 1];
#pragma unroll
    for (int nt = 0; nt < TN; nt++) {
        float of_r = TYPE == 3 ? (float)(p.num - 64 * G) : 0.f;  // of filter n0 + 32*nt + r
        if (TYPE == 2) {
            const int f = n0 + nt * 32 + r;
            const int total = nonzero[nt] + __shfl_xor(nonzero[nt], 32, 64);
            of_r = (float)((f < p.KN ? p.btn[f] : 0) - total);
        }
        if (SWAP) {
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int i = 0; i < 4; i++) bias[nt][(4 * j + i) % (SWAP ? 16 : 1)] = TYPE == 2 ? __shfl(of_r, 8 * j + 4 * kb + i, 64) : of_r;
        } else {
            bias[nt][0] = of_r;
        }
    }
    // filters of tile nt that exist, as a mask over the bits of a packed half-word
    uint32_t live_cols[TN];
#pragma unroll
    for (int nt = 0; nt < TN; nt++) {
        const int left = p.KN - (n0 + nt * 32);
        live_cols[nt] = left >= 32 ? 0xffffffffu : (left <= 0 ? 0u : (1u << left) - 1u);
    }
    const int out_words = (p.KN + 63) >> 6;
    // fp32 output: byte offset of this lane's filter in each of the 16 rows of Y its accumulator elements belong to,
    // from the tile's first row; the same for every tile
    const uint32_t y_row_bytes = (uint32_t)p.KN * 4u;
    uint32_t y_off[SWAP ? 1 : 16];
    if (!SWAP) {
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) y_off[(4 * j + i) % (SWAP ? 1 : 16)] = (uint32_t)(8 * j + 4 * kb + i) * y_row_bytes + (uint32_t)(n0 + r) * 4u;
    }

    // One tile: multiply the activation in `use` and store.  No branch inside, so every tile issues the same number of
    // memory operations and the compiler's wait for a tile's loads leaves the stores of the tiles before it in flight.
    auto run_tile = [&](int tile_index, const uint32_t (&cur)[G][APL], float th_cur) {
        const int tile = __builtin_amdgcn_readfirstlane(tile_index);
        f32x16 acc[TN];
#pragma unroll
        for (int nt = 0; nt < TN; nt++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[nt][e] = bias[nt][e % (SWAP ? 16 : 1)];
#pragma unroll
        for (int w = 0; w < G; w++) {
            uint32_t p0 = cur[w][0], p1 = cur[w][APL - 1];
            if (APL == 2) {
                const u32x2 sw = __builtin_amdgcn_permlane32_swap(p0, p1, false, false);
                p0 = sw[0];
                p1 = sw[1];
            }
            const i32x8 af = expand_operand<TYPE, 0>(p0, p1, consts);
#pragma unroll
            for (int nt = 0; nt < TN; nt++) {
                const i32x8 wf = {wq[w][nt][0], wq[w][nt][1], wq[w][nt][2], wq[w][nt][3], 0, 0, 0, 0};
                acc[nt] = SWAP ? __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf, af, acc[nt], 4, 4, 0, 0, 0, 0)
                               : __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af, wf, acc[nt], 4, 4, 0, 0, 0, 0);
            }
        }
        if (TYPE == 0) {  // both operands are +-2: four times the sums
#pragma unroll
            for (int nt = 0; nt < TN; nt++) acc[nt] *= 0.25f;
        }
        // Every store goes through a buffer descriptor that ends with the tile's last live row, so pixels past M
        // (and, by an offset select, filters past KN) are dropped by the range check instead of branched round: with
        // no branch in the loop every iteration issues the same number of memory operations, and the wait for the
        // next tile's loads can let all of this tile's stores stay in flight.
        const int m_first = tile * 32;
        const int rows_left = p.M - m_first < 32 ? p.M - m_first : 32;
        if (PACKED) {
            // The values of pixel m are thresholded exactly as the quantizer would threshold them as the next
            // layer's NHWC activation (TAB_GEMM.cu:184-192, 231); this lane holds filters 8j+4kb+i of every tile,
            // the other half-wave's lane of the same pixel the rest of each 32-bit half.
            const float th = th_cur;
            uint32_t sign_half[TN], nz_half[TN];
#pragma unroll
            for (int nt = 0; nt < TN; nt++) {
                uint32_t sg = 0, nz = 0;
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float v = acc[nt][4 * j + i];
                        const uint32_t bit = 1u << (8 * j + i);  // shifted by 4*kb below
                        if (OUT == kOutBits1) {
                            sg |= v < th ? bit : 0u;
                        } else {
                            const bool pos = v > th, neg = !pos && v < -th;
                            sg |= neg ? bit : 0u;
                            nz |= (pos || neg) ? bit : 0u;
                        }
                    }
                sg <<= 4 * kb;
                nz <<= 4 * kb;
                sign_half[nt] = (sg | (uint32_t)__shfl_xor((int)sg, 32, 64)) & live_cols[nt];
                if (OUT == kOutBits2) nz_half[nt] = (nz | (uint32_t)__shfl_xor((int)nz, 32, 64)) & live_cols[nt];
            }
            constexpr uint32_t element = OUT == kOutBits1 ? 8u : 16u;
            const uint32_t row_bytes = (uint32_t)out_words * element;
            const __amdgpu_buffer_rsrc_t out = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(reinterpret_cast<char *>(p.qy) + (size_t)m_first * row_bytes), 0, (int)((uint32_t)rows_left * row_bytes), kBufferFlags);
            // n0 is a multiple of 64: tiles 2t, 2t+1 are the halves of word n0/64 + t; the lower half-wave stores
#pragma unroll
            for (int t = 0; t < TN / 2; t++) {
                const int word = (n0 >> 6) + t;
                const uint32_t off = (kb == 0 && word < out_words) ? (uint32_t)r * row_bytes + (uint32_t)word * element : kNoData;
                if (OUT == kOutBits1)
                    __builtin_amdgcn_raw_buffer_store_b64(u32x2{sign_half[2 * t], sign_half[2 * t + 1]}, out, off, 0, 0);
                else
                    __builtin_amdgcn_raw_buffer_store_b128(u32x4{sign_half[2 * t], sign_half[2 * t + 1], nz_half[2 * t], nz_half[2 * t + 1]},
                                                           out, off, 0, 0);
            }
        } else {
            // element 4j+i is pixel 8j+4kb+i of the tile, filter n0 + 32*nt + r: a store writes 128 contiguous bytes of
            // two rows; rows past the tile's last live one lie beyond the descriptor
            const __amdgpu_buffer_rsrc_t out = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(p.y + (size_t)m_first * p.KN), 0, (int)((uint32_t)rows_left * y_row_bytes), kBufferFlags);
#pragma unroll
            for (int nt = 0; nt < TN; nt++) {
                const bool col_ok = OUT == kOutRows || n0 + nt * 32 + r < p.KN;
#pragma unroll
                for (int e = 0; e < 16; e++)
                    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc[nt][e]), out, col_ok ? y_off[e % (SWAP ? 1 : 16)] : kNoData, nt * 128, 0);
            }
        }
    };

    // tiles of this wave: tile, tile + waves, ...; each round requests the next tile (unconditionally: a tile past the
    // end reads nothing), multiplies the current one, and only then, after its stores are issued, makes the next one
    // current (moved up, the copies would wait for the loads right after they were issued); the stores of a tile drain
    // under the tiles after it
    while (tile < tiles) {
        load_tile(tile + waves, buf1, th1);
        __builtin_amdgcn_sched_barrier(0);
        run_tile(tile, buf0, th0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int w = 0; w < G; w++)
#pragma unroll
            for (int pl = 0; pl < APL; pl++) buf0[w][pl] = buf1[w][pl];
        th0 = th1;
        tile += waves;
    }
}

// Workgroups along M for `tiles` 32-pixel tiles: one tile per wave while the launch is small; from `cap` workgroups on,
// the fewest rounds with the waves evenly loaded.
inline unsigned regs_grid_x(int tiles, int cap)
{
    const int wanted = (tiles + 3) / 4;
    if (wanted <= cap) return (unsigned)wanted;
    const int rounds = (tiles + 4 * cap - 1) / (4 * cap);
    return (unsigned)(((tiles + rounds - 1) / rounds + 3) / 4);
}

template <int TYPE, int G, int TN, int OUT>
hipError_t launch_mfma_regs_tile(ConvArgs a, hipStream_t stream)
{
    const int tiles_n = (a.KN + 32 * TN - 1) / (32 * TN);
    if (tiles_n > 65535) return hipErrorInvalidValue;
    // workgroups the chip holds at once (resident workgroups per CU x CUs), looked up on the first launch and kept in
    // one atomic word: threads that race here compute the same value, and a reader sees either 0 or all of it
    static std::atomic<int> resident{0};
    int held = resident.load(std::memory_order_relaxed);
    if (held == 0) {
        int blocks = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, conv_mfma_regs<TYPE, G, TN, OUT>, kConvThreads, 0) != hipSuccess) {
            (void)hipGetLastError();
            blocks = 2;
        }
        held = device_compute_units() * (blocks < 1 ? 1 : blocks);
        resident.store(held, std::memory_order_relaxed);
    }
    const int tiles = (a.M + 31) / 32;
    const int cap = (held + tiles_n - 1) / tiles_n;
    a.kcw = G;
    a.nchunks = 1;
    conv_mfma_regs<TYPE, G, TN, OUT><<<dim3(regs_grid_x(tiles, cap < 1 ? 1 : cap), (unsigned)tiles_n), dim3(kConvThreads), 0, stream>>>(a);
    return hipGetLastError();
}

// True when the register-resident kernel takes this launch.
inline bool mfma_regs_supported(int type, const ConvArgs &a) { return type >= 0 && type <= 3 && a.G <= kRegsMaxWords; }

template <int TYPE, int G, int TN>
hipError_t launch_mfma_regs_out(const ConvArgs &a, hipStream_t stream)
{
    if (a.qy != nullptr)
        return a.out_bits == 1 ? launch_mfma_regs_tile<TYPE, G, TN, kOutBits1>(a, stream) : launch_mfma_regs_tile<TYPE, G, TN, kOutBits2>(a, stream);
    if (a.KN % (32 * TN) == 0) return launch_mfma_regs_tile<TYPE, G, TN, kOutRows>(a, stream);
    return launch_mfma_regs_tile<TYPE, G, TN, kOutFloat>(a, stream);
}

// Filter tiles per wave: two (a whole 64-filter word of packed output); four when K is at most four words and the layer
// has the filters, since a tile's loads, address arithmetic and activation expansions then serve twice the MFMAs.
template <int TYPE, int G>
hipError_t launch_mfma_regs_words(const ConvArgs &a, hipStream_t stream)
{
    if constexpr (G <= 4)
        if (a.KN > 64) return launch_mfma_regs_out<TYPE, G, 4>(a, stream);
    return launch_mfma_regs_out<TYPE, G, 2>(a, stream);
}

template <int TYPE>
hipError_t launch_mfma_regs(const ConvArgs &a, hipStream_t stream)
{
    if (a.G > kRegsMaxWords) return hipErrorInvalidValue;
    switch (a.G) {
    case 1: return launch_mfma_regs_words<TYPE, 1>(a, stream);
    case 2: return launch_mfma_regs_words<TYPE, 2>(a, stream);
    case 3:
    case 4: return launch_mfma_regs_words<TYPE, 4>(a, stream);
    case 9: return launch_mfma_regs_words<TYPE, 9>(a, stream);
    default: return launch_mfma_regs_words<TYPE, 8>(a, stream);
    }
}

}  // namespace
}  // namespace tab
