// Quantizer / bit-packer for gfx950 (wave64): fp32 NHWC -> packed int64 bit planes.
//
// Semantics follow the reference kernels TerOnlyKernel (TAB_GEMM.cu:163-208) and
// BinOnlyKernel (TAB_GEMM.cu:211-247) with the per-item threshold ths[n] of the CPU path
// (TAB_CPU.cpp:67,72), plus BTN_Weight (TAB_GEMM.cu:150-160) for every item.
//
// The tensor is a sequence of "rows" of 64 consecutive channels; row r becomes packed
// word r (C % 64 == 0) so the whole op is one streaming pass: 256 B in, 8 or 16 B out.
#include "tab_pack.h"

namespace tab {
namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / 64;
constexpr int kLoadsPerLane = 8;                // float4 loads in flight per lane
constexpr int kRowsPerWave = 4 * kLoadsPerLane; // each wave-wide float4 load covers 4 rows
constexpr long kSmallLaunchBlocks = 512;        // at or below this many 128-row workgroups a launch is latency-bound

__device__ __forceinline__ int wave_sum(int v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;
}

// Fast path, C % 64 == 0 and X 16-byte aligned.
// Lane layout: a 16-lane DPP row reads one 64-channel row as 16 float4 (256 B contiguous),
// a wave reads 4 consecutive rows per load (1 KB contiguous) and keeps kLoadsPerLane loads
// in flight; pack_row turns the compare bits of the row's lanes into its packed element.
// BITS = 1 or 2 (the reference's bit widths), or the format of conv type 4 or 5; LOADS = 8 (128 rows per
// workgroup) for streaming, 2 for launches too small to fill the chip.
template <int BITS, int LOADS = kLoadsPerLane>
__global__ __launch_bounds__(kThreads) void quantize_rows64(const floatx4 *__restrict__ x,
                                                            const float *__restrict__ ths,
                                                            uint32_t *__restrict__ q, long rows,
                                                            long rows_per_item, Div32 div_item)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: so are row0 and the item test below
    const int sub = lane >> 4;  // which of the 4 rows of a load
    const int l = lane & 15;    // float4 within the row
    const long row0 = ((long)blockIdx.x * kWavesPerBlock + wave) * (4 * LOADS);
    if (row0 >= rows) return;
    long row_last = row0 + (4 * LOADS) - 1;
    if (row_last > rows - 1) row_last = rows - 1;

    floatx4 v[LOADS];
#pragma unroll
    for (int u = 0; u < LOADS; u++) {
        const long r = row0 + u * 4 + sub;
        // rows past the end read the last row again (not stored): straight-line loads, no branch per load
        const floatx4 *src = &x[(r < rows ? r : rows - 1) * 16 + l];
        // a small tensor is likely to sit in the caches (it was just written, or is read again): plain loads;
        // a large one streams past them: non-temporal loads (plain ones are 8-11 % slower at 400 MB and more)
        v[u] = LOADS == 2 ? *src : __builtin_nontemporal_load(src);
    }

    // The wave's items (scalar; div_item.mul == 0 says that rows reach 2^31 and the division takes 64 bits): with the
    // short division the threshold is in flight together with the loads of x instead of behind a long one.
    const long item_first = div_item.mul ? (long)div32((uint32_t)row0, div_item) : row0 / rows_per_item;
    const long item_last = div_item.mul ? (long)div32((uint32_t)row_last, div_item) : row_last / rows_per_item;
    const bool one_item = item_last == item_first;
    const float t_first = ths[item_first];

    auto finish = [&](int u, float t) {
        const long r = row0 + u * 4 + sub;
        uint32_t sign, nz, out[4];
        compare4<BITS>(v[u], t, sign, nz);
        pack_row<BITS>(sign, nz, l, out);  // lane 0 stores the whole element (8 or 16 bytes) at once
        if (BITS != 1) {
            if (r < rows && l == 0) *reinterpret_cast<uintx4 *>(q + r * 4) = uintx4{out[0], out[1], out[2], out[3]};
        } else {
            if (r < rows && l == 0) *reinterpret_cast<uintx2 *>(q + r * 2) = uintx2{out[0], out[1]};
        }
    };
    // two copies of the loop under a scalar branch: the common one has no load but x in flight, so each load is
    // waited for on its own
    if (one_item) {
#pragma unroll
        for (int u = 0; u < LOADS; u++) finish(u, t_first);
    } else {
#pragma unroll
        for (int u = 0; u < LOADS; u++) {
            const long r = row0 + u * 4 + sub;
            finish(u, ths[(r < rows ? r : rows - 1) / rows_per_item]);
        }
    }
}

// The same row quantizer for a 1x1 convolution with stride and no padding, which reads only the
// pixels (oh*s1, ow*s2): one wave per 4*LOADS consecutive words of one output line (n, oh); the packed
// result is the compact [N][OH][OW][PC] activation, i.e. what the conv reads with stride 1.
// grid = (ceil(OW*PC / (4*LOADS)), N*OH), one wave per workgroup; OW*PC < 65536 (fastdiv range).
template <int BITS, int LOADS = kLoadsPerLane>
__global__ __launch_bounds__(64) void quantize_rows64_strided(const floatx4 *__restrict__ x, const float *__restrict__ ths,
                                                              uint32_t *__restrict__ q, int H, int W, int PC, int OH,
                                                              int OW, int s1, int s2, FastDiv div_pc)
{
    const int lane = threadIdx.x;
    const int sub = lane >> 4, l = lane & 15;
    const int n = blockIdx.y / OH, oh = blockIdx.y - n * OH;  // uniform
    const int line_words = OW * PC;
    const long in_line = ((long)n * H + (long)oh * s1) * W;   // first input pixel of the line
    const long out_line = (long)blockIdx.y * line_words;
    const int j0 = blockIdx.x * (4 * LOADS);
    const float t = ths[n];

    floatx4 v[LOADS];
#pragma unroll
    for (int u = 0; u < LOADS; u++) {
        const int j = min(j0 + u * 4 + sub, line_words - 1);  // words past the line read its last word again (not stored)
        const int ow = (int)fastdiv((uint32_t)j, div_pc), pc = j - ow * PC;
        const long r = (in_line + (long)ow * s2) * PC + pc;
        v[u] = LOADS == 2 ? x[r * 16 + l] : __builtin_nontemporal_load(&x[r * 16 + l]);
    }
#pragma unroll
    for (int u = 0; u < LOADS; u++) {
        const int j = j0 + u * 4 + sub;
        const long r = out_line + j;
        uint32_t sign, nz, out[4];
        compare4<BITS>(v[u], t, sign, nz);
        pack_row<BITS>(sign, nz, l, out);
        if (BITS != 1) {
            if (j < line_words && l == 0) *reinterpret_cast<uintx4 *>(q + r * 4) = uintx4{out[0], out[1], out[2], out[3]};
        } else {
            if (j < line_words && l == 0) *reinterpret_cast<uintx2 *>(q + r * 2) = uintx2{out[0], out[1]};
        }
    }
}

// OR over the LP lanes (a power of two up to 16, aligned inside a DPP row) of a group; every lane gets the result.
template <int LP>
__device__ __forceinline__ uint32_t or_reduce_group(uint32_t v)
{
    if (LP >= 2) v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);    // quad_perm [1,0,3,2]
    if (LP >= 4) v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);    // quad_perm [2,3,0,1]
    if (LP >= 8) v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true);   // row_half_mirror
    if (LP >= 16) v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, true);  // row_mirror
    return v;
}

// General path (any C, any alignment of x; pixels * PC < 2^31): a group of LP lanes takes one (pixel, word) row of
// up to 4 * LP channels, lane l the channels l, l + LP, l + 2 LP, l + 3 LP of the word (so a wave-wide load reads
// runs of 4 * LP bytes, and neighbouring groups neighbouring rows); LP = 16 serves words of up to 64 channels,
// smaller groups tensors of few channels (LP = 1: a lane per pixel).  Eight rows per group are in flight.  The
// lanes' compare bits are ORed over the group; unused high bits of a tail word stay 0 (TAB_GEMM.cu:203-206).
template <int BITS, int LP>
__global__ __launch_bounds__(kThreads) void quantize_groups(const float *__restrict__ x, const float *__restrict__ ths,
                                                            uint32_t *__restrict__ q, long rows, long pixels_per_item,
                                                            int C, int PC)
{
    constexpr int GROUPS = 64 / LP;  // rows per wave-wide load
    constexpr int U = 8;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int group = lane / LP, l = lane % LP;
    const long row0 = ((long)blockIdx.x * kWavesPerBlock + wave) * (GROUPS * U);
    if (row0 >= rows) return;
    long row_last = row0 + GROUPS * U - 1;
    if (row_last > rows - 1) row_last = rows - 1;

    float v[U][4];
    int channels[U];  // of the row's word
    long pixel[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const long r = row0 + u * GROUPS + group;
        const uint32_t rc = (uint32_t)(r < rows ? r : rows - 1);  // rows past the end read the last row again (not stored)
        const uint32_t px = PC == 1 ? rc : rc / (uint32_t)PC;
        const int c0 = (int)(rc - px * (uint32_t)PC) * kWordBits;
        channels[u] = C - c0 < kWordBits ? C - c0 : kWordBits;
        pixel[u] = px;
        const float *src = x + (long)px * C + c0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int ch = l + LP * e;  // past the word: its last channel again, masked below
            v[u][e] = __builtin_nontemporal_load(src + (ch < channels[u] ? ch : channels[u] - 1));
        }
    }

    const long item_first = (row0 / PC) / pixels_per_item;
    const bool one_item = ((row_last / PC) / pixels_per_item) == item_first;  // scalar
    const float t_first = ths[item_first];

    auto finish = [&](int u, float t) {
        uint32_t w[4] = {0, 0, 0, 0};  // sign low, sign high, nonzero low, nonzero high
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int ch = l + LP * e;
            const bool valid = ch < channels[u];
            const int half = LP * e >= 32 ? 1 : 0;             // LP * e is 0, 16, 32, 48 when channels reach 32
            const int shift = l + (LP * e - 32 * half);
            if (BITS == 2) {
                const bool pos = v[u][e] > t;
                const bool neg = !pos && (v[u][e] < -t);
                w[half] |= (uint32_t)(valid && neg) << shift;
                w[2 + half] |= (uint32_t)(valid && (pos || neg)) << shift;
            } else {
                w[half] |= (uint32_t)(valid && (v[u][e] < t)) << shift;
            }
        }
        const long r = row0 + u * GROUPS + group;
        const uint32_t s_lo = or_reduce_group<LP>(w[0]), s_hi = LP == 16 ? or_reduce_group<LP>(w[1]) : 0u;
        if (BITS == 2) {
            const uint32_t n_lo = or_reduce_group<LP>(w[2]), n_hi = LP == 16 ? or_reduce_group<LP>(w[3]) : 0u;
            if (r < rows && l == 0) *reinterpret_cast<uintx4 *>(q + r * 4) = uintx4{s_lo, s_hi, n_lo, n_hi};
        } else {
            if (r < rows && l == 0) *reinterpret_cast<uintx2 *>(q + r * 2) = uintx2{s_lo, s_hi};
        }
    };
    if (one_item) {
#pragma unroll
        for (int u = 0; u < U; u++) finish(u, t_first);
    } else {
#pragma unroll
        for (int u = 0; u < U; u++) finish(u, ths[pixel[u] / pixels_per_item]);
    }
}

// Fallback of the general path for tensors of 2^31 rows or more: one wave per (pixel, word); lane i tests channel
// word*64 + i and the two wave-wide ballots are the packed words, LSB first
// (onebit[i] = 1 << i, TAB_GEMM.cu:252-258).  Unused high bits of a tail word stay 0
// (TAB_GEMM.cu:203-206).
template <int BITS>
__global__ __launch_bounds__(kThreads) void quantize_ballot(const float *__restrict__ x,
                                                            const float *__restrict__ ths,
                                                            uint64_t *__restrict__ q, long pixels,
                                                            long pixels_per_item, int C, int PC)
{
    const int lane = threadIdx.x & 63;
    const long nwaves = (long)gridDim.x * kWavesPerBlock;
    const long units = pixels * PC;
    for (long unit = (long)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6); unit < units; unit += nwaves) {
        const long pixel = unit / PC;
        const int word = (int)(unit - pixel * PC);
        const long item = pixel / pixels_per_item;
        const float t = ths[item];
        const int c = word * kWordBits + lane;
        const bool live = c < C;
        const float v = live ? x[pixel * C + c] : 0.f;
        if (BITS == 2) {
            const bool pos = live && (v > t);
            const bool neg = live && !pos && (v < -t);
            const uint64_t nz = __ballot(pos || neg);
            const uint64_t sign = __ballot(neg);
            if (lane == 0) {
                q[unit * 2 + 0] = sign;
                q[unit * 2 + 1] = nz;
            }
        } else {
            const uint64_t neg = __ballot(live && (v < t));
            if (lane == 0) q[unit] = neg;
        }
    }
}

// Packers of the two CPU-only conv types, whose word layouts follow from the reference's GEMMs (it has
// no quantizer for them: TAB_Conv calls Parallel_Binarize_NCHW and Parallel_Ternarize_RTN,
// TAB_CPU.cpp:522,527, which no file defines).  One wave per output word, ballots as above.
// FORMAT 4, DoReFa 2-bit (DRFGEMM_baseline, TAB_CPU.cpp:345-354): [pixel][ceil(C/64)][2], plane 0 the
//   weight-2 bit and plane 1 the weight-1 bit of level = (v >= 0.5t) + (v >= 1.5t) + (v >= 2.5t).
// FORMAT 5, RTN (RTNGEMM_baseline, TAB_CPU.cpp:364-379; 32 channels per word, 520-521):
//   [pixel][ceil(C/32)], channel c in word c/32 as the field (bit 2*(c%32) = nonzero, bit 2*(c%32)+1 =
//   sign) of the ternarizer's value; lane j of the wave tests channel j/2 for bit j.
template <int FORMAT>
__global__ __launch_bounds__(kThreads) void quantize_ballot_format(const float *__restrict__ x, const float *__restrict__ ths,
                                                                   uint64_t *__restrict__ q, long pixels,
                                                                   long pixels_per_item, int C, int PC)
{
    const int lane = threadIdx.x & 63;
    const long nwaves = (long)gridDim.x * kWavesPerBlock;
    const long units = pixels * PC;
    for (long unit = (long)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6); unit < units; unit += nwaves) {
        const long pixel = unit / PC;
        const int word = (int)(unit - pixel * PC);
        const float t = ths[pixel / pixels_per_item];
        if (FORMAT == 4) {
            const int c = word * kWordBits + lane;
            const bool live = c < C;
            const float v = live ? x[pixel * C + c] : 0.f;
            const int level = live ? (int)(v >= 0.5f * t) + (int)(v >= 1.5f * t) + (int)(v >= 2.5f * t) : 0;
            const uint64_t hi = __ballot(level >> 1), lo = __ballot(level & 1);
            if (lane == 0) {
                q[unit * 2 + 0] = hi;
                q[unit * 2 + 1] = lo;
            }
        } else {
            const int c = word * 32 + (lane >> 1);
            const bool live = c < C;
            const float v = live ? x[pixel * C + c] : 0.f;
            const bool pos = live && (v > t);
            const bool neg = live && !pos && (v < -t);
            const uint64_t fields = __ballot((lane & 1) ? neg : (pos || neg));
            if (lane == 0) q[unit] = fields;
        }
    }
}

// The same quantizers on an NCHW tensor, the layout the reference's CPU quantizers read
// (Parallel_Ternarize_NCHWB_to_NHWCB / Parallel_Binarize_NCHW_to_NHWC, TAB_CPU.cpp:20-206), into the same NHWC
// packed output.  A thread owns VEC consecutive pixels of one image and one 64-channel word: it walks the
// word's channels, VEC floats per load (consecutive threads read consecutive pixels of one channel plane,
// so every load instruction is contiguous), and shifts each compare bit into the words it holds in
// registers: no cross-lane step at all.  Pixels are numbered through all images (VEC divides H*W, so a
// thread's pixels share an image), which keeps every workgroup full whatever H*W is.
// grid = ceil(N*H*W / (VEC * 256)) * PC workgroups, the word index fastest: the workgroups that write the PC
// words of the same pixels run side by side, so their 8- or 16-byte stores meet in L2 as whole lines.
template <int BITS, int VEC>
__global__ __launch_bounds__(kThreads) void quantize_nchw(const float *__restrict__ x, const float *__restrict__ ths,
                                                          uint64_t *__restrict__ q, int N, int C, long HW, int PC)
{
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    const int pc = blockIdx.x % PC;
    const long g0 = ((long)(blockIdx.x / PC) * kThreads + threadIdx.x) * VEC;  // first pixel, counted through all images
    if (g0 >= (long)N * HW) return;
    const long n = g0 / HW, s0 = g0 - n * HW;
    const float t = ths[n];
    const int c0 = pc * kWordBits;
    const int channels = C - c0 < kWordBits ? C - c0 : kWordBits;
    const float *src = x + (n * C + c0) * HW + s0;
    uint64_t sign[VEC], nz[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) sign[e] = nz[e] = 0;
    constexpr int kInFlight = VEC == 1 ? 32 : 8;  // the one-pixel form serves small, latency-bound tensors
    auto step = [&](const int j0) {
        float v[kInFlight][VEC];
#pragma unroll
        for (int u = 0; u < kInFlight; u++) {
            const int j = j0 + u < channels ? j0 + u : channels - 1;  // clamped: the bit is masked below
            if (VEC == 1) {
                v[u][0] = src[(long)j * HW];  // the one-pixel form serves small tensors, likely cache-resident: plain loads
            } else {
                const vec_t w = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(src + (long)j * HW));
#pragma unroll
                for (int e = 0; e < VEC; e++) v[u][e] = w[e];
            }
        }
#pragma unroll
        for (int u = 0; u < kInFlight; u++) {
            const uint64_t bit = j0 + u < channels ? (uint64_t)1 << (j0 + u) : 0;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                if (BITS == 2) {
                    const bool pos = v[u][e] > t;
                    const bool neg = !pos && (v[u][e] < -t);
                    if (pos || neg) nz[e] |= bit;
                    if (neg) sign[e] |= bit;
                } else {
                    if (v[u][e] < t) sign[e] |= bit;
                }
            }
        }
    };
    if (channels == kWordBits) {  // a whole word: unrolled, every bit position a constant
#pragma unroll
        for (int j0 = 0; j0 < kWordBits; j0 += kInFlight) step(j0);
    } else {
        for (int j0 = 0; j0 < channels; j0 += kInFlight) step(j0);
    }
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        const long pixel = g0 + e;
        if (BITS == 2) {
            q[(pixel * PC + pc) * 2 + 0] = sign[e];
            q[(pixel * PC + pc) * 2 + 1] = nz[e];
        } else {
            q[pixel * PC + pc] = sign[e];
        }
    }
}

// The NCHW quantizer for PC a multiple of U = 2 or 4 and at least one wave of work per SIMD: a thread packs U
// neighbouring words of its four pixels, one after the other, and the wave then turns its 256 pixels x U words
// (x 2 planes) around in LDS, so that a store instruction writes whole runs of the output - U * BITS words per pixel,
// the entire kilobyte when PC == U - instead of one 8-byte word per lane at the stride of a pixel.  Measured on
// 256 x 256 x 56 x 56: the loads alone take 120 us; with quantize_nchw's word-per-lane stores 152 us (one plane) /
// 166 us (two), with this kernel 135-137 / 153 us.
// One wave per workgroup (with four, the 784 workgroups of that tensor load the CUs 4 : 3), 4 KB of LDS, gone through
// in WPP / 2 rounds of 64 / rounds lanes each.  grid = ceil(N*H*W / 256) * (PC / U), the word group fastest.
template <int BITS, int U>
__global__ __launch_bounds__(64) void quantize_nchw_gather(const float *__restrict__ x, const float *__restrict__ ths,
                                                                 uint64_t *__restrict__ q, int N, int C, long HW, int PC)
{
    constexpr int VEC = 4, kInFlight = 8;
    constexpr int WPP = U * BITS;      // words a thread packs per pixel, contiguous in q
    constexpr int ROUNDS = WPP / 2;    // 64 / ROUNDS lanes x 4 pixels x WPP words = 512 words a round
    constexpr int LPR = 64 / ROUNDS;
    static_assert(U == 2 || U == 4, "one word per thread is quantize_nchw");
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    __shared__ __attribute__((aligned(16))) uint64_t stage[512];
    const int groups = PC / U;
    const int pc0 = (blockIdx.x % groups) * U;
    const int lane = threadIdx.x;
    const long total = (long)N * HW;
    const long wave_pixel0 = (long)(blockIdx.x / groups) * (64 * VEC);  // below total: the grid is ceil(total / 256) * groups
    const long mine = wave_pixel0 + lane * VEC;
    const long g0 = mine < total ? mine : wave_pixel0;  // lanes past the end repeat the wave's first pixels and store nothing
    const long n = g0 / HW, s0 = g0 - n * HW;
    const float t = ths[n];
    // The U words are U * 64 consecutive channels: batches of kInFlight channels, the next batch's loads issued before
    // the compares of this one (two register buffers), so the memory pipe never waits for the packing.
    const int cbase = pc0 * kWordBits;
    const float *src = x + n * C * HW + s0;
    auto load = [&](float (&v)[kInFlight][VEC], const int b) {
#pragma unroll
        for (int k = 0; k < kInFlight; k++) {
            int c = cbase + b * kInFlight + k;
            c = c < C ? c : C - 1;  // past the last channel (tail word, prefetch after the last batch): masked in pack() or unused
            const vec_t w = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(src + (long)c * HW));
#pragma unroll
            for (int e = 0; e < VEC; e++) v[k][e] = w[e];
        }
    };
    uint64_t words[VEC][WPP];
    uint64_t sign[VEC], nz[VEC];
    auto pack = [&](const float (&v)[kInFlight][VEC], const int b) {
        uint32_t s[VEC], z[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) s[e] = z[e] = 0;
#pragma unroll
        for (int k = 0; k < kInFlight; k++) {
            const uint32_t bit = cbase + b * kInFlight + k < C ? 1u << k : 0u;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                if (BITS == 2) {
                    const bool pos = v[k][e] > t;
                    const bool neg = !pos && (v[k][e] < -t);
                    if (pos || neg) z[e] |= bit;
                    if (neg) s[e] |= bit;
                } else {
                    if (v[k][e] < t) s[e] |= bit;
                }
            }
        }
        const int shift = (b * kInFlight) % kWordBits;
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            sign[e] |= (uint64_t)s[e] << shift;
            if (BITS == 2) nz[e] |= (uint64_t)z[e] << shift;
        }
    };
    constexpr int kBatches = kWordBits / kInFlight;  // per word
    float v0[kInFlight][VEC], v1[kInFlight][VEC];
    load(v0, 0);
#pragma unroll
    for (int u = 0; u < U; u++) {
#pragma unroll
        for (int e = 0; e < VEC; e++) sign[e] = nz[e] = 0;
#pragma unroll 1
        for (int b = u * kBatches; b < (u + 1) * kBatches; b += 2) {
            load(v1, b + 1);
            pack(v0, b);
            load(v0, b + 2);  // after the last batch too (a valid channel, unused): guarding it costs more than the 8 loads
            pack(v1, b + 1);
        }
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            words[e][u * BITS] = sign[e];
            if (BITS == 2) words[e][u * BITS + 1] = nz[e];
        }
    }
    uint64_t *st = stage;
#pragma unroll
    for (int r = 0; r < ROUNDS; r++) {
        __builtin_amdgcn_wave_barrier();
        if (lane / LPR == r) {
            const int l = lane % LPR;
#pragma unroll
            for (int e = 0; e < VEC; e++)
#pragma unroll
                for (int j = 0; j < WPP; j += 2)
                    *reinterpret_cast<ulonglong2 *>(st + (l * VEC + e) * WPP + j) = make_ulonglong2(words[e][j], words[e][j + 1]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int w = (i * 64 + lane) * 2;  // two words a lane: 1 KB a store instruction
            const long pixel = wave_pixel0 + r * LPR * VEC + w / WPP;
            const ulonglong2 pair = *reinterpret_cast<const ulonglong2 *>(st + w);
            // an even word index (PC * BITS, pc0 * BITS and w % WPP are even) into a 16-byte aligned q
            if (pixel < total) *reinterpret_cast<ulonglong2 *>(q + (pixel * PC + pc0) * BITS + w % WPP) = pair;
        }
    }
}

__global__ void fill_zero_i32(int32_t *p, long n)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// btn[n] = sum over item n of popcount(nonzero-plane word) (BTN_Weight, TAB_GEMM.cu:150-160,
// for every n).  q is the ternary output [items][words_per_item][2]; one workgroup per
// (item, split) reads its words as 16-byte (sign, nonzero) pairs.  With one split the result
// is stored directly; with several (very long items) the partial sums are added atomically
// into btn, which the caller zeroed beforehand.
__global__ __launch_bounds__(kThreads) void btn_popcount(const ulonglong2 *__restrict__ q,
                                                         int32_t *__restrict__ btn,
                                                         long words_per_item, int splits)
{
    __shared__ int partial[kWavesPerBlock];
    const long item = blockIdx.x / splits;
    const int split = blockIdx.x % splits;
    const long per_split = (words_per_item + splits - 1) / splits;
    const long w0 = split * per_split;
    long w1 = w0 + per_split;
    if (w1 > words_per_item) w1 = words_per_item;
    const ulonglong2 *src = q + item * words_per_item;
    int count = 0;
    for (long w = w0 + threadIdx.x; w < w1; w += kThreads) count += __popcll(src[w].y);
    count = wave_sum(count);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = count;
    __syncthreads();
    if (threadIdx.x == 0) {
        int total = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; w++) total += partial[w];
        if (splits == 1)
            btn[item] = total;
        else if (total)
            atomicAdd(&btn[item], total);
    }
}

// ---- thresholds: ths[n] = scale * mean(|x[n]|) ------------------------------------------------
// The step right before Quantize in the reference's demo flow (the caller computes it in
// torch).  Two fixed-order stages so that the result does not depend on scheduling: `splits`
// workgroups per item each reduce a contiguous slice to one fp32 partial (per-thread serial
// sums of float4, then a tree over lanes and waves), then one thread per item adds the
// partials in index order in fp64.
__global__ __launch_bounds__(kThreads) void abs_sum_partial(const float *__restrict__ x, float *__restrict__ partial,
                                                            long per_item, int splits)
{
    __shared__ float wave_part[kWavesPerBlock];
    const long item = blockIdx.x / splits;
    const int split = blockIdx.x % splits;
    const long slice = ((per_item + splits - 1) / splits + 3) & ~3L;  // multiple of 4 elements
    const long begin = split * slice;
    long end = begin + slice;
    if (end > per_item) end = per_item;
    const float *src = x + item * per_item;
    float sum = 0.f;
    if (((uintptr_t)(src + begin) & 15) == 0) {
        const long n4 = begin < end ? (end - begin) / 4 : 0;
        const floatx4 *src4 = reinterpret_cast<const floatx4 *>(src + begin);
        for (long i = threadIdx.x; i < n4; i += kThreads) {
            const floatx4 v = __builtin_nontemporal_load(&src4[i]);
            sum += (__builtin_fabsf(v[0]) + __builtin_fabsf(v[1])) + (__builtin_fabsf(v[2]) + __builtin_fabsf(v[3]));
        }
        for (long i = begin + n4 * 4 + threadIdx.x; i < end; i += kThreads) sum += __builtin_fabsf(src[i]);
    } else {
        for (long i = begin + threadIdx.x; i < end; i += kThreads) sum += __builtin_fabsf(src[i]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_down(sum, off, 64);
    if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; w++) total += wave_part[w];
        partial[blockIdx.x] = total;
    }
}

__global__ void abs_mean_finish(const float *__restrict__ partial, float *__restrict__ ths, long items, int splits,
                                double scale_over_count)
{
    const long n = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= items) return;
    double total = 0.0;
    for (int s = 0; s < splits; s++) total += (double)partial[n * splits + s];
    ths[n] = (float)(total * scale_over_count);
}

}  // namespace

int threshold_splits(long items, long per_item)
{
    int splits = 1;
    while (splits < 1024 && items * splits < 2048 && per_item / (splits * 2) >= 8L * kThreads) splits *= 2;
    return splits;
}

hipError_t launch_threshold(const float *x, long items, long per_item, float scale, float *ths, float *partial,
                            hipStream_t stream)
{
    const int splits = threshold_splits(items, per_item);
    abs_sum_partial<<<dim3((unsigned)(items * splits)), dim3(kThreads), 0, stream>>>(x, partial, per_item, splits);
    abs_mean_finish<<<dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream>>>(partial, ths, items, splits,
                                                                                   (double)scale / (double)per_item);
    return hipGetLastError();
}

template <int LP>
void launch_quantize_groups_of(const float *x, const float *ths, int bitwidth, long rows, long pixels_per_item, int C, int PC,
                               uint32_t *q, hipStream_t stream)
{
    const long per_block = (long)kWavesPerBlock * (64 / LP) * 8;
    const dim3 grid((unsigned)((rows + per_block - 1) / per_block)), block(kThreads);
    if (bitwidth == 2)
        quantize_groups<2, LP><<<grid, block, 0, stream>>>(x, ths, q, rows, pixels_per_item, C, PC);
    else
        quantize_groups<1, LP><<<grid, block, 0, stream>>>(x, ths, q, rows, pixels_per_item, C, PC);
}

// The general-path kernel with the smallest group of lanes whose 4 channels a lane cover the widest word.
void launch_quantize_groups(const float *x, const float *ths, int bitwidth, long rows, long pixels_per_item, int C, int PC,
                            uint32_t *q, hipStream_t stream)
{
    const int widest = C < kWordBits ? C : kWordBits;
    if (widest <= 4) launch_quantize_groups_of<1>(x, ths, bitwidth, rows, pixels_per_item, C, PC, q, stream);
    else if (widest <= 8) launch_quantize_groups_of<2>(x, ths, bitwidth, rows, pixels_per_item, C, PC, q, stream);
    else if (widest <= 16) launch_quantize_groups_of<4>(x, ths, bitwidth, rows, pixels_per_item, C, PC, q, stream);
    else if (widest <= 32) launch_quantize_groups_of<8>(x, ths, bitwidth, rows, pixels_per_item, C, PC, q, stream);
    else launch_quantize_groups_of<16>(x, ths, bitwidth, rows, pixels_per_item, C, PC, q, stream);
}

// x: fp32 [items][pixels_per_item][C]; qx: [items*pixels_per_item][PC][bitwidth];
// btn: [items] or nullptr (then no counts are produced).
hipError_t launch_quantize(const float *x, const float *ths, int bitwidth, long pixels_per_item,
                           long items, int C, uint64_t *qx, int32_t *btn, hipStream_t stream)
{
    const int PC = (C + kWordBits - 1) / kWordBits;
    const long pixels = items * pixels_per_item;
    const long words_per_item = pixels_per_item * PC;
    // very long items are split over several workgroups for the btn pass
    int splits = 1;
    if (btn && bitwidth == 2 && items < 512) {
        while (splits < 64 && items * splits < 512 && words_per_item / (splits * 2) >= 2 * kThreads) splits *= 2;
    }
    if (btn && (bitwidth != 2 || splits > 1)) {
        // zeros for 1-bit (TAB_GEMM.cu:283); a kernel rather than a memset node so that the
        // call can be captured in a graph
        fill_zero_i32<<<dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream>>>(btn, items);
    }
    const bool fast = (C % kWordBits == 0) && ((uintptr_t)x % 16 == 0);
    if (fast) {
        const long rows = pixels * PC;
        const Div32 div_item = rows < 0x7fffffffL ? make_div32((uint32_t)words_per_item) : Div32{0, 0};
        const long blocks = (rows + kRowsPerWave * kWavesPerBlock - 1) / (kRowsPerWave * kWavesPerBlock);
        const dim3 block(kThreads);
        const floatx4 *x4 = reinterpret_cast<const floatx4 *>(x);
        uint32_t *q32 = reinterpret_cast<uint32_t *>(qx);
        if (blocks <= kSmallLaunchBlocks) {
            // a tensor too small to fill the chip with 128-row workgroups: 32 rows per workgroup, two loads per lane
            // (3.1 MB of fp32: 5.5 -> 4.2 us)
            const dim3 grid((unsigned)((rows + 8 * kWavesPerBlock - 1) / (8 * kWavesPerBlock)));
            if (bitwidth == 2)
                quantize_rows64<2, 2><<<grid, block, 0, stream>>>(x4, ths, q32, rows, words_per_item, div_item);
            else
                quantize_rows64<1, 2><<<grid, block, 0, stream>>>(x4, ths, q32, rows, words_per_item, div_item);
        } else {
            const dim3 grid((unsigned)blocks);
            if (bitwidth == 2)
                quantize_rows64<2><<<grid, block, 0, stream>>>(x4, ths, q32, rows, words_per_item, div_item);
            else
                quantize_rows64<1><<<grid, block, 0, stream>>>(x4, ths, q32, rows, words_per_item, div_item);
        }
    } else if (pixels * PC < 0x7fffffffL) {
        launch_quantize_groups(x, ths, bitwidth, pixels * PC, pixels_per_item, C, PC, reinterpret_cast<uint32_t *>(qx), stream);
    } else {
        const long units = pixels * PC;
        long blocks = (units + kWavesPerBlock - 1) / kWavesPerBlock;
        if (blocks > 256 * 32) blocks = 256 * 32;  // grid-stride beyond 32 blocks per CU
        const dim3 grid((unsigned)blocks), block(kThreads);
        if (bitwidth == 2)
            quantize_ballot<2><<<grid, block, 0, stream>>>(x, ths, qx, pixels, pixels_per_item, C, PC);
        else
            quantize_ballot<1><<<grid, block, 0, stream>>>(x, ths, qx, pixels, pixels_per_item, C, PC);
    }
    if (btn && bitwidth == 2) {
        btn_popcount<<<dim3((unsigned)(items * splits)), dim3(kThreads), 0, stream>>>(
            reinterpret_cast<const ulonglong2 *>(qx), btn, words_per_item, splits);
    }
    return hipGetLastError();
}

hipError_t launch_quantize_nchw(const float *x, const float *ths, int bitwidth, int N, int C, long HW, uint64_t *qx,
                                int32_t *btn, hipStream_t stream)
{
    const int PC = (C + kWordBits - 1) / kWordBits;
    const long words_per_item = HW * PC;
    int splits = 1;
    if (btn && bitwidth == 2 && N < 512) {
        while (splits < 64 && (long)N * splits < 512 && words_per_item / (splits * 2) >= 2 * kThreads) splits *= 2;
    }
    if (btn && (bitwidth != 2 || splits > 1))
        fill_zero_i32<<<dim3((unsigned)((N + 255) / 256)), dim3(256), 0, stream>>>(btn, N);
    // four pixels per thread when the planes allow aligned 16-byte loads and the launch still fills the chip
    const long pixels = (long)N * HW;
    const bool vec4 = HW % 4 == 0 && (uintptr_t)x % 16 == 0 && ((pixels + 4 * kThreads - 1) / (4 * kThreads)) * PC >= 2048;
    const long per_block = (vec4 ? 4 : 1) * (long)kThreads;
    const long blocks = (pixels + per_block - 1) / per_block;
    if (blocks * PC > 0x7fffffffL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)(blocks * PC)), block(kThreads);
    // PC even, enough pixels for a wave on every SIMD: the form that gathers each wave's output into whole runs
    const int unit = PC % 4 == 0 ? 4 : PC % 2 == 0 ? 2 : 1;
    const long gather_waves = (pixels + 255) / 256 * (PC / unit);
    if (gather_waves > 0x7fffffffL) return hipErrorInvalidValue;
    if (HW % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)qx % 16 == 0 && unit > 1 && gather_waves >= 1024) {
        const dim3 ggrid((unsigned)gather_waves), gblock(64);
        if (unit == 4 && bitwidth == 2) quantize_nchw_gather<2, 4><<<ggrid, gblock, 0, stream>>>(x, ths, qx, N, C, HW, PC);
        else if (unit == 4) quantize_nchw_gather<1, 4><<<ggrid, gblock, 0, stream>>>(x, ths, qx, N, C, HW, PC);
        else if (bitwidth == 2) quantize_nchw_gather<2, 2><<<ggrid, gblock, 0, stream>>>(x, ths, qx, N, C, HW, PC);
        else quantize_nchw_gather<1, 2><<<ggrid, gblock, 0, stream>>>(x, ths, qx, N, C, HW, PC);
    } else if (vec4) {
        if (bitwidth == 2) quantize_nchw<2, 4><<<grid, block, 0, stream>>>(x, ths, qx, N, C, HW, PC);
        else quantize_nchw<1, 4><<<grid, block, 0, stream>>>(x, ths, qx, N, C, HW, PC);
    } else {
        if (bitwidth == 2) quantize_nchw<2, 1><<<grid, block, 0, stream>>>(x, ths, qx, N, C, HW, PC);
        else quantize_nchw<1, 1><<<grid, block, 0, stream>>>(x, ths, qx, N, C, HW, PC);
    }
    if (btn && bitwidth == 2) {
        btn_popcount<<<dim3((unsigned)(N * splits)), dim3(kThreads), 0, stream>>>(reinterpret_cast<const ulonglong2 *>(qx), btn,
                                                                                 words_per_item, splits);
    }
    return hipGetLastError();
}

hipError_t launch_quantize_format(const float *x, const float *ths, int format, long pixels_per_item, long items, int C,
                                  uint64_t *qx, hipStream_t stream)
{
    const int PC = format == 5 ? (C + 31) / 32 : (C + kWordBits - 1) / kWordBits;
    const long pixels = items * pixels_per_item;
    if (format != 4 && format != 5) return hipErrorInvalidValue;
    if ((C % kWordBits == 0) && ((uintptr_t)x % 16 == 0)) {
        // whole 64-channel rows: the streaming kernel; a row is 16 bytes of either format
        const long rows = pixels * (C / kWordBits);
        const long blocks = (rows + kRowsPerWave * kWavesPerBlock - 1) / (kRowsPerWave * kWavesPerBlock);
        const dim3 grid((unsigned)blocks), block(kThreads);
        const floatx4 *x4 = reinterpret_cast<const floatx4 *>(x);
        uint32_t *q32 = reinterpret_cast<uint32_t *>(qx);
        const long rows_per_item = pixels_per_item * (C / kWordBits);
        const Div32 div_item = rows < 0x7fffffffL ? make_div32((uint32_t)rows_per_item) : Div32{0, 0};
        if (blocks <= kSmallLaunchBlocks) {  // too small to fill the chip: 32 rows per workgroup, as in launch_quantize
            const dim3 small((unsigned)((rows + 8 * kWavesPerBlock - 1) / (8 * kWavesPerBlock)));
            if (format == 4)
                quantize_rows64<4, 2><<<small, block, 0, stream>>>(x4, ths, q32, rows, rows_per_item, div_item);
            else
                quantize_rows64<5, 2><<<small, block, 0, stream>>>(x4, ths, q32, rows, rows_per_item, div_item);
        } else if (format == 4) {
            quantize_rows64<4><<<grid, block, 0, stream>>>(x4, ths, q32, rows, rows_per_item, div_item);
        } else {
            quantize_rows64<5><<<grid, block, 0, stream>>>(x4, ths, q32, rows, rows_per_item, div_item);
        }
        return hipGetLastError();
    }
    const long units = pixels * PC;
    long blocks = (units + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > 256 * 32) blocks = 256 * 32;  // grid-stride beyond 32 blocks per CU
    const dim3 grid((unsigned)blocks), block(kThreads);
    if (format == 4)
        quantize_ballot_format<4><<<grid, block, 0, stream>>>(x, ths, qx, pixels, pixels_per_item, C, PC);
    else if (format == 5)
        quantize_ballot_format<5><<<grid, block, 0, stream>>>(x, ths, qx, pixels, pixels_per_item, C, PC);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

bool quantize_strided_supported(const float *x, int H, int W, int C, int OH, int OW)
{
    const long PC = C / kWordBits;
    return C % kWordBits == 0 && (uintptr_t)x % 16 == 0 && OW * PC < 65536 && PC < 65536;
}

hipError_t launch_quantize_strided(const float *x, const float *ths, int bitwidth, int N, int H, int W, int C, int OH,
                                   int OW, int s1, int s2, uint64_t *qx, hipStream_t stream)
{
    const int PC = C / kWordBits;
    const dim3 block(64);
    const floatx4 *x4 = reinterpret_cast<const floatx4 *>(x);
    uint32_t *q32 = reinterpret_cast<uint32_t *>(qx);
    const long waves = (long)((OW * PC + kRowsPerWave - 1) / kRowsPerWave) * N * OH;
    if (waves <= kSmallLaunchBlocks * kWavesPerBlock) {  // latency-bound: four times the waves, two loads per lane each
        const dim3 grid((unsigned)((OW * PC + 7) / 8), (unsigned)(N * OH));
        if (bitwidth == 2)
            quantize_rows64_strided<2, 2><<<grid, block, 0, stream>>>(x4, ths, q32, H, W, PC, OH, OW, s1, s2, make_fastdiv(PC));
        else
            quantize_rows64_strided<1, 2><<<grid, block, 0, stream>>>(x4, ths, q32, H, W, PC, OH, OW, s1, s2, make_fastdiv(PC));
        return hipGetLastError();
    }
    const dim3 grid((unsigned)((OW * PC + kRowsPerWave - 1) / kRowsPerWave), (unsigned)(N * OH));
    if (bitwidth == 2)
        quantize_rows64_strided<2><<<grid, block, 0, stream>>>(x4, ths, q32, H, W, PC, OH, OW, s1, s2, make_fastdiv(PC));
    else
        quantize_rows64_strided<1><<<grid, block, 0, stream>>>(x4, ths, q32, H, W, PC, OH, OW, s1, s2, make_fastdiv(PC));
    return hipGetLastError();
}

}  // namespace tab
