// Matrix-core variant of the fused pad + im2row + bitwise GEMM: the packed bit planes are
// expanded to int8 in registers and multiplied with v_mfma_i32_32x32x32_i8.
//
// The four TAB formulas (TAB_GEMM.cu:25-147) written as integer dot products, with
// a_k = a1*(1 - 2*a0), b_k = b1*(1 - 2*b0) the decoded ternary values (any bit pattern) and
// a01, b01 the raw bits of a binary operand:
//   TNN  y = sum a_k*b_k
//   TBN  y = sum a_k - 2 * sum a_k*b01
//   BTN  y = btn[n] - 2 * (sum a01*b_k + popcount(b0 & b1))
//   BNN  y = NUM - 2 * (popcount(a) + popcount(b) - 2 * sum a01*b01)
// All sums are exact in int32.  Zero-padded taps and the unused high bits of a tail word are
// zero bits on both sides and contribute nothing, as in the popcount formulas.
//
// Tiling: 256 threads, 128x128 tile of Y, operands staged in LDS exactly as for the popcount
// kernel (tab_conv_stage.h).  Wave w owns the 64x64 quadrant (w&1, w>>1) as 2x2 MFMA tiles.
// Per 32-bit k-slice a lane reads the slice word of its row (A) / column (B) - lane%32 - and
// expands the 16 bits lane/32 selects into the 16 int8 of its MFMA operand: 4 bits -> 4 bytes
// with one v_bfe, one 24-bit multiply by 0x204081 (copies of the nibble at bit 0, 7, 14, 21)
// and one mask.
#include "tab_conv_stage.h"

namespace tab {
namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

// bits [shift, shift+16) of word -> 16 bytes of 0/1
__device__ __forceinline__ i32x4 expand01(uint32_t word, uint32_t shift)
{
    i32x4 r;
#pragma unroll
    for (int d = 0; d < 4; d++) {
        const uint32_t nib = __builtin_amdgcn_ubfe(word, shift + 4 * d, 4);
        r[d] = (int)(__umul24(nib, 0x00204081u) & 0x01010101u);
    }
    return r;
}

// the same 16 positions of a ternary operand -> bytes +1, 0, -1 (0xFF)
__device__ __forceinline__ i32x4 expand_ternary(uint32_t sign, uint32_t nz, uint32_t shift)
{
    const i32x4 z = expand01(nz, shift), g = expand01(sign & nz, shift);
    i32x4 r;
#pragma unroll
    for (int d = 0; d < 4; d++) r[d] = z[d] | ((g[d] << 8) - g[d]);  // (x << 8) - x = 0xFF per set byte
    return r;
}

__device__ __forceinline__ int popcount16(uint32_t word, uint32_t shift)
{
    return __builtin_popcount(__builtin_amdgcn_ubfe(word, shift, 16));
}

template <int TYPE, int KCH>
__global__ __launch_bounds__(kConvThreads) void conv_mfma(const ConvArgs p)
{
    constexpr int APL = Planes<TYPE>::A, BPL = Planes<TYPE>::B;
    constexpr int BM = 128, BN = 128;
    using Stager = TileStager<TYPE, BM, BN, KCH>;
    constexpr int Q = Stager::Q, A_DWORDS = Stager::A_DWORDS, B_DWORDS = Stager::B_DWORDS;

    __shared__ __attribute__((aligned(16))) uint32_t lds[2 * (A_DWORDS + B_DWORDS)];
    __shared__ int row_side[4][64];  // per wave: row-side sums for the epilogue

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31;                  // row of an A tile / column of a B tile
    const uint32_t shift = 16 * (lane >> 5);  // which 16 of the 32 k this lane feeds
    const int wm = wave & 1, wn = wave >> 1;
    const int tile_m = blockIdx.x % p.tiles_m, tile_n = blockIdx.x / p.tiles_m;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    Stager st;
    st.init(p, tid, m0, n0);

    i32x16 acc[2][2];
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[mt][nt][e] = 0;
    int a_side[2] = {0, 0}, b_side[2] = {0, 0};

    st.fetch(p, 0);
    st.stage(lds);
    __syncthreads();

    for (int chunk = 0; chunk < p.nchunks; chunk++) {
        const bool more = chunk + 1 < p.nchunks;
        if (more) st.fetch(p, chunk + 1);

        const uint32_t *la = lds + (chunk & 1) * (A_DWORDS + B_DWORDS), *lb = la + A_DWORDS;
        const int words_here = (p.G - chunk * p.kcw < p.kcw) ? p.G - chunk * p.kcw : p.kcw;
        const int nq = 2 * words_here;
        for (int q = 0; q < nq; q++) {
            uint32_t aw[APL][2], bw[BPL][2];
#pragma unroll
            for (int pl = 0; pl < APL; pl++)
#pragma unroll
                for (int mt = 0; mt < 2; mt++) aw[pl][mt] = la[(pl * Q + q) * BM + wm * 64 + mt * 32 + r];
#pragma unroll
            for (int pl = 0; pl < BPL; pl++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++) bw[pl][nt] = lb[(pl * Q + q) * BN + wn * 64 + nt * 32 + r];

            i32x4 af[2], bf[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                if (APL == 2) {
                    af[t] = expand_ternary(aw[0][t], aw[APL - 1][t], shift);
                    if (TYPE == 1)  // sum of a_k over this lane's 16 positions
                        a_side[t] += popcount16(aw[APL - 1][t], shift) - 2 * popcount16(aw[0][t] & aw[APL - 1][t], shift);
                } else {
                    af[t] = expand01(aw[0][t], shift);
                    if (TYPE == 3) a_side[t] += popcount16(aw[0][t], shift);
                }
                if (BPL == 2) {
                    bf[t] = expand_ternary(bw[0][t], bw[BPL - 1][t], shift);
                    if (TYPE == 2) b_side[t] += popcount16(bw[0][t] & bw[BPL - 1][t], shift);
                } else {
                    bf[t] = expand01(bw[0][t], shift);
                    if (TYPE == 3) b_side[t] += popcount16(bw[0][t], shift);
                }
            }
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++)
                    acc[mt][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[mt], bf[nt], acc[mt][nt], 0, 0, 0);
        }

        if (more) st.stage(lds + ((chunk + 1) & 1) * (A_DWORDS + B_DWORDS));
        __syncthreads();
    }

    // ---- epilogue ------------------------------------------------------------------------
    // the two lanes r and r+32 hold the two halves of every side sum
#pragma unroll
    for (int t = 0; t < 2; t++) {
        a_side[t] += __shfl_xor(a_side[t], 32, 64);
        b_side[t] += __shfl_xor(b_side[t], 32, 64);
    }
    if (TYPE == 1 || TYPE == 3) {  // row sums live in the lane of their row; outputs need them by row index
        if (lane < 32) {
            row_side[wave][r] = a_side[0];
            row_side[wave][32 + r] = a_side[1];
        }
        __syncthreads();
    }
    // accumulator element 4*j + i of lane (kb, r) is C[8*j + 4*kb + i][r]
#pragma unroll
    for (int nt = 0; nt < 2; nt++) {
        const int col = n0 + wn * 64 + nt * 32 + r;
        const bool col_ok = col < p.KN;
        const int bias = (TYPE == 2 && col_ok) ? p.btn[col] : 0;
#pragma unroll
        for (int mt = 0; mt < 2; mt++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int row_l = mt * 32 + 8 * j + 4 * (lane >> 5) + i;
                    const int m = m0 + wm * 64 + row_l;
                    const int d = acc[mt][nt][4 * j + i];
                    int v;
                    if (TYPE == 0) v = d;
                    else if (TYPE == 1) v = row_side[wave][row_l] - 2 * d;
                    else if (TYPE == 2) v = bias - 2 * (d + b_side[nt]);
                    else v = p.num - 2 * (row_side[wave][row_l] + b_side[nt] - 2 * d);
                    if (col_ok && m < p.M) p.y[(size_t)m * p.KN + col] = (float)v;
                }
    }
}

template <int TYPE>
hipError_t launch_mfma(ConvArgs a, hipStream_t stream)
{
    constexpr int KCH = 4;
    a.nchunks = (a.G + KCH - 1) / KCH;
    a.kcw = (a.G + a.nchunks - 1) / a.nchunks;
    a.nchunks = (a.G + a.kcw - 1) / a.kcw;
    a.tiles_m = (a.M + 127) / 128;
    const long blocks = (long)a.tiles_m * ((a.KN + 127) / 128);
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    conv_mfma<TYPE, KCH><<<dim3((unsigned)blocks), dim3(kConvThreads), 0, stream>>>(a);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_conv_mfma(int type, const ConvArgs &args, hipStream_t stream)
{
    switch (type) {
    case 0: return launch_mfma<0>(args, stream);
    case 1: return launch_mfma<1>(args, stream);
    case 2: return launch_mfma<2>(args, stream);
    case 3: return launch_mfma<3>(args, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace tab
