// Fused zero-pad + im2row + popcount GEMM for gfx950 (wave64), all four TAB types.
//
// Replaces PadKernel + Img2RowKernel (TAB_GEMM.cuh:73-115) and TNNGEMM/TBNGEMM/BTNGEMM/
// BNNGEMM (TAB_GEMM.cu:25-147): Y[m][kn] = f(sum over k of popcount(op(A[m][k], B[kn][k])))
// with A the im2row view of the packed activation, never materialised: padding and stride
// live in the address math, out-of-range taps read all-zero words (TAB_CPU.cpp:39,155).
//
// Work decomposition: a 256-thread workgroup owns a BM x BN tile of Y (BM = 16*TM output
// pixels, BN = 64*NG filters); thread (ty, tx) of the 16x16 grid owns rows ty*TM.. and the
// column quads g*64 + tx*4.. .  K is walked in chunks of `kcw` packed 64-bit words; each
// chunk of both operands is staged in LDS, split into 32-bit halves and stored k-major
// ([plane][q][row], q = 2*word + half) so that a thread fetches its TM rows / 4 columns of
// one k-slice with 128-bit LDS reads (A reads broadcast over the 16 tx lanes, B reads are
// 256 B contiguous per 16 lanes).  The inner loop is pure VALU: XOR/AND + v_bcnt_u32_b32
// with the count accumulated in the instruction's addend.
#include "tab_conv_shape_model.h"
#include "tab_conv_stage.h"

#include <atomic>

namespace tab {
namespace {

constexpr int kThreads = kConvThreads;

// Inner-loop primitives.  Measured on MI355X (tab_amd/lib/valu_peak and register-level probes):
// a SIMD issues v_xor/v_and/v_bitop3 in 2 cycles and v_bcnt_u32_b32 in 4, but only when one
// scalar `s_nop 0` sits between the logic op and its v_bcnt (xor+bcnt back to back: 8.6 cycles
// per wave; xor, s_nop, bcnt: 6.4; a nop after the bcnt as well: 8.4 again), and only with an
// even number of waves per SIMD.  The compiler puts a nop of its own between any two asm
// statements, so each statement below covers four word pairs of one row: (logic, nop, bcnt) x 4.
// v_bcnt carries the accumulator as its addend.
#define TAB_XB(n) "v_xor_b32 %[t], %[a], %[b" #n "]\n\ts_nop 0\n\tv_bcnt_u32_b32 %[c" #n "], %[t], %[c" #n "]\n\t"
#define TAB_TB(n, m) \
    "v_bitop3_b32 %[t], %[a], %[b" #n "], %[" m "] bitop3:0x28\n\ts_nop 0\n\tv_bcnt_u32_b32 %[c" #n "], %[t], %[c" #n "]\n\t"
#define TAB_TNN(n)                                                                                            \
    "v_and_b32 %[u], %[a1], %[m" #n "]\n\ts_nop 0\n\tv_bcnt_u32_b32 %[z" #n "], %[u], %[z" #n "]\n\t"         \
    "v_bitop3_b32 %[t], %[a], %[b" #n "], %[u] bitop3:0x28\n\ts_nop 0\n\tv_bcnt_u32_b32 %[c" #n "], %[t], %[c" #n "]\n\t"

// c[j] += popcount(a ^ b[j]), j = 0..3                                        (BNN, TAB_GEMM.cu:142)
__device__ __forceinline__ void bnn_quad(int *c, uint32_t a, const uint32_t *b)
{
    uint32_t t;
    asm(TAB_XB(0) TAB_XB(1) TAB_XB(2) TAB_XB(3)
        : [c0] "+v"(c[0]), [c1] "+v"(c[1]), [c2] "+v"(c[2]), [c3] "+v"(c[3]), [t] "=&v"(t)
        : [a] "v"(a), [b0] "v"(b[0]), [b1] "v"(b[1]), [b2] "v"(b[2]), [b3] "v"(b[3]));
}
// c[j] += popcount((a ^ b[j]) & m), j = 0..3: one v_bitop3_b32 (truth table 0x28 for operands
// 0xF0, 0xCC, 0xAA) per pair                                             (TBN, TAB_GEMM.cu:81-84)
__device__ __forceinline__ void tbn_quad(int *c, uint32_t a, uint32_t m, const uint32_t *b)
{
    uint32_t t;
    asm(TAB_TB(0, "m") TAB_TB(1, "m") TAB_TB(2, "m") TAB_TB(3, "m")
        : [c0] "+v"(c[0]), [c1] "+v"(c[1]), [c2] "+v"(c[2]), [c3] "+v"(c[3]), [t] "=&v"(t)
        : [a] "v"(a), [m] "v"(m), [b0] "v"(b[0]), [b1] "v"(b[1]), [b2] "v"(b[2]), [b3] "v"(b[3]));
}
// c[j] += popcount((a ^ b[j]) & m[j]), j = 0..3                          (BTN, TAB_GEMM.cu:113-114)
__device__ __forceinline__ void btn_quad(int *c, uint32_t a, const uint32_t *b, const uint32_t *m)
{
    uint32_t t;
    asm(TAB_TB(0, "m0") TAB_TB(1, "m1") TAB_TB(2, "m2") TAB_TB(3, "m3")
        : [c0] "+v"(c[0]), [c1] "+v"(c[1]), [c2] "+v"(c[2]), [c3] "+v"(c[3]), [t] "=&v"(t)
        : [a] "v"(a), [b0] "v"(b[0]), [b1] "v"(b[1]), [b2] "v"(b[2]), [b3] "v"(b[3]), [m0] "v"(m[0]),
          [m1] "v"(m[1]), [m2] "v"(m[2]), [m3] "v"(m[3]));
}
// both = a1 & m[j]; z[j] += popcount(both); c[j] += popcount((a ^ b[j]) & both)   (TNN, TAB_GEMM.cu:48-51)
__device__ __forceinline__ void tnn_quad(int *z, int *c, uint32_t a, uint32_t a1, const uint32_t *b, const uint32_t *m)
{
    uint32_t t, u;
    asm(TAB_TNN(0) TAB_TNN(1) TAB_TNN(2) TAB_TNN(3)
        : [z0] "+v"(z[0]), [z1] "+v"(z[1]), [z2] "+v"(z[2]), [z3] "+v"(z[3]), [c0] "+v"(c[0]), [c1] "+v"(c[1]),
          [c2] "+v"(c[2]), [c3] "+v"(c[3]), [t] "=&v"(t), [u] "=&v"(u)
        : [a] "v"(a), [a1] "v"(a1), [b0] "v"(b[0]), [b1] "v"(b[1]), [b2] "v"(b[2]), [b3] "v"(b[3]), [m0] "v"(m[0]),
          [m1] "v"(m[1]), [m2] "v"(m[2]), [m3] "v"(m[3]));
}
// acc += popcount(x)
__device__ __forceinline__ void popcount_acc(int &acc, uint32_t x)
{
    asm("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc) : "v"(x));
}

// TM rows x 4*NG columns per thread; KCH = packed 64-bit words of K per chunk, at most;
// PIPE = operand fragments double-buffered in registers (costs APL*TM + BPL*4*NG VGPRs).
// 256 threads: one wave per SIMD (512-thread workgroups were measured slightly slower).
template <int TYPE, int TM, int NG, int KCH, bool PIPE>
__global__ __launch_bounds__(kThreads) void conv_popcount(const ConvArgs p)
{
    constexpr int APL = Planes<TYPE>::A, BPL = Planes<TYPE>::B;
    constexpr int BM = 16 * TM, BN = 64 * NG, TN = 4 * NG;
    using Stager = TileStager<TYPE, BM, BN, KCH>;
    constexpr int kMaxQ = Stager::Q, A_DWORDS = Stager::A_DWORDS, B_DWORDS = Stager::B_DWORDS;
    static_assert(TM % 4 == 0 || TM == 2, "TM is read with 64- or 128-bit LDS loads");

    // + one spare k-slice of the wider operand: the pipelined loop reads one slice ahead
    __shared__ __attribute__((aligned(16))) uint32_t lds[2 * (A_DWORDS + B_DWORDS) + (BM > BN ? BM : BN)];

    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    // consecutive workgroups walk M first so neighbours share the weight tile in L2
    const int tile_n = (int)div32(blockIdx.x, p.div_tiles_m), tile_m = (int)blockIdx.x - tile_n * p.tiles_m;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    Stager st;
    st.init(p, tid, m0, n0);

    // ---- accumulators --------------------------------------------------------------------
    // acc: popcount of the "negative" word (TNN/TBN/BTN) or of a^b (BNN);
    // nzc: TNN popcount(a1 & b1) per output; TBN popcount(a1) per row (independent of kn).
    int acc[TM][TN];
    int nzc[TYPE == 0 ? TM : 1][TYPE == 0 ? TN : 1];
    int row_nz[TYPE == 1 ? TM : 1];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            acc[i][j] = 0;
            if (TYPE == 0) nzc[i][j] = 0;
        }
    if (TYPE == 1) {
#pragma unroll
        for (int i = 0; i < TM; i++) row_nz[i] = 0;
    }

    // One k-slice (32 bits of K) of this thread's operands.
    struct Frag {
        uint32_t a[APL][TM], b[BPL][TN];
    };
    auto read_frag = [&](Frag &f, const uint32_t *la, const uint32_t *lb, int q) {
#pragma unroll
        for (int pl = 0; pl < APL; pl++) {
            const uint32_t *src = la + (pl * kMaxQ + q) * BM + ty * TM;
            if (TM == 2) {
                const u32x2 v = *reinterpret_cast<const u32x2 *>(src);
                f.a[pl][0] = v[0]; f.a[pl][1] = v[1];
            } else {
#pragma unroll
                for (int i4 = 0; i4 < TM / 4; i4++) {
                    const u32x4 v = *reinterpret_cast<const u32x4 *>(src + 4 * i4);
#pragma unroll
                    for (int e = 0; e < 4; e++) f.a[pl][4 * i4 + e] = v[e];
                }
            }
        }
#pragma unroll
        for (int pl = 0; pl < BPL; pl++)
#pragma unroll
            for (int g = 0; g < NG; g++) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(lb + (pl * kMaxQ + q) * BN + g * 64 + tx * 4);
#pragma unroll
                for (int e = 0; e < 4; e++) f.b[pl][4 * g + e] = v[e];
            }
    };
    auto mac = [&](const Frag &f) {
        if (TYPE == 1) {
#pragma unroll
            for (int i = 0; i < TM; i++) popcount_acc(row_nz[i], f.a[APL - 1][i]);
        }
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j += 4) {
                if (TYPE == 0)
                    tnn_quad(&nzc[i][j], &acc[i][j], f.a[0][i], f.a[1][i], &f.b[0][j], &f.b[1][j]);
                else if (TYPE == 1)
                    tbn_quad(&acc[i][j], f.a[0][i], f.a[1][i], &f.b[0][j]);  // popcount(a1) is summed once per row above
                else if (TYPE == 2)
                    btn_quad(&acc[i][j], f.a[0][i], &f.b[0][j], &f.b[1][j]);
                else
                    bnn_quad(&acc[i][j], f.a[0][i], &f.b[0][j]);
            }
    };

    st.fetch(p, 0);
    st.stage(lds);
    __syncthreads();

    for (int chunk = 0; chunk < p.nchunks; chunk++) {
        const bool more = chunk + 1 < p.nchunks;
        if (more) st.fetch(p, chunk + 1);

        const uint32_t *la = lds + (chunk & 1) * (A_DWORDS + B_DWORDS), *lb = la + A_DWORDS;
        const int words_here = (p.G - chunk * p.kcw < p.kcw) ? p.G - chunk * p.kcw : p.kcw;
        const int nq = 2 * words_here;
        // Register double buffering: the LDS reads of k-slice q+1 are issued before the VALU
        // work of slice q, so a single wave per SIMD still keeps the VALU busy.  nq is even.
        // The read of slice nq after the last pair stays inside the LDS allocation (one spare
        // slice is reserved) and its value is never used.
        if (PIPE) {
            Frag f0, f1;
            // drain outstanding scalar loads first: they share the LDS counter and return out
            // of order, which would force full waits inside the loop
            __builtin_amdgcn_s_waitcnt(0xc07f);
            read_frag(f0, la, lb, 0);
            for (int q = 0; q < nq; q += 2) {
                read_frag(f1, la, lb, q + 1);
                __builtin_amdgcn_sched_barrier(0);
                mac(f0);
                __builtin_amdgcn_sched_barrier(0);
                read_frag(f0, la, lb, q + 2);
                __builtin_amdgcn_sched_barrier(0);
                mac(f1);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            for (int q = 0; q < nq; q++) {
                Frag f;
                read_frag(f, la, lb, q);
                mac(f);
            }
        }

        if (more) st.stage(lds + ((chunk + 1) & 1) * (A_DWORDS + B_DWORDS));
        __syncthreads();
    }

    // ---- epilogue: integer result -> fp32, Y[m*KN + kn] (TAB_GEMM.cu:53,86,116,144) --------
    const bool vec_ok = (p.KN & 3) == 0;
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const int kn = n0 + g * 64 + tx * 4;
        int bias[4] = {0, 0, 0, 0};
        if (TYPE == 2) {
#pragma unroll
            for (int e = 0; e < 4; e++) bias[e] = (kn + e < p.KN) ? p.btn[kn + e] : 0;
        }
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const int m = m0 + ty * TM + i;
            if (m >= p.M) continue;
            float out[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int j = 4 * g + e;
                int v;
                if (TYPE == 0) v = nzc[i][j] - 2 * acc[i][j];
                else if (TYPE == 1) v = row_nz[i] - 2 * acc[i][j];
                else if (TYPE == 2) v = bias[e] - 2 * acc[i][j];
                else v = p.num - 2 * acc[i][j];
                out[e] = (float)v;
            }
            float *dst = p.y + (size_t)m * p.KN + kn;
            if (vec_ok && kn + 3 < p.KN) {
                *reinterpret_cast<f32x4 *>(dst) = f32x4{out[0], out[1], out[2], out[3]};
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (kn + e < p.KN) dst[e] = out[e];
            }
        }
    }
}

// Extra (unused) dynamic LDS per workgroup that makes the number of resident workgroups per
// CU - one wave per SIMD each - even: the VALU pairing above only pays off with an even number
// of waves per SIMD (2 or 4; 3 measured as slow as no pairing at all).
struct Occupancy {
    int dyn_lds;        // bytes of padding LDS per workgroup
    int blocks_per_cu;  // resident workgroups per CU with that padding (0 = unknown)
};

template <typename Kernel>
Occupancy even_occupancy(Kernel kernel)
{
    for (int dyn = 0; dyn <= 48 * 1024; dyn += 2048) {
        int blocks = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, kernel, kThreads, dyn) != hipSuccess) {
            (void)hipGetLastError();
            return {0, 0};
        }
        if (blocks <= 2 || (blocks & 1) == 0) return {dyn, blocks};
    }
    return {0, 0};
}

template <int TYPE, int TM, int NG, int KCH, bool PIPE = true>
hipError_t launch_tile(ConvArgs a, hipStream_t stream)
{
    constexpr int BM = 16 * TM, BN = 64 * NG;
    static const Occupancy occ = even_occupancy(conv_popcount<TYPE, TM, NG, KCH, PIPE>);
    // chunk length: at most KCH words, chunks of equal length
    a.nchunks = (a.G + KCH - 1) / KCH;
    a.kcw = (a.G + a.nchunks - 1) / a.nchunks;
    a.nchunks = (a.G + a.kcw - 1) / a.kcw;
    a.tiles_m = (a.M + BM - 1) / BM;
    a.div_tiles_m = make_div32((uint32_t)a.tiles_m);
    const long tiles_n = (a.KN + BN - 1) / BN;
    const long blocks = (long)a.tiles_m * tiles_n;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    conv_popcount<TYPE, TM, NG, KCH, PIPE><<<dim3((unsigned)blocks), dim3(kThreads), occ.dyn_lds, stream>>>(a);
    return hipGetLastError();
}

// Kernel choice of tab_set_conv_kernel, (tm << 8) | (ng + 1) in one atomic word so that a launch on another
// thread sees either the old or the new pair, never a mix; 0 = the automatic choice.
std::atomic<int> g_forced_kernel{0};
struct Forced { int tm, ng; };
inline Forced forced_kernel()
{
    const int v = g_forced_kernel.load(std::memory_order_relaxed);
    return {v >> 8, (v & 0xff) - 1};
}

// Tile shapes.  Every shape keeps <= 128 VGPRs, i.e. at least 4 workgroups (4 waves per SIMD)
// per CU; shapes with 128 accumulators at 2 waves per SIMD and 512-thread workgroups were
// measured 10-25 % slower.  Three shapes are used:
//   big    128x128 (128x64 for TNN, which keeps two counts per output), chunks of 4 words;
//          fragments register double-buffered only where that still fits 128 VGPRs (BNN)
//   medium 64x64, chunks of 4 words, double-buffered fragments, 8 workgroups per CU
//   small  32x64, chunks of 8 words
// Measured over the ResNet-18 / sweep shapes at N = 32..256: the medium tile wins everywhere
// except on the very largest launches (>= 3 rounds of big tiles over the whole chip), and the
// small tile wins once even medium tiles give the CUs fewer than two workgroups each.
template <int TYPE>
hipError_t launch_big(const ConvArgs &a, hipStream_t stream)
{
    if constexpr (TYPE == 0)
        return launch_tile<TYPE, 8, 1, 4, false>(a, stream);
    else if constexpr (TYPE == 3)
        return launch_tile<TYPE, 8, 2, 4, true>(a, stream);
    else
        return launch_tile<TYPE, 8, 2, 4, false>(a, stream);
}

template <int TYPE>
hipError_t launch_type(const ConvArgs &a, hipStream_t stream)
{
    constexpr int BIG_BN = (TYPE == 0) ? 64 : 128;
    const int force_tm = forced_kernel().tm;
    if (force_tm == 8) return launch_big<TYPE>(a, stream);
    if (force_tm == 4) return launch_tile<TYPE, 4, 1, 4, true>(a, stream);
    if (force_tm == 2) return launch_tile<TYPE, 2, 1, 8, true>(a, stream);
    auto tiles = [&](int bm, int bn) { return (long)((a.M + bm - 1) / bm) * ((a.KN + bn - 1) / bn); };
    if (a.KN > BIG_BN / 2 && tiles(128, BIG_BN) >= 3072) return launch_big<TYPE>(a, stream);
    if (tiles(64, 64) >= 512) return launch_tile<TYPE, 4, 1, 4, true>(a, stream);
    return launch_tile<TYPE, 2, 1, 8, true>(a, stream);
}

}  // namespace

void force_conv_tile(int tm, int ng)
{
    g_forced_kernel.store(tm == 0 ? 0 : ((tm << 8) | ((ng + 1) & 0xff)), std::memory_order_relaxed);
}

int device_compute_units()
{
    static std::atomic<int> cached{0};
    int cus = cached.load(std::memory_order_relaxed);
    if (cus == 0) {
        int device = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&device) == hipSuccess && hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0) {
            cus = prop.multiProcessorCount;
        } else {
            (void)hipGetLastError();
            cus = 256;
        }
        cached.store(cus, std::memory_order_relaxed);
    }
    return cus;
}

std::atomic<int> g_tail_round{0};
void set_tail_round(int workgroups) { g_tail_round.store(workgroups > 0 ? workgroups : 0, std::memory_order_relaxed); }
int tail_round()
{
    const int forced = g_tail_round.load(std::memory_order_relaxed);
    return forced > 0 ? forced : device_compute_units();
}

bool conv_kernel_forced() { return g_forced_kernel.load(std::memory_order_relaxed) != 0; }

// fp32 accumulators hold integers up to 2^24 exactly; a product is at most 1 (9 for the 2-bit levels of
// type 4, see conv_mfma_exact_levels) and there are 64 per word
bool conv_mfma_exact(const ConvArgs &a) { return (long)a.G * 64 <= (1L << 22); }
bool conv_mfma_exact_levels(const ConvArgs &a) { return (long)a.G * 64 * 9 < (1L << 24); }

hipError_t launch_conv_mfma(int type, const ConvArgs &args, int shape, hipStream_t stream)
{
    if (!conv_mfma_exact(args)) return hipErrorInvalidValue;
    switch (type) {
    case 0: return launch_conv_mfma_tnn(args, shape, stream);
    case 1: return launch_conv_mfma_tbn(args, shape, stream);
    case 2: return launch_conv_mfma_btn(args, shape, stream);
    case 3: return launch_conv_mfma_bnn(args, shape, stream);
    case 4: return conv_mfma_exact_levels(args) ? launch_conv_mfma_drf(args, shape, stream) : hipErrorInvalidValue;
    case 5: return launch_conv_mfma_rtn(args, shape, stream);
    default: return hipErrorInvalidValue;
    }
}

// Workgroup tile of the matrix-core kernel: the shape with the lowest predicted duration under a cost model fitted to
// the measured duration of every shape on some 290 (type, layer) cases (tab_conv_shape_model.h: the ResNet-18 layers at
// N = 16 / 64 / 256, the VGG stack, the 28x28 sweep and layers of other geometries).  What the model's features say:
// the busiest CU decides (ceil(tiles / CUs) tiles of a shape land on it, and it is refilled when it holds no more), K
// scales the loop, the size of Y the epilogue (with a price of its own where K is at most nine words and the launch is
// little but epilogue), and a launch smaller than the chip is as long as one tile.  Features and coefficients are all
// non-negative, so a prediction is positive and monotone in K, tiles and Y for any geometry; on top of that no prediction
// is taken below what the matrix cores of the busiest CU need at their peak rate plus a launch.
// A shape whose filter tile is at least twice the 64-rounded filter count is no candidate.
// cost_us (optional): the predicted duration of the chosen shape.
int conv_mfma_shape(int conv_type, const ConvArgs &a, float *cost_us)
{
    // the CPU-only types follow the type with the same planes: 4 like TNN, 5 like BNN
    const int type = conv_type == 4 ? 0 : (conv_type == 5 ? 3 : conv_type);
    // K of at most nine words and packed output: the kernel with the weights resident in registers, whose epilogue
    // thresholds a pixel's filters inside a lane, runs 1.4-2x faster than the tiled shapes once the launch is a few
    // rounds of waves (N=256 56x56x64->64 3x3: 24 against 38 us) and level with them on small ones; with fp32 output
    // both are bound by writing Y and measure within 5 % of each other, so the tiled shapes keep those launches
    if (conv_type <= 3 && a.G <= 9 && a.qy != nullptr && (a.M >= 65536 || a.G <= 2)) {
        if (cost_us) *cost_us = 0.f;
        return 7;
    }
    const long kn64 = ((long)a.KN + 63) / 64 * 64;
    const long cus = device_compute_units();
    // (packed output ranks the shapes as fp32 output does: the model's terms in Y also stand for what grows with M * KN)
    const float y_mb = (float)a.M * (float)a.KN * 4e-6f;
    int best = 2;
    float best_cost = 0.f;
    bool any = false;
    for (int i = 0; i < kConvShapes; i++) {
        const int shape = kConvShapeIds[i];
        const int bm = kConvShapeTile[i][0], bn = kConvShapeTile[i][1], held = kConvShapeTile[i][2];
        if (bn >= 2 * kn64) continue;
        if (shape == 3 && a.qy != nullptr) continue;        // the packed epilogues need tiles 64 filters wide
        if (shape >= 8 && a.PC % 2 != 0) continue;          // the split-K shapes move whole pairs of words inside a tap
        const long tiles = (long)((a.M + bm - 1) / bm) * ((a.KN + bn - 1) / bn);
        float cost = 0.f, floor_us;
        if (shape == 10 || shape == 11) {
            // the mixed launches: whole tiles on every CU, then 64x64 quarter tiles (four to a 128x128 tile, eight to a
            // 128x256 one); candidates where they have both and K words x bit planes of the two operands exceed 36 (below
            // that the launch is bound by writing Y, whatever the balance of its last round)
            const long pieces = bm / 64 * (bn / 64);
            const long whole = tiles / cus, quarters = (pieces * (tiles % cus) + cus - 1) / cus;
            const int planes = type == 0 ? 4 : (type == 3 ? 2 : 3);
            if (a.G * planes <= 36 || whole == 0 || quarters == 0) continue;  // (an odd number of words per pixel: excluded above)
            if (shape == 11 && a.PC % 4 != 0) continue;                       // the 128x256 tiles take four-word chunks inside a tap
            const float f[kConvShapeFeatures] = {(float)a.G * (float)whole, (float)a.G * (float)quarters, (float)quarters, (float)whole, y_mb, y_mb,
                                                 1.f, 1.f, 0.f};
            for (int k = 0; k < kConvShapeFeatures; k++) cost += kConvShapeCost[type][i][k] * f[k];
            floor_us = 1.f + (float)(4 * pieces * whole + 4 * quarters) * (float)a.G * (32.f / 4.f / 2400.f);
        } else {
            const float n = (float)((tiles + cus - 1) / cus), rounds = (float)(((tiles + cus - 1) / cus + held - 1) / held);
            const float busy = tiles >= cus ? 1.f : (float)tiles / (float)cus;
            const float f[kConvShapeFeatures] = {(float)a.G * n, (float)a.G * rounds, rounds, n, y_mb, y_mb * busy, busy, 1.f,
                                                 a.G <= 9 ? y_mb : 0.f};
            for (int k = 0; k < kConvShapeFeatures; k++) cost += kConvShapeCost[type][i][k] * f[k];
            // the busiest CU's n tiles of (bm/32)(bn/32) MFMA tiles x G words, 32 cycles each on four SIMDs at 2.4 GHz, and a launch
            floor_us = 1.f + n * (float)(bm / 32 * (bn / 32)) * (float)a.G * (32.f / 4.f / 2400.f);
        }
        if (cost < floor_us) cost = floor_us;
        if (!any || cost < best_cost) {
            any = true;
            best = shape;
            best_cost = cost;
        }
    }
    if (cost_us) *cost_us = best_cost;
    return best;
}

hipError_t launch_conv(int type, const ConvArgs &args, hipStream_t stream)
{
    const Forced forced = forced_kernel();
    const int force_tm = forced.tm, force_ng = forced.ng;
    if (args.qy != nullptr) {  // packed output exists in the matrix-core kernel's 64-wide shapes only
        if (!conv_mfma_exact(args)) return hipErrorInvalidValue;
        const int shape = (force_tm == 9 && force_ng >= 0 && force_ng != 3 && force_ng <= 11) ? force_ng : conv_mfma_shape(type, args);
        return launch_conv_mfma(type, args, shape, stream);
    }
    if (force_tm == 9) return launch_conv_mfma(type, args, force_ng < 0 ? conv_mfma_shape(type, args) : force_ng, stream);
    // default path: matrix cores; the popcount kernel takes over when K is too long for exact fp32
    // accumulation (and when a benchmark forces one of its tiles)
    if (force_tm == 0 && conv_mfma_exact(args)) return launch_conv_mfma(type, args, conv_mfma_shape(type, args), stream);
    // types 4 and 5 exist on the matrix cores only
    if (type > 3) return launch_conv_mfma(type, args, conv_mfma_shape(type, args), stream);
    switch (type) {
    case 0: return launch_type<0>(args, stream);
    case 1: return launch_type<1>(args, stream);
    case 2: return launch_type<2>(args, stream);
    case 3: return launch_type<3>(args, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace tab
