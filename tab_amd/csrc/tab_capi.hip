// C ABI of the library (declared in include/tab_amd.h): argument checks, workspace
// carving and kernel launches.  No allocation, no synchronisation, no host<->device copy.
#include "../../include/tab_amd.h"
#include "tab_common.h"

#include <cstdarg>
#include <cstdio>
#include <mutex>

// Packed-activation scratch of tab_conv2d_static, one copy per GPU the library is loaded on.  In host code this
// name is only a handle for hipGetSymbolAddress; the device address is looked up once per device (static_scratch
// below) and that pointer is what the kernels get.
static __device__ __align__(256) unsigned char scratch[TAB_STATIC_SCRATCH_BYTES];

namespace {

thread_local char g_last_error[512] = "";

int fail(int status, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return status;
}

int device_fail(hipError_t e, const char *what)
{
    return fail(TAB_ERR_DEVICE, "%s: %s", what, hipGetErrorString(e));
}

constexpr long kMaxIndex = 0x7fffffffL;  // kernels index rows/pixels with 32-bit ints

struct ConvShape {
    int PC, OH, OW, abits, wbits;
    long M, G;
};

// Shared validation of the conv geometry (TAB_GEMM.cu:354-379).
int check_conv(int type, int p1, int p2, int s1, int s2, int N, int H, int W, int C, int KN,
               int KH, int KW, ConvShape *s)
{
    if (type < 0 || type > 5)
        return fail(TAB_ERR_BAD_ARGUMENT, "type must be 0 (TNN), 1 (TBN), 2 (BTN), 3 (BNN), 4 (DRF) or 5 (RTN), got %d", type);
    if (N < 1 || H < 1 || W < 1 || C < 1 || KN < 1 || KH < 1 || KW < 1)
        return fail(TAB_ERR_BAD_ARGUMENT, "N, H, W, C, KN, KH, KW must be positive");
    if (p1 < 0 || p2 < 0 || s1 < 1 || s2 < 1)
        return fail(TAB_ERR_BAD_ARGUMENT, "padding must be >= 0 and stride >= 1");
    s->PC = type == TAB_RTN ? (C + 31) / 32 : tab_packed_channels(C);
    s->OH = tab_out_extent(H, p1, KH, s1);
    s->OW = tab_out_extent(W, p2, KW, s2);
    if (s->OH < 1 || s->OW < 1)
        return fail(TAB_ERR_BAD_SHAPE, "empty output: OH=%d OW=%d", s->OH, s->OW);
    s->abits = (type < 2 || type == TAB_DRF) ? 2 : 1;  // planes per word position, TAB_CPU.cpp:345-354 for type 4
    s->wbits = (type == 0 || type == 2 || type == TAB_DRF) ? 2 : 1;
    s->M = (long)N * s->OH * s->OW;
    s->G = (long)KH * KW * s->PC;
    if (s->M > kMaxIndex - 512 || s->G >= 65536 || s->PC >= 65536 || KW >= 65536 ||
        (long)N * H * W > kMaxIndex || (long)H * W * s->PC * 2 > kMaxIndex)
        return fail(TAB_ERR_BAD_SHAPE, "problem too large for 32-bit row indices (M=%ld, K words=%ld)", s->M, s->G);
    // type 4 multiplies levels up to 3: 9 * 64 * G has to stay below 2^24 for the fp32 accumulators
    if (type == TAB_DRF && s->G * 64 * 9 >= (1L << 24))
        return fail(TAB_ERR_BAD_SHAPE, "K of %ld words is too long for exact accumulation of type 4", s->G);
    // a workgroup addresses the images its (at most 256) output pixels touch with 32-bit byte offsets
    const long image_bytes = (long)H * W * s->PC * s->abits * 8;
    if (image_bytes * (256 / ((long)s->OH * s->OW) + 2) > 0xffffffffL)
        return fail(TAB_ERR_BAD_SHAPE, "packed image of %ld bytes is too large for 32-bit offsets", image_bytes);
    // a wave addresses its (at most 128) rows of Y with 32-bit byte offsets below 2 GiB
    if ((long)KN * 4 * 128 >= (1L << 31))
        return fail(TAB_ERR_BAD_SHAPE, "KN=%d is too large for 32-bit offsets into a tile of Y", KN);
    return TAB_OK;
}

}  // namespace

extern "C" {

const char *tab_status_string(int status)
{
    switch (status) {
    case TAB_OK: return "TAB_OK";
    case TAB_ERR_BAD_ARGUMENT: return "TAB_ERR_BAD_ARGUMENT";
    case TAB_ERR_BAD_SHAPE: return "TAB_ERR_BAD_SHAPE";
    case TAB_ERR_WORKSPACE: return "TAB_ERR_WORKSPACE";
    case TAB_ERR_DEVICE: return "TAB_ERR_DEVICE";
    default: return "TAB_ERR_UNKNOWN";
    }
}

const char *tab_last_error(void) { return g_last_error; }

const char *tab_version(void) { return "tab_amd 0.1 gfx950"; }

/* Test hook, absent from include/tab_amd.h: the kernels' multiply-shift division evaluated on the host (x < 2^31, 1 <= d < 2^31). */
uint32_t tab_internal_div32(uint32_t x, uint32_t d) { return tab::div32(x, tab::make_div32(d)); }

/* Test hook, absent from include/tab_amd.h: the matrix-core workgroup shape the library would pick for an M x KN output with
 * G = taps * PC words of K (packed: thresholded output), and the duration in microseconds its model predicts for it. */
int tab_internal_conv_shape(int type, int M, int KN, int G, int PC, int packed, float *cost_us)
{
    tab::ConvArgs a = {};
    a.M = M; a.KN = KN; a.G = G; a.PC = PC;
    a.qy = packed ? reinterpret_cast<uint32_t *>(&a) : nullptr;  // only tested against null
    return tab::conv_mfma_shape(type, a, cost_us);
}

/* Test hook, absent from include/tab_amd.h: the number of workgroups the mixed launch (TAB_CONV_MATRIX tile 10) counts as one
 * round of the chip; 0 = the device's compute units.  Small values let small test shapes mix whole tiles and quarters. */
void tab_internal_set_tail_round(int workgroups) { tab::set_tail_round(workgroups); }

int tab_set_conv_kernel(int kernel, int tile)
{
    static const int popcount_tm[4] = {7, 8, 4, 2};  // 7: the popcount kernel's own choice
    if (kernel == TAB_CONV_AUTO && tile == -1) tab::force_conv_tile(0, 0);
    else if (kernel == TAB_CONV_MATRIX && tile >= -1 && tile <= 11) tab::force_conv_tile(9, tile);
    else if (kernel == TAB_CONV_POPCOUNT && tile >= -1 && tile <= 2) tab::force_conv_tile(popcount_tm[tile + 1], 0);
    else return fail(TAB_ERR_BAD_ARGUMENT, "no conv kernel %d with tile %d", kernel, tile);
    return TAB_OK;
}

int tab_packed_channels(int C) { return (C + tab::kWordBits - 1) / tab::kWordBits; }

int tab_out_extent(int in, int pad, int k, int stride)
{
    if (stride < 1) return 0;
    return (in + 2 * pad - k + 1) / stride;
}

int tab_quantize(const float *dev_X, const float *dev_ths, int bitwidth, int N, int H, int W,
                 int C, int64_t *dev_QX, int32_t *dev_BTN, void *stream)
{
    if (bitwidth != 1 && bitwidth != 2) return fail(TAB_ERR_BAD_ARGUMENT, "bitwidth must be 1 or 2, got %d", bitwidth);
    if (N < 1 || H < 1 || W < 1 || C < 1) return fail(TAB_ERR_BAD_ARGUMENT, "N, H, W, C must be positive");
    if (!dev_X || !dev_ths || !dev_QX) return fail(TAB_ERR_BAD_ARGUMENT, "null device pointer");  // dev_BTN may be NULL
    if (((uintptr_t)dev_X % 4) || ((uintptr_t)dev_QX % (8 * bitwidth)))
        return fail(TAB_ERR_BAD_ARGUMENT, "X must be aligned to its floats and QX to a whole packed element (%d bytes)", 8 * bitwidth);
    hipError_t e = tab::launch_quantize(dev_X, dev_ths, bitwidth, (long)H * W, N, C,
                                        reinterpret_cast<uint64_t *>(dev_QX), dev_BTN,
                                        static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return device_fail(e, "quantize launch");
    return TAB_OK;
}

int tab_quantize_nchw(const float *dev_X, const float *dev_ths, int bitwidth, int N, int C, int H, int W,
                      int64_t *dev_QX, int32_t *dev_BTN, void *stream)
{
    if (bitwidth != 1 && bitwidth != 2) return fail(TAB_ERR_BAD_ARGUMENT, "bitwidth must be 1 or 2, got %d", bitwidth);
    if (N < 1 || H < 1 || W < 1 || C < 1) return fail(TAB_ERR_BAD_ARGUMENT, "N, C, H, W must be positive");
    if (!dev_X || !dev_ths || !dev_QX) return fail(TAB_ERR_BAD_ARGUMENT, "null device pointer");  // dev_BTN may be NULL
    if (((uintptr_t)dev_X % 4) || ((uintptr_t)dev_QX % (8 * bitwidth)))
        return fail(TAB_ERR_BAD_ARGUMENT, "X must be aligned to its floats and QX to a whole packed element (%d bytes)", 8 * bitwidth);
    if (((long)N * H * W + 255) / 256 * tab_packed_channels(C) > kMaxIndex)
        return fail(TAB_ERR_BAD_SHAPE, "tensor too large for one launch (N*H*W/256 * ceil(C/64) workgroups)");
    hipError_t e = tab::launch_quantize_nchw(dev_X, dev_ths, bitwidth, N, C, (long)H * W, reinterpret_cast<uint64_t *>(dev_QX),
                                             dev_BTN, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return device_fail(e, "quantize launch");
    return TAB_OK;
}

size_t tab_threshold_workspace_bytes(int N, long per_item)
{
    if (N < 1 || per_item < 1) return 0;
    return (size_t)N * tab::threshold_splits(N, per_item) * sizeof(float);
}

int tab_threshold(const float *dev_X, int N, long per_item, float scale, float *dev_ths, void *workspace,
                  size_t workspace_bytes, void *stream)
{
    if (N < 1 || per_item < 1) return fail(TAB_ERR_BAD_ARGUMENT, "N and per_item must be positive");
    if (!dev_X || !dev_ths) return fail(TAB_ERR_BAD_ARGUMENT, "null device pointer");
    const size_t need = tab_threshold_workspace_bytes(N, per_item);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace % 4))
        return fail(TAB_ERR_WORKSPACE, "workspace must hold %zu bytes (got %zu)", need, workspace_bytes);
    hipError_t e = tab::launch_threshold(dev_X, N, per_item, scale, dev_ths, static_cast<float *>(workspace),
                                         static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return device_fail(e, "threshold launch");
    return TAB_OK;
}

int tab_operand_words(int type, int operand, int C)
{
    if (type < 0 || type > 5 || operand < 0 || operand > 1 || C < 1) return 0;
    if (type == TAB_RTN) return (C + 31) / 32;
    const bool two_planes = type == TAB_DRF || (operand == 0 ? type < 2 : (type == 0 || type == 2));
    return tab_packed_channels(C) * (two_planes ? 2 : 1);
}

size_t tab_conv2d_workspace_bytes(int type, int N, int H, int W, int C)
{
    if (type < 0 || type > 5 || N < 1 || H < 1 || W < 1 || C < 1) return 0;
    return (size_t)N * H * W * tab_operand_words(type, 0, C) * sizeof(int64_t);
}

int tab_quantize_format(const float *dev_X, const float *dev_ths, int type, int N, int H, int W, int C,
                        int64_t *dev_QX, void *stream)
{
    if (type != TAB_DRF && type != TAB_RTN) return fail(TAB_ERR_BAD_ARGUMENT, "type must be 4 (DRF) or 5 (RTN), got %d", type);
    if (N < 1 || H < 1 || W < 1 || C < 1) return fail(TAB_ERR_BAD_ARGUMENT, "N, H, W, C must be positive");
    if (!dev_X || !dev_ths || !dev_QX) return fail(TAB_ERR_BAD_ARGUMENT, "null device pointer");
    if (((uintptr_t)dev_X % 4) || ((uintptr_t)dev_QX % 16))
        return fail(TAB_ERR_BAD_ARGUMENT, "X must be aligned to its floats and QX to 16 bytes");
    hipError_t e = tab::launch_quantize_format(dev_X, dev_ths, type, (long)H * W, N, C, reinterpret_cast<uint64_t *>(dev_QX),
                                               static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return device_fail(e, "quantize launch");
    return TAB_OK;
}

/* Pointer checks shared by every conv entry point; they run before anything is launched. */
static int check_conv_pointers(const ConvShape &s, int type, const void *dev_QX, const void *dev_QW, const void *dev_btn,
                               const void *dev_Y, const void *dev_QY)
{
    if (!dev_QX || !dev_QW || (!dev_Y && !dev_QY)) return fail(TAB_ERR_BAD_ARGUMENT, "null device pointer");
    if (type == TAB_BTN && !dev_btn) return fail(TAB_ERR_BAD_ARGUMENT, "btn is required for type 2 (BTN)");
    if (((uintptr_t)dev_QX % (8 * s.abits)) || ((uintptr_t)dev_QW % (8 * s.wbits)) || ((uintptr_t)dev_Y % 16))
        return fail(TAB_ERR_BAD_ARGUMENT, "QX/QW must be aligned to a whole packed element and Y to 16 bytes");
    return TAB_OK;
}

/* Shared body of the packed-activation entry points: Y as fp32 (dev_Y) or thresholded and packed (dev_QY). */
static int conv_packed(const int64_t *dev_QX, const int64_t *dev_QW, const int32_t *dev_btn, int type, int padding1,
                       int padding2, int stride1, int stride2, int N, int H, int W, int C, int KN, int KH, int KW,
                       float *dev_Y, const float *dev_out_ths, int out_bitwidth, int64_t *dev_QY, void *stream)
{
    ConvShape s;
    int rc = check_conv(type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW, &s);
    if (rc != TAB_OK) return rc;
    rc = check_conv_pointers(s, type, dev_QX, dev_QW, dev_btn, dev_Y, dev_QY);
    if (rc != TAB_OK) return rc;
    if (dev_QY) {
        if (out_bitwidth != 1 && out_bitwidth != 2)
            return fail(TAB_ERR_BAD_ARGUMENT, "out_bitwidth must be 1 or 2, got %d", out_bitwidth);
        if (!dev_out_ths) return fail(TAB_ERR_BAD_ARGUMENT, "null device pointer");
        if ((uintptr_t)dev_QY % (8 * out_bitwidth)) return fail(TAB_ERR_BAD_ARGUMENT, "QY must be aligned to a whole packed element");
    }

    tab::ConvArgs a;
    a.qx = reinterpret_cast<const uint64_t *>(dev_QX);
    a.qw = reinterpret_cast<const uint64_t *>(dev_QW);
    a.btn = dev_btn;
    a.y = dev_Y;
    a.qy = reinterpret_cast<uint32_t *>(dev_QY);
    a.out_ths = dev_out_ths;
    a.out_bits = out_bitwidth;
    a.N = N; a.H = H; a.W = W; a.PC = s.PC;
    a.KN = KN; a.KH = KH; a.KW = KW;
    a.p1 = padding1; a.p2 = padding2; a.s1 = stride1; a.s2 = stride2;
    a.OH = s.OH; a.OW = s.OW;
    a.M = (int)s.M;
    a.G = (int)s.G;
    a.kcw = 0; a.nchunks = 0; a.tiles_m = 0;
    a.num = KH * KW * C;
    a.div_pc = tab::make_fastdiv((uint32_t)s.PC);
    a.div_kw = tab::make_fastdiv((uint32_t)KW);
    a.div_pixels = tab::make_div32((uint32_t)(s.OH * s.OW));
    a.div_ow = tab::make_div32((uint32_t)s.OW);
    a.div_tiles_m = tab::make_div32(1);
    a.tiles_n = 0;
    a.xcd_share = 0; a.filter_tiles = 1; a.tail_big = 0; a.tail_chunks = 0;
    // A Y that fits the 256 MB last-level cache beside the operands but not the L2s is written through the caches
    // (the cache takes the stores faster than HBM: Y of 190-206 MB 1-11 % sooner); every other Y with non-temporal
    // stores: a smaller one leaves no dirty L2 to flush when the launch ends (7-25 % sooner), a larger one would only
    // push the operands out (Y of 411 MB: 7-28 % sooner).  At 103 MB the two policies measured within 3 %.
    const long y_bytes = s.M * (long)KN * 4;
    a.y_cached = y_bytes >= (128L << 20) && y_bytes <= (240L << 20);
    a.div_filter_tiles = tab::make_div32(1);
    hipError_t e = tab::launch_conv(type, a, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return device_fail(e, "conv launch");
    return TAB_OK;
}

int tab_conv2d_packed(const int64_t *dev_QX, const int64_t *dev_QW, const int32_t *dev_btn,
                      int type, int padding1, int padding2, int stride1, int stride2, int N,
                      int H, int W, int C, int KN, int KH, int KW, float *dev_Y, void *stream)
{
    if (!dev_Y) return fail(TAB_ERR_BAD_ARGUMENT, "null device pointer");
    return conv_packed(dev_QX, dev_QW, dev_btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW,
                       dev_Y, nullptr, 0, nullptr, stream);
}

int tab_conv2d_packed_out(const int64_t *dev_QX, const int64_t *dev_QW, const int32_t *dev_btn,
                          int type, int padding1, int padding2, int stride1, int stride2, int N,
                          int H, int W, int C, int KN, int KH, int KW, const float *dev_out_ths,
                          int out_bitwidth, int64_t *dev_QY, void *stream)
{
    if (!dev_QY) return fail(TAB_ERR_BAD_ARGUMENT, "null device pointer");
    return conv_packed(dev_QX, dev_QW, dev_btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW,
                       nullptr, dev_out_ths, out_bitwidth, dev_QY, stream);
}

/* Device address of `scratch` on the current device, looked up on the first call made with that device current. */
static int static_scratch(void **out)
{
    constexpr int kMaxDevices = 64;
    static std::mutex mutex;
    static void *address[kMaxDevices] = {};
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return device_fail(e, "hipGetDevice");
    if (device < 0 || device >= kMaxDevices) return fail(TAB_ERR_DEVICE, "device index %d out of range", device);
    std::lock_guard<std::mutex> lock(mutex);
    if (address[device] == nullptr) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return device_fail(e, "hipGetSymbolAddress(scratch)");
        if (ptr == nullptr) return fail(TAB_ERR_DEVICE, "hipGetSymbolAddress(scratch) gave no address");
        address[device] = ptr;
    }
    *out = address[device];
    return TAB_OK;
}

/* Body of tab_conv2d and tab_conv2d_static (workspace == NULL and builtin: the library's own scratch): quantize
 * into the workspace, then the fused conv kernel. */
static int conv_from_floats(const float *dev_X, const int64_t *dev_QW, const float *dev_ths, const int32_t *dev_btn, int type,
                            int padding1, int padding2, int stride1, int stride2, int N, int H, int W, int C, int KN, int KH,
                            int KW, float *dev_Y, void *workspace, size_t workspace_bytes, bool builtin, void *stream)
{
    ConvShape s;
    int rc = check_conv(type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW, &s);
    if (rc != TAB_OK) return rc;
    if (!dev_X || !dev_ths) return fail(TAB_ERR_BAD_ARGUMENT, "null device pointer");
    if ((uintptr_t)dev_X % 4) return fail(TAB_ERR_BAD_ARGUMENT, "X must be aligned to its floats");
    const size_t need = tab_conv2d_workspace_bytes(type, N, H, W, C);
    if (builtin) {
        if (need > TAB_STATIC_SCRATCH_BYTES)
            return fail(TAB_ERR_WORKSPACE, "the packed activation needs %zu bytes, the built-in scratch holds %zu; use tab_conv2d with a workspace",
                        need, (size_t)TAB_STATIC_SCRATCH_BYTES);
        rc = static_scratch(&workspace);
        if (rc != TAB_OK) return rc;
    } else if (!workspace || workspace_bytes < need || ((uintptr_t)workspace % 16)) {
        return fail(TAB_ERR_WORKSPACE, "workspace must be 16-byte aligned and hold %zu bytes (got %zu)", need, workspace_bytes);
    }
    // everything the second stage would reject is rejected here, before the quantizer is enqueued
    rc = check_conv_pointers(s, type, workspace, dev_QW, dev_btn, dev_Y, nullptr);
    if (rc != TAB_OK) return rc;
    if (type > 3) {  // the CPU-only types: their own packers, then the same fused kernel
        hipError_t e = tab::launch_quantize_format(dev_X, dev_ths, type, (long)H * W, N, C, reinterpret_cast<uint64_t *>(workspace),
                                                   static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return device_fail(e, "quantize launch");
        return tab_conv2d_packed(reinterpret_cast<const int64_t *>(workspace), dev_QW, dev_btn, type, padding1, padding2, stride1,
                                 stride2, N, H, W, C, KN, KH, KW, dev_Y, stream);
    }
    // A small 1x1 convolution without padding: quantize and multiply in one launch, the packed activation stays in LDS
    // (only under the automatic kernel choice: a forced kernel is what the caller wants to see run)
    if (!tab::conv_kernel_forced() && tab::conv1x1_fused_supported(type, dev_X, C, KH, KW, padding1, padding2, s.M, KN)) {
        hipError_t e = tab::launch_conv1x1_fused(type, dev_X, dev_ths, reinterpret_cast<const uint64_t *>(dev_QW), dev_btn, dev_Y, N, H,
                                                 W, C, KN, stride1, stride2, s.OH, s.OW, static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return device_fail(e, "conv launch");
        return TAB_OK;
    }
    // A 1x1 convolution with stride and no padding reads one pixel in stride1*stride2: quantize only
    // those, into a compact activation, and convolve it with stride 1 (same outputs, a fraction of
    // the reads of X).
    if (KH == 1 && KW == 1 && padding1 == 0 && padding2 == 0 && (stride1 > 1 || stride2 > 1) && N * (long)s.OH < 65536 &&
        tab::quantize_strided_supported(dev_X, H, W, C, s.OH, s.OW)) {
        hipError_t e = tab::launch_quantize_strided(dev_X, dev_ths, s.abits, N, H, W, C, s.OH, s.OW, stride1, stride2,
                                                    reinterpret_cast<uint64_t *>(workspace), static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return device_fail(e, "quantize launch");
        return tab_conv2d_packed(reinterpret_cast<const int64_t *>(workspace), dev_QW, dev_btn, type, 0, 0, 1, 1, N, s.OH,
                                 s.OW, C, KN, 1, 1, dev_Y, stream);
    }
    // stage 1: quantize + pack the activation (TAB_GEMM.cu:419-426); no btn for activations
    hipError_t e = tab::launch_quantize(dev_X, dev_ths, s.abits, (long)H * W, N, C,
                                        reinterpret_cast<uint64_t *>(workspace), nullptr,
                                        static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return device_fail(e, "quantize launch");
    // stage 2: pad + im2row + GEMM, fused
    return tab_conv2d_packed(reinterpret_cast<const int64_t *>(workspace), dev_QW, dev_btn, type,
                             padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW, dev_Y,
                             stream);
}

int tab_conv2d(const float *dev_X, const int64_t *dev_QW, const float *dev_ths,
               const int32_t *dev_btn, int type, int padding1, int padding2, int stride1,
               int stride2, int N, int H, int W, int C, int KN, int KH, int KW, float *dev_Y,
               void *workspace, size_t workspace_bytes, void *stream)
{
    return conv_from_floats(dev_X, dev_QW, dev_ths, dev_btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW,
                            dev_Y, workspace, workspace_bytes, false, stream);
}

int tab_conv2d_launches(const float *dev_X, int type, int padding1, int padding2, int stride1, int stride2, int N, int H, int W,
                        int C, int KN, int KH, int KW)
{
    ConvShape s;
    if (check_conv(type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW, &s) != TAB_OK) return 0;
    return !tab::conv_kernel_forced() && tab::conv1x1_fused_supported(type, dev_X, C, KH, KW, padding1, padding2, s.M, KN) ? 1 : 2;
}

size_t tab_static_scratch_bytes(void) { return TAB_STATIC_SCRATCH_BYTES; }

int tab_conv2d_static(const float *dev_X, const int64_t *dev_QW, const float *dev_ths, const int32_t *dev_btn, int type,
                      int padding1, int padding2, int stride1, int stride2, int N, int H, int W, int C, int KN, int KH, int KW,
                      float *dev_Y, void *stream)
{
    return conv_from_floats(dev_X, dev_QW, dev_ths, dev_btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW,
                            dev_Y, nullptr, 0, true, stream);
}

}  // extern "C"
