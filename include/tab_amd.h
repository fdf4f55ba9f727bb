/*
 * tab_amd.h - C ABI of the MI355X (gfx950) TAB quantize + bitwise-convolution library.
 *
 * All pointers named dev_* are device (HBM) addresses on the current HIP device; the
 * library never copies to or from the host.  `stream` is a hipStream_t passed as void*
 * (NULL = the default stream).  Every call only enqueues work on `stream` and returns
 * without synchronising.  Functions returning int give TAB_OK or a negative
 * tab_status; tab_status_string() names it and tab_last_error() holds a longer message
 * for the calling thread.
 *
 * Data layouts are the reference's (ntuliuteam/TAB):
 *   X    fp32  [N][H][W][C]                                  TAB_GEMM.cu:163-208
 *   QX   int64 [N][H][W][PC][bits], PC = ceil(C/64), channel c -> word c/64, bit c%64
 *        (LSB first); bits = 2: plane 0 = sign marker, plane 1 = nonzero marker;
 *        bits = 1: bit set <=> value -1                     TAB_GEMM.cu:196-197,238,321
 *   QW   the same layout with (N,H,W,C) = (KN,KH,KW,C)
 *   Y    fp32  [N*OH*OW][KN]  (labelled (N,KN,OH,OW) by the caller)   TAB_GEMM.cu:53,526
 * and, for the two types that exist only in the reference's CPU file (TAB_CPU.cpp:332-383), the
 * layouts their GEMMs read:
 *   type 4 (DoReFa 2-bit)  int64 [N][H][W][PC][2], plane 0 = weight-2 bit, plane 1 = weight-1 bit of an
 *        unsigned level 0..3, on both operands          TAB_CPU.cpp:345-354
 *   type 5 (RTN)  int64 [N][H][W][ceil(C/32)], channel c -> word c/32, bit 2*(c%32) = nonzero marker,
 *        bit 2*(c%32)+1 = sign marker, on both operands  TAB_CPU.cpp:364-379, 520-521
 */
#ifndef TAB_AMD_H
#define TAB_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum tab_status {
    TAB_OK = 0,
    TAB_ERR_BAD_ARGUMENT = -1, /* NULL pointer, non-positive extent, bad type/bitwidth */
    TAB_ERR_BAD_SHAPE = -2,    /* empty output, or a size that overflows the index range */
    TAB_ERR_WORKSPACE = -3,    /* workspace missing or smaller than required */
    TAB_ERR_DEVICE = -4        /* a HIP call failed; see tab_last_error() */
} tab_status;

/* Conv types, TAB_GPU.cpp:27 ("0: TNN, 1, TBN, 2: BTN, 3: BNN"): first letter =
 * activation precision, second = weight precision. */
enum { TAB_TNN = 0, TAB_TBN = 1, TAB_BTN = 2, TAB_BNN = 3 };
/* The CPU path's two further types (TAB_CPU.cpp:577-584 / 603-610): DoReFa-Net 2-bit and RTN. */
enum { TAB_DRF = 4, TAB_RTN = 5 };

const char *tab_status_string(int status);
const char *tab_last_error(void);
/* "tab_amd <version> gfx950"; lets a binding check what it loaded. */
const char *tab_version(void);

/* PC = ceil(C/64) (TAB_GEMM.cu:262-265). */
int tab_packed_channels(int C);

/* int64 words per pixel of the activation (operand 0) or per tap of the weight (operand 1) for conv
 * type 0..5: planes * ceil(C/64), or ceil(C/32) for type 5 (TAB_GEMM.cu:367-379, TAB_CPU.cpp:520-521).
 * 0 on bad arguments. */
int tab_operand_words(int type, int operand, int C);

/* Output extent (in + 2*pad - k + 1) / stride, integer division (TAB_GEMM.cu:354-357). */
int tab_out_extent(int in, int pad, int k, int stride);

/*
 * Replaces QuanWithCuda_TAB (TAB_GEMM.cu:250-322), the body of
 * TAB_Quantize(X, thresholds, bitwidth, N, H, W, C) (TAB_GPU.cpp:53-58).
 *   dev_X    fp32 [N*H*W*C]
 *   dev_ths  fp32 [>=N], threshold of item n is ths[n] (TAB_CPU.cpp:67,72)
 *   bitwidth 2: ternarize (v > t -> +1, else v < -t -> -1, else 0); 1: binarize (v < t -> -1)
 *   dev_QX   int64 [N*H*W*PC*bitwidth], aligned to a whole packed element (8*bitwidth bytes; the same holds
 *            for tab_quantize_nchw, 16 bytes for tab_quantize_format); every element is written
 *   dev_BTN  int32 [N]; bitwidth 2: popcount of item n's nonzero plane (TAB_GEMM.cu:150-160,
 *            for every n); bitwidth 1: zeros (TAB_GEMM.cu:283).  NULL: not wanted (an activation's
 *            counts are read by nobody); the launches that produce them are then skipped.  The same
 *            holds for tab_quantize_nchw.
 */
int tab_quantize(const float *dev_X, const float *dev_ths, int bitwidth, int N, int H, int W,
                 int C, int64_t *dev_QX, int32_t *dev_BTN, void *stream);

/*
 * tab_quantize on an activation stored NCHW, the layout the reference's CPU quantizers read
 * (Parallel_Ternarize_NCHWB_to_NHWCB / Parallel_Binarize_NCHW_to_NHWC, TAB_CPU.cpp:20-206; its CPU binding
 * takes N, C, H, W, TAB_CPU.cpp:621): dev_X fp32 [N][C][H][W]; dev_QX and dev_BTN exactly what tab_quantize
 * gives for the same values stored NHWC, so the conv entry points take it unchanged and a caller holding
 * NCHW tensors needs no transposed copy.  No spatial padding is applied here (the conv kernel pads).
 */
int tab_quantize_nchw(const float *dev_X, const float *dev_ths, int bitwidth, int N, int C, int H, int W,
                      int64_t *dev_QX, int32_t *dev_BTN, void *stream);

/*
 * Packers for conv types 4 and 5, activations and weights alike (weights as (N,H,W,C) = (KN,KH,KW,C)).
 * The reference defines the word layouts through DRFGEMM_baseline / RTNGEMM_baseline
 * (TAB_CPU.cpp:332-383) but ships no quantizer for them (TAB_Conv calls Parallel_Binarize_NCHW and
 * Parallel_Ternarize_RTN, TAB_CPU.cpp:522,527, which no file defines), so the value rules are this
 * library's:
 *   type 4: level = (v >= 0.5t) + (v >= 1.5t) + (v >= 2.5t) with t = ths[n], the uniform 2-bit
 *           quantizer with step t (each bound rounded to fp32; NaN -> 0)
 *   type 5: the ternarizer's rule (v > t -> +1, else v < -t -> -1, TAB_GEMM.cu:184-192)
 *   dev_QX  int64 [N*H*W*tab_operand_words(type, 0, C)], every element is written
 */
int tab_quantize_format(const float *dev_X, const float *dev_ths, int type, int N, int H, int W, int C,
                        int64_t *dev_QX, void *stream);

/*
 * Per-item threshold ths[n] = scale * mean(|X[n]|) over per_item consecutive fp32 values: the
 * step before Quantize/Conv2d, which the reference leaves to the caller (README.md:45,
 * "threshold values of each filter or each input image"; the usual ternary rule is
 * scale = 0.7).  It has no counterpart function in the reference.  Floating point: a
 * fixed-order fp32 tree per slice and an fp64 sum of the slices, reproducible from run to
 * run; agrees with an fp64 reference to a relative 1e-5.
 *   workspace: tab_threshold_workspace_bytes(N, per_item) bytes of device scratch.
 */
size_t tab_threshold_workspace_bytes(int N, long per_item);
int tab_threshold(const float *dev_X, int N, long per_item, float scale, float *dev_ths,
                  void *workspace, size_t workspace_bytes, void *stream);
int tab_conv2d_launches(const float *dev_X, int type, int padding1, int padding2, int stride1, int stride2,
                        int N, int H, int W, int C, int KN, int KH, int KW);

/*
 * Bytes of device scratch tab_conv2d needs for the packed activation
 * (the reference cudaMallocs pad_a/img_a per call, TAB_GEMM.cu:391-397).  0 on bad arguments.
 */
size_t tab_conv2d_workspace_bytes(int type, int N, int H, int W, int C);

/*
 * Replaces ConvWithCuda_TAB (TAB_GEMM.cu:325-527), the body of
 * TAB_Conv2d(X, QW, thresholds, btn, type, padding1, padding2, stride1, stride2,
 *            N, H, W, C, KN, KH, KW) (TAB_GPU.cpp:34-42).
 *   dev_X   fp32 [N*H*W*C]; quantized on the fly: ternary for TNN/TBN, binary for BTN/BNN
 *           (TAB_GEMM.cu:419-426)
 *   dev_QW  int64 [KN*KH*KW*PC*wbits], wbits = 2 for TNN/BTN, 1 for TBN/BNN (374-379)
 *   dev_ths fp32 [>=N]
 *   dev_btn int32 [>=KN], read only for BTN (TAB_GEMM.cu:116); may be NULL otherwise
 *   dev_Y   fp32 [N*OH*OW*KN], OH = tab_out_extent(H, padding1, KH, stride1), OW likewise;
 *           16-byte aligned (the kernels store four floats at a time); every element is written
 *   workspace / workspace_bytes: device scratch of at least tab_conv2d_workspace_bytes()
 *           bytes, 16-byte aligned; owned by the caller, reusable once the stream has
 *           passed this call
 * Padded taps read all-zero words: value 0 for ternary, +1 for binary activations
 * (TAB_CPU.cpp:39,155); BNN's constant is KH*KW*C (TAB_GEMM.cu:509).
 * Types 4 and 5 (CPU-only in the reference, TAB_CPU.cpp:507-614) are accepted too: X goes through
 * tab_quantize_format, dev_QW holds the same format, zero words are the value 0, and Y is
 * DRFGEMM_baseline's / RTNGEMM_baseline's integer as fp32.  Type 4 needs 9 * 64 * K words < 2^24.
 * Launches: the quantizer, then the fused pad + im2row + GEMM kernel; a small 1x1 convolution without
 * padding (64, 128, 256 or 512 channels, types 0..3) quantizes and multiplies in ONE kernel and leaves
 * the workspace untouched.  tab_conv2d_launches() says which (1 or 2; 0 on bad arguments), for tools that
 * attribute time per launch; dev_X matters only through its alignment.
 */
int tab_conv2d(const float *dev_X, const int64_t *dev_QW, const float *dev_ths,
               const int32_t *dev_btn, int type, int padding1, int padding2, int stride1,
               int stride2, int N, int H, int W, int C, int KN, int KH, int KW, float *dev_Y,
               void *workspace, size_t workspace_bytes, void *stream);

/*
 * tab_conv2d for callers that cannot allocate device memory or pass a workspace: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose
 * ConvWithCuda_TAB cudaMallocs its scratch on every call, TAB_GEMM.cu:391-397).  Arguments and results are
 * exactly tab_conv2d's; the packed activation goes to a scratch array built into the library
 * (TAB_STATIC_SCRATCH_BYTES bytes of device memory per GPU, held until the process ends) instead of a
 * caller-owned workspace.  The call allocates nothing and frees nothing.
 *   - tab_conv2d_workspace_bytes(type, N, H, W, C) must not exceed TAB_STATIC_SCRATCH_BYTES, else
 *     TAB_ERR_WORKSPACE and nothing is launched (use tab_conv2d with a workspace for larger activations).
 *   - All calls on one GPU share that GPU's array: two calls whose kernels may overlap (different streams,
 *     different host threads without ordering) race on it.  Calls on one stream are ordered and safe.
 *   - The first call made on a device looks the array's address up once (no stream work, no allocation); make
 *     that first call outside a graph capture.
 */
#define TAB_STATIC_SCRATCH_BYTES (32u << 20)
size_t tab_static_scratch_bytes(void);
int tab_conv2d_static(const float *dev_X, const int64_t *dev_QW, const float *dev_ths,
                      const int32_t *dev_btn, int type, int padding1, int padding2, int stride1,
                      int stride2, int N, int H, int W, int C, int KN, int KH, int KW, float *dev_Y,
                      void *stream);

/*
 * The second half of tab_conv2d on an activation that is already packed (the output of
 * tab_quantize with bitwidth 2 for TNN/TBN, 1 for BTN/BNN): zero padding, im2row and the
 * popcount GEMM (PadKernel + Img2RowKernel + GEMMWithCuda, TAB_GEMM.cuh:22-115) fused in
 * one kernel.  dev_QX int64 [N*H*W*PC*abits], aligned to a whole packed element (8*abits bytes; dev_QW likewise,
 * 8*wbits bytes; dev_Y 16 bytes); other arguments as in tab_conv2d.  Unlike the reference's .toType() calls
 * (TAB_GEMM.cu:341-347) no entry point converts element types: buffers must hold the types named here.  Types 4 and 5:
 * dev_QX int64 [N*H*W*tab_operand_words(type, 0, C)] from tab_quantize_format.
 */
int tab_conv2d_packed(const int64_t *dev_QX, const int64_t *dev_QW, const int32_t *dev_btn,
                      int type, int padding1, int padding2, int stride1, int stride2, int N,
                      int H, int W, int C, int KN, int KH, int KW, float *dev_Y, void *stream);

/*
 * tab_conv2d_packed with the output quantized and packed in the kernel's epilogue instead of written
 * as fp32: dev_QY is what tab_quantize(Y, dev_out_ths, out_bitwidth, N, OH, OW, KN) would give for
 * the Y of tab_conv2d_packed - Y's memory order (n, oh, ow, kn) read as the NHWC activation of the
 * next layer (TAB_GEMM.cu:53,526 for the order; TAB_GEMM.cu:184-192, 231 for the compares) - bit
 * for bit, without Y ever reaching memory.  It chains layers packed-in / packed-out; the
 * reference has no counterpart (every TAB_Conv2d returns fp32 and the caller re-quantizes).
 *   dev_out_ths fp32 [>=N]: threshold for the outputs of image n
 *   dev_QY      int64 [N*OH*OW*ceil(KN/64)*out_bitwidth], aligned to a whole packed element
 *               (8*out_bitwidth bytes); every element is written
 * All six types; types 4 and 5 take dev_QX / dev_QW as tab_conv2d_packed does, and their output, too, is packed as
 * tab_quantize packs it (bit planes for a following layer of types 0..3).
 */
int tab_conv2d_packed_out(const int64_t *dev_QX, const int64_t *dev_QW, const int32_t *dev_btn,
                          int type, int padding1, int padding2, int stride1, int stride2, int N,
                          int H, int W, int C, int KN, int KH, int KW, const float *dev_out_ths,
                          int out_bitwidth, int64_t *dev_QY, void *stream);

/*
 * Which kernel tab_conv2d / tab_conv2d_packed launch.  Both give bit-identical Y; the switch exists
 * for verification and tuning and has no counterpart in the reference (which has one GEMM kernel
 * per type, TAB_GEMM.cu:25-147).  Process-wide: the choice is one atomic word, a conv call on another
 * thread sees either the old or the new choice.  While a choice other than TAB_CONV_AUTO is held,
 * tab_conv2d always runs the quantizer and the chosen conv kernel as two launches.
 *   TAB_CONV_AUTO      (tile -1) the library's choice: matrix cores, tile picked from the shape
 *   TAB_CONV_MATRIX    bit planes expanded to FP4 operands of v_mfma_f32_32x32x64_f8f6f4;
 *                      tile 0: 128x128, 1: 128x64, 2: 64x64, 3: 32x32 with K split over the
 *                      four waves, 4: 256x64, 5: 256x128, 6: 128x256, 7: weights resident in registers
 *                      (K of at most nine words; longer K takes the library's choice), 8: 64x64 and
 *                      9: 128x128 with K split over four / two groups of waves inside the workgroup (an
 *                      even number of words per pixel; otherwise tiles 2 and 0), 10: 128x128 for the
 *                      whole rounds of the chip and 64x64 quarters, K split over the waves, for the rest
 *                      of the last round (an even number of words per pixel; otherwise tile 0), 11: the
 *                      same with whole tiles of 128x256 (words per pixel in fours; otherwise tile 6); -1:
 *                      picked from the shape
 *   TAB_CONV_POPCOUNT  the reference's xor/and + popcount formulation on the vector ALU;
 *                      tile 0: big, 1: medium, 2: small; -1: picked from the shape
 *                      (types 4 and 5 exist on the matrix cores only and ignore this choice)
 */
enum { TAB_CONV_AUTO = 0, TAB_CONV_MATRIX = 1, TAB_CONV_POPCOUNT = 2 };
int tab_set_conv_kernel(int kernel, int tile);

#ifdef __cplusplus
}
#endif
#endif /* TAB_AMD_H */
