// PyTorch C++ extension front end: the reference's operator boundary (TAB_GPU.cpp:34-65) on
// top of the C ABI of include/tab_amd.h.  Same exported names (`Quantize`, `Conv2d`), same
// positional parameter lists, same return tensors; the CPU module's names (TAB_CPU.cpp:636-639)
// are exported as aliases.  PyTorch only supplies device memory (caching allocator) and the
// current HIP stream; all compute is in libtab_amd.so.
#include <torch/extension.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <vector>

#include "../../include/tab_amd.h"

// CHECK_INPUT of the reference (TAB_GPU.cpp:7-9)
#define CHECK_CUDA(x) TORCH_CHECK(x.device().is_cuda(), #x " must be a CUDA tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")
#define CHECK_INPUT(x) \
    CHECK_CUDA(x);     \
    CHECK_CONTIGUOUS(x)
// The reference converts dtypes with .toType() on a temporary (TAB_GEMM.cu:279-280,341-347),
// which dangles whenever a conversion really happens; exact dtypes are required instead.
#define CHECK_DTYPE(x, t) TORCH_CHECK(x.scalar_type() == t, #x " must have dtype " #t)

namespace {

void check_status(int status)
{
    TORCH_CHECK(status == TAB_OK, tab_status_string(status), ": ", tab_last_error());
}

void *current_stream(const torch::Tensor &t)
{
    return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

}  // namespace

std::vector<torch::Tensor> TAB_Quantize(torch::Tensor X, torch::Tensor thresholds, int bitwidth, int N,
                                        int H, int W, int C)
{
    CHECK_INPUT(X);
    CHECK_INPUT(thresholds);
    CHECK_DTYPE(X, torch::kFloat32);
    CHECK_DTYPE(thresholds, torch::kFloat32);
    TORCH_CHECK(bitwidth == 1 || bitwidth == 2, "bitwidth must be 1 or 2, got ", bitwidth);
    TORCH_CHECK(N > 0 && H > 0 && W > 0 && C > 0, "N, H, W, C must be positive");
    TORCH_CHECK(X.numel() == (int64_t)N * H * W * C, "X has ", X.numel(), " elements, expected N*H*W*C = ",
                (int64_t)N * H * W * C);
    TORCH_CHECK(thresholds.numel() >= N, "thresholds has ", thresholds.numel(), " elements, expected at least N = ", N);
    TORCH_CHECK(thresholds.device() == X.device(), "X and thresholds must be on the same device");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(X.device());
    const int PC = tab_packed_channels(C);
    auto QX = torch::empty({N, H, W, PC, bitwidth}, X.options().dtype(torch::kInt64));
    auto BTN = torch::empty({N}, X.options().dtype(torch::kInt32));
    check_status(tab_quantize(X.data_ptr<float>(), thresholds.data_ptr<float>(), bitwidth, N, H, W, C,
                              QX.data_ptr<int64_t>(), BTN.data_ptr<int32_t>(), current_stream(X)));
    return {QX, BTN};
}

namespace {

// Checks shared by the conv entry points; returns (OH, OW).
std::pair<int, int> check_conv(const torch::Tensor &QW, const torch::Tensor &btn, int type, int padding1, int padding2,
                               int stride1, int stride2, int N, int H, int W, int C, int KN, int KH, int KW)
{
    // types 4 (DoReFa 2-bit) and 5 (RTN) are the further cases of the CPU binding's TAB_Conv2d (TAB_CPU.cpp:577-584, 621-633)
    TORCH_CHECK(type >= 0 && type <= 5, "type must be 0 (TNN), 1 (TBN), 2 (BTN), 3 (BNN), 4 (DRF) or 5 (RTN), got ", type);
    TORCH_CHECK(N > 0 && H > 0 && W > 0 && C > 0 && KN > 0 && KH > 0 && KW > 0 && padding1 >= 0 && padding2 >= 0 &&
                    stride1 > 0 && stride2 > 0,
                "sizes must be positive, padding >= 0 and stride >= 1");
    const int wwords = tab_operand_words(type, 1, C);
    TORCH_CHECK(QW.numel() == (int64_t)KN * KH * KW * wwords, "QW has ", QW.numel(), " words, type ", type,
                " expects KN*KH*KW*", wwords, " = ", (int64_t)KN * KH * KW * wwords);
    TORCH_CHECK(type != TAB_BTN || btn.numel() >= KN, "btn has ", btn.numel(), " elements, expected at least KN = ", KN);
    const int OH = tab_out_extent(H, padding1, KH, stride1), OW = tab_out_extent(W, padding2, KW, stride2);
    TORCH_CHECK(OH > 0 && OW > 0, "empty output: OH=", OH, ", OW=", OW);
    return {OH, OW};
}

}  // namespace

torch::Tensor TAB_Conv2d(torch::Tensor X, torch::Tensor QW, torch::Tensor thresholds, torch::Tensor btn, int type,
                         int padding1, int padding2, int stride1, int stride2, int N, int H, int W, int C, int KN,
                         int KH, int KW)
{
    CHECK_INPUT(X);
    CHECK_INPUT(QW);
    CHECK_INPUT(thresholds);
    CHECK_INPUT(btn);
    CHECK_DTYPE(X, torch::kFloat32);
    CHECK_DTYPE(QW, torch::kInt64);
    CHECK_DTYPE(thresholds, torch::kFloat32);
    CHECK_DTYPE(btn, torch::kInt32);
    const auto [OH, OW] = check_conv(QW, btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW);
    TORCH_CHECK(X.numel() == (int64_t)N * H * W * C, "X has ", X.numel(), " elements, expected N*H*W*C = ",
                (int64_t)N * H * W * C);
    TORCH_CHECK(thresholds.numel() >= N, "thresholds has ", thresholds.numel(), " elements, expected at least N = ", N);
    TORCH_CHECK(QW.device() == X.device() && thresholds.device() == X.device() && btn.device() == X.device(),
                "X, QW, thresholds and btn must be on the same device");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(X.device());
    auto Y = torch::empty({N, KN, OH, OW}, X.options());
    const size_t ws_bytes = tab_conv2d_workspace_bytes(type, N, H, W, C);
    auto ws = torch::empty({(int64_t)ws_bytes}, X.options().dtype(torch::kUInt8));
    check_status(tab_conv2d(X.data_ptr<float>(), QW.data_ptr<int64_t>(), thresholds.data_ptr<float>(),
                            btn.data_ptr<int32_t>(), type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH,
                            KW, Y.data_ptr<float>(), ws.data_ptr(), ws_bytes, current_stream(X)));
    return Y;
}

// ---- the entry points beyond the reference's two: same conventions, one C ABI call each -----------------------

// Quantize on an NCHW tensor, the layout and argument order of the reference's CPU binding (TAB_CPU.cpp:20-206, 621).
std::vector<torch::Tensor> TAB_QuantizeNCHW(torch::Tensor X, torch::Tensor thresholds, int bitwidth, int N, int C,
                                            int H, int W)
{
    CHECK_INPUT(X);
    CHECK_INPUT(thresholds);
    CHECK_DTYPE(X, torch::kFloat32);
    CHECK_DTYPE(thresholds, torch::kFloat32);
    TORCH_CHECK(bitwidth == 1 || bitwidth == 2, "bitwidth must be 1 or 2, got ", bitwidth);
    TORCH_CHECK(N > 0 && H > 0 && W > 0 && C > 0, "N, C, H, W must be positive");
    TORCH_CHECK(X.numel() == (int64_t)N * H * W * C, "X has ", X.numel(), " elements, expected N*C*H*W = ",
                (int64_t)N * H * W * C);
    TORCH_CHECK(thresholds.numel() >= N, "thresholds has ", thresholds.numel(), " elements, expected at least N = ", N);
    TORCH_CHECK(thresholds.device() == X.device(), "X and thresholds must be on the same device");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(X.device());
    auto QX = torch::empty({N, H, W, tab_packed_channels(C), bitwidth}, X.options().dtype(torch::kInt64));
    auto BTN = torch::empty({N}, X.options().dtype(torch::kInt32));
    check_status(tab_quantize_nchw(X.data_ptr<float>(), thresholds.data_ptr<float>(), bitwidth, N, C, H, W,
                                   QX.data_ptr<int64_t>(), BTN.data_ptr<int32_t>(), current_stream(X)));
    return {QX, BTN};
}

// Packer of conv types 4 and 5 (layouts of DRFGEMM_baseline / RTNGEMM_baseline, TAB_CPU.cpp:332-383).
torch::Tensor TAB_QuantizeFormat(torch::Tensor X, torch::Tensor thresholds, int type, int N, int H, int W, int C)
{
    CHECK_INPUT(X);
    CHECK_INPUT(thresholds);
    CHECK_DTYPE(X, torch::kFloat32);
    CHECK_DTYPE(thresholds, torch::kFloat32);
    TORCH_CHECK(type == TAB_DRF || type == TAB_RTN, "type must be 4 (DRF) or 5 (RTN), got ", type);
    TORCH_CHECK(N > 0 && H > 0 && W > 0 && C > 0, "N, H, W, C must be positive");
    TORCH_CHECK(X.numel() == (int64_t)N * H * W * C, "X has ", X.numel(), " elements, expected N*H*W*C = ",
                (int64_t)N * H * W * C);
    TORCH_CHECK(thresholds.numel() >= N, "thresholds has ", thresholds.numel(), " elements, expected at least N = ", N);
    TORCH_CHECK(thresholds.device() == X.device(), "X and thresholds must be on the same device");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(X.device());
    auto QX = type == TAB_DRF ? torch::empty({N, H, W, tab_packed_channels(C), 2}, X.options().dtype(torch::kInt64))
                              : torch::empty({N, H, W, (C + 31) / 32}, X.options().dtype(torch::kInt64));
    check_status(tab_quantize_format(X.data_ptr<float>(), thresholds.data_ptr<float>(), type, N, H, W, C,
                                     QX.data_ptr<int64_t>(), current_stream(X)));
    return QX;
}

// thresholds[n] = scale * mean|X[n]|, the rule README.md:45 leaves to the caller.
torch::Tensor TAB_Threshold(torch::Tensor X, int N, double scale)
{
    CHECK_INPUT(X);
    CHECK_DTYPE(X, torch::kFloat32);
    TORCH_CHECK(N > 0 && X.numel() > 0 && X.numel() % N == 0, "X has ", X.numel(), " elements, not a positive multiple of N = ", N);
    const long per_item = (long)(X.numel() / N);
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(X.device());
    auto ths = torch::empty({N}, X.options());
    const size_t ws_bytes = tab_threshold_workspace_bytes(N, per_item);
    auto ws = torch::empty({(int64_t)ws_bytes}, X.options().dtype(torch::kUInt8));
    check_status(tab_threshold(X.data_ptr<float>(), N, per_item, (float)scale, ths.data_ptr<float>(), ws.data_ptr(), ws_bytes,
                               current_stream(X)));
    return ths;
}

// Conv2d on an activation already packed by Quantize / QuantizeFormat (TAB_GEMM.cu:447-509 only).
torch::Tensor TAB_Conv2dPacked(torch::Tensor QX, torch::Tensor QW, torch::Tensor btn, int type, int padding1, int padding2,
                               int stride1, int stride2, int N, int H, int W, int C, int KN, int KH, int KW)
{
    CHECK_INPUT(QX);
    CHECK_INPUT(QW);
    CHECK_INPUT(btn);
    CHECK_DTYPE(QX, torch::kInt64);
    CHECK_DTYPE(QW, torch::kInt64);
    CHECK_DTYPE(btn, torch::kInt32);
    const auto [OH, OW] = check_conv(QW, btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW);
    const int awords = tab_operand_words(type, 0, C);
    TORCH_CHECK(QX.numel() == (int64_t)N * H * W * awords, "QX has ", QX.numel(), " words, type ", type, " expects N*H*W*", awords);
    TORCH_CHECK(QW.device() == QX.device() && btn.device() == QX.device(), "QX, QW and btn must be on the same device");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(QX.device());
    auto Y = torch::empty({N, KN, OH, OW}, QX.options().dtype(torch::kFloat32));
    check_status(tab_conv2d_packed(QX.data_ptr<int64_t>(), QW.data_ptr<int64_t>(), btn.data_ptr<int32_t>(), type, padding1,
                                   padding2, stride1, stride2, N, H, W, C, KN, KH, KW, Y.data_ptr<float>(), current_stream(QX)));
    return Y;
}

// Conv2dPacked with the output thresholded and packed in the epilogue: the next layer's activation, no fp32 Y.
torch::Tensor TAB_Conv2dPackedOut(torch::Tensor QX, torch::Tensor QW, torch::Tensor btn, int type, int padding1, int padding2,
                                  int stride1, int stride2, int N, int H, int W, int C, int KN, int KH, int KW,
                                  torch::Tensor out_thresholds, int out_bitwidth)
{
    CHECK_INPUT(QX);
    CHECK_INPUT(QW);
    CHECK_INPUT(btn);
    CHECK_INPUT(out_thresholds);
    CHECK_DTYPE(QX, torch::kInt64);
    CHECK_DTYPE(QW, torch::kInt64);
    CHECK_DTYPE(btn, torch::kInt32);
    CHECK_DTYPE(out_thresholds, torch::kFloat32);
    TORCH_CHECK(out_bitwidth == 1 || out_bitwidth == 2, "out_bitwidth must be 1 or 2, got ", out_bitwidth);
    const auto [OH, OW] = check_conv(QW, btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW);
    const int awords = tab_operand_words(type, 0, C);
    TORCH_CHECK(QX.numel() == (int64_t)N * H * W * awords, "QX has ", QX.numel(), " words, type ", type, " expects N*H*W*", awords);
    TORCH_CHECK(out_thresholds.numel() >= N, "out_thresholds has ", out_thresholds.numel(), " elements, need N = ", N);
    TORCH_CHECK(QW.device() == QX.device() && btn.device() == QX.device() && out_thresholds.device() == QX.device(),
                "QX, QW, btn and out_thresholds must be on the same device");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(QX.device());
    auto QY = torch::empty({N, OH, OW, tab_packed_channels(KN), out_bitwidth}, QX.options());
    check_status(tab_conv2d_packed_out(QX.data_ptr<int64_t>(), QW.data_ptr<int64_t>(), btn.data_ptr<int32_t>(), type, padding1,
                                       padding2, stride1, stride2, N, H, W, C, KN, KH, KW, out_thresholds.data_ptr<float>(),
                                       out_bitwidth, QY.data_ptr<int64_t>(), current_stream(QX)));
    return QY;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("Quantize", &TAB_Quantize, "Ternarization or binarization of NHWC fp32 data, packed 64 channels per int64");
    m.def("Conv2d", &TAB_Conv2d, "Conv2d of all TAB types (0 TNN, 1 TBN, 2 BTN, 3 BNN; 4 DRF and 5 RTN of the CPU path)");
    m.def("TAB_Quantize", &TAB_Quantize, "alias of Quantize");
    m.def("TAB_Conv2d", &TAB_Conv2d, "alias of Conv2d");
    m.def("QuantizeNCHW", &TAB_QuantizeNCHW, "Quantize on NCHW fp32 data (X, thresholds, bitwidth, N, C, H, W)");
    m.def("QuantizeFormat", &TAB_QuantizeFormat, "Packer of conv types 4 (DRF) and 5 (RTN)");
    m.def("Threshold", &TAB_Threshold, "thresholds[n] = scale * mean|X[n]|", pybind11::arg("X"), pybind11::arg("N"),
          pybind11::arg("scale") = 0.7);
    m.def("Conv2dPacked", &TAB_Conv2dPacked, "Conv2d on an already packed activation");
    m.def("Conv2dPackedOut", &TAB_Conv2dPackedOut, "Conv2dPacked with the output quantized and packed in the epilogue");
}
