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
    TORCH_CHECK(type >= 0 && type <= 3, "type must be 0 (TNN), 1 (TBN), 2 (BTN) or 3 (BNN), got ", type);
    TORCH_CHECK(N > 0 && H > 0 && W > 0 && C > 0 && KN > 0 && KH > 0 && KW > 0 && padding1 >= 0 && padding2 >= 0 &&
                    stride1 > 0 && stride2 > 0,
                "sizes must be positive, padding >= 0 and stride >= 1");
    const int PC = tab_packed_channels(C);
    const int wbits = (type == TAB_TNN || type == TAB_BTN) ? 2 : 1;
    TORCH_CHECK(X.numel() == (int64_t)N * H * W * C, "X has ", X.numel(), " elements, expected N*H*W*C = ",
                (int64_t)N * H * W * C);
    TORCH_CHECK(QW.numel() == (int64_t)KN * KH * KW * PC * wbits, "QW has ", QW.numel(), " words, type ", type,
                " expects KN*KH*KW*PC*", wbits, " = ", (int64_t)KN * KH * KW * PC * wbits);
    TORCH_CHECK(thresholds.numel() >= N, "thresholds has ", thresholds.numel(), " elements, expected at least N = ", N);
    TORCH_CHECK(type != TAB_BTN || btn.numel() >= KN, "btn has ", btn.numel(), " elements, expected at least KN = ", KN);
    TORCH_CHECK(QW.device() == X.device() && thresholds.device() == X.device() && btn.device() == X.device(),
                "X, QW, thresholds and btn must be on the same device");
    const int OH = tab_out_extent(H, padding1, KH, stride1), OW = tab_out_extent(W, padding2, KW, stride2);
    TORCH_CHECK(OH > 0 && OW > 0, "empty output: OH=", OH, ", OW=", OW);
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(X.device());
    auto Y = torch::empty({N, KN, OH, OW}, X.options());
    const size_t ws_bytes = tab_conv2d_workspace_bytes(type, N, H, W, C);
    auto ws = torch::empty({(int64_t)ws_bytes}, X.options().dtype(torch::kUInt8));
    check_status(tab_conv2d(X.data_ptr<float>(), QW.data_ptr<int64_t>(), thresholds.data_ptr<float>(),
                            btn.data_ptr<int32_t>(), type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH,
                            KW, Y.data_ptr<float>(), ws.data_ptr(), ws_bytes, current_stream(X)));
    return Y;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("Quantize", &TAB_Quantize, "Ternarization or binarization of NHWC fp32 data, packed 64 channels per int64");
    m.def("Conv2d", &TAB_Conv2d, "Conv2d of all TAB types (0 TNN, 1 TBN, 2 BTN, 3 BNN)");
    m.def("TAB_Quantize", &TAB_Quantize, "alias of Quantize");
    m.def("TAB_Conv2d", &TAB_Conv2d, "alias of Conv2d");
}
