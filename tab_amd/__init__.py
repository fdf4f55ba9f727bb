"""tab_amd - MI355X (gfx950) implementation of TAB's quantize + bitwise-conv operators.

Host-side mirror of the reference's operator interface (TAB_GPU.cpp:34-65): the same two
calls, positional argument lists, return tensors and error behaviour, on top of the C ABI
in include/tab_amd.h.  PyTorch only supplies device memory and the current stream.

    QW, BTN_W = Quantize(w, w_ths, bitwidth, KN, KH, KW, C)
    y = Conv2d(x, QW, x_ths, BTN_W, type, pad1, pad2, stride1, stride2, N, H, W, C, KN, KH, KW)
"""
import torch

from . import _capi

_lib = _capi.load()
TabError = _capi.TabError

TNN, TBN, BTN, BNN = 0, 1, 2, 3
DRF, RTN = 4, 5  # the types of the reference's CPU path only (TAB_CPU.cpp:332-383)


def version():
    return _lib.tab_version().decode()


def _check_input(t, name):
    # CHECK_INPUT of the reference (TAB_GPU.cpp:7-9): device + contiguity, as RuntimeError
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _check_dtype(t, dtype, name):
    # The reference converts with .toType() on a temporary (TAB_GEMM.cu:279-280,341-347),
    # which dangles when a conversion really happens; exact dtypes are required instead.
    if t.dtype != dtype:
        raise RuntimeError(f"{name} must have dtype {dtype}, got {t.dtype}")


def _stream():
    return torch.cuda.current_stream().cuda_stream


def packed_channels(C):
    return _lib.tab_packed_channels(int(C))


def operand_words(type, operand, C):
    """int64 words per pixel of the activation (operand 0) or per tap of the weight (operand 1)."""
    return _lib.tab_operand_words(int(type), int(operand), int(C))


def out_shape(H, W, KH, KW, pad1, pad2, stride1, stride2):
    """(OH, OW) by the reference's integer-division formula (TAB_GEMM.cu:354-357)."""
    return (_lib.tab_out_extent(H, pad1, KH, stride1), _lib.tab_out_extent(W, pad2, KW, stride2))


def Quantize(X, thresholds, bitwidth, N, H, W, C):
    """Ternarize (bitwidth 2) or binarize (bitwidth 1) NHWC fp32 data and pack 64 channels
    per int64 word.  Returns [QX, BTN]: QX int64 (N,H,W,PC,bitwidth), BTN int32 (N,)
    (TAB_GPU.cpp:53-58, TAB_GEMM.cu:250-322)."""
    _check_input(X, "X")
    _check_input(thresholds, "thresholds")
    _check_dtype(X, torch.float32, "X")
    _check_dtype(thresholds, torch.float32, "thresholds")
    bitwidth, N, H, W, C = int(bitwidth), int(N), int(H), int(W), int(C)
    if bitwidth not in (1, 2):
        raise RuntimeError(f"bitwidth must be 1 or 2, got {bitwidth}")
    if min(N, H, W, C) < 1:
        raise RuntimeError("N, H, W, C must be positive")
    if X.numel() != N * H * W * C:
        raise RuntimeError(f"X has {X.numel()} elements, expected N*H*W*C = {N * H * W * C}")
    if thresholds.numel() < N:
        raise RuntimeError(f"thresholds has {thresholds.numel()} elements, expected at least N = {N}")
    if thresholds.device != X.device:
        raise RuntimeError("X and thresholds must be on the same device")
    PC = packed_channels(C)
    with torch.cuda.device(X.device):
        QX = torch.empty((N, H, W, PC, bitwidth), dtype=torch.int64, device=X.device)
        BTN = torch.empty((N,), dtype=torch.int32, device=X.device)
        _capi.check(_lib, _lib.tab_quantize(X.data_ptr(), thresholds.data_ptr(), bitwidth, N, H, W, C,
                                            QX.data_ptr(), BTN.data_ptr(), _stream()))
    return [QX, BTN]


def QuantizeActivation(X, thresholds, bitwidth, N, H, W, C, nchw=False):
    """QX of Quantize (or, with nchw, of QuantizeNCHW with X given as N, C, H, W) without the BTN vector: an
    activation's counts are read by nobody, and passing NULL for them to the C ABI skips the launches that
    produce them."""
    _check_input(X, "X")
    _check_input(thresholds, "thresholds")
    _check_dtype(X, torch.float32, "X")
    _check_dtype(thresholds, torch.float32, "thresholds")
    bitwidth, N, H, W, C = int(bitwidth), int(N), int(H), int(W), int(C)
    if bitwidth not in (1, 2):
        raise RuntimeError(f"bitwidth must be 1 or 2, got {bitwidth}")
    if min(N, H, W, C) < 1:
        raise RuntimeError("N, H, W, C must be positive")
    if X.numel() != N * H * W * C:
        raise RuntimeError(f"X has {X.numel()} elements, expected N*H*W*C = {N * H * W * C}")
    if thresholds.numel() < N:
        raise RuntimeError(f"thresholds has {thresholds.numel()} elements, expected at least N = {N}")
    if thresholds.device != X.device:
        raise RuntimeError("X and thresholds must be on the same device")
    with torch.cuda.device(X.device):
        QX = torch.empty((N, H, W, packed_channels(C), bitwidth), dtype=torch.int64, device=X.device)
        if nchw:
            _capi.check(_lib, _lib.tab_quantize_nchw(X.data_ptr(), thresholds.data_ptr(), bitwidth, N, C, H, W, QX.data_ptr(), None, _stream()))
        else:
            _capi.check(_lib, _lib.tab_quantize(X.data_ptr(), thresholds.data_ptr(), bitwidth, N, H, W, C, QX.data_ptr(), None, _stream()))
    return QX


def QuantizeNCHW(X, thresholds, bitwidth, N, C, H, W):
    """Quantize on an NCHW fp32 tensor (the layout the reference's CPU quantizers read, TAB_CPU.cpp:20-206, and
    the argument order of its CPU binding, TAB_CPU.cpp:621): returns [QX, BTN] exactly as
    Quantize(X.permute(0, 2, 3, 1), thresholds, bitwidth, N, H, W, C) would, without the transposed copy."""
    _check_input(X, "X")
    _check_input(thresholds, "thresholds")
    _check_dtype(X, torch.float32, "X")
    _check_dtype(thresholds, torch.float32, "thresholds")
    bitwidth, N, C, H, W = int(bitwidth), int(N), int(C), int(H), int(W)
    if bitwidth not in (1, 2):
        raise RuntimeError(f"bitwidth must be 1 or 2, got {bitwidth}")
    if min(N, C, H, W) < 1:
        raise RuntimeError("N, C, H, W must be positive")
    if X.numel() != N * C * H * W:
        raise RuntimeError(f"X has {X.numel()} elements, expected N*C*H*W = {N * C * H * W}")
    if thresholds.numel() < N:
        raise RuntimeError(f"thresholds has {thresholds.numel()} elements, expected at least N = {N}")
    if thresholds.device != X.device:
        raise RuntimeError("X and thresholds must be on the same device")
    PC = packed_channels(C)
    with torch.cuda.device(X.device):
        QX = torch.empty((N, H, W, PC, bitwidth), dtype=torch.int64, device=X.device)
        BTN = torch.empty((N,), dtype=torch.int32, device=X.device)
        _capi.check(_lib, _lib.tab_quantize_nchw(X.data_ptr(), thresholds.data_ptr(), bitwidth, N, C, H, W,
                                                 QX.data_ptr(), BTN.data_ptr(), _stream()))
    return [QX, BTN]


def QuantizeFormat(X, thresholds, type, N, H, W, C):
    """Packer of conv types 4 (DoReFa 2-bit levels; QX int64 (N,H,W,PC,2), plane 0 = weight-2 bit)
    and 5 (RTN 2-bit fields; QX int64 (N,H,W,ceil(C/32))), for activations and weights alike.  The
    layouts are the ones DRFGEMM_baseline / RTNGEMM_baseline read (TAB_CPU.cpp:332-383); the
    reference has no quantizer for them, the value rules (uniform step thresholds[n]; the
    ternarizer's compares) are this library's."""
    _check_input(X, "X")
    _check_input(thresholds, "thresholds")
    _check_dtype(X, torch.float32, "X")
    _check_dtype(thresholds, torch.float32, "thresholds")
    type, N, H, W, C = int(type), int(N), int(H), int(W), int(C)
    if type not in (DRF, RTN):
        raise RuntimeError(f"type must be 4 (DRF) or 5 (RTN), got {type}")
    if min(N, H, W, C) < 1:
        raise RuntimeError("N, H, W, C must be positive")
    if X.numel() != N * H * W * C:
        raise RuntimeError(f"X has {X.numel()} elements, expected N*H*W*C = {N * H * W * C}")
    if thresholds.numel() < N:
        raise RuntimeError(f"thresholds has {thresholds.numel()} elements, expected at least N = {N}")
    if thresholds.device != X.device:
        raise RuntimeError("X and thresholds must be on the same device")
    shape = (N, H, W, packed_channels(C), 2) if type == DRF else (N, H, W, (C + 31) // 32)
    with torch.cuda.device(X.device):
        QX = torch.empty(shape, dtype=torch.int64, device=X.device)
        _capi.check(_lib, _lib.tab_quantize_format(X.data_ptr(), thresholds.data_ptr(), type, N, H, W, C,
                                                   QX.data_ptr(), _stream()))
    return QX


def Threshold(X, N, scale=0.7):
    """ths[n] = scale * mean(|X[n]|) per item (image or filter), fp32 (N,), computed on the
    device in one pass: the threshold rule the reference leaves to the caller (README.md:45).
    Reproducible from run to run; within 1e-5 relative of an fp64 reference."""
    _check_input(X, "X")
    _check_dtype(X, torch.float32, "X")
    N = int(N)
    if N < 1 or X.numel() % N != 0 or X.numel() == 0:
        raise RuntimeError(f"X has {X.numel()} elements, not a positive multiple of N = {N}")
    per_item = X.numel() // N
    with torch.cuda.device(X.device):
        ths = torch.empty((N,), dtype=torch.float32, device=X.device)
        ws_bytes = _lib.tab_threshold_workspace_bytes(N, per_item)
        ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=X.device)
        _capi.check(_lib, _lib.tab_threshold(X.data_ptr(), N, per_item, float(scale), ths.data_ptr(),
                                             ws.data_ptr(), ws_bytes, _stream()))
    return ths


def _conv_checks(QW, btn, type, N, H, W, C, KN, KH, KW, pad1, pad2, stride1, stride2):
    if type not in (0, 1, 2, 3, 4, 5):
        raise RuntimeError(f"type must be 0 (TNN), 1 (TBN), 2 (BTN), 3 (BNN), 4 (DRF) or 5 (RTN), got {type}")
    if min(N, H, W, C, KN, KH, KW) < 1 or min(pad1, pad2) < 0 or min(stride1, stride2) < 1:
        raise RuntimeError("sizes must be positive, padding >= 0 and stride >= 1")
    need = KN * KH * KW * operand_words(type, 1, C)
    if QW.numel() != need:
        raise RuntimeError(f"QW has {QW.numel()} words, type {type} expects KN*KH*KW*{operand_words(type, 1, C)} = {need}")
    if type == 2 and btn.numel() < KN:
        raise RuntimeError(f"btn has {btn.numel()} elements, expected at least KN = {KN}")
    OH, OW = out_shape(H, W, KH, KW, pad1, pad2, stride1, stride2)
    if OH < 1 or OW < 1:
        raise RuntimeError(f"empty output: OH={OH}, OW={OW}")
    return OH, OW


def Conv2d(X, QW, thresholds, btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW):
    """Quantize the NHWC fp32 activation on the fly (ternary for types 0/1, binary for 2/3; types 4
    and 5 of the CPU path through QuantizeFormat) and convolve it with the packed weights.  Returns fp32 shaped
    (N,KN,OH,OW) whose memory is ordered (n,oh,ow,kn), exactly as the reference's reshape
    of its GEMM result (TAB_GPU.cpp:34-42, TAB_GEMM.cu:325-527)."""
    for t, name in ((X, "X"), (QW, "QW"), (thresholds, "thresholds"), (btn, "btn")):
        _check_input(t, name)
    _check_dtype(X, torch.float32, "X")
    _check_dtype(QW, torch.int64, "QW")
    _check_dtype(thresholds, torch.float32, "thresholds")
    _check_dtype(btn, torch.int32, "btn")
    (type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW) = (
        int(v) for v in (type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW))
    OH, OW = _conv_checks(QW, btn, type, N, H, W, C, KN, KH, KW, padding1, padding2, stride1, stride2)
    if X.numel() != N * H * W * C:
        raise RuntimeError(f"X has {X.numel()} elements, expected N*H*W*C = {N * H * W * C}")
    if thresholds.numel() < N:
        raise RuntimeError(f"thresholds has {thresholds.numel()} elements, expected at least N = {N}")
    for t, name in ((QW, "QW"), (thresholds, "thresholds"), (btn, "btn")):
        if t.device != X.device:
            raise RuntimeError(f"X and {name} must be on the same device")
    with torch.cuda.device(X.device):
        Y = torch.empty((N, KN, OH, OW), dtype=torch.float32, device=X.device)
        ws_bytes = _lib.tab_conv2d_workspace_bytes(type, N, H, W, C)
        ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=X.device)
        _capi.check(_lib, _lib.tab_conv2d(X.data_ptr(), QW.data_ptr(), thresholds.data_ptr(), btn.data_ptr(),
                                          type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW,
                                          Y.data_ptr(), ws.data_ptr(), ws_bytes, _stream()))
    return Y


def conv2d_launches(X, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW):
    """Kernels one Conv2d call with these arguments enqueues: 1 (quantize and convolution in one launch) or 2."""
    return _lib.tab_conv2d_launches(X.data_ptr(), *(int(v) for v in (type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW)))


def static_scratch_bytes():
    """Size of the scratch array built into the library that Conv2dStatic packs the activation into."""
    return _lib.tab_static_scratch_bytes()


def Conv2dStatic(X, QW, thresholds, btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW, out=None):
    """Conv2d through tab_conv2d_static: the packed activation goes to the library's built-in device scratch
    (static_scratch_bytes() bytes per GPU) instead of a workspace tensor, so the C call allocates nothing.
    With `out` (fp32, N*OH*OW*KN elements) given, this wrapper allocates nothing either.  Calls that may
    overlap on one GPU race on the shared scratch."""
    for t, name in ((X, "X"), (QW, "QW"), (thresholds, "thresholds"), (btn, "btn")):
        _check_input(t, name)
    _check_dtype(X, torch.float32, "X")
    _check_dtype(QW, torch.int64, "QW")
    _check_dtype(thresholds, torch.float32, "thresholds")
    _check_dtype(btn, torch.int32, "btn")
    (type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW) = (
        int(v) for v in (type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW))
    OH, OW = _conv_checks(QW, btn, type, N, H, W, C, KN, KH, KW, padding1, padding2, stride1, stride2)
    if X.numel() != N * H * W * C:
        raise RuntimeError(f"X has {X.numel()} elements, expected N*H*W*C = {N * H * W * C}")
    if thresholds.numel() < N:
        raise RuntimeError(f"thresholds has {thresholds.numel()} elements, expected at least N = {N}")
    with torch.cuda.device(X.device):
        if out is None:
            out = torch.empty((N, KN, OH, OW), dtype=torch.float32, device=X.device)
        else:
            _check_input(out, "out")
            _check_dtype(out, torch.float32, "out")
            if out.numel() != N * KN * OH * OW:
                raise RuntimeError(f"out has {out.numel()} elements, expected {N * KN * OH * OW}")
        _capi.check(_lib, _lib.tab_conv2d_static(X.data_ptr(), QW.data_ptr(), thresholds.data_ptr(), btn.data_ptr(),
                                                 type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW,
                                                 out.data_ptr(), _stream()))
    return out


def Conv2dPacked(QX, QW, btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW):
    """Conv2d on an activation already packed by Quantize (bitwidth 2 for types 0/1,
    1 for types 2/3) or by QuantizeFormat (types 4/5): the pad + im2row + GEMM stages of
    TAB_GEMM.cu:447-509 only."""
    for t, name in ((QX, "QX"), (QW, "QW"), (btn, "btn")):
        _check_input(t, name)
    _check_dtype(QX, torch.int64, "QX")
    _check_dtype(QW, torch.int64, "QW")
    _check_dtype(btn, torch.int32, "btn")
    (type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW) = (
        int(v) for v in (type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW))
    OH, OW = _conv_checks(QW, btn, type, N, H, W, C, KN, KH, KW, padding1, padding2, stride1, stride2)
    if QX.numel() != N * H * W * operand_words(type, 0, C):
        raise RuntimeError(f"QX has {QX.numel()} words, type {type} expects N*H*W*{operand_words(type, 0, C)}")
    with torch.cuda.device(QX.device):
        Y = torch.empty((N, KN, OH, OW), dtype=torch.float32, device=QX.device)
        _capi.check(_lib, _lib.tab_conv2d_packed(QX.data_ptr(), QW.data_ptr(), btn.data_ptr(), type,
                                                 padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW,
                                                 Y.data_ptr(), _stream()))
    return Y


def Conv2dPackedOut(QX, QW, btn, type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW,
                    out_thresholds, out_bitwidth):
    """Conv2dPacked whose output is quantized and packed in the kernel's epilogue: returns QY int64
    (N, OH, OW, ceil(KN/64), out_bitwidth), equal bit for bit to
    Quantize(Conv2dPacked(...), out_thresholds, out_bitwidth, N, OH, OW, KN)[0] - the conv output's
    (n, oh, ow, kn) memory read as the next layer's NHWC activation - without the fp32 tensor ever
    being written.  out_thresholds: fp32 [>=N], one threshold per image."""
    for t, name in ((QX, "QX"), (QW, "QW"), (btn, "btn"), (out_thresholds, "out_thresholds")):
        _check_input(t, name)
    _check_dtype(QX, torch.int64, "QX")
    _check_dtype(QW, torch.int64, "QW")
    _check_dtype(btn, torch.int32, "btn")
    _check_dtype(out_thresholds, torch.float32, "out_thresholds")
    (type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW, out_bitwidth) = (
        int(v) for v in (type, padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW, out_bitwidth))
    OH, OW = _conv_checks(QW, btn, type, N, H, W, C, KN, KH, KW, padding1, padding2, stride1, stride2)
    awords = operand_words(type, 0, C)
    if QX.numel() != N * H * W * awords:
        raise RuntimeError(f"QX has {QX.numel()} words, type {type} expects N*H*W*{awords}")
    if out_thresholds.numel() < N:
        raise RuntimeError(f"out_thresholds has {out_thresholds.numel()} elements, need N={N}")
    if out_bitwidth not in (1, 2):
        raise RuntimeError(f"out_bitwidth must be 1 or 2, got {out_bitwidth}")
    with torch.cuda.device(QX.device):
        QY = torch.empty((N, OH, OW, packed_channels(KN), out_bitwidth), dtype=torch.int64, device=QX.device)
        _capi.check(_lib, _lib.tab_conv2d_packed_out(QX.data_ptr(), QW.data_ptr(), btn.data_ptr(), type,
                                                     padding1, padding2, stride1, stride2, N, H, W, C, KN, KH, KW,
                                                     out_thresholds.data_ptr(), out_bitwidth, QY.data_ptr(), _stream()))
    return QY


CONV_AUTO, CONV_MATRIX, CONV_POPCOUNT = 0, 1, 2


def set_conv_kernel(kernel=CONV_AUTO, tile=-1):
    """Pick the conv kernel (process-wide): CONV_AUTO, CONV_MATRIX (tile 0..11 or -1) or
    CONV_POPCOUNT (tile 0..2 or -1).  Every choice gives bit-identical outputs."""
    _capi.check(_lib, _lib.tab_set_conv_kernel(int(kernel), int(tile)))


# names of the reference's CPU module (TAB_CPU.cpp:636-639)
TAB_Quantize = Quantize
TAB_Conv2d = Conv2d

__all__ = ["Quantize", "QuantizeNCHW", "QuantizeActivation", "conv2d_launches", "QuantizeFormat", "Conv2d", "Conv2dStatic", "static_scratch_bytes", "Conv2dPacked", "Conv2dPackedOut", "Threshold", "TAB_Quantize", "TAB_Conv2d", "TabError",
           "packed_channels", "out_shape", "version", "TNN", "TBN", "BTN", "BNN", "set_conv_kernel",
           "CONV_AUTO", "CONV_MATRIX", "CONV_POPCOUNT"]
