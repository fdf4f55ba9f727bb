"""ctypes front end of the CPU oracle (oracle/tab_oracle.c) and, when it was built, of the
reference's own CPU functions (oracle/_ref/libtab_ref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by bench.py's
cpu_baseline leg as the checker.  The product package (tab_amd) never imports it.

All functions take and return numpy arrays; layouts follow the reference
(TAB_GEMM.cu:163-247,321,526): X is NHWC fp32, QX is int64 (N,H,W,PC,bits), conv output is
fp32 shaped (N,KN,OH,OW) over memory ordered (n,oh,ow,kn).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libtab_ref.so")

_c_f32 = ctypes.POINTER(ctypes.c_float)
_c_i64 = ctypes.POINTER(ctypes.c_int64)
_c_i32 = ctypes.POINTER(ctypes.c_int32)
_int, _long = ctypes.c_int, ctypes.c_long


def build(force=False):
    """Compile liboracle.so (and _ref/libtab_ref.so when /root/reference is present)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"])
    if os.path.isdir("/root/reference"):
        subprocess.check_call(["make", "-C", _HERE, "ref"])


def _ptr(a, ctype):
    return a.ctypes.data_as(ctype)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_num_threads.restype = _int
        L.oracle_out_extent.restype = _int
        L.oracle_out_extent.argtypes = [_int] * 4
        for name in ("oracle_quantize_ternary", "oracle_quantize_binary", "oracle_quantize_drf", "oracle_quantize_rtn"):
            getattr(L, name).argtypes = [_c_f32, _c_f32, _int, _int, _int, _int, _c_i64]
            getattr(L, name).restype = None
        L.oracle_btn_weight.argtypes = [_c_i64, _int, _long, _c_i32]
        L.oracle_btn_weight.restype = None
        L.oracle_pad.argtypes = [_c_i64, _int, _int, _int, _int, _int, _int, _c_i64]
        L.oracle_pad.restype = None
        L.oracle_img2row.argtypes = [_c_i64] + [_int] * 8 + [_c_i64]
        L.oracle_img2row.restype = None
        L.oracle_gemm_tnn.argtypes = [_c_i64, _c_i64, _long, _int, _int, _c_i32]
        L.oracle_gemm_tbn.argtypes = [_c_i64, _c_i64, _long, _int, _int, _c_i32]
        L.oracle_gemm_btn.argtypes = [_c_i64, _c_i64, _c_i32, _long, _int, _int, _c_i32]
        L.oracle_gemm_bnn.argtypes = [_c_i64, _c_i64, _long, _int, _int, _int, _c_i32]
        L.oracle_gemm_drf.argtypes = [_c_i64, _c_i64, _long, _int, _int, _c_i32]
        L.oracle_gemm_rtn.argtypes = [_c_i64, _c_i64, _long, _int, _int, _c_i32]
        L.oracle_conv2d.argtypes = [_c_f32, _c_i64, _c_f32, _c_i32] + [_int] * 12 + [_c_f32]
        L.oracle_conv2d.restype = _int
        L.oracle_conv2d_packed.argtypes = [_c_i64, _c_i64, _c_i32] + [_int] * 12 + [_c_f32]
        L.oracle_conv2d_packed.restype = _int
        _lib = L
    return _lib


def num_threads():
    return lib().oracle_num_threads()


def packed_channels(C):
    return (C + 63) // 64


def out_extent(size, pad, k, stride):
    return lib().oracle_out_extent(size, pad, k, stride)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def quantize(x, ths, bitwidth, N, H, W, C):
    """Reference Quantize (TAB_GEMM.cu:250-322): returns (QX (N,H,W,PC,bits) int64, BTN (N,) int32)."""
    if bitwidth not in (1, 2):
        raise ValueError("bitwidth must be 1 or 2")
    x, ths = _f32(x), _f32(ths)
    assert x.size == N * H * W * C and ths.size >= N
    PC = packed_channels(C)
    qx = np.empty((N, H, W, PC, bitwidth), dtype=np.int64)
    btn = np.zeros((N,), dtype=np.int32)
    fn = lib().oracle_quantize_ternary if bitwidth == 2 else lib().oracle_quantize_binary
    fn(_ptr(x, _c_f32), _ptr(ths, _c_f32), N, H, W, C, _ptr(qx, _c_i64))
    if bitwidth == 2:
        lib().oracle_btn_weight(_ptr(qx, _c_i64), N, H * W * PC, _ptr(btn, _c_i32))
    return qx, btn


TYPE_DRF, TYPE_RTN = 4, 5  # the CPU-only types of TAB_Conv (TAB_CPU.cpp:332-383)


def words_per_pixel(type, C, operand):
    """int64 words per pixel of operand 'a' (activation) or 'w' (weight) for conv type 0..5."""
    if type == TYPE_RTN:
        return (C + 31) // 32
    if type == TYPE_DRF:
        return 2 * packed_channels(C)
    two_planes = type < 2 if operand == "a" else type in (0, 2)
    return packed_channels(C) * (2 if two_planes else 1)


def quantize_format(x, ths, type, N, H, W, C):
    """Packers of the two CPU-only types: 4 -> DoReFa levels (N,H,W,PC,2), 5 -> RTN fields
    (N,H,W,ceil(C/32)).  The reference defines the layouts (through its GEMMs) but no
    quantizer; the value rules are documented in tab_oracle.c."""
    x, ths = _f32(x), _f32(ths)
    assert x.size == N * H * W * C and ths.size >= N
    if type == TYPE_DRF:
        qx = np.empty((N, H, W, packed_channels(C), 2), dtype=np.int64)
        lib().oracle_quantize_drf(_ptr(x, _c_f32), _ptr(ths, _c_f32), N, H, W, C, _ptr(qx, _c_i64))
    elif type == TYPE_RTN:
        qx = np.empty((N, H, W, (C + 31) // 32), dtype=np.int64)
        lib().oracle_quantize_rtn(_ptr(x, _c_f32), _ptr(ths, _c_f32), N, H, W, C, _ptr(qx, _c_i64))
    else:
        raise ValueError("type must be 4 or 5")
    return qx


def quantize_nchw(x, ths, bitwidth, N, C, H, W):
    """Quantize of an NCHW tensor, the layout the reference's CPU quantizers read (TAB_CPU.cpp:20-206): the
    same (N,H,W,PC,bits) words as quantize() on the values stored NHWC."""
    x = np.ascontiguousarray(_f32(x).reshape(N, C, H, W).transpose(0, 2, 3, 1))
    return quantize(x, ths, bitwidth, N, H, W, C)


def pad(a, N, H, W, D, p1, p2):
    a = _i64(a)
    y = np.empty((N, H + 2 * p1, W + 2 * p2, D), dtype=np.int64)
    lib().oracle_pad(_ptr(a, _c_i64), N, H, W, D, p1, p2, _ptr(y, _c_i64))
    return y


def img2row(a, N, PH, PW, D, KH, KW, s1, s2):
    a = _i64(a)
    OH, OW = (PH - KH + 1) // s1, (PW - KW + 1) // s2
    rows = np.empty((N * OH * OW, KH * KW * D), dtype=np.int64)
    lib().oracle_img2row(_ptr(a, _c_i64), N, PH, PW, D, KH, KW, s1, s2, _ptr(rows, _c_i64))
    return rows


def gemm(type, a, b, M, N, K, btn=None, NUM=0):
    """One of the six popcount GEMMs (TAB_CPU.cpp:242-383); returns int32 [M,N]."""
    a, b = _i64(a), _i64(b)
    y = np.empty((M, N), dtype=np.int32)
    L = lib()
    if type == 0:
        L.oracle_gemm_tnn(_ptr(a, _c_i64), _ptr(b, _c_i64), M, N, K, _ptr(y, _c_i32))
    elif type == 1:
        L.oracle_gemm_tbn(_ptr(a, _c_i64), _ptr(b, _c_i64), M, N, K, _ptr(y, _c_i32))
    elif type == 2:
        btn = _i32(btn)
        L.oracle_gemm_btn(_ptr(a, _c_i64), _ptr(b, _c_i64), _ptr(btn, _c_i32), M, N, K, _ptr(y, _c_i32))
    elif type == 3:
        L.oracle_gemm_bnn(_ptr(a, _c_i64), _ptr(b, _c_i64), M, N, K, NUM, _ptr(y, _c_i32))
    elif type == TYPE_DRF:
        L.oracle_gemm_drf(_ptr(a, _c_i64), _ptr(b, _c_i64), M, N, K, _ptr(y, _c_i32))
    elif type == TYPE_RTN:
        L.oracle_gemm_rtn(_ptr(a, _c_i64), _ptr(b, _c_i64), M, N, K, _ptr(y, _c_i32))
    else:
        raise ValueError("type must be 0..5")
    return y


def conv2d(x, qw, ths, btn, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW):
    """Reference Conv2d (TAB_GEMM.cu:325-527); returns fp32 (N,KN,OH,OW) over (n,oh,ow,kn) memory."""
    x, qw, ths, btn = _f32(x), _i64(qw), _f32(ths), _i32(btn)
    OH, OW = out_extent(H, p1, KH, s1), out_extent(W, p2, KW, s2)
    y = np.empty((N, KN, OH, OW), dtype=np.float32)
    rc = lib().oracle_conv2d(_ptr(x, _c_f32), _ptr(qw, _c_i64), _ptr(ths, _c_f32), _ptr(btn, _c_i32),
                             type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW, _ptr(y, _c_f32))
    if rc != 0:
        raise ValueError("oracle_conv2d rejected the arguments")
    return y


def conv2d_packed(qx, qw, btn, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW):
    """Conv2d on a packed activation (pad, im2row, GEMM), types 0..5; fp32 (N,KN,OH,OW)."""
    qx, qw = _i64(qx), _i64(qw)
    btn = _i32(btn if btn is not None else np.zeros(KN))
    assert qx.size == N * H * W * words_per_pixel(type, C, "a")
    assert qw.size == KN * KH * KW * words_per_pixel(type, C, "w")
    OH, OW = out_extent(H, p1, KH, s1), out_extent(W, p2, KW, s2)
    y = np.empty((N, KN, OH, OW), dtype=np.float32)
    rc = lib().oracle_conv2d_packed(_ptr(qx, _c_i64), _ptr(qw, _c_i64), _ptr(btn, _c_i32), type, p1, p2, s1, s2,
                                    N, H, W, C, KN, KH, KW, _ptr(y, _c_f32))
    if rc != 0:
        raise ValueError("oracle_conv2d_packed rejected the arguments")
    return y


# --------------------------------------------------------------------------------------
# The reference's own CPU functions (present only when oracle/_ref was built).
_ref = None


def have_ref():
    return os.path.exists(_REF_PATH)


def ref():
    global _ref
    if _ref is None:
        R = ctypes.CDLL(_REF_PATH)
        R.ref_gemm_tnn.argtypes = [_c_i64, _c_i64, _int, _int, _int, _c_i32]
        R.ref_gemm_tbn.argtypes = [_c_i64, _c_i64, _int, _int, _int, _c_i32]
        R.ref_gemm_btn.argtypes = [_c_i64, _c_i64, _c_i32, _int, _int, _int, _c_i32]
        R.ref_gemm_bnn.argtypes = [_c_i64, _c_i64, _int, _int, _int, _int, _c_i32]
        if hasattr(R, "ref_gemm_drf"):
            R.ref_gemm_drf.argtypes = [_c_i64, _c_i64, _int, _int, _int, _c_i32]
            R.ref_gemm_rtn.argtypes = [_c_i64, _c_i64, _int, _int, _int, _c_i32]
        R.ref_img2row_3x3.argtypes = [_c_i64] + [_int] * 8 + [_c_i64]
        R.ref_ternarize_nchw.argtypes = [_c_f32, _int, _int, _c_f32] + [_int] * 4 + [_c_i64]
        R.ref_binarize_nchw.argtypes = [_c_f32, _int, _int] + [_int] * 4 + [_c_i64]
        _ref = R
    return _ref


def ref_gemm(type, a, b, M, N, K, btn=None, NUM=0):
    a, b = _i64(a).copy(), _i64(b).copy()
    y = np.empty((M, N), dtype=np.int32)
    R = ref()
    if type == 0:
        R.ref_gemm_tnn(_ptr(a, _c_i64), _ptr(b, _c_i64), M, N, K, _ptr(y, _c_i32))
    elif type == 1:
        R.ref_gemm_tbn(_ptr(a, _c_i64), _ptr(b, _c_i64), M, N, K, _ptr(y, _c_i32))
    elif type == 2:
        btn = _i32(btn).copy()
        R.ref_gemm_btn(_ptr(a, _c_i64), _ptr(b, _c_i64), _ptr(btn, _c_i32), M, N, K, _ptr(y, _c_i32))
    elif type == 3:
        R.ref_gemm_bnn(_ptr(a, _c_i64), _ptr(b, _c_i64), M, N, K, NUM, _ptr(y, _c_i32))
    elif type == TYPE_DRF:
        R.ref_gemm_drf(_ptr(a, _c_i64), _ptr(b, _c_i64), M, N, K, _ptr(y, _c_i32))
    else:
        R.ref_gemm_rtn(_ptr(a, _c_i64), _ptr(b, _c_i64), M, N, K, _ptr(y, _c_i32))
    return y


def ref_img2row_3x3(a, N, PH, PW, D, KH, KW, s1, s2):
    a = _i64(a).copy()
    OH, OW = (PH - KH + 1) // s1, (PW - KW + 1) // s2
    rows = np.empty((N * OH * OW, KH * KW * D), dtype=np.int64)
    ref().ref_img2row_3x3(_ptr(a, _c_i64), N, D, PH, PW, KH, KW, s1, s2, _ptr(rows, _c_i64))
    return rows


def ref_ternarize_nchw(x_nchw, p1, p2, ths, N, C, H, W):
    x_nchw, ths = _f32(x_nchw).copy(), _f32(ths).copy()
    PC = packed_channels(C)
    out = np.empty((N, H + 2 * p1, W + 2 * p2, PC, 2), dtype=np.int64)
    ref().ref_ternarize_nchw(_ptr(x_nchw, _c_f32), p1, p2, _ptr(ths, _c_f32), N, C, H, W, _ptr(out, _c_i64))
    return out


def ref_binarize_nchw(x_nchw, p1, p2, N, C, H, W):
    x_nchw = _f32(x_nchw).copy()
    PC = packed_channels(C)
    out = np.empty((N, H + 2 * p1, W + 2 * p2, PC), dtype=np.int64)
    ref().ref_binarize_nchw(_ptr(x_nchw, _c_f32), p1, p2, N, C, H, W, _ptr(out, _c_i64))
    return out
