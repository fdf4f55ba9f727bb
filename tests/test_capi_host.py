"""CPU-side checks of the boundary: the shared library loads, exports every symbol that
include/tab_amd.h declares, its host-only entry points answer, and both the C ABI and the
Python mirror reject bad arguments before anything is launched (no GPU is touched)."""
import ctypes
import os
import re

import pytest
import torch

import tab_amd
from tab_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "tab_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tab_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert {"tab_quantize", "tab_conv2d", "tab_conv2d_packed", "tab_conv2d_workspace_bytes"} <= set(names)
    lib = ctypes.CDLL(_capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/tab_amd.h but not exported"
    assert sorted(_capi.SIGNATURES) == names


def test_host_only_entry_points():
    lib = _capi.load()
    assert lib.tab_version().decode().endswith("gfx950")
    assert [lib.tab_packed_channels(c) for c in (1, 63, 64, 65, 256)] == [1, 1, 1, 2, 4]
    # (in + 2*pad - k + 1) / stride, integer division (TAB_GEMM.cu:354-357)
    assert lib.tab_out_extent(7, 1, 3, 2) == 3
    assert lib.tab_out_extent(56, 1, 3, 2) == 28
    assert lib.tab_out_extent(28, 1, 1, 2) == 15
    assert lib.tab_status_string(0) == b"TAB_OK"
    assert lib.tab_status_string(-3) == b"TAB_ERR_WORKSPACE"
    # activation scratch: N*H*W*PC*abits int64 words
    assert lib.tab_conv2d_workspace_bytes(0, 2, 5, 5, 70) == 2 * 5 * 5 * 2 * 2 * 8
    assert lib.tab_conv2d_workspace_bytes(3, 2, 5, 5, 70) == 2 * 5 * 5 * 2 * 1 * 8
    # the CPU-only types: two planes of ceil(C/64) words (4), one plane of ceil(C/32) words (5)
    assert lib.tab_conv2d_workspace_bytes(4, 2, 5, 5, 70) == 2 * 5 * 5 * 2 * 2 * 8
    assert lib.tab_conv2d_workspace_bytes(5, 2, 5, 5, 70) == 2 * 5 * 5 * 3 * 8
    assert lib.tab_conv2d_workspace_bytes(6, 2, 5, 5, 70) == 0
    assert [lib.tab_operand_words(t, 0, 70) for t in range(7)] == [4, 4, 2, 2, 4, 3, 0]
    assert [lib.tab_operand_words(t, 1, 70) for t in range(7)] == [4, 2, 4, 2, 4, 3, 0]
    assert lib.tab_operand_words(0, 2, 70) == 0


def test_c_abi_rejects_bad_arguments_without_launching():
    lib = _capi.load()
    p = 4096  # never dereferenced: every call below fails validation first
    assert lib.tab_quantize(p, p, 3, 1, 1, 1, 64, p, p, None) == -1
    assert b"bitwidth" in lib.tab_last_error()
    assert lib.tab_quantize(None, p, 2, 1, 1, 1, 64, p, p, None) == -1
    assert lib.tab_quantize(p, p, 2, 0, 1, 1, 64, p, p, None) == -1
    # QX aligned to a whole packed element (8 bytes 1-bit, 16 bytes 2-bit and the type-4/5 formats)
    assert lib.tab_quantize(p, p, 2, 1, 1, 1, 64, p + 8, p, None) == -1 and b"aligned" in lib.tab_last_error()
    assert lib.tab_quantize(p, p, 1, 1, 1, 1, 64, p + 4, p, None) == -1
    assert lib.tab_quantize(p + 2, p, 1, 1, 1, 1, 64, p, p, None) == -1
    assert lib.tab_quantize_nchw(p, p, 2, 1, 64, 1, 1, p + 8, p, None) == -1
    assert lib.tab_quantize_format(p, p, 4, 1, 1, 1, 64, p + 8, None) == -1 and b"aligned" in lib.tab_last_error()
    conv = lambda **kw: lib.tab_conv2d(  # noqa: E731
        kw.get("x", p), p, p, p, kw.get("type", 0), kw.get("p1", 1), 1, kw.get("s1", 1), 1,
        1, kw.get("H", 8), 8, 64, 4, 3, 3, p, kw.get("ws", p), kw.get("ws_bytes", 1 << 20), None)
    assert conv(type=6) == -1 and conv(type=-1) == -1
    assert conv(s1=0) == -1
    assert conv(p1=-1) == -1
    assert conv(H=1, p1=0) == -2 and b"empty output" in lib.tab_last_error()
    assert conv(ws=None) == -3
    assert conv(ws_bytes=8) == -3 and b"workspace" in lib.tab_last_error()
    assert conv(x=None) == -1
    # BTN needs btn
    assert lib.tab_conv2d_packed(p, p, None, 2, 1, 1, 1, 1, 1, 8, 8, 64, 4, 3, 3, p, None) == -1
    with pytest.raises(_capi.TabError, match="TAB_ERR_BAD_ARGUMENT"):
        _capi.check(lib, lib.tab_quantize(p, p, 0, 1, 1, 1, 64, p, p, None))
    # packed output: bit width, thresholds, output pointer, alignment of a 2-bit element
    out = lambda **kw: lib.tab_conv2d_packed_out(  # noqa: E731
        p, p, p, 3, 1, 1, 1, 1, 1, 8, 8, 64, 4, 3, 3, kw.get("ths", p), kw.get("bits", 1), kw.get("qy", p), None)
    assert out(bits=3) == -1 and b"out_bitwidth" in lib.tab_last_error()
    assert out(ths=None) == -1
    assert out(qy=None) == -1
    assert out(qy=p + 8, bits=2) == -1 and b"aligned" in lib.tab_last_error()
    # the CPU-only types: packed output takes the same checks; type 4 bounds K so that 9 * 64 * K words stays below 2^24
    assert lib.tab_conv2d_packed_out(p, p, p, 4, 1, 1, 1, 1, 1, 8, 8, 64, 4, 3, 3, p, 3, p, None) == -1
    assert b"out_bitwidth" in lib.tab_last_error()
    assert lib.tab_conv2d_packed_out(p, p, p, 5, 1, 1, 1, 1, 1, 8, 8, 64, 4, 3, 3, None, 1, p, None) == -1
    assert lib.tab_conv2d_packed(p, p, p, 4, 0, 0, 1, 1, 1, 4, 4, 64 * 29200, 4, 1, 1, p, None) == -2
    assert b"exact accumulation" in lib.tab_last_error()
    assert lib.tab_conv2d_packed(p, p, p, 5, 0, 0, 1, 1, 1, 4, 4, 32 * 65536, 4, 1, 1, p, None) == -2
    assert lib.tab_quantize_nchw(p, p, 3, 1, 64, 1, 1, p, p, None) == -1 and b"bitwidth" in lib.tab_last_error()
    assert lib.tab_quantize_nchw(p, p, 2, 60000, 64 * 100, 1000, 1000, p, p, None) == -2
    assert lib.tab_quantize_nchw(p, p, 2, 1, 64, 1, 1, None, p, None) == -1
    assert lib.tab_quantize_format(p, p, 3, 1, 1, 1, 64, p, None) == -1 and b"4 (DRF) or 5 (RTN)" in lib.tab_last_error()
    assert lib.tab_quantize_format(p, None, 4, 1, 1, 1, 64, p, None) == -1
    assert lib.tab_quantize_format(p, p, 5, 1, 0, 1, 64, p, None) == -1
    # threshold: workspace
    assert lib.tab_threshold_workspace_bytes(0, 10) == 0
    assert lib.tab_threshold(p, 4, 100, ctypes.c_float(0.7), p, None, 0, None) == -3
    # a packed image too large for 32-bit offsets inside one workgroup
    assert lib.tab_conv2d_packed(p, p, p, 3, 0, 0, 1, 1, 1, 30000, 30000, 64, 4, 1, 1, p, None) == -2
    assert b"32-bit" in lib.tab_last_error()
    # a wave addresses its rows of Y with 32-bit byte offsets: 128 rows of KN floats stay below 2 GiB
    assert lib.tab_conv2d_packed(p, p, p, 3, 0, 0, 1, 1, 1, 4, 4, 64, 1 << 22, 1, 1, p, None) == -2
    assert b"KN" in lib.tab_last_error()


def test_conv2d_launches_names_the_one_launch_cases():
    """tab_conv2d_launches: 1 for a small 1x1 convolution without padding on 64..512 channels (types 0..3), else 2."""
    lib = _capi.load()
    p = 4096
    launches = lambda type, p1, s, N, HW, C, KN, K, x=p: lib.tab_conv2d_launches(x, type, p1, p1, s, s, N, HW, HW, C, KN, K, K)  # noqa: E731
    assert launches(3, 0, 2, 16, 14, 256, 512, 1) == 1
    assert launches(0, 0, 1, 4, 28, 64, 100, 1) == 1
    assert launches(3, 1, 1, 16, 14, 256, 256, 3) == 2      # 3x3
    assert launches(3, 1, 2, 16, 14, 256, 512, 1) == 2      # padding
    assert launches(3, 0, 2, 16, 14, 192, 512, 1) == 2      # three words per pixel
    assert launches(4, 0, 2, 16, 14, 256, 512, 1) == 2      # the CPU-only types
    assert launches(3, 0, 1, 256, 28, 128, 256, 1) == 2     # a launch too large for it
    assert launches(3, 0, 2, 16, 14, 256, 512, 1, x=p + 4) == 2  # X not aligned for 16-byte loads
    assert launches(7, 0, 2, 16, 14, 256, 512, 1) == 0      # bad arguments
    try:
        assert lib.tab_set_conv_kernel(1, 2) == 0
        assert launches(3, 0, 2, 16, 14, 256, 512, 1) == 2  # a forced conv kernel keeps the two launches
    finally:
        assert lib.tab_set_conv_kernel(0, -1) == 0


def test_set_conv_kernel_validates_without_a_gpu():
    lib = _capi.load()
    try:
        for kernel, tile, ok in [(0, -1, True), (1, -1, True), (1, 6, True), (1, 7, True), (1, 11, True), (1, 12, False), (2, 2, True), (2, 3, False),
                                 (0, 0, False), (3, -1, False)]:
            assert (lib.tab_set_conv_kernel(kernel, tile) == 0) == ok, (kernel, tile)
        assert b"no conv kernel" in lib.tab_last_error()
    finally:
        assert lib.tab_set_conv_kernel(0, -1) == 0


def test_python_mirror_names_and_input_checks():
    # exported names of the CUDA module (TAB_GPU.cpp:62-65) and of the CPU module (TAB_CPU.cpp:636-639)
    for name in ("Quantize", "Conv2d", "TAB_Quantize", "TAB_Conv2d"):
        assert callable(getattr(tab_amd, name))
    x = torch.zeros(1, 4, 4, 64)
    ths = torch.zeros(1)
    # CHECK_INPUT (TAB_GPU.cpp:7-9): a CPU tensor is refused with the reference's message
    with pytest.raises(RuntimeError, match="X must be a CUDA tensor"):
        tab_amd.Quantize(x, ths, 2, 1, 4, 4, 64)
    with pytest.raises(RuntimeError, match="X must be a CUDA tensor"):
        tab_amd.Conv2d(x, torch.zeros(4, dtype=torch.int64), ths, torch.zeros(4, dtype=torch.int32),
                       0, 1, 1, 1, 1, 1, 4, 4, 64, 4, 3, 3)
    assert tab_amd.out_shape(112, 112, 3, 3, 1, 1, 1, 1) == (112, 112)
    assert tab_amd.packed_channels(256) == 4
    with pytest.raises(RuntimeError, match="X must be a CUDA tensor"):
        tab_amd.QuantizeFormat(x, ths, 4, 1, 4, 4, 64)
    assert (tab_amd.DRF, tab_amd.RTN) == (4, 5) and tab_amd.operand_words(5, 0, 64) == 2


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(ImportError, match="no fallback"):
        _capi.load(str(tmp_path / "libtab_amd.so"))


def test_extension_module_names_and_cpu_rejection():
    """The pybind module exports the reference's names (TAB_GPU.cpp:62-65) and applies
    CHECK_INPUT (TAB_GPU.cpp:7-9) before touching the device."""
    import TAB_CUDA as TAB

    public = [n for n in dir(TAB) if not n.startswith("_")]
    assert "Conv2d" in public and "Quantize" in public
    with pytest.raises(RuntimeError, match="X must be a CUDA tensor"):
        TAB.Quantize(torch.zeros(1, 4, 4, 64), torch.zeros(1), 2, 1, 4, 4, 64)


def test_multiply_shift_division_is_exact_below_2_31():
    """The conv kernels decode output rows with x / d = (x * mul) >> shift; the same inline function evaluated on the
    host must equal integer division for every divisor and numerator below 2^31, edge cases first."""
    import random
    lib = ctypes.CDLL(_capi.LIB_PATH)
    f = lib.tab_internal_div32
    f.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
    f.restype = ctypes.c_uint32
    rng = random.Random(7)
    top = 2 ** 31 - 1
    divisors = list(range(1, 300)) + [2 ** k for k in range(31)] + [2 ** k + 1 for k in range(30)] + \
        [2 ** k - 1 for k in range(2, 32)] + [784, 3136, 12544, 50176, 200704, 802816] + \
        [rng.randrange(1, 2 ** 31) for _ in range(1500)]
    for d in divisors:
        xs = {0, 1, d - 1, d, min(d + 1, top), top, top - 1, (top // d) * d, max((top // d) * d - 1, 0)}
        xs.update(rng.randrange(0, 2 ** 31) for _ in range(12))
        xs.update(min(k * d + o, top) for k in (1, 2, 3, 7) for o in (-1, 0, 1) if k * d + o >= 0)
        for x in xs:
            assert f(x, d) == x // d, (x, d)
