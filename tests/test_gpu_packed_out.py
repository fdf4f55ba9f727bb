"""GPU parity of Conv2dPackedOut (conv with the quantize + pack of its output fused into the
epilogue) against the oracle's conv followed by the oracle's quantizer.  Bit-exact."""
import numpy as np
import pytest
import torch

import oracle
import tab_amd
from helpers import TYPE_NAMES, act_bits, make_layer, weight_bits

pytestmark = pytest.mark.gpu


def _out_thresholds(N, kind):
    """Per-image thresholds: conv outputs are integers, so integer thresholds put values exactly
    on the boundary of the strict compares (TAB_GEMM.cu:184-192, 231)."""
    if kind == "zero":
        return torch.zeros(N)
    if kind == "integer":
        return torch.tensor([float(3 * n - 4) for n in range(N)])
    return torch.tensor([5.5 + 2.25 * n for n in range(N)])


def _packed_out_case(type, N, H, W, C, KN, KH, KW, p1, p2, s1, s2, out_bits, ths_kind, seed=0):
    print(f"[case] Conv2dPackedOut {TYPE_NAMES[type]} N={N} {H}x{W}x{C}->{KN} k{KH}x{KW} pad({p1},{p2}) "
          f"stride({s1},{s2}) out_bits={out_bits} ths={ths_kind}", flush=True)
    x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, KH, KW, seed=seed)
    qw, btn = oracle.quantize(w.numpy(), w_ths.numpy(), weight_bits(type), KN, KH, KW, C)
    y = oracle.conv2d(x.numpy(), qw, x_ths.numpy(), btn, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    OH, OW = tab_amd.out_shape(H, W, KH, KW, p1, p2, s1, s2)
    out_ths = _out_thresholds(N, ths_kind)
    # the conv output's memory is (n, oh, ow, kn): the next layer's NHWC activation
    want, _ = oracle.quantize(np.ascontiguousarray(y).reshape(N, OH, OW, KN), out_ths.numpy(), out_bits, N, OH, OW, KN)

    QX, _ = tab_amd.Quantize(x.cuda(), x_ths.cuda(), act_bits(type), N, H, W, C)
    got = tab_amd.Conv2dPackedOut(QX, torch.from_numpy(qw).cuda(), torch.from_numpy(btn).cuda(), type, p1, p2, s1, s2,
                                  N, H, W, C, KN, KH, KW, out_ths.cuda(), out_bits)
    torch.cuda.synchronize()
    assert got.dtype == torch.int64 and tuple(got.shape) == (N, OH, OW, (KN + 63) // 64, out_bits)
    assert np.array_equal(got.cpu().numpy(), want)
    return got


CASES = [
    # N, H, W, C, KN, KH, KW, p1, p2, s1, s2
    (2, 12, 12, 128, 64, 3, 3, 1, 1, 1, 1),    # one full word of filters
    (3, 9, 6, 70, 5, 3, 3, 1, 0, 1, 2),        # KN < 32: tail bits of the only word stay zero
    (2, 10, 10, 192, 130, 3, 3, 1, 1, 1, 1),   # three words of filters, the last one 2 bits
    (5, 5, 5, 256, 96, 3, 3, 0, 0, 1, 1),      # 9 output pixels per image: a tile spans several images
    (2, 16, 16, 64, 200, 1, 1, 0, 0, 2, 2),    # 1x1 stride 2
    (2, 5, 5, 64, 72, 3, 3, 3, 3, 1, 1),       # padding as wide as the kernel
    (40, 2, 2, 128, 65, 2, 2, 0, 0, 1, 1),     # one output pixel per image: a tile of rows spans 40 images and thresholds
    (3, 1, 17, 128, 33, 1, 3, 0, 1, 1, 1),     # images of one line
    (2, 13, 13, 256, 129, 3, 3, 1, 1, 4, 4),   # stride beyond the kernel
]


@pytest.fixture
def restore_kernel_choice():
    yield
    tab_amd.set_conv_kernel(tab_amd.CONV_AUTO, -1)


@pytest.mark.parametrize("out_bits", [1, 2])
@pytest.mark.parametrize("type", [0, 1, 2, 3])
@pytest.mark.parametrize("case", CASES)
def test_packed_out(type, case, out_bits):
    for kind in ("zero", "integer", "fraction"):
        _packed_out_case(type, *case, out_bits, kind, seed=type + out_bits)


@pytest.mark.parametrize("tile", [0, 1, 2, 4, 5, 6, 7, 8, 9, 10, 11])
@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_packed_out_every_tile(type, tile, restore_kernel_choice):
    """Every shape packs its output: C = 192 and 256 take the kernel that multiplies with the weights first and packs
    inside a lane (BTN hands its per-filter bias round through LDS there), C = 70 the one that packs by ballot."""
    tab_amd.set_conv_kernel(tab_amd.CONV_MATRIX, tile)
    for out_bits in (1, 2):
        for case in (CASES[1], CASES[2], CASES[3], (1, 28, 28, 256, 256, 3, 3, 1, 1, 1, 1)):
            _packed_out_case(type, *case, out_bits, "integer", seed=9 + out_bits)


def test_packed_out_ignores_popcount_choice(restore_kernel_choice):
    """The packed epilogue lives in the matrix-core kernel; asking for the popcount kernel must not
    change the result of this entry point."""
    tab_amd.set_conv_kernel(tab_amd.CONV_POPCOUNT, -1)
    _packed_out_case(3, *CASES[2], 1, "zero")


def test_two_layers_chained_packed():
    """BNN layer -> packed output -> BNN layer, no fp32 activation in between, against the oracle
    doing conv, quantize, conv."""
    N, H, W, C1, C2, C3 = 2, 14, 14, 128, 192, 80
    x, x_ths, w1, w1_ths = make_layer(3, N, H, W, C1, C2, 3, 3, seed=1)
    _, _, w2, w2_ths = make_layer(3, N, H, W, C2, C3, 3, 3, seed=2)
    qw1, btn1 = oracle.quantize(w1.numpy(), w1_ths.numpy(), 1, C2, 3, 3, C1)
    qw2, btn2 = oracle.quantize(w2.numpy(), w2_ths.numpy(), 1, C3, 3, 3, C2)
    zeros = np.zeros(N, dtype=np.float32)
    y1 = oracle.conv2d(x.numpy(), qw1, zeros, btn1, 3, 1, 1, 1, 1, N, H, W, C1, C2, 3, 3)
    want = oracle.conv2d(np.ascontiguousarray(y1).reshape(N, H, W, C2), qw2, zeros, btn2, 3, 1, 1, 1, 1, N, H, W, C2, C3, 3, 3)

    z = torch.zeros(N, device="cuda")
    QX, _ = tab_amd.Quantize(x.cuda(), z, 1, N, H, W, C1)
    Q1 = tab_amd.Conv2dPackedOut(QX, torch.from_numpy(qw1).cuda(), torch.from_numpy(btn1).cuda(), 3, 1, 1, 1, 1,
                                 N, H, W, C1, C2, 3, 3, z, 1)
    y2 = tab_amd.Conv2dPacked(Q1, torch.from_numpy(qw2).cuda(), torch.from_numpy(btn2).cuda(), 3, 1, 1, 1, 1,
                              N, H, W, C2, C3, 3, 3)
    assert np.array_equal(y2.cpu().numpy(), want)


def test_packed_out_rejects_bad_arguments():
    N, H, W, C, KN = 1, 4, 4, 64, 64
    QX = torch.zeros((N, H, W, 1, 1), dtype=torch.int64, device="cuda")
    QW = torch.zeros((KN, 3, 3, 1, 1), dtype=torch.int64, device="cuda")
    btn = torch.zeros(KN, dtype=torch.int32, device="cuda")
    ths = torch.zeros(N, device="cuda")
    with pytest.raises(RuntimeError, match="out_bitwidth"):
        tab_amd.Conv2dPackedOut(QX, QW, btn, 3, 1, 1, 1, 1, N, H, W, C, KN, 3, 3, ths, 3)
    with pytest.raises(RuntimeError, match="out_thresholds has"):
        tab_amd.Conv2dPackedOut(QX, QW, btn, 3, 1, 1, 1, 1, N, H, W, C, KN, 3, 3, torch.zeros(0, device="cuda"), 1)
    with pytest.raises(RuntimeError, match="dtype"):
        tab_amd.Conv2dPackedOut(QX, QW, btn, 3, 1, 1, 1, 1, N, H, W, C, KN, 3, 3, ths.double(), 1)


SHORT_K_PACKED = [
    # K of at most nine words (the register-resident kernel's own packed epilogue)
    (2, 12, 12, 64, 64, 3, 3, 1, 1, 1, 1),     # 9 words, one word of filters
    (3, 9, 7, 33, 70, 3, 3, 1, 0, 2, 1),       # ragged KN: the second word holds six filters, tiles span images
    (2, 8, 8, 320, 130, 1, 1, 0, 0, 1, 1),     # three words of filters, the last with two
    (5, 3, 3, 64, 31, 3, 3, 1, 1, 1, 1),       # fewer than 32 filters
    (4, 6, 6, 512, 256, 1, 1, 0, 0, 1, 1),     # four full words
    (1, 5, 5, 100, 97, 1, 1, 0, 0, 1, 1),      # 97 filters: one half-word used in the last word
]


@pytest.mark.parametrize("out_bits", [1, 2])
@pytest.mark.parametrize("type", [0, 1, 2, 3])
@pytest.mark.parametrize("case", SHORT_K_PACKED)
def test_packed_out_short_k(type, case, out_bits):
    for kind in ("zero", "integer", "fraction"):
        _packed_out_case(type, *case, out_bits, kind, seed=3 * type + out_bits)
