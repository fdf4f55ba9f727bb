"""The mixed launches of the matrix-core conv kernel (tab_set_conv_kernel(TAB_CONV_MATRIX, 10 or 11)): 128x128 (10) or 128x256
(11) tiles for the whole rounds of the chip, 64x64 split-K quarter tiles for the rest of the last round.  A round is the chip's compute units, far
more tiles than an oracle-sized layer has, so these tests shrink the round through the library's test hook: layers of a few
tiles then mix whole tiles and quarters, with ragged edges in both.  Bit-exact against the CPU oracle."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
import tab_amd
from helpers import TYPE_NAMES, make_layer, weight_bits
from tab_amd import _capi

pytestmark = pytest.mark.gpu


@pytest.fixture(params=[10, 11])
def tail_round(request):
    lib = ctypes.CDLL(_capi.LIB_PATH)
    lib.tab_internal_set_tail_round.argtypes = [ctypes.c_int]
    lib.tab_internal_set_tail_round.restype = None
    tab_amd.set_conv_kernel(tab_amd.CONV_MATRIX, request.param)
    yield lib.tab_internal_set_tail_round
    lib.tab_internal_set_tail_round(0)
    tab_amd.set_conv_kernel(tab_amd.CONV_AUTO, -1)


GEOMETRIES = [
    # N, H, W, C, KN, KH, KW, p1, p2, s1, s2              tiles of 128 x 128
    (2, 14, 14, 256, 256, 3, 3, 1, 1, 1, 1),             # 4 x 2, rows ragged
    (3, 13, 11, 250, 200, 3, 3, 1, 1, 1, 1),             # 4 x 2, rows, filters and channels ragged
    (5, 9, 9, 512, 130, 3, 3, 1, 1, 2, 2),               # 1 x 2: the second filter tile holds two filters, its second quarter column none
    (1, 28, 28, 256, 64, 1, 1, 0, 0, 1, 1),              # 7 x 1, four words of K: one zero-padded chunk of eight in the quarters
    (7, 8, 8, 256, 384, 3, 3, 1, 0, 1, 1),               # 3 x 3 (3 x 2 of 128 x 256, the second half filled)
    (4, 10, 10, 256, 600, 3, 3, 1, 1, 1, 1),             # 4 x 5 (4 x 3 of 128 x 256: the last filter tile holds 88 filters)
    (2, 12, 12, 768, 96, 2, 2, 0, 1, 1, 1),              # twelve words per pixel, 2x2 taps
    (3, 16, 16, 128, 256, 3, 3, 1, 1, 1, 1),             # two words per pixel: the whole tiles take chunks of six words across taps
    (2, 10, 10, 384, 130, 3, 3, 1, 1, 1, 1),             # six words per pixel
    (2, 9, 9, 128, 70, 2, 2, 0, 0, 1, 1),                # two words per pixel, K = 8 words: whole tiles in chunks of two
]


@pytest.mark.parametrize("round_size", [1, 3, 5])
@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_mixed_launch_against_oracle(type, round_size, tail_round):
    tail_round(round_size)
    for N, H, W, C, KN, KH, KW, p1, p2, s1, s2 in GEOMETRIES:
        print(f"[case] mixed launch {TYPE_NAMES[type]} round {round_size} N={N} {H}x{W}x{C}->{KN} k{KH}x{KW}", flush=True)
        x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, KH, KW, seed=round_size + type, relu=(type == 1))
        qw, btn = oracle.quantize(w.numpy(), w_ths.numpy(), weight_bits(type), KN, KH, KW, C)
        args = (type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
        want = oracle.conv2d(x.numpy(), qw, x_ths.numpy(), btn, *args)
        y = tab_amd.Conv2d(x.cuda(), torch.from_numpy(qw).cuda(), x_ths.cuda(), torch.from_numpy(btn).cuda(), *args)
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy(), want)


@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_mixed_launch_packed_output(type, tail_round):
    """Packed output (the next layer's operand) from the mixed launch equals quantizing its fp32 output."""
    N, H, W, C, KN = 3, 12, 12, 256, 192
    x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, 3, 3, seed=9 + type, relu=(type == 1))
    QW, BTN = tab_amd.Quantize(w.cuda(), w_ths.cuda(), weight_bits(type), KN, 3, 3, C)
    for round_size in (2, 3):
        tail_round(round_size)
        y = tab_amd.Conv2d(x.cuda(), QW, x_ths.cuda(), BTN, type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3)
        qx = tab_amd.QuantizeActivation(x.cuda(), x_ths.cuda(), 2 if type in (0, 1) else 1, N, H, W, C)
        for out_bits, ths in ((2, 7.5), (1, 0.0)):
            next_ths = torch.full((N,), ths, device="cuda")
            want = tab_amd.QuantizeActivation(y, next_ths, out_bits, N, H, W, KN)
            got = tab_amd.Conv2dPackedOut(qx, QW, BTN, type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3, next_ths, out_bits)
            torch.cuda.synchronize()
            assert torch.equal(got, want), (type, round_size, out_bits)


def test_mixed_launch_formats_4_and_5(tail_round):
    tail_round(3)
    for type in (4, 5):
        N, H, W, C, KN = 2, 14, 14, 256 if type == 4 else 128, 160
        g = torch.Generator("cpu").manual_seed(type)
        x = torch.randn((N, H, W, C), generator=g).abs() if type == 4 else torch.randn((N, H, W, C), generator=g)
        w = torch.randn((KN, 3, 3, C), generator=g).abs() if type == 4 else torch.randn((KN, 3, 3, C), generator=g)
        x_ths, w_ths = torch.full((N,), 0.6), torch.full((KN,), 0.5)
        qw = oracle.quantize_format(w.numpy(), w_ths.numpy(), type, KN, 3, 3, C)
        btn = np.zeros(KN, dtype=np.int32)
        args = (type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3)
        want = oracle.conv2d(x.numpy(), qw, x_ths.numpy(), btn, *args)
        y = tab_amd.Conv2d(x.cuda(), torch.from_numpy(qw).cuda(), x_ths.cuda(), torch.from_numpy(btn).cuda(), *args)
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy(), want), type


@pytest.mark.parametrize("geometry,picked", [((256, 14, 14, 256, 256), 10), ((64, 28, 28, 512, 512), 11)])
def test_chosen_for_a_layer_of_a_few_rounds_and_equal_to_the_large_tile(geometry, picked):
    """At benchmark sizes the library picks the mixed launches by itself (N=256 14x14x256: 784 tiles of 128x128 on 256 compute
    units, three whole rounds and a sixteenth; N=64 28x28x512: 784 tiles of 128x256); the output equals the plain 128x128
    launch's."""
    N, H, W, C, KN = geometry
    g = torch.Generator("cuda").manual_seed(3)
    x = torch.randn((N, H, W, C), generator=g, device="cuda")
    w = torch.randn((KN, 3, 3, C), generator=g, device="cuda")
    ths = torch.full((N,), 0.4, device="cuda")
    for type in (0, 3):
        QW, BTN = tab_amd.Quantize(w, torch.full((KN,), 0.3, device="cuda"), weight_bits(type), KN, 3, 3, C)
        try:
            tab_amd.set_conv_kernel(tab_amd.CONV_AUTO, -1)
            y = tab_amd.Conv2d(x, QW, ths, BTN, type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3)
            tab_amd.set_conv_kernel(tab_amd.CONV_MATRIX, 0)
            y0 = tab_amd.Conv2d(x, QW, ths, BTN, type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3)
        finally:
            tab_amd.set_conv_kernel(tab_amd.CONV_AUTO, -1)
        assert torch.equal(y, y0)
    lib = ctypes.CDLL(_capi.LIB_PATH)
    lib.tab_internal_conv_shape.restype = ctypes.c_int
    lib.tab_internal_conv_shape.argtypes = [ctypes.c_int] * 6 + [ctypes.POINTER(ctypes.c_float)]
    cost = ctypes.c_float()
    assert lib.tab_internal_conv_shape(3, N * H * W, KN, 9 * (C // 64), C // 64, 0, ctypes.byref(cost)) == picked
