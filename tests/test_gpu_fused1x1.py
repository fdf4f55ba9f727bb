"""The one-launch quantize + 1x1 conv kernel (tab_conv_fused1x1.hip) that Conv2d takes for small 1x1 layers without
padding: bit-exact against the CPU oracle (quantize, then conv), and equal to the two-kernel path it replaces."""
import numpy as np
import pytest
import torch

import oracle
import tab_amd
from helpers import TYPE_NAMES, act_bits, make_layer, weight_bits

pytestmark = pytest.mark.gpu


@pytest.fixture
def restore_kernel_choice():
    yield
    tab_amd.set_conv_kernel(tab_amd.CONV_AUTO, -1)


def _two_kernel_path(x, QW, x_ths, BTN, args):
    """Conv2d under a forced kernel choice, which keeps the call on quantize + conv."""
    tab_amd.set_conv_kernel(tab_amd.CONV_MATRIX, -1)
    try:
        return tab_amd.Conv2d(x, QW, x_ths, BTN, *args)
    finally:
        tab_amd.set_conv_kernel(tab_amd.CONV_AUTO, -1)


def _case(type, N, H, W, C, KN, s1, s2, seed=0, relu=False, x=None, x_ths=None):
    print(f"[case] fused 1x1 {TYPE_NAMES[type]} N={N} {H}x{W}x{C}->{KN} stride({s1},{s2})", flush=True)
    x0, ths0, w, w_ths = make_layer(type, N, H, W, C, KN, 1, 1, seed=seed, relu=relu)
    x = x0 if x is None else x
    x_ths = ths0 if x_ths is None else x_ths
    qw_o, btn_o = oracle.quantize(w.numpy(), w_ths.numpy(), weight_bits(type), KN, 1, 1, C)
    args = (type, 0, 0, s1, s2, N, H, W, C, KN, 1, 1)
    want = oracle.conv2d(x.numpy(), qw_o, x_ths.numpy(), btn_o, *args)
    QW, BTN = torch.from_numpy(qw_o).cuda(), torch.from_numpy(btn_o).cuda()
    y = tab_amd.Conv2d(x.cuda(), QW, x_ths.cuda(), BTN, *args)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), want)
    assert torch.equal(y, _two_kernel_path(x.cuda(), QW, x_ths.cuda(), BTN, args))


CASES = [
    # N, H, W, C, KN, s1, s2
    (16, 14, 14, 256, 512, 2, 2),   # the three 1x1 stride-2 layers of the ResNet-18 set, N = 16
    (16, 28, 28, 128, 256, 2, 2),
    (4, 56, 56, 64, 128, 2, 2),
    (3, 9, 11, 64, 20, 2, 3),       # one word; 60 output pixels: the second tile partly empty; 20 of 128 filters
    (2, 7, 8, 128, 70, 1, 2),       # two words, ragged filter count across waves
    (5, 5, 5, 256, 130, 1, 1),      # four words, stride 1, a second filter group of two filters
    (2, 6, 6, 512, 33, 3, 3),       # eight words, stride 3
    (40, 1, 1, 64, 5, 1, 1),        # one pixel per image: a tile spans 32 images and their thresholds
    (1, 1, 1, 64, 1, 1, 1),         # a single output element
    (2, 10, 3, 512, 300, 2, 1),     # images of three columns
]


@pytest.mark.parametrize("type", [0, 1, 2, 3])
@pytest.mark.parametrize("case", CASES)
def test_fused_1x1_against_oracle(type, case, restore_kernel_choice):
    _case(type, *case, seed=31 + type, relu=(type == 1))


@pytest.mark.parametrize("type", [0, 3])
def test_fused_1x1_ties_and_special_values(type, restore_kernel_choice):
    """Values on the thresholds, signed zeros, infinities and NaN go through the quantizer's own compares
    (TAB_GEMM.cu:184-192, 231): strict, ordered, ties and NaN give 0 (ternary) or +1 (binary)."""
    N, H, W, C, KN = 2, 6, 6, 128, 40
    g = torch.Generator("cpu").manual_seed(5)
    x = torch.randn((N, H, W, C), generator=g)
    ths = torch.tensor([0.5, 0.25]) if act_bits(type) == 2 else torch.tensor([0.0, 0.25])
    flat = x.view(N, -1)
    for n in range(N):
        t = float(ths[n])
        specials = torch.tensor([t, -t, 0.0, -0.0, float("inf"), float("-inf"), float("nan"), np.nextafter(np.float32(t), np.float32(1)),
                                 np.nextafter(np.float32(-t), np.float32(-1))], dtype=torch.float32)
        idx = torch.randperm(flat.shape[1], generator=g)[: 40 * len(specials)]
        flat[n, idx] = specials.repeat(40)
    _case(type, N, H, W, C, KN, 2, 2, seed=3, x=x.contiguous(), x_ths=ths.float())


def test_fused_1x1_arbitrary_weight_bits(restore_kernel_choice):
    """QW and btn are caller data: any 64-bit pattern follows the reference's formulas (TAB_GEMM.cu:25-147)."""
    N, H, W, C, KN = 3, 8, 8, 256, 72
    rng = np.random.default_rng(2)
    for type in range(4):
        x, x_ths, _, _ = make_layer(type, N, H, W, C, KN, 1, 1, seed=8)
        qw = rng.integers(-2**63, 2**63 - 1, size=(KN, 1, 1, C // 64, weight_bits(type)), dtype=np.int64, endpoint=True)
        btn = rng.integers(0, 1000, size=KN).astype(np.int32)
        args = (type, 0, 0, 2, 2, N, H, W, C, KN, 1, 1)
        want = oracle.conv2d(x.numpy(), qw, x_ths.numpy(), btn, *args)
        y = tab_amd.Conv2d(x.cuda(), torch.from_numpy(qw).cuda(), x_ths.cuda(), torch.from_numpy(btn).cuda(), *args)
        assert np.array_equal(y.cpu().numpy(), want), f"type {type}"


def test_large_1x1_keeps_the_two_kernel_path_and_agrees():
    """Beyond the fused kernel's launch size Conv2d runs quantize + conv; either way the images are independent:
    a slice of the batch small enough for the fused kernel gives the same rows."""
    N, H, W, C, KN = 192, 28, 28, 128, 256
    g = torch.Generator("cuda").manual_seed(1)
    x = torch.randn((N, H, W, C), generator=g, device="cuda")
    w = torch.randn((KN, 1, 1, C), generator=g, device="cuda")
    QW, BTN = tab_amd.Quantize(w, torch.zeros(KN, device="cuda"), 1, KN, 1, 1, C)
    ths = torch.zeros(N, device="cuda")
    y = tab_amd.Conv2d(x, QW, ths, BTN, 3, 0, 0, 1, 1, N, H, W, C, KN, 1, 1)
    for first in (0, N - 4):
        part = tab_amd.Conv2d(x[first:first + 4].contiguous(), QW, ths[first:first + 4].contiguous(), BTN, 3, 0, 0, 1, 1, 4, H, W, C,
                              KN, 1, 1)
        assert torch.equal(y[first:first + 4], part)
