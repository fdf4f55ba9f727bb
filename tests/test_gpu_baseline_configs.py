"""GPU parity on the benchmark's own configurations: every layer shape of the ResNet-18 set (N=16, ternary
activations on ReLU inputs included), the VGG-16-style TNN stack (N=32) and the large-batch sweep
(N in {64, 128, 256}, 28x28, C = KN in {256, 512}, 3x3 and 1x1, stride 1 and 2, pad (1,1) / (1,0) / (0,0)).

Whole tensors are compared with the CPU oracle where it finishes in seconds.  At full batch the reference
pipeline (TAB_GEMM.cu:325-527, M up to 1.6 M rows) is checked through properties that do not depend on size:
images are independent, so images computed alone must equal the same images inside the batch; the first and
the last image are compared with the oracle; every output obeys |y| <= KH*KW*C and, for BNN,
y = KH*KW*C (mod 2)."""
import numpy as np
import pytest
import torch

import oracle
import tab_amd
from helpers import TYPE_NAMES, act_bits, make_layer, weight_bits

pytestmark = pytest.mark.gpu


def _against_oracle(type, N, H, W, C, KN, KH, KW, p1, p2, s1, s2, seed=0, relu=False):
    print(f"[case] Conv2d {TYPE_NAMES[type]} N={N} {H}x{W}x{C}->{KN} k{KH}x{KW} pad({p1},{p2}) stride({s1},{s2}) relu={relu}",
          flush=True)
    x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, KH, KW, seed=seed, relu=relu)
    qw_o, btn_o = oracle.quantize(w.numpy(), w_ths.numpy(), weight_bits(type), KN, KH, KW, C)
    want = oracle.conv2d(x.numpy(), qw_o, x_ths.numpy(), btn_o, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    QW, BTN = tab_amd.Quantize(w.cuda(), w_ths.cuda(), weight_bits(type), KN, KH, KW, C)
    y = tab_amd.Conv2d(x.cuda(), QW, x_ths.cuda(), BTN, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    torch.cuda.synchronize()
    assert tuple(y.shape) == want.shape
    assert np.array_equal(QW.cpu().numpy(), qw_o) and np.array_equal(BTN.cpu().numpy(), btn_o)
    got = y.cpu().numpy()
    assert np.array_equal(got, want), f"max |diff| = {np.abs(got - want).max()}"


def _full_batch_properties(type, N, H, W, C, KN, KH, KW, p1, p2, s1, s2, seed=0, relu=False):
    print(f"[case] full batch {TYPE_NAMES[type]} N={N} {H}x{W}x{C}->{KN} k{KH}x{KW} pad({p1},{p2}) stride({s1},{s2})", flush=True)
    g = torch.Generator("cuda").manual_seed(seed)
    x = torch.randn((N, H, W, C), generator=g, device="cuda")
    if relu:
        x = torch.relu(x)
    w = torch.randn((KN, KH, KW, C), generator=g, device="cuda")
    ab, wb = act_bits(type), weight_bits(type)
    x_ths = (0.7 * x.abs().reshape(N, -1).mean(dim=1)).contiguous() if ab == 2 else torch.zeros(N, device="cuda")
    w_ths = (0.7 * w.abs().reshape(KN, -1).mean(dim=1)).contiguous() if wb == 2 else torch.zeros(KN, device="cuda")
    QW, BTN = tab_amd.Quantize(w, w_ths, wb, KN, KH, KW, C)
    y = tab_amd.Conv2d(x, QW, x_ths, BTN, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    # images computed alone (a smaller launch, usually another tile shape) equal the same images in the batch
    for first in (0, N // 2 - 1, N - 2):
        part = tab_amd.Conv2d(x[first:first + 2].contiguous(), QW, x_ths[first:first + 2].contiguous(), BTN, type,
                              p1, p2, s1, s2, 2, H, W, C, KN, KH, KW)
        torch.cuda.synchronize()
        assert torch.equal(y[first:first + 2], part), f"images {first}, {first + 1} differ from the same images computed alone"
    qw_h, btn_h = QW.cpu().numpy(), BTN.cpu().numpy()
    for n in (0, N - 1):  # the last image: another threshold and the far end of every index range
        want = oracle.conv2d(x[n:n + 1].cpu().numpy(), qw_h, x_ths[n:n + 1].cpu().numpy(), btn_h, type, p1, p2, s1, s2,
                             1, H, W, C, KN, KH, KW)
        assert np.array_equal(y[n:n + 1].cpu().numpy(), want), f"image {n} differs from the oracle"
    assert bool((y.abs() <= KH * KW * C).all())
    if type == 3:
        assert bool(((y.to(torch.int64) - KH * KW * C) % 2 == 0).all())
    del x, y
    torch.cuda.empty_cache()


# ---- TNN VGG-16-style stack, N=32: 224^2x64, 112^2x128, 56^2x256, 28^2x512, 14^2x512 (C -> C, 3x3 pad 1 stride 1) ----
VGG = [(224, 64), (112, 128), (56, 256), (28, 512), (14, 512)]


@pytest.mark.parametrize("HW,C", VGG)
def test_vgg_layers_one_image_against_oracle(HW, C):
    _against_oracle(0, 1, HW, HW, C, C, 3, 3, 1, 1, 1, 1, seed=HW)


@pytest.mark.parametrize("HW,C", VGG)
def test_vgg_layers_full_batch(HW, C):
    _full_batch_properties(0, 32, HW, HW, C, C, 3, 3, 1, 1, 1, 1, seed=HW + 1)


# ---- ResNet-18 set at N=16: ternary activations (TBN) and ternary weights (BTN) on ReLU inputs, every 3x3 shape ----
RESNET18_3X3 = [(56, 64, 64, 1), (28, 128, 128, 1), (14, 256, 256, 1), (7, 512, 512, 1),
                (56, 64, 128, 2), (28, 128, 256, 2), (14, 256, 512, 2)]


@pytest.mark.parametrize("type", [1, 2])
@pytest.mark.parametrize("HW,C,KN,stride", RESNET18_3X3)
def test_resnet18_tbn_btn_relu_all_3x3_shapes(type, HW, C, KN, stride):
    _against_oracle(type, 16, HW, HW, C, KN, 3, 3, 1, 1, stride, stride, seed=7, relu=True)


@pytest.mark.parametrize("type", [0, 1, 2])
@pytest.mark.parametrize("HW,C,KN", [(56, 64, 128), (28, 128, 256), (14, 256, 512)])
def test_resnet18_downsample_1x1_other_types(type, HW, C, KN):
    _against_oracle(type, 16, HW, HW, C, KN, 1, 1, 0, 0, 2, 2, seed=8, relu=(type != 0))


# ---- large-batch sweep: every (C, kernel, stride, padding) point for all four types at a small batch ----
SWEEP_POINTS = [(C, k, s, pads) for C in (256, 512) for k in (3, 1) for s in (1, 2)
                for pads in (((1, 1) if k == 3 else (0, 0)), (1, 0))]


@pytest.mark.parametrize("type", [0, 1, 2, 3])
@pytest.mark.parametrize("C,k,s,pads", SWEEP_POINTS)
def test_sweep_points_small_batch_against_oracle(type, C, k, s, pads):
    _against_oracle(type, 3, 28, 28, C, C, k, k, pads[0], pads[1], s, s, seed=C + 10 * k + s)


@pytest.mark.parametrize("type", [0, 1, 2, 3])
@pytest.mark.parametrize("N,C,k,s,pads", [
    (64, 256, 3, 1, (1, 0)),
    (64, 512, 1, 2, (1, 0)),
    (128, 512, 1, 1, (0, 0)),
    (128, 512, 3, 2, (1, 0)),
    (128, 256, 3, 1, (1, 1)),
    (256, 256, 1, 1, (0, 0)),
])
def test_sweep_points_full_batch(type, N, C, k, s, pads):
    _full_batch_properties(type, N, 28, 28, C, C, k, k, pads[0], pads[1], s, s, seed=N + C + k)
