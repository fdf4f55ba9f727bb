"""GPU parity of Conv2d / Conv2dPacked (through the C ABI) against the CPU oracle.
Integer-valued results stored as fp32: the bar is bit-exact equality."""
import numpy as np
import pytest
import torch

import oracle
import tab_amd
from helpers import TYPE_NAMES, act_bits, make_layer, weight_bits

pytestmark = pytest.mark.gpu


def _conv_case(type, N, H, W, C, KN, KH, KW, p1, p2, s1, s2, seed=0, relu=False):
    print(f"[case] Conv2d {TYPE_NAMES[type]} N={N} {H}x{W}x{C}->{KN} k{KH}x{KW} pad({p1},{p2}) "
          f"stride({s1},{s2}) relu={relu}", flush=True)
    x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, KH, KW, seed=seed, relu=relu)
    qw_o, btn_o = oracle.quantize(w.numpy(), w_ths.numpy(), weight_bits(type), KN, KH, KW, C)
    want = oracle.conv2d(x.numpy(), qw_o, x_ths.numpy(), btn_o, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)

    QW, BTN = tab_amd.Quantize(w.cuda(), w_ths.cuda(), weight_bits(type), KN, KH, KW, C)
    y = tab_amd.Conv2d(x.cuda(), QW, x_ths.cuda(), BTN, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    torch.cuda.synchronize()
    assert y.dtype == torch.float32 and tuple(y.shape) == want.shape
    assert np.array_equal(QW.cpu().numpy(), qw_o) and np.array_equal(BTN.cpu().numpy(), btn_o)
    got = y.cpu().numpy()
    assert np.array_equal(got, want), f"max |diff| = {np.abs(got - want).max()}"
    # the packed entry point on the separately quantized activation gives the same tensor
    QX, _ = tab_amd.Quantize(x.cuda(), x_ths.cuda(), act_bits(type), N, H, W, C)
    y2 = tab_amd.Conv2dPacked(QX, QW, BTN, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    assert torch.equal(y, y2)


@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_config1_shape(type):
    # the single-image benchmark shape: N=1, 32x32x64 -> 64, 3x3, pad 1, stride 1
    _conv_case(type, 1, 32, 32, 64, 64, 3, 3, 1, 1, 1, 1)


EDGE_CASES = [
    # N, H, W, C, KN, KH, KW, p1, p2, s1, s2
    (2, 7, 7, 64, 8, 3, 3, 1, 1, 2, 2),       # OH = 3 (PyTorch would say 4)
    (2, 9, 6, 70, 5, 3, 3, 1, 0, 1, 2),       # C % 64 != 0, KN % 4 != 0, asymmetric pad/stride
    (2, 8, 8, 128, 16, 1, 1, 0, 0, 2, 2),     # 1x1 stride 2
    (1, 6, 5, 200, 7, 2, 3, 2, 1, 1, 1),      # even kernel, pad > k/2
    (3, 5, 5, 64, 4, 1, 1, 1, 0, 2, 1),       # 1x1 with padding
    (1, 3, 3, 64, 1, 3, 3, 0, 0, 1, 1),       # single output element
    (2, 12, 12, 192, 130, 3, 3, 1, 1, 1, 1),  # KN not a multiple of the 64/128 tile
    (1, 10, 10, 64, 66, 5, 5, 2, 2, 1, 1),    # 5x5 kernel
    (5, 4, 4, 1024, 12, 3, 3, 1, 1, 1, 1),    # long K (144 words)
    (3, 9, 11, 192, 20, 1, 1, 0, 0, 2, 3),    # 1x1, no padding, strides (2, 3): only the pixels read are quantized
    (2, 7, 8, 64, 70, 1, 1, 0, 0, 1, 2),      # 1x1, stride on W only
    (2, 9, 9, 384, 72, 3, 3, 1, 1, 1, 1),     # PC = 6: chunks of six words across taps
    (1, 12, 12, 640, 40, 3, 3, 1, 1, 2, 2),   # PC = 10
    (2, 8, 8, 384, 70, 1, 1, 0, 0, 1, 1),     # PC = 6, K = one tap
    (3, 6, 6, 768, 33, 3, 3, 1, 1, 1, 1),     # PC = 12, small launch: twelve-word chunks
    (2, 5, 5, 64, 8, 3, 3, 3, 3, 1, 1),       # padding as wide as the kernel: the outer outputs see padding only
    (2, 13, 13, 128, 8, 3, 3, 1, 1, 4, 4),    # stride beyond the kernel: pixels between the windows are never read
    (3, 1, 17, 128, 12, 1, 3, 0, 1, 1, 1),    # images of one line
    (2, 17, 1, 64, 12, 3, 1, 1, 0, 2, 1),     # images of one column
    (1, 9, 9, 1, 3, 3, 3, 1, 1, 1, 1),        # one channel: 63 tail bits in every word
    (2, 8, 12, 64, 9, 1, 7, 0, 3, 1, 1),      # 1x7 kernel
    (40, 2, 2, 64, 5, 2, 2, 0, 0, 1, 1),      # one output pixel per image: a tile of rows spans 40 images
    (3, 4, 4, 2048, 6, 2, 2, 1, 1, 1, 1),     # PC = 32
]


@pytest.mark.parametrize("type", [0, 1, 2, 3])
@pytest.mark.parametrize("case", EDGE_CASES)
def test_edge_shapes(type, case):
    _conv_case(type, *case, seed=type + 3, relu=(type == 1))


RESNET18_N16 = [
    # the ResNet-18 benchmark set: N=16, 3x3 pad 1 stride 1, plus the stride-2 downsample variants
    (16, 56, 56, 64, 64, 3, 3, 1, 1, 1, 1), (16, 28, 28, 128, 128, 3, 3, 1, 1, 1, 1),
    (16, 14, 14, 256, 256, 3, 3, 1, 1, 1, 1), (16, 7, 7, 512, 512, 3, 3, 1, 1, 1, 1),
    (16, 56, 56, 64, 128, 3, 3, 1, 1, 2, 2), (16, 28, 28, 128, 256, 3, 3, 1, 1, 2, 2),
    (16, 14, 14, 256, 512, 3, 3, 1, 1, 2, 2), (16, 56, 56, 64, 128, 1, 1, 0, 0, 2, 2),
    (16, 28, 28, 128, 256, 1, 1, 0, 0, 2, 2), (16, 14, 14, 256, 512, 1, 1, 0, 0, 2, 2),
]


@pytest.mark.parametrize("case", RESNET18_N16)
def test_resnet18_bnn(case):
    _conv_case(3, *case)


@pytest.mark.parametrize("type", [1, 2])
@pytest.mark.parametrize("case", RESNET18_N16[:4])
def test_resnet18_tbn_btn_relu_inputs(type, case):
    _conv_case(type, *case, relu=True)


@pytest.mark.parametrize("case", [
    (1, 28, 28, 512, 512, 3, 3, 1, 1, 1, 1),   # VGG-style 28x28x512 (config 4) at N=1
    (1, 56, 56, 256, 256, 3, 3, 1, 1, 1, 1),
    (2, 28, 28, 256, 256, 3, 3, 1, 0, 2, 2),   # sweep shape with asymmetric padding (config 5)
    (2, 28, 28, 512, 512, 1, 1, 1, 0, 2, 2),
])
@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_large_channel_layers(type, case):
    _conv_case(type, *case)


KERNEL_VARIANTS = [(tab_amd.CONV_MATRIX, t) for t in range(12)] + [(tab_amd.CONV_POPCOUNT, t) for t in range(3)]
VARIANT_CASES = [
    (2, 9, 6, 70, 5, 3, 3, 1, 0, 1, 2),        # one word per pixel pair: chunks cross taps
    (2, 12, 12, 192, 130, 3, 3, 1, 1, 1, 1),   # PC = 3: odd words per tap
    (3, 10, 10, 128, 40, 3, 3, 1, 1, 1, 1),    # PC = 2: chunks of two words inside a tap
    (2, 9, 9, 512, 72, 3, 3, 1, 1, 2, 2),      # PC = 8: chunks of four words inside a tap
    (1, 3, 3, 8192, 12, 3, 3, 1, 1, 1, 1),     # K = 73728 bits
    (2, 10, 10, 384, 136, 3, 3, 1, 1, 1, 1),   # PC = 6: six-word chunks across taps in every tile shape
    (2, 9, 9, 256, 72, 1, 1, 0, 0, 1, 1),      # K = one chunk of four words: a pipelined loop's prologue meets its last step
    (3, 7, 7, 128, 40, 1, 1, 0, 0, 1, 1),      # K = one chunk of two words (two MFMA steps)
]


@pytest.fixture
def restore_kernel_choice():
    yield
    tab_amd.set_conv_kernel(tab_amd.CONV_AUTO, -1)


@pytest.mark.parametrize("variant", KERNEL_VARIANTS)
@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_every_kernel_variant(type, variant, restore_kernel_choice):
    """Each selectable kernel and tile shape against the oracle, on shapes that take every staging
    path (chunks inside a tap / across taps, ragged M, KN and C)."""
    tab_amd.set_conv_kernel(*variant)
    for case in VARIANT_CASES:
        _conv_case(type, *case, seed=11 + type, relu=(type == 1))


SHORT_K_CASES = [
    # K of at most nine words: the kernel with the weights resident in registers, one wave per 32 output pixels
    (2, 12, 12, 64, 64, 3, 3, 1, 1, 1, 1),     # 9 words, the C = 64 3x3 shape
    (3, 9, 7, 33, 70, 3, 3, 1, 0, 2, 1),       # tail bits in the only word, ragged KN, tiles spanning images
    (2, 10, 10, 128, 100, 2, 2, 1, 1, 1, 1),   # 8 words as 2x2 taps of two words
    (1, 7, 9, 192, 33, 1, 3, 0, 1, 1, 1),      # 9 words as 1x3 taps of three words
    (5, 3, 3, 64, 31, 3, 3, 1, 1, 1, 1),       # 45 output pixels over five images: two tiles, the second partly empty
    (2, 8, 8, 320, 130, 1, 1, 0, 0, 1, 1),     # 5 words run as 8
    (2, 8, 8, 192, 65, 1, 1, 1, 1, 1, 1),      # 3 words run as 4, padded 1x1
    (4, 6, 6, 512, 256, 1, 1, 0, 0, 1, 1),     # 8 words, four filter tiles
    (2, 9, 9, 64, 1, 3, 3, 2, 2, 3, 3),        # one filter, pad 2, stride 3
    (1, 5, 5, 100, 7, 1, 1, 0, 0, 1, 1),       # 2 words
    (3, 4, 4, 64, 64, 1, 1, 0, 0, 1, 1),       # 1 word
]


@pytest.mark.parametrize("type", [0, 1, 2, 3])
@pytest.mark.parametrize("case", SHORT_K_CASES)
def test_short_k_register_resident_kernel(type, case, restore_kernel_choice):
    tab_amd.set_conv_kernel(tab_amd.CONV_MATRIX, 7)
    _conv_case(type, *case, seed=21 + type, relu=(type == 1))


@pytest.mark.parametrize("type", [0, 3])
def test_short_k_waves_walk_several_tiles(type):
    """100352 output pixels are 3136 tiles of 32, more than the waves of a launch: waves loop over tile, tile + waves.
    Too slow for the oracle as a whole: images computed alone equal the same images in the batch; first and last image
    against the oracle."""
    N, H, W, C, KN = 32, 56, 56, 64, 64
    g = torch.Generator("cuda").manual_seed(type)
    x = torch.randn((N, H, W, C), generator=g, device="cuda")
    w = torch.randn((KN, 3, 3, C), generator=g, device="cuda")
    ab, wb = act_bits(type), weight_bits(type)
    x_ths = (0.7 * x.abs().reshape(N, -1).mean(dim=1)).contiguous() if ab == 2 else torch.zeros(N, device="cuda")
    w_ths = (0.7 * w.abs().reshape(KN, -1).mean(dim=1)).contiguous() if wb == 2 else torch.zeros(KN, device="cuda")
    QW, BTN = tab_amd.Quantize(w, w_ths, wb, KN, 3, 3, C)
    y = tab_amd.Conv2d(x, QW, x_ths, BTN, type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3)
    for first in (0, 15, N - 1):
        part = tab_amd.Conv2d(x[first:first + 1].contiguous(), QW, x_ths[first:first + 1].contiguous(), BTN, type,
                              1, 1, 1, 1, 1, H, W, C, KN, 3, 3)
        torch.cuda.synchronize()
        assert torch.equal(y[first:first + 1], part)
    for n in (0, N - 1):
        want = oracle.conv2d(x[n:n + 1].cpu().numpy(), QW.cpu().numpy(), x_ths[n:n + 1].cpu().numpy(), BTN.cpu().numpy(),
                             type, 1, 1, 1, 1, 1, H, W, C, KN, 3, 3)
        assert np.array_equal(y[n:n + 1].cpu().numpy(), want)


def test_kernel_variants_agree_on_random_bits(restore_kernel_choice):
    """Arbitrary 64-bit patterns in QW and btn (sign bits outside the nonzero plane, tail bits set):
    every kernel follows the reference's formulas, so all of them agree with the oracle."""
    N, H, W, C, KN, KH, KW = 2, 6, 6, 256, 40, 3, 3
    rng = np.random.default_rng(5)
    x, x_ths, _, _ = make_layer(0, N, H, W, C, KN, KH, KW, seed=4)
    for type in range(4):
        qw = rng.integers(-2**63, 2**63 - 1, size=(KN, KH, KW, C // 64, weight_bits(type)), dtype=np.int64, endpoint=True)
        btn = rng.integers(0, 1000, size=KN).astype(np.int32)
        ths = x_ths if act_bits(type) == 2 else torch.zeros(N)
        want = oracle.conv2d(x.numpy(), qw, ths.numpy(), btn, type, 1, 1, 1, 1, N, H, W, C, KN, KH, KW)
        for variant in KERNEL_VARIANTS:
            print(f"[case] random QW bits type={type} kernel={variant}", flush=True)
            tab_amd.set_conv_kernel(*variant)
            y = tab_amd.Conv2d(x.cuda(), torch.from_numpy(qw).cuda(), ths.cuda(), torch.from_numpy(btn).cuda(),
                               type, 1, 1, 1, 1, N, H, W, C, KN, KH, KW)
            assert np.array_equal(y.cpu().numpy(), want), f"type {type} kernel {variant}"


def test_set_conv_kernel_rejects_unknown():
    with pytest.raises(tab_amd.TabError, match="no conv kernel"):
        tab_amd.set_conv_kernel(5, 0)
    with pytest.raises(tab_amd.TabError, match="no conv kernel"):
        tab_amd.set_conv_kernel(tab_amd.CONV_MATRIX, 12)


def test_arbitrary_weight_bit_patterns():
    """QW is caller data: the kernels must follow the formulas for any 64-bit pattern, including
    sign bits outside the nonzero plane (the notebook passes a 1-bit QW to the 2-bit types)."""
    N, H, W, C, KN, KH, KW = 2, 6, 6, 128, 20, 3, 3
    rng = np.random.default_rng(0)
    x, x_ths, _, _ = make_layer(0, N, H, W, C, KN, KH, KW, seed=9)
    for type in range(4):
        print(f"[case] random QW bits type={type}", flush=True)
        qw = rng.integers(-2**63, 2**63 - 1, size=(KN, KH, KW, C // 64, weight_bits(type)), dtype=np.int64, endpoint=True)
        btn = rng.integers(0, 1000, size=KN).astype(np.int32)
        ths = x_ths if act_bits(type) == 2 else torch.zeros(N)
        want = oracle.conv2d(x.numpy(), qw, ths.numpy(), btn, type, 1, 1, 1, 1, N, H, W, C, KN, KH, KW)
        y = tab_amd.Conv2d(x.cuda(), torch.from_numpy(qw).cuda(), ths.cuda(), torch.from_numpy(btn).cuda(),
                           type, 1, 1, 1, 1, N, H, W, C, KN, KH, KW)
        assert np.array_equal(y.cpu().numpy(), want)


def test_full_size_sweep_point_properties():
    """N=256, 28x28x512 -> 512, 3x3 (the largest sweep point, 9.5e11 binary ops) is too slow for
    the CPU oracle as a whole.  Images are independent, so: the first two images computed alone
    must equal the same images inside the full batch; the first and the last image are compared
    with the oracle; and every output obeys |y| <= KH*KW*C and, for BNN, y = NUM (mod 2)."""
    N, H, W, C, KN = 256, 28, 28, 512, 512
    print("[case] full-size sweep point N=256 28x28x512->512 3x3, four types", flush=True)
    g = torch.Generator("cuda").manual_seed(0)
    x = torch.randn((N, H, W, C), generator=g, device="cuda")
    w = torch.randn((KN, 3, 3, C), generator=g, device="cuda")
    for type in (3, 0, 1, 2):  # every type takes its own tile shape at this size
        ab, wb = act_bits(type), weight_bits(type)
        x_ths = (0.7 * x.abs().reshape(N, -1).mean(dim=1)).contiguous() if ab == 2 else torch.zeros(N, device="cuda")
        w_ths = (0.7 * w.abs().reshape(KN, -1).mean(dim=1)).contiguous() if wb == 2 else torch.zeros(KN, device="cuda")
        QW, BTN = tab_amd.Quantize(w, w_ths, wb, KN, 3, 3, C)
        y = tab_amd.Conv2d(x, QW, x_ths, BTN, type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3)
        y_small = tab_amd.Conv2d(x[:2].contiguous(), QW, x_ths[:2].contiguous(), BTN, type, 1, 1, 1, 1, 2, H, W, C, KN, 3, 3)
        torch.cuda.synchronize()
        assert torch.equal(y[:2], y_small)
        want = oracle.conv2d(x[:1].cpu().numpy(), QW.cpu().numpy(), x_ths[:1].cpu().numpy(), BTN.cpu().numpy(),
                             type, 1, 1, 1, 1, 1, H, W, C, KN, 3, 3)
        assert np.array_equal(y[:1].cpu().numpy(), want)
        # last image too (a different threshold and the far end of every index range)
        want_last = oracle.conv2d(x[-1:].cpu().numpy(), QW.cpu().numpy(), x_ths[-1:].cpu().numpy(), BTN.cpu().numpy(),
                                  type, 1, 1, 1, 1, 1, H, W, C, KN, 3, 3)
        assert np.array_equal(y[-1:].cpu().numpy(), want_last)
        assert bool((y.abs() <= 9 * C).all())
        if type == 3:
            assert bool(((y.to(torch.int64) - 9 * C) % 2 == 0).all())


@pytest.mark.parametrize("C,KN", [(128, 384), (64, 256)])  # the LDS-direct kernel; the register-staged one (one word per pixel)
def test_short_k_large_output_workgroup_order(C, KN):
    """A 1x1 layer whose Y exceeds 192 MB orders its workgroups by rows of Y (groups of eight row tiles walk the
    filter tiles), and 203840 = 65*56*56 rows leave the last group partly empty.  Too much for the oracle as a
    whole: images are independent, so two images computed alone (the other order: their Y is small) must equal
    the same images inside the batch, the first and the last image are compared with the oracle, and every
    output obeys |y| <= C and, for BNN, y = C (mod 2)."""
    N, H, W = 65, 56, 56
    assert N * H * W * KN * 4 >= 192 << 20 and (N * H * W + 127) // 128 % 8 != 0
    print(f"[case] short-K large-Y order N={N} {H}x{W}x{C}->{KN} 1x1, types 3 and 0", flush=True)
    g = torch.Generator("cuda").manual_seed(3)
    x = torch.randn((N, H, W, C), generator=g, device="cuda")
    w = torch.randn((KN, 1, 1, C), generator=g, device="cuda")
    for type in (3, 0):
        ab, wb = act_bits(type), weight_bits(type)
        x_ths = (0.7 * x.abs().reshape(N, -1).mean(dim=1)).contiguous() if ab == 2 else torch.zeros(N, device="cuda")
        w_ths = (0.7 * w.abs().reshape(KN, -1).mean(dim=1)).contiguous() if wb == 2 else torch.zeros(KN, device="cuda")
        QW, BTN = tab_amd.Quantize(w, w_ths, wb, KN, 1, 1, C)
        y = tab_amd.Conv2d(x, QW, x_ths, BTN, type, 0, 0, 1, 1, N, H, W, C, KN, 1, 1)
        for first in (0, N - 2):
            part = tab_amd.Conv2d(x[first:first + 2].contiguous(), QW, x_ths[first:first + 2].contiguous(), BTN, type,
                                  0, 0, 1, 1, 2, H, W, C, KN, 1, 1)
            torch.cuda.synchronize()
            assert torch.equal(y[first:first + 2], part)
        for n in (0, N - 1):
            want = oracle.conv2d(x[n:n + 1].cpu().numpy(), QW.cpu().numpy(), x_ths[n:n + 1].cpu().numpy(), BTN.cpu().numpy(),
                                 type, 0, 0, 1, 1, 1, H, W, C, KN, 1, 1)
            assert np.array_equal(y[n:n + 1].cpu().numpy(), want)
        assert bool((y.abs() <= C).all())
        if type == 3:
            assert bool(((y.to(torch.int64) - C) % 2 == 0).all())


@pytest.mark.parametrize("C", [128, 64])  # the LDS-direct kernel and the register-staged one
@pytest.mark.parametrize("type", [0, 3])
def test_xcd_order_with_a_ragged_tile_count(type, C, restore_kernel_choice):
    """Launches of 64 tiles and more hand each XCD an eighth of the tiles (workgroup b -> tile (b % 8) * share + b / 8)
    and leave the last tiles % 8 where they are: every tile must still be computed exactly once.  M = 5 * 37 * 37 =
    6845 rows and KN = 192 give 321 (64x64), 162 (128x64), 108 (128x128), 81 (256x64), 54 tiles (below 64: the plain
    order) and 214 * 6 (32x32): counts that leave every remainder."""
    for tile in (-1, 0, 1, 2, 3, 4, 5, 6):
        tab_amd.set_conv_kernel(tab_amd.CONV_MATRIX if tile >= 0 else tab_amd.CONV_AUTO, tile)
        _conv_case(type, 5, 37, 37, C, 192, 3, 3, 1, 1, 1, 1, seed=29 + tile)


def test_conv_rejects_wrong_sizes():
    x = torch.zeros((1, 4, 4, 64), device="cuda")
    ths = torch.zeros(1, device="cuda")
    btn = torch.zeros(4, dtype=torch.int32, device="cuda")
    qw1 = torch.zeros((4, 3, 3, 1, 1), dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="QW has"):
        tab_amd.Conv2d(x, qw1, ths, btn, 0, 1, 1, 1, 1, 1, 4, 4, 64, 4, 3, 3)  # TNN needs 2-bit QW
    with pytest.raises(RuntimeError, match="type must be"):
        tab_amd.Conv2d(x, qw1, ths, btn, 7, 1, 1, 1, 1, 1, 4, 4, 64, 4, 3, 3)
    with pytest.raises(RuntimeError, match="contiguous"):
        tab_amd.Conv2d(x.permute(0, 3, 1, 2), qw1, ths, btn, 3, 1, 1, 1, 1, 1, 4, 4, 64, 4, 3, 3)
    with pytest.raises(RuntimeError, match="dtype"):
        tab_amd.Conv2d(x.double(), qw1, ths, btn, 3, 1, 1, 1, 1, 1, 4, 4, 64, 4, 3, 3)
    qw4 = torch.zeros((4, 3, 3, 4, 1), dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="empty output"):
        tab_amd.Conv2d(x, qw4, ths, btn, 3, 0, 0, 1, 1, 1, 2, 2, 64 * 4, 4, 3, 3)


@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_longest_k_with_every_product_of_one_sign(type):
    """K = 65535 words, the most the library takes, and filters whose products are all +1, all -1, or cancel: the
    sums +-4194240 must come out exact (two ternary operands multiply as +-2 x +-2 and are scaled back, so their
    accumulators reach 16776960, just below 2^24)."""
    C, KN = 64 * 65535, 3
    print(f"[case] Conv2d {TYPE_NAMES[type]} 1x1x{C}->{KN}", flush=True)
    x = np.full((1, 1, 1, C), 1.0, dtype=np.float32)
    w = np.ones((KN, 1, 1, C), dtype=np.float32)
    w[1] = -1.0
    w[2, :, :, 1::2] = -1.0
    ths = np.array([0.5 if act_bits(type) == 2 else 0.0], dtype=np.float32)
    w_ths = np.full(KN, 0.5 if weight_bits(type) == 2 else 0.0, dtype=np.float32)
    qw, btn = oracle.quantize(w, w_ths, weight_bits(type), KN, 1, 1, C)
    want = oracle.conv2d(x, qw, ths, btn, type, 0, 0, 1, 1, 1, 1, 1, C, KN, 1, 1)
    assert want.reshape(-1).tolist() == [float(C), -float(C), 0.0]
    y = tab_amd.Conv2d(torch.from_numpy(x).cuda(), torch.from_numpy(qw).cuda(), torch.from_numpy(ths).cuda(),
                       torch.from_numpy(btn).cuda(), type, 0, 0, 1, 1, 1, 1, 1, C, KN, 1, 1)
    assert np.array_equal(y.cpu().numpy(), want)
