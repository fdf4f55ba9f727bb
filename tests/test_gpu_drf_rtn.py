"""GPU parity of the two CPU-only conv types, 4 (DoReFa 2-bit) and 5 (RTN), through the C ABI against
the CPU oracle (whose GEMMs are pinned against the reference's DRFGEMM_baseline / RTNGEMM_baseline,
TAB_CPU.cpp:332-383).  Integer work: the bar is bit-exact equality."""
import numpy as np
import pytest
import torch

import oracle
import tab_amd
from helpers import TYPE_NAMES

pytestmark = pytest.mark.gpu


def _rand_words(rng, shape):
    return rng.integers(-2**63, 2**63 - 1, size=shape, dtype=np.int64, endpoint=True)


@pytest.fixture
def restore_kernel_choice():
    yield
    tab_amd.set_conv_kernel(tab_amd.CONV_AUTO, -1)


@pytest.mark.parametrize("type", [4, 5])
@pytest.mark.parametrize("C", [1, 31, 32, 33, 64, 65, 200, 256])
def test_packer_equals_oracle(type, C):
    print(f"[case] QuantizeFormat {TYPE_NAMES[type]} C={C}", flush=True)
    rng = np.random.default_rng(C + type)
    N, H, W = 3, 5, 4
    x = (rng.standard_normal((N, H, W, C)) * 1.5).astype(np.float32)
    ths = np.array([0.5, 0.0, 1.25], np.float32)
    flat = x.reshape(N, -1)
    for n in range(N):  # ties at every bound, NaN, infinities, signed zero
        specials = [0.5 * ths[n], 1.5 * ths[n], 2.5 * ths[n], ths[n], -ths[n], np.nan, np.inf, -np.inf, 0.0, -0.0]
        k = min(len(specials), flat.shape[1])
        flat[n, :k] = specials[:k]
    want = oracle.quantize_format(x, ths, type, N, H, W, C)
    got = tab_amd.QuantizeFormat(torch.from_numpy(x).cuda(), torch.from_numpy(ths).cuda(), type, N, H, W, C)
    torch.cuda.synchronize()
    assert got.dtype == torch.int64 and tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)


CASES = [
    # N, H, W, C, KN, KH, KW, p1, p2, s1, s2
    (1, 32, 32, 64, 64, 3, 3, 1, 1, 1, 1),
    (2, 7, 7, 64, 8, 3, 3, 1, 1, 2, 2),
    (2, 9, 6, 70, 5, 3, 3, 1, 0, 1, 2),
    (2, 8, 8, 128, 16, 1, 1, 0, 0, 2, 2),
    (1, 6, 5, 200, 7, 2, 3, 2, 1, 1, 1),
    (2, 12, 12, 192, 130, 3, 3, 1, 1, 1, 1),
    (3, 10, 10, 128, 40, 3, 3, 1, 1, 1, 1),
    (2, 9, 9, 512, 72, 3, 3, 1, 1, 2, 2),
    (4, 28, 28, 256, 256, 3, 3, 1, 1, 1, 1),
]


@pytest.mark.parametrize("type", [4, 5])
@pytest.mark.parametrize("case", CASES)
def test_conv2d_from_floats(type, case):
    N, H, W, C, KN, KH, KW, p1, p2, s1, s2 = case
    print(f"[case] Conv2d {TYPE_NAMES[type]} {case}", flush=True)
    rng = np.random.default_rng(type * 13 + C + KN)
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    w = rng.standard_normal((KN, KH, KW, C)).astype(np.float32)
    if type == 4:  # unsigned levels: spread the inputs over all four
        x, w = np.abs(x) * 1.3, np.abs(w) * 1.3
    x_ths = np.linspace(0.4, 0.8, N).astype(np.float32)
    w_ths = np.linspace(0.3, 0.9, KN).astype(np.float32)
    qw_o = oracle.quantize_format(w, w_ths, type, KN, KH, KW, C)
    want = oracle.conv2d(x, qw_o, x_ths, np.zeros(KN, np.int32), type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    QW = tab_amd.QuantizeFormat(torch.from_numpy(w).cuda(), torch.from_numpy(w_ths).cuda(), type, KN, KH, KW, C)
    btn = torch.zeros(KN, dtype=torch.int32, device="cuda")
    y = tab_amd.Conv2d(torch.from_numpy(x).cuda(), QW, torch.from_numpy(x_ths).cuda(), btn, type, p1, p2, s1, s2,
                       N, H, W, C, KN, KH, KW)
    torch.cuda.synchronize()
    assert np.array_equal(QW.cpu().numpy(), qw_o)
    got = y.cpu().numpy()
    assert got.shape == want.shape and np.array_equal(got, want), f"max |diff| = {np.abs(got - want).max()}"


KERNELS = [(tab_amd.CONV_MATRIX, t) for t in range(12)] + [(tab_amd.CONV_POPCOUNT, -1)]


@pytest.mark.parametrize("type", [4, 5])
@pytest.mark.parametrize("kernel", KERNELS)
def test_conv2d_packed_any_bits_every_tile(type, kernel, restore_kernel_choice):
    """Random 64-bit words (every bit pattern is a valid operand of both types) through every
    workgroup tile of the matrix-core kernel; a popcount-kernel request is ignored for these types."""
    tab_amd.set_conv_kernel(*kernel)
    for case in [(2, 9, 6, 70, 5, 3, 3, 1, 0, 1, 2), (2, 12, 12, 192, 130, 3, 3, 1, 1, 1, 1),
                 (2, 9, 9, 512, 72, 3, 3, 1, 1, 2, 2), (1, 3, 3, 2048, 12, 3, 3, 1, 1, 1, 1)]:
        N, H, W, C, KN, KH, KW, p1, p2, s1, s2 = case
        print(f"[case] Conv2dPacked {TYPE_NAMES[type]} kernel={kernel} {case}", flush=True)
        rng = np.random.default_rng(type + C)
        qx = _rand_words(rng, (N, H, W, tab_amd.operand_words(type, 0, C)))
        qw = _rand_words(rng, (KN, KH, KW, tab_amd.operand_words(type, 1, C)))
        want = oracle.conv2d_packed(qx, qw, None, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
        btn = torch.zeros(KN, dtype=torch.int32, device="cuda")
        y = tab_amd.Conv2dPacked(torch.from_numpy(qx).cuda(), torch.from_numpy(qw).cuda(), btn, type, p1, p2, s1, s2,
                                 N, H, W, C, KN, KH, KW)
        torch.cuda.synchronize()
        got = y.cpu().numpy()
        assert np.array_equal(got, want), f"max |diff| = {np.abs(got - want).max()}"


PACKED_OUT_KERNELS = [(tab_amd.CONV_AUTO, -1)] + [(tab_amd.CONV_MATRIX, t) for t in (0, 1, 2, 4, 5, 6, 8, 9, 10, 11)]


@pytest.mark.parametrize("type", [4, 5])
@pytest.mark.parametrize("kernel", PACKED_OUT_KERNELS)
def test_packed_output_every_tile(type, kernel, restore_kernel_choice):
    """Conv2dPackedOut for the two CPU-path types: the conv's outputs thresholded and packed in the epilogue as Quantize packs
    them (1- and 2-bit planes), against the oracle's conv followed by the oracle's quantizer.  Thresholds sit inside the range
    of the sums, on values the integer sums hit (ties)."""
    tab_amd.set_conv_kernel(*kernel)
    for case in [(2, 9, 6, 70, 5, 3, 3, 1, 0, 1, 2), (2, 12, 12, 192, 130, 3, 3, 1, 1, 1, 1), (3, 9, 9, 512, 72, 3, 3, 1, 1, 2, 2),
                 (2, 10, 10, 256, 200, 3, 3, 1, 1, 1, 1)]:
        N, H, W, C, KN, KH, KW, p1, p2, s1, s2 = case
        print(f"[case] Conv2dPackedOut {TYPE_NAMES[type]} kernel={kernel} {case}", flush=True)
        rng = np.random.default_rng(type * 7 + C)
        qx = _rand_words(rng, (N, H, W, tab_amd.operand_words(type, 0, C)))
        qw = _rand_words(rng, (KN, KH, KW, tab_amd.operand_words(type, 1, C)))
        y = oracle.conv2d_packed(qx, qw, None, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
        OH, OW = tab_amd.out_shape(H, W, KH, KW, p1, p2, s1, s2)
        y = np.ascontiguousarray(y).reshape(N, OH, OW, KN)
        btn = torch.zeros(KN, dtype=torch.int32, device="cuda")
        for out_bits in (1, 2):
            # per image: the median of its sums (binary: about half the bits set) or of their magnitudes (ternary)
            ths = np.array([np.median(y[n]) if out_bits == 1 else np.median(np.abs(y[n])) for n in range(N)], dtype=np.float32)
            want, _ = oracle.quantize(y, ths, out_bits, N, OH, OW, KN)
            got = tab_amd.Conv2dPackedOut(torch.from_numpy(qx).cuda(), torch.from_numpy(qw).cuda(), btn, type, p1, p2, s1, s2,
                                          N, H, W, C, KN, KH, KW, torch.from_numpy(ths).cuda(), out_bits)
            torch.cuda.synchronize()
            assert np.array_equal(got.cpu().numpy(), want), f"{TYPE_NAMES[type]} {case} out_bits={out_bits}"


@pytest.mark.parametrize("type", [4, 5])
def test_saturated_operands_stay_exact(type):
    """All-ones words: every product takes its largest value (9 per bit for type 4), the sums the
    largest the accumulators have to hold for this K."""
    N, H, W, C, KN = 1, 4, 4, 4096, 8
    words_a, words_w = tab_amd.operand_words(type, 0, C), tab_amd.operand_words(type, 1, C)
    qx = torch.full((N, H, W, words_a), 0x5555555555555555 if type == 5 else -1, dtype=torch.int64, device="cuda")
    qw = torch.full((KN, 3, 3, words_w), 0x5555555555555555 if type == 5 else -1, dtype=torch.int64, device="cuda")
    btn = torch.zeros(KN, dtype=torch.int32, device="cuda")
    y = tab_amd.Conv2dPacked(qx, qw, btn, type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3)
    torch.cuda.synchronize()
    per_tap = C * (9 if type == 4 else 1)
    taps = torch.tensor([[(min(h + 1, H - 1) - max(h - 1, 0) + 1) * (min(w + 1, W - 1) - max(w - 1, 0) + 1)
                          for w in range(W)] for h in range(H)], dtype=torch.float32)
    want = (taps * per_tap).reshape(1, H, W, 1).expand(N, H, W, KN)
    assert torch.equal(y.cpu().reshape(N, H, W, KN), want)
