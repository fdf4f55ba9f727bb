"""Pins oracle.quantize (the CPU restatement of TerOnlyKernel/BinOnlyKernel/BTN_Weight,
TAB_GEMM.cu:150-247) without reusing its code: per-element closed forms, bit-order probes,
the demo notebook's stored words and the reference's own CPU quantizers."""
import json
import os

import numpy as np
import pytest

import oracle
from helpers import brute_pack, brute_values, unpack

GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.mark.parametrize("bitwidth", [1, 2])
@pytest.mark.parametrize("C", [1, 63, 64, 65, 128, 200])
def test_matches_closed_form(bitwidth, C):
    rng = np.random.default_rng(C * 10 + bitwidth)
    N, H, W = 3, 2, 5
    x = rng.standard_normal((N, H, W, C)).astype(np.float32)
    ths = np.array([0.3, 0.0, 1.1], dtype=np.float32)
    qx, btn = oracle.quantize(x, ths, bitwidth, N, H, W, C)
    vals = brute_values(x, ths, bitwidth)
    assert qx.shape == (N, H, W, (C + 63) // 64, bitwidth) and qx.dtype == np.int64
    assert np.array_equal(qx, brute_pack(vals, bitwidth))
    if bitwidth == 2:
        assert np.array_equal(btn, (vals != 0).reshape(N, -1).sum(axis=1).astype(np.int32))
    else:
        assert not btn.any()  # zeros for 1-bit (TAB_GEMM.cu:283,309-317)


def test_special_values_and_ties():
    # strict, ordered compares: ties, NaN -> 0 (ternary) / +1 (binary); -0.0 is not < 0
    t = np.float32(0.5)
    x = np.array([t, -t, np.nextafter(t, 1, dtype=np.float32), np.nextafter(-t, -1, dtype=np.float32),
                  np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-45, -1e-45], dtype=np.float32)
    C = x.size
    want_t = np.array([0, 0, 1, -1, 0, 1, -1, 0, 0, 0, 0], dtype=np.int8)
    q2, btn = oracle.quantize(x.reshape(1, 1, 1, C), [t], 2, 1, 1, 1, C)
    assert np.array_equal(unpack(q2, C, 2).ravel(), want_t)
    assert btn[0] == 4
    want_b = np.array([1, -1, 1, -1, 1, 1, -1, -1, -1, -1, -1], dtype=np.int8)
    q1, _ = oracle.quantize(x.reshape(1, 1, 1, C), [t], 1, 1, 1, 1, C)
    assert np.array_equal(unpack(q1, C, 1).ravel(), want_b)
    # threshold 0: -0.0 and +0.0 are +1, NaN is +1
    q0, _ = oracle.quantize(x.reshape(1, 1, 1, C), [0.0], 1, 1, 1, 1, C)
    assert np.array_equal(unpack(q0, C, 1).ravel(), np.array([1, -1, 1, -1, 1, 1, -1, 1, 1, 1, -1], dtype=np.int8))


def test_negative_threshold_first_branch_wins():
    # t < 0: v > t and v < -t can both hold; the reference tests v > t first (+1)
    x = np.array([0.0, -0.2, -0.6, 0.6], dtype=np.float32).reshape(1, 1, 1, 4)
    q, _ = oracle.quantize(x, [-0.5], 2, 1, 1, 1, 4)
    assert np.array_equal(unpack(q, 4, 2).ravel(), [1, 1, -1, 1])


@pytest.mark.parametrize("c", [0, 1, 31, 32, 63, 64, 100, 127])
def test_bit_order_one_hot(c):
    # channel c -> word c/64, bit c%64, LSB first (onebit[i] = 1 << i, TAB_GEMM.cu:252-258);
    # bit 63 makes the int64 negative
    C = 128
    x = np.zeros((1, 1, 1, C), dtype=np.float32)
    x[..., c] = -1.0
    q1, _ = oracle.quantize(x, [0.0], 1, 1, 1, 1, C)
    want = np.zeros(2, dtype=np.uint64)
    want[c // 64] = np.uint64(1) << np.uint64(c % 64)
    assert np.array_equal(q1.view(np.uint64).ravel(), want)
    q2, btn = oracle.quantize(x, [0.5], 2, 1, 1, 1, C)
    assert np.array_equal(q2.view(np.uint64)[0, 0, 0, :, 0], want)  # plane 0: sign
    assert np.array_equal(q2.view(np.uint64)[0, 0, 0, :, 1], want)  # plane 1: nonzero
    assert btn[0] == 1


def test_tail_word_high_bits_zero():
    C = 70
    x = -np.ones((1, 1, 1, C), dtype=np.float32)
    q, _ = oracle.quantize(x, [0.0], 1, 1, 1, 1, C)
    assert q.view(np.uint64)[0, 0, 0, 1, 0] == np.uint64((1 << 6) - 1)


def test_threshold_is_per_item():
    # ths[n] for image n (TAB_CPU.cpp:67,72), not per block row
    x = np.full((3, 4, 2, 64), 0.5, dtype=np.float32)
    q, btn = oracle.quantize(x, [0.4, 0.6, 0.4], 2, 3, 4, 2, 64)
    assert list(btn) == [4 * 2 * 64, 0, 4 * 2 * 64]


def test_notebook_known_answers():
    """Stored cell outputs of the demo notebook: on the same w and threshold 0.5 the 1-bit word
    is the bitwise NOT of the 2-bit nonzero-plane word and the sign plane is 0 for w >= 0.
    The notebook's w is unseeded, so the relation (not the values) is what can be replayed."""
    kat = json.load(open(os.path.join(GOLD, "notebook_kat.json")))
    ter = np.array(kat["ternary_QW_0_0_0"], dtype=np.int64)
    bin_ = np.array(kat["binary_QW_0_0_0"], dtype=np.int64)
    assert np.array_equal(~ter[:, 1], bin_[:, 0]) and not ter[:, 0].any()
    rng = np.random.default_rng(7)
    KN, KH, KW, KC = 64, 3, 3, 256
    w = rng.random((KN, KH, KW, KC), dtype=np.float32)
    ths = np.full(KN, 0.5, dtype=np.float32)
    q2, btn2 = oracle.quantize(w, ths, 2, KN, KH, KW, KC)
    q1, btn1 = oracle.quantize(w, ths, 1, KN, KH, KW, KC)
    assert list(q2.shape) == kat["ternary_shape"] and list(q1.shape) == kat["binary_shape"]
    assert list(btn2.shape) == kat["btn_shape"] and btn2.dtype == np.int32
    assert not q2[..., 0].any()
    assert np.array_equal(~q2[..., 1], q1[..., 0])


def _nhwc_padded(q, p1, p2):
    N, H, W, PC, B = q.shape
    out = np.zeros((N, H + 2 * p1, W + 2 * p2, PC, B), dtype=np.int64)
    out[:, p1:p1 + H, p2:p2 + W] = q
    return out


@pytest.mark.parametrize("name", ["ter_c70", "ter_c128"])
def test_ternary_against_reference_cpu_golden(name):
    """Outputs of the reference's Parallel_Ternarize_NCHWB_to_NHWCB (TAB_CPU.cpp:20-124),
    committed by tests/golden/make_ref_golden.py."""
    g = np.load(os.path.join(GOLD, "ref_golden.npz"))
    C, H, W, p1, p2 = (int(v) for v in g[name + "_dims"])
    x_nhwc = np.ascontiguousarray(g[name + "_x_chw"].transpose(1, 2, 0))[None]
    q, _ = oracle.quantize(x_nhwc, g[name + "_th"], 2, 1, H, W, C)
    assert np.array_equal(_nhwc_padded(q, p1, p2), g[name + "_q"])


def test_binary_sign_against_reference_cpu_golden():
    """Parallel_Binarize_NCHW_to_NHWC (TAB_CPU.cpp:137-206) binarizes by sign; it equals the
    GPU rule v < ths at ths = 0."""
    g = np.load(os.path.join(GOLD, "ref_golden.npz"))
    C, H, W, p1, p2 = (int(v) for v in g["bin_c128_dims"])
    x_nhwc = np.ascontiguousarray(g["bin_c128_x_chw"].transpose(1, 2, 0))[None]
    q, _ = oracle.quantize(x_nhwc, [0.0], 1, 1, H, W, C)
    assert np.array_equal(_nhwc_padded(q, p1, p2)[..., 0], g["bin_c128_q"])


@pytest.mark.parametrize("name,bits", [("ter_c70", 2), ("ter_c128", 2), ("bin_c128", 1)])
def test_nchw_reading_against_reference_cpu_golden(name, bits):
    """quantize_nchw reads [C][H][W] the way the reference's CPU quantizers do (TAB_CPU.cpp:20-206): their
    committed outputs, interior of the padded buffer."""
    g = np.load(os.path.join(GOLD, "ref_golden.npz"))
    C, H, W, p1, p2 = (int(v) for v in g[name + "_dims"])
    ths = g[name + "_th"] if bits == 2 else [0.0]
    q, _ = oracle.quantize_nchw(g[name + "_x_chw"], ths, bits, 1, C, H, W)
    want = g[name + "_q"] if bits == 2 else g[name + "_q"][..., None]
    assert np.array_equal(_nhwc_padded(q, p1, p2), want)


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built (no reference tree)")
def test_ternary_against_reference_cpu_live():
    rng = np.random.default_rng(11)
    C, H, W, p1, p2 = 192, 4, 3, 1, 0
    x = rng.standard_normal((C, H, W)).astype(np.float32)
    buf = np.concatenate([np.zeros((64, H, W), np.float32), x], axis=0)
    ths = np.array([0.55], dtype=np.float32)
    got = oracle.ref_ternarize_nchw(buf, p1, p2, ths, 1, C, H, W)
    q, _ = oracle.quantize(np.ascontiguousarray(x.transpose(1, 2, 0))[None], ths, 2, 1, H, W, C)
    assert np.array_equal(_nhwc_padded(q, p1, p2), got)
