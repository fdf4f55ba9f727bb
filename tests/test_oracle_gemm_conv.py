"""Pins the oracle's pad / im2row / GEMM / conv2d (TAB_GEMM.cuh:73-115, TAB_CPU.cpp:242-328,
TAB_GEMM.cu:325-527) against the reference's own compiled CPU functions (live and as committed
golden vectors), against torch.nn.functional.conv2d on dequantised tensors, and against
identities the arithmetic fixes."""
import json
import os

import numpy as np
import pytest

import oracle
from helpers import act_bits, make_layer, torch_conv_reference, unpack, weight_bits

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _rand_words(rng, shape):
    return rng.integers(-2**63, 2**63 - 1, size=shape, dtype=np.int64, endpoint=True)


@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_gemm_against_reference_golden(type):
    g = np.load(os.path.join(GOLD, "ref_golden.npz"))
    M, N, K, num = (int(v) for v in g[f"gemm{type}_mnk_num"])
    y = oracle.gemm(type, g[f"gemm{type}_a"], g[f"gemm{type}_b"], M, N, K, g[f"gemm{type}_btn"], NUM=num)
    assert np.array_equal(y, g[f"gemm{type}_y"])


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built (no reference tree)")
@pytest.mark.parametrize("type", [0, 1, 2, 3])
@pytest.mark.parametrize("mnk", [(1, 1, 1), (33, 17, 9), (130, 70, 36)])
def test_gemm_against_reference_live(type, mnk):
    M, N, K = mnk
    rng = np.random.default_rng(M * 7 + type)
    a = _rand_words(rng, (M, K, act_bits(type)))
    b = _rand_words(rng, (N, K, weight_bits(type)))
    btn = rng.integers(0, 64 * K, size=N).astype(np.int32)
    assert np.array_equal(oracle.gemm(type, a, b, M, N, K, btn, NUM=64 * K - 3),
                          oracle.ref_gemm(type, a, b, M, N, K, btn, NUM=64 * K - 3))


@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_gemm_equals_integer_dot_product(type):
    """On valid encodings every GEMM is the dot product of the decoded {-1,0,+1} rows."""
    rng = np.random.default_rng(40 + type)
    M, N, C = 9, 6, 192
    K = C // 64
    xa = rng.standard_normal((M, 1, 1, C)).astype(np.float32)
    xb = rng.standard_normal((N, 1, 1, C)).astype(np.float32)
    qa, _ = oracle.quantize(xa, np.full(M, 0.6 if act_bits(type) == 2 else 0.0, np.float32), act_bits(type), M, 1, 1, C)
    qb, btn = oracle.quantize(xb, np.full(N, 0.6 if weight_bits(type) == 2 else 0.0, np.float32), weight_bits(type), N, 1, 1, C)
    va = unpack(qa, C, act_bits(type)).reshape(M, C).astype(np.int32)
    vb = unpack(qb, C, weight_bits(type)).reshape(N, C).astype(np.int32)
    y = oracle.gemm(type, qa, qb, M, N, K, btn, NUM=C)
    assert np.array_equal(y, va @ vb.T)


def test_gemm_identities_between_types():
    """TBN(a,b) == TNN(a, (b, all-ones)); BTN(a,b) == TNN((a, all-ones), b) with btn = popcount
    of b's nonzero plane; BNN == TNN with both nonzero planes all-ones when NUM = 64*K."""
    rng = np.random.default_rng(5)
    M, N, K = 12, 10, 4
    ones = np.int64(-1)
    a2 = _rand_words(rng, (M, K, 2))
    b2 = _rand_words(rng, (N, K, 2))
    a1, b1 = a2[..., :1].copy(), b2[..., :1].copy()
    b_as_t = np.concatenate([b1, np.full_like(b1, ones)], axis=-1)
    a_as_t = np.concatenate([a1, np.full_like(a1, ones)], axis=-1)
    assert np.array_equal(oracle.gemm(1, a2, b1, M, N, K), oracle.gemm(0, a2, b_as_t, M, N, K))
    btn = np.array([sum(bin(int(w) & (2**64 - 1)).count("1") for w in b2[n, :, 1]) for n in range(N)], np.int32)
    assert np.array_equal(oracle.gemm(2, a1, b2, M, N, K, btn), oracle.gemm(0, a_as_t, b2, M, N, K))
    assert np.array_equal(oracle.gemm(3, a1, b1, M, N, K, NUM=64 * K), oracle.gemm(0, a_as_t, b_as_t, M, N, K))


def test_bnn_parity_invariant_from_notebook():
    # y = NUM - 2*cnt, so y has the parity of NUM (the notebook's BNN sample is all even, NUM = 9*256)
    kat = json.load(open(os.path.join(GOLD, "notebook_kat.json")))
    assert all(v % 2 == 0 for v in kat["bnn_y_first"])
    rng = np.random.default_rng(3)
    y = oracle.gemm(3, _rand_words(rng, (5, 3, 1)), _rand_words(rng, (4, 3, 1)), 5, 4, 3, NUM=191)
    assert ((y - 191) % 2 == 0).all() and (np.abs(y) <= 192).all()


@pytest.mark.parametrize("name", ["i2r_s1", "i2r_s2"])
def test_img2row_against_reference_golden(name):
    g = np.load(os.path.join(GOLD, "ref_golden.npz"))
    N, PH, PW, D, KH, KW, s1, s2 = (int(v) for v in g[name + "_dims"])
    assert np.array_equal(oracle.img2row(g[name + "_a"], N, PH, PW, D, KH, KW, s1, s2), g[name + "_rows"])


def test_img2row_k_order_and_pad_by_indexing():
    rng = np.random.default_rng(9)
    N, H, W, D, p1, p2, KH, KW, s1, s2 = 2, 5, 4, 3, 1, 2, 2, 3, 2, 1
    a = _rand_words(rng, (N, H, W, D))
    padded = oracle.pad(a, N, H, W, D, p1, p2)
    assert padded.shape == (N, H + 2 * p1, W + 2 * p2, D)
    assert np.array_equal(padded[:, p1:p1 + H, p2:p2 + W], a)
    assert not padded[:, :p1].any() and not padded[:, :, :p2].any() and not padded[:, -p1:].any()
    PH, PW = H + 2 * p1, W + 2 * p2
    rows = oracle.img2row(padded, N, PH, PW, D, KH, KW, s1, s2)
    OH, OW = (PH - KH + 1) // s1, (PW - KW + 1) // s2
    for n in range(N):
        for oh in range(OH):
            for ow in range(OW):
                patch = padded[n, oh * s1:oh * s1 + KH, ow * s2:ow * s2 + KW]  # (kh,kw,d)
                assert np.array_equal(rows[(n * OH + oh) * OW + ow], patch.ravel())


@pytest.mark.parametrize("case", [
    # (H, pad, K, stride, expected): integer division of (H+2p-K+1) by the stride
    (32, 1, 3, 1, 32), (56, 1, 3, 2, 28), (56, 0, 1, 2, 28), (28, 0, 3, 2, 13), (28, 1, 1, 2, 15),
    (7, 1, 3, 2, 3),  # PyTorch would give 4 here
    (112, 1, 3, 1, 112), (5, 0, 5, 1, 1), (5, 0, 5, 3, 0),
])
def test_out_extent_formula(case):
    H, p, K, s, want = case
    assert oracle.out_extent(H, p, K, s) == want


CONV_CASES = [
    # N, H, W, C, KN, KH, KW, p1, p2, s1, s2
    (1, 32, 32, 64, 64, 3, 3, 1, 1, 1, 1),   # the single-image benchmark shape
    (2, 7, 7, 64, 8, 3, 3, 1, 1, 2, 2),      # OH differs from PyTorch's formula
    (2, 9, 6, 70, 5, 3, 3, 1, 0, 1, 2),      # C % 64 != 0, asymmetric pad and stride
    (2, 8, 8, 128, 16, 1, 1, 0, 0, 2, 2),    # 1x1 stride 2
    (1, 6, 5, 200, 7, 2, 3, 2, 1, 1, 1),     # even kernel, pad larger than k/2
    (3, 5, 5, 64, 4, 1, 1, 1, 0, 2, 1),      # 1x1 with padding
]


@pytest.mark.parametrize("type", [0, 1, 2, 3])
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_equals_torch_conv_on_dequantised(type, case):
    N, H, W, C, KN, KH, KW, p1, p2, s1, s2 = case
    x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, KH, KW, seed=type * 31 + C, relu=(type in (1,)))
    qw, btn = oracle.quantize(w.numpy(), w_ths.numpy(), weight_bits(type), KN, KH, KW, C)
    y = oracle.conv2d(x.numpy(), qw, x_ths.numpy(), btn, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    OH, OW = oracle.out_extent(H, p1, KH, s1), oracle.out_extent(W, p2, KW, s2)
    assert y.shape == (N, KN, OH, OW) and y.dtype == np.float32
    qx, _ = oracle.quantize(x.numpy(), x_ths.numpy(), act_bits(type), N, H, W, C)
    want = torch_conv_reference(unpack(qx, C, act_bits(type)), unpack(qw, C, weight_bits(type)),
                                type, p1, p2, s1, s2, OH, OW)
    assert np.array_equal(y, want)


def test_conv2d_1x1_is_plain_gemm():
    N, H, W, C, KN = 2, 4, 3, 128, 9
    x, x_ths, w, w_ths = make_layer(0, N, H, W, C, KN, 1, 1, seed=77)
    qw, btn = oracle.quantize(w.numpy(), w_ths.numpy(), 2, KN, 1, 1, C)
    qx, _ = oracle.quantize(x.numpy(), x_ths.numpy(), 2, N, H, W, C)
    y = oracle.conv2d(x.numpy(), qw, x_ths.numpy(), btn, 0, 0, 0, 1, 1, N, H, W, C, KN, 1, 1)
    g = oracle.gemm(0, qx, qw, N * H * W, KN, C // 64)
    assert np.array_equal(y.ravel(), g.ravel().astype(np.float32))


def test_conv2d_rejects_bad_arguments():
    x = np.zeros((1, 4, 4, 64), np.float32)
    qw = np.zeros((1, 3, 3, 1, 1), np.int64)
    with pytest.raises(ValueError):
        oracle.conv2d(x, qw, [0.0], [0], 6, 1, 1, 1, 1, 1, 4, 4, 64, 1, 3, 3)
    with pytest.raises(ValueError):
        oracle.conv2d(x, qw, [0.0], [0], 3, 0, 0, 1, 1, 1, 2, 2, 64, 1, 3, 3)  # empty output
