"""Pins the oracle's two CPU-only types, 4 (DoReFa 2-bit) and 5 (RTN): the GEMMs
(TAB_CPU.cpp:332-383) against the reference's own compiled functions (live and as committed
golden vectors) and against integer dot products of the decoded operands; the conv pipeline
against torch.nn.functional.conv2d on decoded tensors.  The two packers have no counterpart in
the reference (TAB_Conv calls functions that no file defines, TAB_CPU.cpp:522,527): they are
checked against per-element closed forms only."""
import os

import numpy as np
import pytest

import oracle
from helpers import (brute_levels, brute_values, pack_drf, pack_rtn, torch_conv_reference, unpack_drf,
                     unpack_rtn)

GOLD = os.path.join(os.path.dirname(__file__), "golden")
PLANES = {4: 2, 5: 1}


def _rand_words(rng, shape):
    return rng.integers(-2**63, 2**63 - 1, size=shape, dtype=np.int64, endpoint=True)


def _decode(type, q, C):
    return unpack_drf(q, C) if type == 4 else unpack_rtn(q, C)


@pytest.mark.parametrize("type", [4, 5])
def test_gemm_against_reference_golden(type):
    g = np.load(os.path.join(GOLD, "ref_golden.npz"))
    M, N, K, _ = (int(v) for v in g[f"gemm{type}_mnk_num"])
    assert np.array_equal(oracle.gemm(type, g[f"gemm{type}_a"], g[f"gemm{type}_b"], M, N, K), g[f"gemm{type}_y"])


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref not built (no reference tree)")
@pytest.mark.parametrize("type", [4, 5])
@pytest.mark.parametrize("mnk", [(1, 1, 1), (33, 17, 9), (130, 70, 36)])
def test_gemm_against_reference_live(type, mnk):
    M, N, K = mnk
    rng = np.random.default_rng(M * 11 + type)
    a = _rand_words(rng, (M, K, PLANES[type]))
    b = _rand_words(rng, (N, K, PLANES[type]))
    assert np.array_equal(oracle.gemm(type, a, b, M, N, K), oracle.ref_gemm(type, a, b, M, N, K))


@pytest.mark.parametrize("type", [4, 5])
def test_gemm_equals_integer_dot_product_on_any_bits(type):
    """Every bit pattern decodes (levels 2*hi+lo; fields nonzero*(1-2*sign), a sign bit without its
    nonzero bit being 0), and the GEMM is the dot product of the decoded rows."""
    rng = np.random.default_rng(90 + type)
    M, N, K = 11, 7, 5
    a = _rand_words(rng, (M, K, PLANES[type]))
    b = _rand_words(rng, (N, K, PLANES[type]))
    per_word = 64 if type == 4 else 32
    if type == 5:
        a, b = a[..., 0], b[..., 0]
    va = _decode(type, a, K * per_word).astype(np.int64)
    vb = _decode(type, b, K * per_word).astype(np.int64)
    assert np.array_equal(oracle.gemm(type, a, b, M, N, K), va @ vb.T)


def test_rtn_gemm_is_tnn_on_deinterleaved_planes():
    """The fields of type 5 carry the same two markers as type 0's planes."""
    rng = np.random.default_rng(3)
    M, N, C = 6, 5, 128
    va = rng.integers(-1, 2, size=(M, C)).astype(np.int8)
    vb = rng.integers(-1, 2, size=(N, C)).astype(np.int8)
    from helpers import brute_pack
    y_rtn = oracle.gemm(5, pack_rtn(va), pack_rtn(vb), M, N, C // 32)
    y_tnn = oracle.gemm(0, brute_pack(va, 2), brute_pack(vb, 2), M, N, C // 64)
    assert np.array_equal(y_rtn, y_tnn) and np.array_equal(y_rtn, va.astype(np.int32) @ vb.T.astype(np.int32))


@pytest.mark.parametrize("C", [1, 31, 32, 33, 63, 64, 65, 100, 200])
def test_packers_equal_closed_forms(C):
    rng = np.random.default_rng(C)
    N, H, W = 3, 2, 3
    x = rng.standard_normal((N, H, W, C)).astype(np.float32) * 1.5
    ths = np.array([0.5, 0.0, 1.25], np.float32)
    flat = x.reshape(N, -1)
    for n in range(N):  # ties at every bound, NaN, infinities, signed zero
        specials = [0.5 * ths[n], 1.5 * ths[n], 2.5 * ths[n], ths[n], -ths[n], np.nan, np.inf, -np.inf, 0.0, -0.0]
        k = min(len(specials), flat.shape[1])
        flat[n, :k] = specials[:k]
    q4 = oracle.quantize_format(x, ths, 4, N, H, W, C)
    assert q4.shape == (N, H, W, (C + 63) // 64, 2)
    assert np.array_equal(q4, pack_drf(brute_levels(x, ths)))
    q5 = oracle.quantize_format(x, ths, 5, N, H, W, C)
    assert q5.shape == (N, H, W, (C + 31) // 32)
    assert np.array_equal(q5, pack_rtn(brute_values(x, ths, 2)))
    assert np.array_equal(unpack_drf(q4, C), brute_levels(x, ths))
    assert np.array_equal(unpack_rtn(q5, C), brute_values(x, ths, 2))


CONV_CASES = [
    # N, H, W, C, KN, KH, KW, p1, p2, s1, s2
    (1, 8, 8, 64, 16, 3, 3, 1, 1, 1, 1),
    (2, 7, 7, 64, 8, 3, 3, 1, 1, 2, 2),
    (2, 9, 6, 70, 5, 3, 3, 1, 0, 1, 2),
    (2, 8, 8, 128, 16, 1, 1, 0, 0, 2, 2),
    (1, 6, 5, 200, 7, 2, 3, 2, 1, 1, 1),
    (3, 5, 5, 33, 4, 1, 1, 1, 0, 2, 1),
]


@pytest.mark.parametrize("type", [4, 5])
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_equals_torch_conv_on_decoded(type, case):
    N, H, W, C, KN, KH, KW, p1, p2, s1, s2 = case
    rng = np.random.default_rng(type * 17 + C)
    x = np.abs(rng.standard_normal((N, H, W, C))).astype(np.float32) if type == 4 else rng.standard_normal((N, H, W, C)).astype(np.float32)
    w = np.abs(rng.standard_normal((KN, KH, KW, C))).astype(np.float32) if type == 4 else rng.standard_normal((KN, KH, KW, C)).astype(np.float32)
    x_ths = np.full(N, 0.6, np.float32)
    w_ths = np.full(KN, 0.5, np.float32)
    qw = oracle.quantize_format(w, w_ths, type, KN, KH, KW, C)
    qx = oracle.quantize_format(x, x_ths, type, N, H, W, C)
    OH, OW = oracle.out_extent(H, p1, KH, s1), oracle.out_extent(W, p2, KW, s2)
    want = torch_conv_reference(_decode(type, qx, C), _decode(type, qw, C), type, p1, p2, s1, s2, OH, OW)
    y = oracle.conv2d(x, qw, x_ths, np.zeros(KN, np.int32), type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    assert y.shape == (N, KN, OH, OW) and np.array_equal(y, want)
    assert np.array_equal(oracle.conv2d_packed(qx, qw, None, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW), want)


@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_conv2d_packed_equals_conv2d_for_the_gpu_types(type):
    from helpers import act_bits, make_layer, weight_bits
    N, H, W, C, KN, KH, KW, p1, p2, s1, s2 = 2, 6, 7, 70, 9, 3, 3, 1, 1, 1, 2
    x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, KH, KW, seed=5 + type)
    qw, btn = oracle.quantize(w.numpy(), w_ths.numpy(), weight_bits(type), KN, KH, KW, C)
    qx, _ = oracle.quantize(x.numpy(), x_ths.numpy(), act_bits(type), N, H, W, C)
    assert np.array_equal(oracle.conv2d_packed(qx, qw, btn, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW),
                          oracle.conv2d(x.numpy(), qw, x_ths.numpy(), btn, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW))
