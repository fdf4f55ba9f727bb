"""Seeded random geometry against the oracle: Conv2d (default kernel choice and a random forced
kernel) and Conv2dPackedOut, all four types.  Bit-exact."""
import numpy as np
import pytest
import torch

import oracle
import tab_amd
from helpers import act_bits, make_layer, weight_bits

pytestmark = pytest.mark.gpu

VARIANTS = [(tab_amd.CONV_AUTO, -1)] + [(tab_amd.CONV_MATRIX, t) for t in range(12)] + [(tab_amd.CONV_POPCOUNT, t) for t in range(3)]


def _random_case(rng):
    while True:
        N = int(rng.integers(1, 5))
        H, W = int(rng.integers(1, 21)), int(rng.integers(1, 21))
        C = int(rng.choice([1, 3, 63, 64, 65, 100, 128, 129, 192, 256, 320, 512]))
        KN = int(rng.choice([1, 2, 7, 31, 32, 33, 64, 65, 100, 129, 200]))
        KH, KW = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        p1, p2 = int(rng.integers(0, 3)), int(rng.integers(0, 3))
        s1, s2 = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        OH, OW = tab_amd.out_shape(H, W, KH, KW, p1, p2, s1, s2)
        if OH >= 1 and OW >= 1 and N * OH * OW * KN * KH * KW * C < 3e8:
            return N, H, W, C, KN, KH, KW, p1, p2, s1, s2


@pytest.mark.parametrize("seed", range(12))
def test_random_geometry(seed):
    rng = np.random.default_rng(1000 + seed)
    try:
        for _ in range(10):
            type = int(rng.integers(0, 4))
            N, H, W, C, KN, KH, KW, p1, p2, s1, s2 = case = _random_case(rng)
            variant = VARIANTS[int(rng.integers(0, len(VARIANTS)))]
            out_bits = int(rng.integers(1, 3))
            print(f"[case] random type={type} {case} kernel={variant} out_bits={out_bits}", flush=True)
            x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, KH, KW, seed=seed * 100 + type, relu=bool(rng.integers(0, 2)))
            qw, btn = oracle.quantize(w.numpy(), w_ths.numpy(), weight_bits(type), KN, KH, KW, C)
            want = oracle.conv2d(x.numpy(), qw, x_ths.numpy(), btn, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
            QW, BTN = torch.from_numpy(qw).cuda(), torch.from_numpy(btn).cuda()
            tab_amd.set_conv_kernel(*variant)
            y = tab_amd.Conv2d(x.cuda(), QW, x_ths.cuda(), BTN, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
            assert np.array_equal(y.cpu().numpy(), want), f"type {type} {case} {variant}"
            OH, OW = tab_amd.out_shape(H, W, KH, KW, p1, p2, s1, s2)
            out_ths = torch.from_numpy(rng.integers(-6, 7, size=N).astype(np.float32))
            want_q, _ = oracle.quantize(np.ascontiguousarray(want).reshape(N, OH, OW, KN), out_ths.numpy(), out_bits, N, OH, OW, KN)
            QX, _ = tab_amd.Quantize(x.cuda(), x_ths.cuda(), act_bits(type), N, H, W, C)
            q = tab_amd.Conv2dPackedOut(QX, QW, BTN, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW, out_ths.cuda(), out_bits)
            assert np.array_equal(q.cpu().numpy(), want_q), f"packed out type {type} {case} {variant}"
    finally:
        tab_amd.set_conv_kernel(tab_amd.CONV_AUTO, -1)
