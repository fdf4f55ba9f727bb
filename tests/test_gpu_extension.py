"""The pybind11 C++ extension (imported as TAB_CUDA, the reference's module name) on the GPU:
the demo notebook's call sequence (TAB Demo CUDA.ipynb cells 5-18) with seeded inputs, checked
against the CPU oracle, plus the notebook's stored shapes/dtypes/relations."""
import json
import os

import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def test_notebook_flow_matches_oracle():
    import TAB_CUDA as TAB

    assert {"Conv2d", "Quantize"} <= set(dir(TAB))  # cell 3
    kat = json.load(open(os.path.join(GOLD, "notebook_kat.json")))
    g = torch.Generator("cpu").manual_seed(0)
    KN, KH, KW, KC = 64, 3, 3, 256
    w = torch.rand([KN, KH, KW, KC], generator=g)
    w_ths = 0.5 * torch.ones([KN])
    # cell 5/7: ternary weights
    QW2, BTN_W2 = TAB.Quantize(w.cuda(), w_ths.cuda(), 2, KN, KH, KW, KC)
    assert list(QW2.size()) == kat["ternary_shape"] and list(BTN_W2.size()) == kat["btn_shape"]
    assert QW2.dtype == torch.int64 and QW2.is_cuda and BTN_W2.dtype == torch.int32
    assert not bool(QW2[..., 0].any())  # rand() >= 0: no -1, sign plane all zero
    # cell 9/10: binary weights are the complement of the ternary nonzero plane
    QW1, BTN_W1 = TAB.Quantize(w.cuda(), w_ths.cuda(), 1, KN, KH, KW, KC)
    assert list(QW1.size()) == kat["binary_shape"]
    assert torch.equal(QW1[..., 0], ~QW2[..., 1])
    q2_o, btn2_o = oracle.quantize(w.numpy(), w_ths.numpy(), 2, KN, KH, KW, KC)
    q1_o, _ = oracle.quantize(w.numpy(), w_ths.numpy(), 1, KN, KH, KW, KC)
    assert np.array_equal(QW2.cpu().numpy(), q2_o) and np.array_equal(BTN_W2.cpu().numpy(), btn2_o)
    assert np.array_equal(QW1.cpu().numpy(), q1_o) and not bool(BTN_W1.any())
    # cell 12-18 at a reduced batch (N=2 instead of 16) so the oracle stays fast
    N, H, W, C = 2, 112, 112, 256
    x = torch.rand([N, H, W, C], generator=g)
    x_ths = 0.5 * torch.ones([N])
    for conv_type in range(4):
        print(f"[case] TAB_CUDA.Conv2d type={conv_type}", flush=True)
        QW, BTN_W = (QW2, BTN_W2) if conv_type in (0, 2) else (QW1, BTN_W1)
        y = TAB.Conv2d(x.cuda(), QW, x_ths.cuda(), BTN_W, conv_type, 1, 1, 1, 1, N, H, W, C, KN, KH, KW)
        assert list(y.size()) == [N] + kat["conv_shape"][1:] and y.dtype == torch.float32
        want = oracle.conv2d(x.numpy(), QW.cpu().numpy(), x_ths.numpy(), BTN_W.cpu().numpy(), conv_type,
                             1, 1, 1, 1, N, H, W, C, KN, KH, KW)
        assert np.array_equal(y.cpu().numpy(), want)
        if conv_type == 3:
            assert bool((y.to(torch.int64) % 2 == 0).all())  # NUM = 9*256 is even (cell 18's sample)


def test_extension_equals_ctypes_front_end():
    import TAB_CUDA as TAB

    import tab_amd

    g = torch.Generator("cpu").manual_seed(3)
    N, H, W, C, KN = 3, 9, 7, 192, 40
    x = torch.randn([N, H, W, C], generator=g).cuda()
    w = torch.randn([KN, 3, 3, C], generator=g).cuda()
    x_ths = (0.7 * x.abs().reshape(N, -1).mean(dim=1)).contiguous()
    w_ths = (0.7 * w.abs().reshape(KN, -1).mean(dim=1)).contiguous()
    QWa, BTNa = TAB.Quantize(w, w_ths, 2, KN, 3, 3, C)
    QWb, BTNb = tab_amd.Quantize(w, w_ths, 2, KN, 3, 3, C)
    assert torch.equal(QWa, QWb) and torch.equal(BTNa, BTNb)
    ya = TAB.Conv2d(x, QWa, x_ths, BTNa, 0, 1, 0, 2, 1, N, H, W, C, KN, 3, 3)
    yb = tab_amd.Conv2d(x, QWb, x_ths, BTNb, 0, 1, 0, 2, 1, N, H, W, C, KN, 3, 3)
    assert torch.equal(ya, yb)


def test_extension_input_checks():
    import TAB_CUDA as TAB

    x = torch.zeros((1, 4, 4, 64), device="cuda")
    ths = torch.zeros(1, device="cuda")
    btn = torch.zeros(4, dtype=torch.int32, device="cuda")
    qw = torch.zeros((4, 3, 3, 1, 1), dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="X must be a CUDA tensor"):
        TAB.Conv2d(x.cpu(), qw, ths, btn, 3, 1, 1, 1, 1, 1, 4, 4, 64, 4, 3, 3)
    with pytest.raises(RuntimeError, match="must be contiguous"):
        TAB.Quantize(x.permute(0, 3, 1, 2), ths, 1, 1, 4, 4, 64)
    with pytest.raises(RuntimeError, match="QW has"):
        TAB.Conv2d(x, qw, ths, btn, 0, 1, 1, 1, 1, 1, 4, 4, 64, 4, 3, 3)
    with pytest.raises(RuntimeError, match="type must be"):
        TAB.Conv2d(x, qw, ths, btn, 9, 1, 1, 1, 1, 1, 4, 4, 64, 4, 3, 3)
    with pytest.raises(RuntimeError, match="bitwidth"):
        TAB.Quantize(x, ths, 3, 1, 4, 4, 64)
    y = TAB.Conv2d(x, qw, ths, btn, 3, 1, 1, 1, 1, 1, 4, 4, 64, 4, 3, 3)
    assert tuple(y.shape) == (1, 4, 4, 4)


def test_every_extension_entry_point_equals_ctypes_front_end():
    """The pybind module exports everything the ctypes mirror does; each function, called through TAB_CUDA,
    returns the tensors the mirror returns (same C ABI underneath), and Conv2d takes types 4 and 5 like the
    reference's CPU binding (TAB_CPU.cpp:577-584, 621-633)."""
    import TAB_CUDA as TAB

    import tab_amd

    assert {"QuantizeNCHW", "QuantizeFormat", "Threshold", "Conv2dPacked", "Conv2dPackedOut", "TAB_Quantize",
            "TAB_Conv2d"} <= set(dir(TAB))
    g = torch.Generator("cpu").manual_seed(11)
    N, H, W, C, KN = 3, 10, 9, 192, 72
    x = torch.randn([N, H, W, C], generator=g).cuda()
    w = torch.randn([KN, 3, 3, C], generator=g).cuda()
    # Threshold
    ths_a, ths_b = TAB.Threshold(x, N, 0.7), tab_amd.Threshold(x, N, 0.7)
    assert torch.equal(ths_a, ths_b) and torch.equal(TAB.Threshold(x, N), ths_b)
    w_ths = TAB.Threshold(w, KN, 0.7)
    # QuantizeNCHW
    x_nchw = x.permute(0, 3, 1, 2).contiguous()
    for bits in (1, 2):
        qa, ba = TAB.QuantizeNCHW(x_nchw, ths_a, bits, N, C, H, W)
        qb, bb = tab_amd.QuantizeNCHW(x_nchw, ths_a, bits, N, C, H, W)
        qc, _ = TAB.Quantize(x, ths_a, bits, N, H, W, C)
        assert torch.equal(qa, qb) and torch.equal(ba, bb) and torch.equal(qa, qc)
    zeros = torch.zeros(max(N, KN), device="cuda")
    for type in range(4):
        print(f"[case] TAB_CUDA packed entry points type={type}", flush=True)
        ab, wb = (2 if type < 2 else 1), (2 if type in (0, 2) else 1)
        QW, BTN = TAB.Quantize(w, w_ths if wb == 2 else zeros, wb, KN, 3, 3, C)
        QX, _ = TAB.Quantize(x, ths_a if ab == 2 else zeros, ab, N, H, W, C)
        ya = TAB.Conv2dPacked(QX, QW, BTN, type, 1, 0, 1, 2, N, H, W, C, KN, 3, 3)
        yb = tab_amd.Conv2dPacked(QX, QW, BTN, type, 1, 0, 1, 2, N, H, W, C, KN, 3, 3)
        assert torch.equal(ya, yb) and tuple(ya.shape) == tuple(yb.shape)
        assert torch.equal(ya, TAB.TAB_Conv2d(x, QW, ths_a if ab == 2 else zeros, BTN, type, 1, 0, 1, 2, N, H, W, C, KN, 3, 3))
        out_ths = torch.full((N,), 3.0, device="cuda")
        for out_bits in (1, 2):
            qa = TAB.Conv2dPackedOut(QX, QW, BTN, type, 1, 0, 1, 2, N, H, W, C, KN, 3, 3, out_ths, out_bits)
            qb = tab_amd.Conv2dPackedOut(QX, QW, BTN, type, 1, 0, 1, 2, N, H, W, C, KN, 3, 3, out_ths, out_bits)
            assert torch.equal(qa, qb) and tuple(qa.shape) == tuple(qb.shape)
    # types 4 and 5: packer and Conv2d
    btn = torch.zeros(KN, dtype=torch.int32, device="cuda")
    for type in (4, 5):
        print(f"[case] TAB_CUDA types of the CPU path type={type}", flush=True)
        xs, ws = (x.abs(), w.abs()) if type == 4 else (x, w)
        x_t, w_t = torch.full((N,), 0.6, device="cuda"), torch.full((KN,), 0.5, device="cuda")
        QWa, QWb = TAB.QuantizeFormat(ws, w_t, type, KN, 3, 3, C), tab_amd.QuantizeFormat(ws, w_t, type, KN, 3, 3, C)
        assert torch.equal(QWa, QWb) and tuple(QWa.shape) == tuple(QWb.shape)
        ya = TAB.Conv2d(xs, QWa, x_t, btn, type, 1, 1, 2, 1, N, H, W, C, KN, 3, 3)
        yb = tab_amd.Conv2d(xs, QWa, x_t, btn, type, 1, 1, 2, 1, N, H, W, C, KN, 3, 3)
        assert torch.equal(ya, yb)
        qw_o = oracle.quantize_format(ws.cpu().numpy(), w_t.cpu().numpy(), type, KN, 3, 3, C)
        want = oracle.conv2d(xs.cpu().numpy(), qw_o, x_t.cpu().numpy(), np.zeros(KN, np.int32), type, 1, 1, 2, 1, N, H, W, C, KN, 3, 3)
        assert np.array_equal(ya.cpu().numpy(), want)
        QX = TAB.QuantizeFormat(xs, x_t, type, N, H, W, C)
        assert torch.equal(TAB.Conv2dPacked(QX, QWa, btn, type, 1, 1, 2, 1, N, H, W, C, KN, 3, 3), ya)
        # packed output for these types too: both front ends agree with quantizing the fp32 result
        OH, OW = tab_amd.out_shape(H, W, 3, 3, 1, 1, 2, 1)
        out_t = torch.full((N,), float(ya.abs().median()), device="cuda")
        for out_bits in (1, 2):
            qa = TAB.Conv2dPackedOut(QX, QWa, btn, type, 1, 1, 2, 1, N, H, W, C, KN, 3, 3, out_t, out_bits)
            qb = tab_amd.Conv2dPackedOut(QX, QWa, btn, type, 1, 1, 2, 1, N, H, W, C, KN, 3, 3, out_t, out_bits)
            want_q, _ = tab_amd.Quantize(ya.view(N, OH, OW, KN), out_t, out_bits, N, OH, OW, KN)
            assert torch.equal(qa, qb) and torch.equal(qa.reshape(want_q.shape), want_q)
