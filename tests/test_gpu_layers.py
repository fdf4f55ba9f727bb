"""Threshold kernel and the nn.Module wrappers on the GPU."""
import numpy as np
import pytest
import torch

import oracle
import tab_amd
from helpers import torch_conv_reference, unpack
from tab_amd.nn import TABConv2d, TABLinear

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [(1, 64), (3, 7), (16, 56 * 56 * 64), (5, 1000003), (64, 3 * 3 * 256), (2, 4096 * 33 + 1)])
def test_threshold_matches_fp64_mean(shape):
    """Floating point: tolerance 1e-5 relative to the fp64 value of 0.7*mean|x| (fp32 slice sums,
    fp64 combination); two runs must agree bit for bit (fixed summation order)."""
    N, per = shape
    print(f"[case] Threshold N={N} per_item={per}", flush=True)
    x = torch.randn((N, per), generator=torch.Generator("cpu").manual_seed(per % 1000)) * 3.0
    xd = x.cuda()
    t1 = tab_amd.Threshold(xd, N, 0.7)
    t2 = tab_amd.Threshold(xd, N, 0.7)
    torch.cuda.synchronize()
    want = 0.7 * x.double().abs().mean(dim=1)
    assert t1.dtype == torch.float32 and tuple(t1.shape) == (N,)
    assert torch.equal(t1, t2)
    np.testing.assert_allclose(t1.cpu().double().numpy(), want.numpy(), rtol=1e-5, atol=0)


def test_threshold_unaligned_view_and_errors():
    base = torch.randn(4 * 1001 + 1, generator=torch.Generator("cpu").manual_seed(0)).cuda()
    x = base[1:]  # 4-byte aligned only
    t = tab_amd.Threshold(x, 4, 1.0)
    want = x.cpu().double().reshape(4, -1).abs().mean(dim=1)
    np.testing.assert_allclose(t.cpu().double().numpy(), want.numpy(), rtol=1e-5)
    with pytest.raises(RuntimeError, match="multiple of N"):
        tab_amd.Threshold(base, 4)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        tab_amd.Threshold(base.cpu(), 1)


@pytest.mark.parametrize("conv_type", [0, 1, 2, 3])
def test_conv_module_matches_dequantised_torch_conv(conv_type):
    print(f"[case] TABConv2d type={conv_type}", flush=True)
    g = torch.Generator("cpu").manual_seed(conv_type)
    N, C, H, W, KN = 3, 128, 9, 11, 24
    x = torch.randn((N, C, H, W), generator=g)
    w = torch.randn((KN, C, 3, 3), generator=g)
    layer = TABConv2d.from_float(w, conv_type, stride=(2, 1), padding=(1, 0))
    y = layer(x.cuda())
    torch.cuda.synchronize()
    OH, OW = tab_amd.out_shape(H, W, 3, 3, 1, 0, 2, 1)
    assert tuple(y.shape) == (N, KN, OH, OW)
    # independent reference: decode the packed tensors the layer used and convolve with torch
    abits = 2 if conv_type < 2 else 1
    wbits = 2 if conv_type in (0, 2) else 1
    x_nhwc = x.permute(0, 2, 3, 1).contiguous()
    ths = tab_amd.Threshold(x_nhwc.cuda(), N, 0.7) if abits == 2 else torch.zeros(N, device="cuda")
    qx, _ = oracle.quantize(x_nhwc.numpy(), ths.cpu().numpy(), abits, N, H, W, C)
    wq = unpack(layer.QW.cpu().numpy(), C, wbits)
    want = torch_conv_reference(unpack(qx, C, abits), wq, conv_type, 1, 0, 2, 1, OH, OW)
    want_nchw = torch.from_numpy(want).reshape(N, OH, OW, KN).permute(0, 3, 1, 2)
    assert torch.equal(y.cpu(), want_nchw)
    # NHWC flavour returns the same numbers without the permutes
    layer_nhwc = TABConv2d(layer.QW, layer.BTN_W, conv_type, C, KN, 3, (2, 1), (1, 0), data_format="NHWC")
    y2 = layer_nhwc(x_nhwc.cuda())
    assert torch.equal(y2.permute(0, 3, 1, 2), y)


def test_linear_module_is_integer_dot_product():
    g = torch.Generator("cpu").manual_seed(5)
    N, F, O = 7, 320, 33
    x = torch.randn((N, F), generator=g)
    w = torch.randn((O, F), generator=g)
    fc = TABLinear.from_float(w, tab_amd.BNN)
    y = fc(x.cuda())
    sx = torch.where(x < 0, -1.0, 1.0)
    sw = torch.where(w < 0, -1.0, 1.0)
    assert torch.equal(y.cpu(), sx @ sw.t())


def test_packed_chain_equals_layer_by_layer():
    """Three binary-activation layers (BNN, BTN, BNN) chained packed-to-packed return exactly what
    the same modules return one after the other (threshold 0 on both paths), and a ternary layer in
    the middle with a calibrated threshold matches the oracle's conv -> quantize -> conv."""
    from tab_amd.nn import TABPackedChain

    g = torch.Generator("cpu").manual_seed(3)
    x = torch.randn((3, 64, 12, 12), generator=g)
    w1 = torch.randn((128, 64, 3, 3), generator=g)
    w2 = torch.randn((96, 128, 3, 3), generator=g)
    w3 = torch.randn((40, 96, 1, 1), generator=g)
    l1 = TABConv2d.from_float(w1, tab_amd.BNN, stride=1, padding=1)
    l2 = TABConv2d.from_float(w2, tab_amd.BTN, stride=2, padding=1)
    l3 = TABConv2d.from_float(w3, tab_amd.BNN)
    print("[case] TABPackedChain BNN -> BTN -> BNN", flush=True)
    chain = TABPackedChain([l1, l2, l3])
    got = chain(x.cuda())
    want = l3(l2(l1(x.cuda())))
    torch.cuda.synchronize()
    assert got.shape == want.shape and torch.equal(got, want)

    # a ternary-activation layer second: its input threshold is the constant given to the chain
    print("[case] TABPackedChain BNN -> TNN with a calibrated threshold", flush=True)
    t2 = TABConv2d.from_float(w2, tab_amd.TNN, stride=1, padding=1)
    chain = TABPackedChain([l1, t2], ternary_thresholds={1: 24.0}, data_format="NHWC")
    xh = x.permute(0, 2, 3, 1).contiguous()
    got = chain(xh.cuda()).cpu().numpy()
    N, H, W = 3, 12, 12
    zeros = np.zeros(N, dtype=np.float32)
    y1 = oracle.conv2d(xh.numpy(), l1.QW.cpu().numpy(), zeros, l1.BTN_W.cpu().numpy(), 3, 1, 1, 1, 1, N, H, W, 64, 128, 3, 3)
    y2 = oracle.conv2d(np.ascontiguousarray(y1).reshape(N, H, W, 128), t2.QW.cpu().numpy(), np.full(N, 24.0, np.float32),
                       t2.BTN_W.cpu().numpy(), 0, 1, 1, 1, 1, N, H, W, 128, 96, 3, 3)
    assert np.array_equal(got.reshape(-1), np.ascontiguousarray(y2).reshape(-1))
    with pytest.raises(ValueError, match="ternary_thresholds"):
        TABPackedChain([l1, t2])
    with pytest.raises(ValueError, match="input channels"):
        TABPackedChain([l1, l3])
