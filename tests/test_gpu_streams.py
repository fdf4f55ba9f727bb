"""The library only enqueues work on the stream it is handed: calls on a side stream, and calls captured into a
HIP graph and replayed several times with new inputs and eager work in between, must give what the same calls
give eagerly on the default stream.  Bit-exact (integer work); the threshold reduction is reproducible, so it is
compared bit for bit as well."""
import pytest
import torch

import tab_amd
from helpers import act_bits, make_layer, weight_bits

pytestmark = pytest.mark.gpu

GEOM = (4, 14, 14, 128, 96, 3, 3, 1, 1, 1, 1)  # N, H, W, C, KN, KH, KW, p1, p2, s1, s2


def _everything(type, x, x_ths, QW, BTN, out_ths):
    """One call of every entry point that launches kernels, on the current stream."""
    N, H, W, C, KN, KH, KW, p1, p2, s1, s2 = GEOM
    y = tab_amd.Conv2d(x, QW, x_ths, BTN, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    QX, btn_x = tab_amd.Quantize(x, x_ths, act_bits(type), N, H, W, C)
    QN, _ = tab_amd.QuantizeNCHW(x.view(N, C, H, W), x_ths, act_bits(type), N, C, H, W)
    yp = tab_amd.Conv2dPacked(QX, QW, BTN, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
    qy = tab_amd.Conv2dPackedOut(QX, QW, BTN, type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW, out_ths, 2)
    th = tab_amd.Threshold(x, N, 0.7)
    return [y, QX, btn_x, QN, yp, qy, th]


def _inputs(type, seed):
    N, H, W, C, KN, KH, KW = GEOM[:7]
    x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, KH, KW, seed=seed)
    QW, BTN = tab_amd.Quantize(w.cuda(), w_ths.cuda(), weight_bits(type), KN, KH, KW, C)
    out_ths = torch.linspace(1.0, 9.0, N).cuda()
    return x.cuda(), x_ths.cuda(), QW, BTN, out_ths


@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_side_stream_equals_default_stream(type):
    x, x_ths, QW, BTN, out_ths = _inputs(type, seed=20 + type)
    want = _everything(type, x, x_ths, QW, BTN, out_ths)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        got = _everything(type, x, x_ths, QW, BTN, out_ths)
    side.synchronize()
    for g, w in zip(got, want):
        assert torch.equal(g, w)


@pytest.mark.parametrize("type", [0, 3])
def test_graph_replays_equal_eager(type):
    x, x_ths, QW, BTN, out_ths = _inputs(type, seed=30 + type)
    static_x, static_ths = x.clone(), x_ths.clone()
    # warm up on a side stream, as graph capture asks, then capture every entry point once
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _everything(type, static_x, static_ths, QW, BTN, out_ths)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = _everything(type, static_x, static_ths, QW, BTN, out_ths)
    for replay in range(4):
        new_x, new_ths, _, _, _ = _inputs(type, seed=100 * replay + type)
        want = _everything(type, new_x, new_ths, QW, BTN, out_ths)  # eager work between the replays
        static_x.copy_(new_x)
        static_ths.copy_(new_ths)
        graph.replay()
        torch.cuda.synchronize()
        for g, w in zip(captured, want):
            assert torch.equal(g, w), f"replay {replay}"
