"""tab_conv2d_static (the packed activation in the library's built-in device scratch, no allocation in the call)
against tab_conv2d (caller-owned workspace) through the C ABI: bit-identical outputs, on calls in a row that
share the scratch, the later ones with smaller inputs."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import make_layer, weight_bits

pytestmark = pytest.mark.gpu


def _both(lib, check, type, N, H, W, C, KN, KH, KW, p1, p2, s1, s2, seed, relu=False):
    import tab_amd

    x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, KH, KW, seed=seed, relu=relu)
    QW, BTN = tab_amd.Quantize(w.cuda(), w_ths.cuda(), weight_bits(type), KN, KH, KW, C)
    xd, td = x.cuda(), x_ths.cuda()
    OH, OW = tab_amd.out_shape(H, W, KH, KW, p1, p2, s1, s2)
    ws_bytes = lib.tab_conv2d_workspace_bytes(type, N, H, W, C)
    assert 0 < ws_bytes <= lib.tab_static_scratch_bytes()
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    y_ws = torch.full((N * OH * OW * KN,), float("nan"), device="cuda")
    y_static = torch.full((N * OH * OW * KN,), float("nan"), device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    check(lib, lib.tab_conv2d(xd.data_ptr(), QW.data_ptr(), td.data_ptr(), BTN.data_ptr(), type, p1, p2, s1, s2,
                              N, H, W, C, KN, KH, KW, y_ws.data_ptr(), ws.data_ptr(), ws_bytes, stream))
    # a first static call looks the scratch's address up (and, like the call above, has the kernels' code loaded):
    # everything the next one touches exists by then, and that call must not allocate or free, neither through
    # torch's allocator nor behind its back (the driver's own count of free device memory sees a hipMalloc or
    # hipFree made inside the library)
    check(lib, lib.tab_conv2d_static(xd.data_ptr(), QW.data_ptr(), td.data_ptr(), BTN.data_ptr(), type, p1, p2, s1, s2,
                                     N, H, W, C, KN, KH, KW, y_static.data_ptr(), stream))
    torch.cuda.synchronize()
    y_static.fill_(float("nan"))
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    check(lib, lib.tab_conv2d_static(xd.data_ptr(), QW.data_ptr(), td.data_ptr(), BTN.data_ptr(), type, p1, p2, s1, s2,
                                     N, H, W, C, KN, KH, KW, y_static.data_ptr(), stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    assert not torch.isnan(y_static).any()
    assert torch.equal(y_ws, y_static), f"type {type} N={N} {H}x{W}x{C}->{KN} k{KH}x{KW} s{s1}{s2}: outputs differ"
    return y_static


@pytest.mark.parametrize("type", [0, 1, 2, 3])
def test_static_scratch_matches_workspace_on_calls_in_a_row(type):
    from tab_amd import _capi

    lib = _capi.load()
    # a large call first, then smaller ones that find its packed activation still in the scratch
    _both(lib, _capi.check, type, 4, 28, 28, 256, 128, 3, 3, 1, 1, 1, 1, seed=10 + type, relu=type in (1, 2))
    _both(lib, _capi.check, type, 2, 14, 14, 128, 64, 3, 3, 1, 1, 2, 2, seed=20 + type)
    _both(lib, _capi.check, type, 1, 9, 7, 70, 33, 1, 1, 0, 0, 2, 2, seed=30 + type)   # the strided 1x1 quantizer
    y = _both(lib, _capi.check, type, 1, 8, 8, 64, 64, 3, 3, 1, 0, 1, 1, seed=40 + type)
    # and against the oracle, once
    import oracle

    x, x_ths, w, w_ths = make_layer(type, 1, 8, 8, 64, 64, 3, 3, seed=40 + type)
    qw, btn = oracle.quantize(w.numpy(), w_ths.numpy(), weight_bits(type), 64, 3, 3, 64)
    want = oracle.conv2d(x.numpy(), qw, x_ths.numpy(), btn, type, 1, 0, 1, 1, 1, 8, 8, 64, 64, 3, 3)
    assert np.array_equal(y.cpu().numpy().reshape(want.shape), want)


@pytest.mark.parametrize("type", [0, 3])
def test_static_scratch_under_graph_capture(type):
    """The use the entry point is made for: captured into a HIP graph after a first eager call, replayed several times
    with the program's own eager work and synchronisations in between, every replay equal to tab_conv2d's result."""
    import tab_amd
    from tab_amd import _capi

    lib = _capi.load()
    N, H, W, C, KN = 3, 14, 14, 128, 96
    x, x_ths, w, w_ths = make_layer(type, N, H, W, C, KN, 3, 3, seed=50 + type)
    QW, BTN = tab_amd.Quantize(w.cuda(), w_ths.cuda(), weight_bits(type), KN, 3, 3, C)
    xd, td = x.cuda(), x_ths.cuda()
    want = tab_amd.Conv2d(xd, QW, td, BTN, type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3)
    out = torch.zeros_like(want)
    args = (xd.data_ptr(), QW.data_ptr(), td.data_ptr(), BTN.data_ptr(), type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3, out.data_ptr())
    _capi.check(lib, lib.tab_conv2d_static(*args, torch.cuda.current_stream().cuda_stream))  # address lookup, outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _capi.check(lib, lib.tab_conv2d_static(*args, torch.cuda.current_stream().cuda_stream))
    for replay in range(4):
        out.fill_(float("nan"))
        # eager work that reuses the scratch between the replays: a different, smaller call
        tab_amd.Conv2dStatic(xd[:1].contiguous(), QW, td[:1].contiguous(), BTN, type, 1, 1, 1, 1, 1, H, W, C, KN, 3, 3)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {replay}"


def test_static_scratch_formats_4_and_5():
    import tab_amd
    from tab_amd import _capi

    lib = _capi.load()
    for type, (N, H, W, C, KN) in ((4, (2, 12, 12, 128, 64)), (5, (2, 12, 12, 128, 64)), (5, (1, 6, 6, 64, 32))):
        g = torch.Generator("cpu").manual_seed(type)
        x = torch.randn((N, H, W, C), generator=g).abs() if type == 4 else torch.randn((N, H, W, C), generator=g)
        w = torch.randn((KN, 3, 3, C), generator=g).abs() if type == 4 else torch.randn((KN, 3, 3, C), generator=g)
        x_ths, w_ths = torch.full((N,), 0.6), torch.full((KN,), 0.5)
        QW = tab_amd.QuantizeFormat(w.cuda(), w_ths.cuda(), type, KN, 3, 3, C)
        btn = torch.zeros(KN, dtype=torch.int32, device="cuda")
        want = tab_amd.Conv2d(x.cuda(), QW, x_ths.cuda(), btn, type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3)
        got = tab_amd.Conv2dStatic(x.cuda(), QW, x_ths.cuda(), btn, type, 1, 1, 1, 1, N, H, W, C, KN, 3, 3)
        torch.cuda.synchronize()
        assert torch.equal(want, got)


def test_static_scratch_rejects_what_does_not_fit():
    from tab_amd import _capi

    lib = _capi.load()
    limit = lib.tab_static_scratch_bytes()
    assert limit == 32 << 20
    # TNN N=256 56x56x256: 256*56*56*4*2*8 = 51 MB of packed activation
    N, H, W, C, KN = 256, 56, 56, 256, 64
    assert lib.tab_conv2d_workspace_bytes(0, N, H, W, C) > limit
    dummy = torch.zeros(1024, device="cuda")
    rc = lib.tab_conv2d_static(dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(), dummy.data_ptr(), 0, 1, 1, 1, 1,
                               N, H, W, C, KN, 3, 3, dummy.data_ptr(), None)
    assert rc == -3 and b"built-in scratch" in lib.tab_last_error()
    torch.cuda.synchronize()
