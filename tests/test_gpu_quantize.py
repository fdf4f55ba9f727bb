"""GPU parity of Quantize (through the C ABI) against the CPU oracle: bit-exact QX and BTN."""
import numpy as np
import pytest
import torch

import oracle
import tab_amd

pytestmark = pytest.mark.gpu


def _run(x, ths, bitwidth, N, H, W, C):
    print(f"[case] Quantize bitwidth={bitwidth} N={N} H={H} W={W} C={C}", flush=True)
    qx, btn = tab_amd.Quantize(x.cuda(), ths.cuda(), bitwidth, N, H, W, C)
    torch.cuda.synchronize()
    assert qx.dtype == torch.int64 and tuple(qx.shape) == (N, H, W, (C + 63) // 64, bitwidth)
    assert btn.dtype == torch.int32 and tuple(btn.shape) == (N,)
    want_q, want_btn = oracle.quantize(x.numpy(), ths.numpy(), bitwidth, N, H, W, C)
    assert np.array_equal(qx.cpu().numpy(), want_q)
    assert np.array_equal(btn.cpu().numpy(), want_btn)


@pytest.mark.parametrize("bitwidth", [1, 2])
@pytest.mark.parametrize("shape", [
    (1, 32, 32, 64), (3, 5, 7, 64), (2, 3, 3, 128), (16, 14, 14, 256), (5, 7, 7, 512),
    (64, 3, 3, 256),            # the notebook's weight tensor
    (1, 1, 1, 64), (7, 1, 3, 192),
    (2, 4, 5, 1), (2, 3, 3, 63), (3, 2, 2, 65), (2, 5, 3, 70), (1, 3, 3, 200),  # C % 64 != 0
    # every lane-group width of the general path, full and ragged, several items per wave and waves per item
    (3, 9, 11, 2), (2, 17, 13, 3), (5, 8, 8, 4), (2, 9, 7, 5), (3, 6, 5, 8), (2, 7, 9, 13), (4, 5, 5, 16),
    (2, 6, 7, 17), (3, 5, 4, 31), (2, 8, 5, 32), (3, 4, 5, 33), (2, 13, 11, 100), (70, 2, 2, 129), (1, 40, 40, 3),
    (5, 60, 61, 3), (3, 30, 31, 100), (4, 33, 35, 24),  # many workgroups, items ending inside a wave
])
def test_quantize_matches_oracle(bitwidth, shape):
    N, H, W, C = shape
    g = torch.Generator("cpu").manual_seed(N * 1000 + C + bitwidth)
    x = torch.randn((N, H, W, C), generator=g)
    ths = (0.7 * x.abs().reshape(N, -1).mean(dim=1)) if bitwidth == 2 else torch.zeros(N)
    if N > 1:
        ths = ths * torch.linspace(0.5, 1.5, N)  # distinct thresholds per item
        if bitwidth == 1:
            ths = torch.linspace(-0.3, 0.3, N)
    _run(x, ths.float().contiguous(), bitwidth, N, H, W, C)


@pytest.mark.parametrize("bitwidth", [1, 2])
@pytest.mark.parametrize("C", [64, 70])
def test_quantize_special_values(bitwidth, C):
    t = 0.5
    specials = torch.tensor([t, -t, float(np.nextafter(np.float32(t), np.float32(1))),
                             float(np.nextafter(np.float32(-t), np.float32(-1))),
                             float("nan"), float("inf"), float("-inf"), 0.0, -0.0, 1e-45, -1e-45])
    x = specials.repeat(4 * C // specials.numel() + 1)[: 4 * C].reshape(1, 2, 2, C).contiguous()
    for th in (t, 0.0, -t):
        _run(x, torch.tensor([th]), bitwidth, 1, 2, 2, C)


def test_quantize_relu_zero_heavy_and_btn():
    g = torch.Generator("cpu").manual_seed(5)
    x = torch.relu(torch.randn((4, 9, 9, 128), generator=g))
    ths = 0.7 * x.abs().reshape(4, -1).mean(dim=1)
    _run(x, ths, 2, 4, 9, 9, 128)


def test_quantize_full_size_properties():
    """256x56x56x256 (the roofline shape) is too large for a full oracle compare inside a test,
    so check properties that do not depend on size: the sign plane is a subset of the nonzero
    plane and of the 1-bit (x < 0) words, BTN equals the number of nonzero ternary values counted
    on the fp32 input, and 4096 sampled pixels equal the oracle bit for bit."""
    N, H, W, C = 256, 56, 56, 256
    print(f"[case] Quantize full size N={N} H={H} W={W} C={C}", flush=True)
    g = torch.Generator("cuda").manual_seed(0)
    x = torch.randn((N, H, W, C), generator=g, device="cuda")
    ths = (0.7 * x.abs().reshape(N, -1).mean(dim=1)).contiguous()
    q2, btn = tab_amd.Quantize(x, ths, 2, N, H, W, C)
    q1, btn1 = tab_amd.Quantize(x, torch.zeros(N, device="cuda"), 1, N, H, W, C)
    torch.cuda.synchronize()
    sign, nz = q2[..., 0], q2[..., 1]
    assert bool(((sign & ~nz) == 0).all())
    assert not bool(btn1.any())
    # negative values: sign-plane bits are a subset of the 1-bit (x < 0) bits
    assert bool(((sign & ~q1[..., 0]) == 0).all())
    # BTN = number of nonzero ternary values per image, counted on the fp32 input
    nonzero = ((x > ths.view(N, 1, 1, 1)) | (x < -ths.view(N, 1, 1, 1))).reshape(N, -1).sum(dim=1)
    assert torch.equal(btn.to(torch.int64), nonzero)
    # sampled pixels against the oracle
    idx = torch.randint(0, N * H * W, (4096,), generator=torch.Generator("cpu").manual_seed(1))
    n_of = (idx // (H * W))
    xs = x.reshape(-1, C)[idx.cuda()].cpu().numpy()
    for bitwidth, q, t in ((2, q2, ths.cpu()), (1, q1, torch.zeros(N))):
        want, _ = oracle.quantize(xs.reshape(-1, 1, 1, C), t[n_of].numpy(), bitwidth, idx.numel(), 1, 1, C)
        got = q.reshape(N * H * W, C // 64, bitwidth)[idx.cuda()].cpu().numpy()
        assert np.array_equal(got, want.reshape(got.shape))


@pytest.mark.parametrize("bitwidth", [1, 2])
def test_quantize_without_btn(bitwidth):
    """dev_BTN == NULL (QuantizeActivation): the same packed words, no count vector, for NHWC and NCHW input."""
    N, H, W, C = 3, 9, 7, 200
    g = torch.Generator("cpu").manual_seed(bitwidth)
    x = torch.randn((N, H, W, C), generator=g)
    ths = (0.7 * x.abs().reshape(N, -1).mean(dim=1)).float() if bitwidth == 2 else torch.zeros(N)
    want, _ = oracle.quantize(x.numpy(), ths.numpy(), bitwidth, N, H, W, C)
    got = tab_amd.QuantizeActivation(x.cuda(), ths.cuda(), bitwidth, N, H, W, C)
    assert np.array_equal(got.cpu().numpy(), want)
    x_nchw = x.permute(0, 3, 1, 2).contiguous()
    got = tab_amd.QuantizeActivation(x_nchw.cuda(), ths.cuda(), bitwidth, N, H, W, C, nchw=True)
    assert np.array_equal(got.cpu().numpy(), want)
