"""GPU parity of QuantizeNCHW (through the C ABI) against the CPU oracle, whose NCHW reading order is pinned
against the reference's own CPU quantizers (TAB_CPU.cpp:20-206).  Bit-exact."""
import numpy as np
import pytest
import torch

import oracle
import tab_amd

pytestmark = pytest.mark.gpu

CASES = [
    # N, C, H, W
    (1, 64, 4, 4), (2, 70, 3, 5), (3, 128, 7, 7), (2, 1, 5, 3), (2, 200, 6, 6), (4, 256, 14, 14), (1, 63, 2, 2), (2, 65, 8, 4),
    (16, 64, 56, 56), (2, 512, 28, 28),
]


@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("case", CASES)
def test_nchw_equals_oracle_and_nhwc_path(bits, case):
    N, C, H, W = case
    print(f"[case] QuantizeNCHW bits={bits} N={N} C={C} {H}x{W}", flush=True)
    rng = np.random.default_rng(C * 7 + H + bits)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    ths = (0.7 * np.abs(x).reshape(N, -1).mean(axis=1)).astype(np.float32) if bits == 2 else np.linspace(-0.2, 0.2, N).astype(np.float32)
    flat = x.reshape(N, -1)
    for n in range(N):  # ties, NaN, infinities, signed zeros
        specials = [ths[n], -ths[n], np.nan, np.inf, -np.inf, 0.0, -0.0]
        k = min(len(specials), flat.shape[1])
        flat[n, :k] = specials[:k]
    want_q, want_btn = oracle.quantize_nchw(x, ths, bits, N, C, H, W)
    X = torch.from_numpy(x).cuda()
    T = torch.from_numpy(ths).cuda()
    QX, BTN = tab_amd.QuantizeNCHW(X, T, bits, N, C, H, W)
    torch.cuda.synchronize()
    assert QX.dtype == torch.int64 and tuple(QX.shape) == want_q.shape
    assert np.array_equal(QX.cpu().numpy(), want_q)
    assert np.array_equal(BTN.cpu().numpy(), want_btn)
    # the same words as the NHWC entry point on the transposed tensor
    QX2, BTN2 = tab_amd.Quantize(X.permute(0, 2, 3, 1).contiguous(), T, bits, N, H, W, C)
    assert torch.equal(QX, QX2) and torch.equal(BTN, BTN2)


def test_nchw_unaligned_view_takes_the_scalar_path():
    """A tensor whose storage is not 16-byte aligned (H*W % 4 == 0 notwithstanding) must give the same words."""
    N, C, H, W = 2, 128, 4, 4
    base = torch.randn(N * C * H * W + 1, device="cuda")
    x = base[1:].view(N, C, H, W)
    assert x.data_ptr() % 16 != 0 and x.is_contiguous()
    ths = torch.full((N,), 0.3, device="cuda")
    QX, BTN = tab_amd.QuantizeNCHW(x, ths, 2, N, C, H, W)
    want_q, want_btn = oracle.quantize_nchw(x.cpu().numpy(), ths.cpu().numpy(), 2, N, C, H, W)
    assert np.array_equal(QX.cpu().numpy(), want_q) and np.array_equal(BTN.cpu().numpy(), want_btn)


LARGE_CASES = [
    # N, C, H, W: enough pixels for the kernels that only large tensors reach
    (4, 128, 256, 256),  # two words per thread, gathered stores
    (3, 200, 300, 300),  # four words per thread, a tail word of 8 channels, a last wave with lanes past the end
    (2, 512, 260, 260),  # two groups of four words per pixel
    (2, 192, 600, 600),  # PC odd: four pixels per thread, one word, stored by the thread itself
]


@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("case", LARGE_CASES)
def test_nchw_large_tensors(bits, case):
    """Every image against the NHWC entry point on the transposed tensor (itself checked against the oracle in
    test_gpu_quantize.py), the first and the last image against the oracle directly."""
    N, C, H, W = case
    print(f"[case] QuantizeNCHW large bits={bits} N={N} C={C} {H}x{W}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(C + bits)
    X = torch.randn((N, C, H, W), generator=g, device="cuda")
    T = 0.7 * X.abs().reshape(N, -1).mean(dim=1) if bits == 2 else torch.linspace(-0.2, 0.2, N, device="cuda")
    for n in range(N):
        X[n].view(-1)[:7] = torch.tensor([T[n].item(), -T[n].item(), float("nan"), float("inf"), float("-inf"), 0.0, -0.0],
                                         device="cuda")
    QX, BTN = tab_amd.QuantizeNCHW(X, T, bits, N, C, H, W)
    QX2, BTN2 = tab_amd.Quantize(X.permute(0, 2, 3, 1).contiguous(), T, bits, N, H, W, C)
    torch.cuda.synchronize()
    assert torch.equal(QX, QX2) and torch.equal(BTN, BTN2)
    for n in (0, N - 1):
        want_q, want_btn = oracle.quantize_nchw(X[n:n + 1].cpu().numpy(), T[n:n + 1].cpu().numpy(), bits, 1, C, H, W)
        assert np.array_equal(QX[n:n + 1].cpu().numpy(), want_q)
        assert np.array_equal(BTN[n:n + 1].cpu().numpy(), want_btn)
