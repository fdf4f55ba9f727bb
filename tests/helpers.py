"""Shared input builders and independent references for the tests.

Nothing here restates the oracle's C code: `dequantize_*` and `torch_conv_reference` go
through torch.nn.functional.conv2d on {-1,0,+1} tensors, and `brute_*` are per-element
closed forms in numpy.
"""
import numpy as np
import torch

TYPE_NAMES = {0: "TNN", 1: "TBN", 2: "BTN", 3: "BNN"}


def act_bits(type):
    return 2 if type < 2 else 1


def weight_bits(type):
    return 2 if type in (0, 2) else 1


def make_layer(type, N, H, W, C, KN, KH, KW, seed=0, relu=False):
    """Seeded inputs as the benchmark defines them: X ~ N(0,1) (optionally ReLU'd) NHWC,
    Wt ~ N(0,1) [KN,KH,KW,C]; ternary thresholds 0.7*mean|.| per image / per filter,
    binary thresholds 0."""
    gx = torch.Generator("cpu").manual_seed(seed)
    gw = torch.Generator("cpu").manual_seed(seed + 1)
    x = torch.randn((N, H, W, C), generator=gx, dtype=torch.float32)
    if relu:
        x = torch.relu(x)
    w = torch.randn((KN, KH, KW, C), generator=gw, dtype=torch.float32)
    if act_bits(type) == 2:
        x_ths = 0.7 * x.abs().reshape(N, -1).mean(dim=1)
    else:
        x_ths = torch.zeros(N)
    if weight_bits(type) == 2:
        w_ths = 0.7 * w.abs().reshape(KN, -1).mean(dim=1)
    else:
        w_ths = torch.zeros(KN)
    return x.contiguous(), x_ths.float().contiguous(), w.contiguous(), w_ths.float().contiguous()


# ---- per-element closed forms (TAB_GEMM.cu:184-192, 231) ------------------------------------
def brute_values(x, ths, bitwidth):
    """Quantized values in {-1,0,+1} (ternary) or {-1,+1} (binary), same shape as x (N first)."""
    x = np.asarray(x, dtype=np.float32)
    t = np.asarray(ths, dtype=np.float32)[: x.shape[0]].reshape((-1,) + (1,) * (x.ndim - 1))
    with np.errstate(invalid="ignore"):
        if bitwidth == 2:
            pos = x > t
            neg = (~pos) & (x < -t)
            return pos.astype(np.int8) - neg.astype(np.int8)
        return np.where(x < t, -1, 1).astype(np.int8)


def brute_pack(values, bitwidth):
    """Pack {-1,0,+1} values (..., C) into uint64 words (..., PC, bits), channel c -> word c//64,
    bit c%64, plane 0 = (value == -1), plane 1 = (value != 0)."""
    v = np.asarray(values)
    C = v.shape[-1]
    PC = (C + 63) // 64
    padded = np.zeros(v.shape[:-1] + (PC * 64,), dtype=np.int8)
    padded[..., :C] = v
    padded = padded.reshape(v.shape[:-1] + (PC, 64))
    weights = (np.uint64(1) << np.arange(64, dtype=np.uint64))
    sign = ((padded == -1).astype(np.uint64) * weights).sum(axis=-1, dtype=np.uint64)
    if bitwidth == 1:
        return sign[..., None].view(np.int64)
    nz = ((padded != 0).astype(np.uint64) * weights).sum(axis=-1, dtype=np.uint64)
    return np.stack([sign, nz], axis=-1).view(np.int64)


def unpack(q, C, bitwidth):
    """Inverse of brute_pack: int64 (..., PC, bits) -> values (..., C) in {-1,0,+1}."""
    q = np.ascontiguousarray(q).view(np.uint64)
    shifts = np.arange(64, dtype=np.uint64)
    bits = ((q[..., None] >> shifts) & np.uint64(1)).astype(np.int8)  # (..., PC, bits, 64)
    sign = bits[..., 0, :].reshape(q.shape[:-2] + (-1,))[..., :C]
    if bitwidth == 1:
        return (1 - 2 * sign).astype(np.int8)
    nz = bits[..., 1, :].reshape(q.shape[:-2] + (-1,))[..., :C]
    return (nz * (1 - 2 * sign)).astype(np.int8)


def torch_conv_reference(xq, wq, type, p1, p2, s1, s2, OH, OW):
    """Conv of dequantised tensors with torch: xq (N,H,W,C), wq (KN,KH,KW,C) in {-1,0,+1}.
    Padding value is 0 for ternary activations and +1 for binary ones (an all-zero packed
    word means +1 there).  Result cropped to the reference's (OH, OW) and laid out
    (n,oh,ow,kn) under an (N,KN,OH,OW) shape, like the reference's reshape."""
    x = torch.from_numpy(np.asarray(xq)).to(torch.float64).permute(0, 3, 1, 2)
    w = torch.from_numpy(np.asarray(wq)).to(torch.float64).permute(0, 3, 1, 2)
    pad_value = 0.0 if act_bits(type) == 2 else 1.0
    x = torch.nn.functional.pad(x, (p2, p2, p1, p1), value=pad_value)
    y = torch.nn.functional.conv2d(x, w, stride=(s1, s2))[:, :, :OH, :OW]
    N, KN = y.shape[0], y.shape[1]
    flat = y.permute(0, 2, 3, 1).contiguous().to(torch.float32)
    return flat.reshape(N, KN, OH, OW).numpy()
