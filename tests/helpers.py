"""Shared input builders and independent references for the tests.

Nothing here restates the oracle's C code: `dequantize_*` and `torch_conv_reference` go
through torch.nn.functional.conv2d on {-1,0,+1} tensors, and `brute_*` are per-element
closed forms in numpy.
"""
import numpy as np
import torch

TYPE_NAMES = {0: "TNN", 1: "TBN", 2: "BTN", 3: "BNN", 4: "DRF", 5: "RTN"}


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


# ---- the CPU-only types: DoReFa 2-bit levels (4) and RTN 2-bit fields (5) -------------------
def brute_levels(x, ths):
    """Levels 0..3 of the uniform quantizer with step ths[n]: bounds 0.5t, 1.5t, 2.5t in fp32."""
    x = np.asarray(x, dtype=np.float32)
    t = np.asarray(ths, dtype=np.float32)[: x.shape[0]].reshape((-1,) + (1,) * (x.ndim - 1))
    with np.errstate(invalid="ignore"):
        return ((x >= np.float32(0.5) * t).astype(np.int8) + (x >= np.float32(1.5) * t) + (x >= np.float32(2.5) * t)).astype(np.int8)


def _pack_bits(bits, per_word):
    """bits (..., L) of 0/1 -> uint64 words (..., ceil(L/per_word)), bit i of a word = element i."""
    L = bits.shape[-1]
    nw = (L + per_word - 1) // per_word
    padded = np.zeros(bits.shape[:-1] + (nw * per_word,), dtype=np.uint64)
    padded[..., :L] = bits
    padded = padded.reshape(bits.shape[:-1] + (nw, per_word))
    return (padded << np.arange(per_word, dtype=np.uint64)).sum(axis=-1, dtype=np.uint64)


def pack_drf(levels):
    """Levels (..., C) in 0..3 -> int64 (..., PC, 2): plane 0 the weight-2 bit, plane 1 the weight-1 bit."""
    lv = np.asarray(levels).astype(np.uint64)
    return np.stack([_pack_bits(lv >> np.uint64(1), 64), _pack_bits(lv & np.uint64(1), 64)], axis=-1).view(np.int64)


def pack_rtn(values):
    """Values (..., C) in {-1,0,+1} -> int64 (..., ceil(C/32)): field c%32 of word c//32, even bit =
    nonzero, odd bit = sign."""
    v = np.asarray(values)
    fields = np.stack([(v != 0), (v < 0)], axis=-1).astype(np.uint64).reshape(v.shape[:-1] + (-1,))
    return _pack_bits(fields, 64).view(np.int64)


def unpack_drf(q, C):
    """int64 (..., PC, 2) -> levels (..., C): 2 * plane 0 + plane 1, any bit pattern."""
    q = np.ascontiguousarray(q).view(np.uint64)
    bits = ((q[..., None] >> np.arange(64, dtype=np.uint64)) & np.uint64(1)).astype(np.int8)
    hi = bits[..., 0, :].reshape(q.shape[:-2] + (-1,))[..., :C]
    lo = bits[..., 1, :].reshape(q.shape[:-2] + (-1,))[..., :C]
    return (2 * hi + lo).astype(np.int8)


def unpack_rtn(q, C):
    """int64 (..., PC32) -> values (..., C): nonzero bit * (1 - 2 * sign bit), any bit pattern."""
    q = np.ascontiguousarray(q).view(np.uint64)
    bits = ((q[..., None] >> np.arange(64, dtype=np.uint64)) & np.uint64(1)).astype(np.int8)
    bits = bits.reshape(q.shape[:-1] + (-1, 2))[..., :C, :]
    return (bits[..., 0] * (1 - 2 * bits[..., 1])).astype(np.int8)


def torch_conv_reference(xq, wq, type, p1, p2, s1, s2, OH, OW):
    """Conv of dequantised tensors with torch: xq (N,H,W,C), wq (KN,KH,KW,C) in {-1,0,+1}.
    Padding value is 0 for ternary activations and +1 for binary ones (an all-zero packed
    word means +1 there).  Result cropped to the reference's (OH, OW) and laid out
    (n,oh,ow,kn) under an (N,KN,OH,OW) shape, like the reference's reshape."""
    x = torch.from_numpy(np.asarray(xq)).to(torch.float64).permute(0, 3, 1, 2)
    w = torch.from_numpy(np.asarray(wq)).to(torch.float64).permute(0, 3, 1, 2)
    pad_value = 1.0 if type in (2, 3) else 0.0
    x = torch.nn.functional.pad(x, (p2, p2, p1, p1), value=pad_value)
    y = torch.nn.functional.conv2d(x, w, stride=(s1, s2))[:, :, :OH, :OW]
    N, KN = y.shape[0], y.shape[1]
    flat = y.permute(0, 2, 3, 1).contiguous().to(torch.float32)
    return flat.reshape(N, KN, OH, OW).numpy()
