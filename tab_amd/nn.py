"""Layer wrappers around the two operators: the caller the reference's demo notebook gestures
at (it imports torch.nn and autograd.Function, TAB Demo CUDA.ipynb cell 1, but ships none).
Inference only (the operators have no backward).

    layer = TABConv2d.from_float(weight_kn_c_kh_kw, conv_type=tab_amd.TNN, stride=1, padding=1)
    y = layer(x)            # x: (N, C, H, W) fp32 on the GPU -> (N, KN, OH, OW), logical NCHW
"""
import torch
from torch import nn

from . import (BNN, BTN, TBN, TNN, Conv2d, Conv2dPacked, Conv2dPackedOut, Quantize, QuantizeActivation, Threshold,
               out_shape)

_ACT_BITS = {TNN: 2, TBN: 2, BTN: 1, BNN: 1}
_WEIGHT_BITS = {TNN: 2, TBN: 1, BTN: 2, BNN: 1}


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else (int(v[0]), int(v[1]))


class TABConv2d(nn.Module):
    """2-D convolution with ternary/binary activations and weights.  Holds the packed weights
    (QW) and the BTN popcounts as buffers; the activation threshold is `act_scale * mean|x|` per
    image for ternary activations and 0 for binary ones.  `data_format` is the layout of the
    input and of the returned tensor: "NCHW" (PyTorch's; quantized directly from that layout, the
    result a permuted view of the operators' NHWC output) or "NHWC"."""

    def __init__(self, QW, BTN_W, conv_type, in_channels, out_channels, kernel_size, stride=1, padding=0,
                 act_scale=0.7, data_format="NCHW"):
        super().__init__()
        if conv_type not in _ACT_BITS:
            raise ValueError("conv_type must be 0 (TNN), 1 (TBN), 2 (BTN) or 3 (BNN)")
        if data_format not in ("NCHW", "NHWC"):
            raise ValueError("data_format must be 'NCHW' or 'NHWC'")
        self.conv_type = int(conv_type)
        self.in_channels, self.out_channels = int(in_channels), int(out_channels)
        self.kernel_size, self.stride, self.padding = _pair(kernel_size), _pair(stride), _pair(padding)
        self.act_scale, self.data_format = float(act_scale), data_format
        self.register_buffer("QW", QW)
        self.register_buffer("BTN_W", BTN_W)

    @classmethod
    def from_float(cls, weight, conv_type, stride=1, padding=0, weight_scale=0.7, act_scale=0.7, data_format="NCHW"):
        """Quantize an fp32 weight of PyTorch's shape (KN, C, KH, KW) on the GPU: ternary weights
        use the threshold weight_scale * mean|w| per filter, binary weights the sign."""
        KN, C, KH, KW = weight.shape
        w = weight.detach().to(torch.float32).permute(0, 2, 3, 1).contiguous().cuda()  # (KN,KH,KW,C)
        bits = _WEIGHT_BITS[conv_type]
        ths = Threshold(w, KN, weight_scale) if bits == 2 else torch.zeros(KN, device=w.device)
        QW, BTN_W = Quantize(w, ths, bits, KN, KH, KW, C)
        return cls(QW, BTN_W, conv_type, C, KN, (KH, KW), stride, padding, act_scale, data_format)

    def forward(self, x):
        nchw = self.data_format == "NCHW"
        if nchw:
            N, C, H, W = x.shape
        else:
            N, H, W, C = x.shape
        if C != self.in_channels:
            raise RuntimeError(f"expected {self.in_channels} input channels, got {C}")
        x = x.to(torch.float32).contiguous()
        abits = _ACT_BITS[self.conv_type]
        if abits == 2:
            ths = Threshold(x, N, self.act_scale)  # mean|x| per image: the same in either layout
        else:
            ths = torch.zeros(N, dtype=torch.float32, device=x.device)
        (KH, KW), (s1, s2), (p1, p2) = self.kernel_size, self.stride, self.padding
        if nchw:
            # quantized straight from NCHW (no transposed fp32 copy), then the packed entry point
            QX = QuantizeActivation(x, ths, abits, N, H, W, C, nchw=True)  # no BTN vector: nobody reads an activation's
            y = Conv2dPacked(QX, self.QW, self.BTN_W, self.conv_type, p1, p2, s1, s2, N, H, W, C,
                             self.out_channels, KH, KW)
        else:
            y = Conv2d(x, self.QW, ths, self.BTN_W, self.conv_type, p1, p2, s1, s2, N, H, W, C,
                       self.out_channels, KH, KW)
        OH, OW = out_shape(H, W, KH, KW, p1, p2, s1, s2)
        # the operator's (N,KN,OH,OW)-shaped result is (n,oh,ow,kn) in memory (TAB_GEMM.cu:526)
        y = y.view(N, OH, OW, self.out_channels)
        return y.permute(0, 3, 1, 2) if self.data_format == "NCHW" else y

    def extra_repr(self):
        names = {TNN: "TNN", TBN: "TBN", BTN: "BTN", BNN: "BNN"}
        return (f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}, stride={self.stride}, "
                f"padding={self.padding}, type={names[self.conv_type]}, data_format={self.data_format}")


class TABLinear(nn.Module):
    """Fully connected layer as a 1x1 convolution on a 1x1 image ("FC equals to 1x1 conv",
    TAB_CPU.cpp:487-488).  Input (N, in_features), output (N, out_features)."""

    def __init__(self, conv):
        super().__init__()
        self.conv = conv

    @classmethod
    def from_float(cls, weight, conv_type, weight_scale=0.7, act_scale=0.7):
        out_features, in_features = weight.shape
        conv = TABConv2d.from_float(weight.reshape(out_features, in_features, 1, 1), conv_type, 1, 0,
                                    weight_scale, act_scale, data_format="NHWC")
        return cls(conv)

    def forward(self, x):
        N, F = x.shape
        return self.conv(x.reshape(N, 1, 1, F)).reshape(N, self.conv.out_channels)


class TABPackedChain(nn.Module):
    """A stack of TABConv2d layers run packed-in / packed-out: the input is quantized once, every
    layer but the last writes its output already thresholded and packed for the next layer (no fp32
    activation between layers), the last one returns fp32.  A layer's output channels must be the
    next layer's input channels.

    The threshold applied to a layer's output is the next layer's activation threshold: 0 when the
    next layer takes binary activations (types BTN, BNN) - then the chain returns exactly what
    calling the layers one after the other returns - and, when it takes ternary activations, the
    calibrated constant given in `ternary_thresholds[i]` for layer i+1 (the per-image
    `act_scale * mean|y|` of an unchained TABConv2d needs the fp32 tensor this class avoids)."""

    def __init__(self, layers, ternary_thresholds=None, data_format="NCHW"):
        super().__init__()
        self.layers = nn.ModuleList(layers)
        if not self.layers:
            raise ValueError("at least one layer")
        for a, b in zip(self.layers[:-1], self.layers[1:]):
            if a.out_channels != b.in_channels:
                raise ValueError(f"{a.out_channels} output channels feed a layer with {b.in_channels} input channels")
        self.ternary_thresholds = dict(ternary_thresholds or {})
        for i, layer in enumerate(self.layers[1:], start=1):
            if _ACT_BITS[layer.conv_type] == 2 and i not in self.ternary_thresholds:
                raise ValueError(f"layer {i} takes ternary activations: give ternary_thresholds[{i}]")
        if data_format not in ("NCHW", "NHWC"):
            raise ValueError("data_format must be 'NCHW' or 'NHWC'")
        self.data_format = data_format

    def forward(self, x):
        nchw = self.data_format == "NCHW"
        if nchw:
            N, C, H, W = x.shape
        else:
            N, H, W, C = x.shape
        first = self.layers[0]
        if C != first.in_channels:
            raise RuntimeError(f"expected {first.in_channels} input channels, got {C}")
        x = x.to(torch.float32).contiguous()
        bits = _ACT_BITS[first.conv_type]
        ths = Threshold(x, N, first.act_scale) if bits == 2 else torch.zeros(N, dtype=torch.float32, device=x.device)
        q = QuantizeActivation(x, ths, bits, N, H, W, C, nchw=nchw)
        for i, layer in enumerate(self.layers):
            (KH, KW), (s1, s2), (p1, p2) = layer.kernel_size, layer.stride, layer.padding
            args = (layer.conv_type, p1, p2, s1, s2, N, H, W, layer.in_channels, layer.out_channels, KH, KW)
            OH, OW = out_shape(H, W, KH, KW, p1, p2, s1, s2)
            if i + 1 == len(self.layers):
                y = Conv2dPacked(q, layer.QW, layer.BTN_W, *args).view(N, OH, OW, layer.out_channels)
                return y.permute(0, 3, 1, 2) if self.data_format == "NCHW" else y
            next_bits = _ACT_BITS[self.layers[i + 1].conv_type]
            out_ths = torch.full((N,), float(self.ternary_thresholds.get(i + 1, 0.0)), dtype=torch.float32, device=x.device)
            q = Conv2dPackedOut(q, layer.QW, layer.BTN_W, *args, out_ths, next_bits)
            H, W = OH, OW
