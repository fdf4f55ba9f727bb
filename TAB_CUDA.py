"""Drop-in for the reference's CUDA module: `import TAB_CUDA as TAB` (TAB Demo CUDA.ipynb,
cell 1; module name from Setup_CUDA.py:9) resolves to the MI355X implementation.

    QW, BTN_W = TAB.Quantize(w.cuda(), w_ths.cuda(), bitwidth, KN, KH, KW, KC)
    y = TAB.Conv2d(x.cuda(), QW, x_ths.cuda(), BTN_W, conv_type, pad1, pad2, str1, str2, N, H, W, C, KN, KH, KW)

The functions are the pybind11 entry points of the C++ extension tab_amd/_C
(tab_amd/csrc/torch_binding.cpp).  There is no fallback: if the extension or libtab_amd.so is
not built, the import fails.
"""
try:
    from tab_amd._C import Conv2d, Quantize  # noqa: F401
    # beyond the reference's two functions: the same C ABI, same conventions
    from tab_amd._C import (Conv2dPacked, Conv2dPackedOut, QuantizeFormat, QuantizeNCHW,  # noqa: F401
                            TAB_Conv2d, TAB_Quantize, Threshold)
except ImportError as exc:  # pragma: no cover
    raise ImportError(
        "tab_amd/_C is not built; run `python -c 'import __graft_entry__ as g; g.build()'` first"
    ) from exc

__all__ = ["Conv2d", "Quantize", "TAB_Conv2d", "TAB_Quantize", "QuantizeNCHW", "QuantizeFormat", "Threshold",
           "Conv2dPacked", "Conv2dPackedOut"]
