"""ctypes binding of the C ABI declared in include/tab_amd.h.

The library is the only compute path: if it is missing or fails to load, importing this
module raises, and nothing here falls back to another implementation.
"""
import ctypes
import os

from .build import LIB_PATH

_vp, _int, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/tab_amd.h one to one
SIGNATURES = {
    "tab_status_string": (ctypes.c_char_p, [_int]),
    "tab_last_error": (ctypes.c_char_p, []),
    "tab_version": (ctypes.c_char_p, []),
    "tab_packed_channels": (_int, [_int]),
    "tab_operand_words": (_int, [_int] * 3),
    "tab_out_extent": (_int, [_int] * 4),
    "tab_quantize": (_int, [_vp, _vp, _int, _int, _int, _int, _int, _vp, _vp, _vp]),
    "tab_quantize_nchw": (_int, [_vp, _vp, _int, _int, _int, _int, _int, _vp, _vp, _vp]),
    "tab_quantize_format": (_int, [_vp, _vp, _int, _int, _int, _int, _int, _vp, _vp]),
    "tab_threshold_workspace_bytes": (_sz, [_int, ctypes.c_long]),
    "tab_threshold": (_int, [_vp, _int, ctypes.c_long, ctypes.c_float, _vp, _vp, _sz, _vp]),
    "tab_conv2d_workspace_bytes": (_sz, [_int] * 5),
    "tab_conv2d": (_int, [_vp] * 4 + [_int] * 12 + [_vp, _vp, _sz, _vp]),
    "tab_conv2d_launches": (_int, [_vp] + [_int] * 12),
    "tab_static_scratch_bytes": (_sz, []),
    "tab_conv2d_static": (_int, [_vp] * 4 + [_int] * 12 + [_vp, _vp]),
    "tab_conv2d_packed": (_int, [_vp] * 3 + [_int] * 12 + [_vp, _vp]),
    "tab_conv2d_packed_out": (_int, [_vp] * 3 + [_int] * 12 + [_vp, _int, _vp, _vp]),
    "tab_set_conv_kernel": (_int, [_int, _int]),
}


def load(path=LIB_PATH):
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `python -m tab_amd.build`) first. There is no fallback implementation.")
    lib = ctypes.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


class TabError(RuntimeError):
    """A C ABI call returned a negative tab_status."""


def check(lib, status):
    if status != 0:
        name = lib.tab_status_string(status).decode()
        raise TabError(f"{name}: {lib.tab_last_error().decode()}")
