"""Writes tests/golden/ref_golden.npz: inputs and outputs of the reference's own CPU functions
(TNN/TBN/BTN/BNN/DRF/RTNGEMM_baseline, TAB_CPU.cpp:242-383; Parallel_Img2Row_NHWCB_3x3,
TAB_CPU.h:27-63; Parallel_Ternarize_NCHWB_to_NHWCB, TAB_CPU.cpp:20-124), run from
oracle/_ref/libtab_ref.so, which oracle/Makefile compiles from /root/reference.

Run in the build container (needs /root/reference):  python tests/golden/make_ref_golden.py
The fixture holds data only, so the checks that use it also run where the reference tree
is absent.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def main():
    oracle.build()
    assert oracle.have_ref(), "oracle/_ref/libtab_ref.so was not built"
    rng = np.random.default_rng(20240607)
    out = {}
    # GEMMs: full 64-bit random words (sign bit 63 included), ragged M/N/K
    for t, (M, N, K) in zip(range(4), [(19, 7, 5), (23, 9, 3), (17, 11, 4), (21, 6, 7)]):
        pa = 2 if t < 2 else 1
        pb = 2 if t in (0, 2) else 1
        a = rng.integers(-2**63, 2**63 - 1, size=(M, K, pa), dtype=np.int64, endpoint=True)
        b = rng.integers(-2**63, 2**63 - 1, size=(N, K, pb), dtype=np.int64, endpoint=True)
        btn = rng.integers(0, 64 * K, size=N).astype(np.int32)
        num = 64 * K - 5
        out[f"gemm{t}_a"], out[f"gemm{t}_b"], out[f"gemm{t}_btn"] = a, b, btn
        out[f"gemm{t}_mnk_num"] = np.array([M, N, K, num], dtype=np.int64)
        out[f"gemm{t}_y"] = oracle.ref_gemm(t, a, b, M, N, K, btn, NUM=num)
    # im2row 3x3 over packed words, stride 1 and stride 2.  The stride-2 extents keep
    # (P - 3 + 1) divisible by the stride: the reference loops `for (w = 0; w < W-KW+1; w += s)`
    # (TAB_CPU.h:39-41), one step more than its own OW = (W-KW+1)/s otherwise, and then writes
    # past the end of its output vector.
    for name, (N, PH, PW, D, s1, s2) in {"i2r_s1": (2, 6, 7, 3, 1, 1), "i2r_s2": (2, 8, 10, 2, 2, 2)}.items():
        a = rng.integers(-2**63, 2**63 - 1, size=(N, PH, PW, D), dtype=np.int64, endpoint=True)
        out[name + "_a"] = a
        out[name + "_dims"] = np.array([N, PH, PW, D, 3, 3, s1, s2], dtype=np.int64)
        out[name + "_rows"] = oracle.ref_img2row_3x3(a, N, PH, PW, D, 3, 3, s1, s2)
    # ternarize: the reference steps to the next 64-channel block before reading
    # (TAB_CPU.cpp:59,92), so with one image and 64 leading filler channels it reads channels
    # 64..64+C-1 of the buffer; those are the logical input recorded here (NCHW).
    for name, (C, H, W, p1, p2, th) in {"ter_c70": (70, 3, 4, 1, 2, 0.4), "ter_c128": (128, 2, 3, 0, 1, 0.8)}.items():
        x = rng.standard_normal((C, H, W)).astype(np.float32)
        x[0, 0, 0], x[1, 0, 0], x[2, 0, 0] = th, -th, 0.0  # ties and zero
        buf = np.concatenate([np.full((64, H, W), 9.0, np.float32), x], axis=0)
        ths = np.array([th], dtype=np.float32)
        out[name + "_x_chw"] = x
        out[name + "_dims"] = np.array([C, H, W, p1, p2], dtype=np.int64)
        out[name + "_th"] = ths
        out[name + "_q"] = oracle.ref_ternarize_nchw(buf, p1, p2, ths, 1, C, H, W)
    # binarize (sign, TAB_CPU.cpp:177): same reading pattern; whole 64-channel blocks only,
    # because the tail loop reads from the start of the buffer instead (TAB_CPU.cpp:193)
    C, H, W, p1, p2 = 128, 3, 2, 1, 1
    x = rng.standard_normal((C, H, W)).astype(np.float32)
    x[0, 0, 0], x[1, 0, 0] = 0.0, -0.0
    buf = np.concatenate([np.full((64, H, W), 9.0, np.float32), x], axis=0)
    out["bin_c128_x_chw"] = x
    out["bin_c128_dims"] = np.array([C, H, W, p1, p2], dtype=np.int64)
    out["bin_c128_q"] = oracle.ref_binarize_nchw(buf, p1, p2, 1, C, H, W)
    # the CPU-only GEMMs (types 4 and 5), drawn last so that the vectors above keep their values
    for t, (M, N, K) in zip((4, 5), [(18, 5, 6), (20, 8, 5)]):
        planes = 2 if t == 4 else 1
        a = rng.integers(-2**63, 2**63 - 1, size=(M, K, planes), dtype=np.int64, endpoint=True)
        b = rng.integers(-2**63, 2**63 - 1, size=(N, K, planes), dtype=np.int64, endpoint=True)
        out[f"gemm{t}_a"], out[f"gemm{t}_b"] = a, b
        out[f"gemm{t}_mnk_num"] = np.array([M, N, K, 0], dtype=np.int64)
        out[f"gemm{t}_y"] = oracle.ref_gemm(t, a, b, M, N, K)
    path = os.path.join(HERE, "ref_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
