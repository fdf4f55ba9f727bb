"""Fits the cost model conv_mfma_shape() chooses the workgroup shape with and writes tab_amd/csrc/tab_conv_shape_model.h.

Input: conv_shape_training_timings.txt, the model's training data: per (type, layer) the measured duration in microseconds of
every shape on one MI355X (median of three rounds taken round-robin over the shapes, clock warmed; conv kernel alone,
tab_set_conv_kernel(TAB_CONV_MATRIX, shape)).
Model, per (type, shape): duration ~ c . f with the features
    f = [G*n, G*rounds, rounds, n, Y, Y*busy, busy, 1, Y*[G <= 9]]
    tiles  = ceil(M / BM) * ceil(KN / BN)            workgroups of the launch
    n      = ceil(tiles / 256)                       tiles on the busiest of the 256 CUs
    rounds = ceil(n / workgroups a CU holds)         how often that CU is refilled
    busy   = min(1, tiles / 256)                     share of the CUs that have work at all
    G      = KH*KW*PC words of K, Y = 4*M*KN bytes / 1e6; the last feature gives the layers whose loop is a handful of
             MFMAs (C = 64 with 3x3, 1x1) their own price per byte of Y: their launches are the epilogue
The mixed launches (shape 10: 128x128 tiles for the whole rounds of the chip, 64x64 split-K quarters for the rest; shape 11:
the same with 128x256 tiles, eight quarters to a tile, words per pixel in fours) have
    f = [G*whole, G*quarters, quarters, whole, Y, Y, 1, 1, Y*[G <= 9]]
    whole    = floor(tiles / 256)                    whole tiles on every CU
    quarters = ceil(4 * (tiles mod 256) / 256)       quarter tiles on the busiest CU after them
and are candidates where both are positive, the words per pixel are even in number and K words x bit planes of the two
operands exceed 36 (the work per byte of Y grows with K and with the planes to expand alone; below that the launch is bound
by writing Y and gains nothing from a better balanced last round: BNN N=256 28x28x128->256 3x3 stride 2, K = 18 words,
16.1 us mixed or plain against 13.9 with 128x64 tiles, where the ternary types gain 6-10 %).
fitted by NON-NEGATIVE least squares on relative error (the N=16 set weighted threefold): every feature is non-negative and
so is every coefficient, hence a predicted duration is positive and grows with K, with the tiles on the busiest CU and
with Y for every geometry, inside the fitted range or far outside it (an unconstrained fit had coefficients of both signs,
whose predictions can cross or go negative where nothing was measured).  A shape whose filter tile is at least twice the
(64-rounded) filter count is not a candidate.  The script prints the regret of the model's choice against the best measured shape:
fitted on everything, and with each set held out in turn.

    python tab_amd/tuning/fit_conv_shape_model.py        # needs numpy only"""
import collections
import os
import re

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
# shape id -> rows x filters of the workgroup tile, workgroups a CU holds (the occupancy the compiler reports for the
# shape's kernels with four-word chunks: registers, or LDS where that is the tighter limit)
SHAPES = {0: (128, 128, 4), 1: (128, 64, 6), 2: (64, 64, 8), 3: (32, 32, 4), 4: (256, 64, 4), 5: (256, 128, 2), 6: (128, 256, 2),
          8: (64, 64, 4), 9: (128, 128, 2), 10: (128, 128, 4), 11: (128, 256, 2)}
MIXED = (10, 11)
PLANES = {0: 4, 1: 3, 2: 3, 3: 2}  # bit planes of activation + weight operand, per type
IDS = sorted(SHAPES)
NFEAT = 9


def parse(path):
    rows, which = [], None
    for line in open(path):
        if line.startswith("##"):
            which = line.split()[1]
            continue
        m = re.match(r"type (\d) N(\d+)_(\d+)x(\d+)x(\d+)->(\d+)_k(\d+)x(\d+)_p(\d)(\d)_s(\d)(\d)\s+\| (.*)", line)
        if not m:
            continue
        t, N, H, W, C, KN, kh, kw, p1, p2, s1, s2 = map(int, m.groups()[:12])
        OH, OW = (H + 2 * p1 - kh + 1) // s1, (W + 2 * p2 - kw + 1) // s2  # TAB_GEMM.cu:354-357
        times = {int(a.split(":")[0]): float(a.split(":")[1]) for a in m.group(13).split()}
        rows.append(dict(set=which, type=t, M=N * OH * OW, KN=KN, G=kh * kw * ((C + 63) // 64), PC=(C + 63) // 64, times=times,
                         name=line.split()[2]))
    return rows


def mixed_rounds(r, s):
    BM, BN, _ = SHAPES[s]
    tiles = -(-r["M"] // BM) * -(-r["KN"] // BN)
    return tiles // 256, -(-(BM // 64 * (BN // 64)) * (tiles % 256) // 256)


def eligible(r, s):
    # (the split-K shapes need an even number of words per pixel; otherwise they run as shapes 2 and 0)
    if s in MIXED and (r["G"] * PLANES[r["type"]] <= 36 or 0 in mixed_rounds(r, s) or (s == 11 and r["PC"] % 4)):
        return False
    return SHAPES[s][1] < 2 * (-(-r["KN"] // 64) * 64) and s in r["times"] and not (s >= 8 and r["PC"] % 2)


def features(r, s):
    BM, BN, held = SHAPES[s]
    Y = r["M"] * r["KN"] * 4e-6
    if s in MIXED:
        whole, quarters = mixed_rounds(r, s)
        return [r["G"] * whole, r["G"] * quarters, quarters, whole, Y, Y, 1.0, 1.0, Y if r["G"] <= 9 else 0.0]
    tiles = -(-r["M"] // BM) * -(-r["KN"] // BN)
    n = -(-tiles // 256)
    rounds = -(-n // held)
    busy = min(1.0, tiles / 256.0)
    return [r["G"] * n, r["G"] * rounds, rounds, n, Y, Y * busy, busy, 1.0, Y if r["G"] <= 9 else 0.0]


def fit(rows):
    from scipy.optimize import nnls

    coef = {}
    for s in SHAPES:
        for t in range(4):
            X = np.array([features(r, s) for r in rows if r["type"] == t and eligible(r, s)])
            y = np.array([r["times"][s] for r in rows if r["type"] == t and eligible(r, s)])
            w = 1.0 / np.maximum(y, 1.0)  # relative error; the latency-bound N=16 set, the benchmark's headline, counts threefold
            w = w * np.array([3.0 if r["set"] == "rn16" else 1.0 for r in rows if r["type"] == t and eligible(r, s)])
            coef[(t, s)] = nnls(X * w[:, None], y * w)[0]
    return coef


def choose(coef, r):
    return min((s for s in SHAPES if eligible(r, s)), key=lambda s: (float(coef[(r["type"], s)] @ np.array(features(r, s))), s))


def best_time(r):
    return min(v for s, v in r["times"].items() if eligible(r, s))


def regret(rows, coef):
    chosen = best = 0.0
    per = collections.defaultdict(lambda: [0.0, 0.0])
    for r in rows:
        c, b = r["times"][choose(coef, r)], best_time(r)
        chosen += c
        best += b
        per[r["set"]][0] += c
        per[r["set"]][1] += b
    return chosen / best - 1, {k: v[0] / v[1] - 1 for k, v in per.items()}


def main():
    rows = parse(os.path.join(HERE, "conv_shape_training_timings.txt"))
    coef = fit(rows)
    total, per = regret(rows, coef)
    sets = sorted(per)
    held_chosen = held_best = 0.0
    held = {}
    for hold in sets:
        c = fit([r for r in rows if r["set"] != hold])
        g, _ = regret([r for r in rows if r["set"] == hold], c)
        held[hold] = g
        for r in rows:
            if r["set"] == hold:
                held_chosen += r["times"][choose(c, r)]
                held_best += best_time(r)
    print(f"{len(rows)} cases; regret of the model's choice, fitted on all: {total:.2%} ({', '.join(f'{k} {v:.1%}' for k, v in sorted(per.items()))})")
    print(f"each set held out of the fit in turn: {held_chosen / held_best - 1:.2%} ({', '.join(f'{k} {v:.1%}' for k, v in sorted(held.items()))})")
    out = os.path.join(os.path.dirname(HERE), "csrc", "tab_conv_shape_model.h")
    import datetime
    import subprocess

    commit = subprocess.run(["git", "-C", HERE, "rev-parse", "--short", "HEAD"], stdout=subprocess.PIPE, text=True).stdout.strip() or "unknown"
    with open(out, "w") as f:
        f.write("// Written by tab_amd/tuning/fit_conv_shape_model.py from tab_amd/tuning/conv_shape_training_timings.txt: do not edit.\n")
        f.write(f"// Fitted {datetime.date.today().isoformat()} on the kernels of commit {commit} (and the working tree on top of it).\n")
        f.write("// Cost model of the matrix-core workgroup shapes: predicted duration (us) = kConvShapeCost[type][i] . f for the shape\n")
        f.write("// kConvShapeIds[i], f = {G*n, G*rounds, rounds, n, Y, Y*busy, busy, 1, Y*[G <= 9]} (n = tiles on the busiest CU,\n")
        f.write("// rounds = refills of that CU, Y = megabytes of output, busy = share of the CUs with work; shapes 10 and 11, the mixed launches:\n")
        f.write("// {G*whole, G*quarters, quarters, whole, Y, Y, 1, 1, Y*[G <= 9]}, whole tiles per CU and quarter tiles after them).  Non-negative least squares:\n")
        f.write("// every feature and every coefficient is >= 0, so a prediction is positive and monotone for any geometry.  Regret of the\n")
        f.write(f"// choice against the best measured shape over the {len(rows)} fitted cases: {total:.2%}; with each layer set held out of\n")
        f.write(f"// the fit in turn: {held_chosen / held_best - 1:.2%}.\n")
        f.write("#pragma once\n\nnamespace tab {\n\n")
        f.write(f"constexpr int kConvShapes = {len(IDS)}, kConvShapeFeatures = {NFEAT};\n")
        f.write("// the shape ids tab_set_conv_kernel(TAB_CONV_MATRIX, id) takes, in the order of the tables below\n")
        f.write("constexpr int kConvShapeIds[kConvShapes] = {" + ", ".join(str(i) for i in IDS) + "};\n")
        f.write("// rows x filters of the workgroup tile and workgroups a CU holds (compiled occupancy), per shape\n")
        f.write("constexpr int kConvShapeTile[kConvShapes][3] = {" + ", ".join("{%d, %d, %d}" % SHAPES[s] for s in IDS) + "};\n")
        f.write("constexpr float kConvShapeCost[4][kConvShapes][kConvShapeFeatures] = {\n")
        for t in range(4):
            f.write("    {\n")
            for s_ in IDS:
                f.write("        {" + ", ".join(("%.6g" % v if "." in "%.6g" % v or "e" in "%.6g" % v else "%.6g.0" % v) + "f" for v in coef[(t, s_)]) + "},\n")
            f.write("    },\n")
        f.write("};\n\n}  // namespace tab\n")
    print("wrote", out)


if __name__ == "__main__":
    main()
