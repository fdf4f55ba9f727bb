"""Times every matrix-core workgroup shape (tab_set_conv_kernel(TAB_CONV_MATRIX, 0..6)) on sets of layers and prints one
line per (type, layer): the durations in microseconds, median of three rounds taken round-robin over the shapes with the
clock warmed.  Needs an MI355X.  The output, concatenated over the sets, is conv_shape_timings.txt, which
fit_conv_shape_model.py turns into tab_amd/csrc/tab_conv_shape_model.h.

    python tab_amd/tuning/collect_conv_shape_timings.py <set> [types, default 3,0,1,2]  >> conv_shape_timings.txt

sets: rn16 / rn64 / rn256 (the ResNet-18 layers at that batch), vgg (N=32), sweep (28x28, C = 256 / 512, N = 64 and 256),
sweep128, other1, other2 (layers of other geometries: channel counts that are no power of two, 5x5, odd sizes)."""
import os
import statistics
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
import torch  # noqa: E402

import tab_amd as tab  # noqa: E402
from bench import RESNET18_LAYERS, Layer, graph_time_ms, layer_name  # noqa: E402

SWEEP = [(256, 3, 1, 1, 0), (512, 3, 2, 1, 0), (512, 1, 1, 0, 0), (256, 1, 2, 1, 0), (512, 3, 1, 1, 1)]
SETS = {
    "rn16": [(16, l) for l in RESNET18_LAYERS],
    "rn64": [(64, l) for l in RESNET18_LAYERS],
    "rn256": [(256, l) for l in RESNET18_LAYERS],
    "vgg": [(32, (hw, hw, c, c, 3, 3, 1, 1, 1, 1)) for hw, c in [(224, 64), (112, 128), (56, 256), (28, 512), (14, 512)]],
    "sweep": [(n, (28, 28, c, c, k, k, p1, p2, s, s)) for n in (64, 256) for (c, k, s, p1, p2) in SWEEP],
    "sweep128": [(128, (28, 28, c, c, k, k, p1, p2, s, s)) for (c, k, s, p1, p2) in SWEEP + [(256, 3, 2, 1, 1), (256, 3, 1, 1, 1)]],
    "other1": [(48, (40, 40, 384, 384, 3, 3, 1, 1, 1, 1)), (200, (20, 20, 640, 320, 3, 3, 1, 1, 1, 1)),
               (96, (32, 32, 256, 128, 3, 3, 1, 1, 2, 2)), (24, (64, 64, 128, 256, 3, 3, 1, 1, 1, 1)),
               (512, (14, 14, 512, 512, 1, 1, 0, 0, 1, 1)), (8, (96, 96, 128, 128, 5, 5, 2, 2, 1, 1)),
               (100, (24, 24, 768, 192, 3, 3, 0, 0, 1, 1)), (40, (36, 36, 256, 1024, 1, 1, 0, 0, 1, 1))],
    "other2": [(64, (20, 20, 512, 384, 3, 3, 1, 1, 1, 1)), (12, (80, 80, 128, 128, 3, 3, 1, 1, 1, 1)),
               (160, (16, 16, 384, 640, 3, 3, 1, 1, 1, 1)), (32, (48, 48, 256, 256, 3, 3, 1, 1, 2, 2)),
               (300, (10, 10, 1024, 256, 3, 3, 1, 1, 1, 1)), (6, (128, 128, 128, 64, 3, 3, 1, 1, 1, 1)),
               (72, (30, 30, 128, 512, 1, 1, 0, 0, 1, 1)), (20, (50, 50, 384, 192, 3, 3, 1, 1, 1, 1)),
               (128, (12, 12, 768, 768, 3, 3, 1, 1, 1, 1)), (4, (60, 60, 256, 320, 3, 3, 1, 1, 1, 1))],
}


def main():
    which = sys.argv[1]
    types = [int(t) for t in (sys.argv[2] if len(sys.argv) > 2 else "3,0,1,2").split(",")]
    shapes = list(range(7))
    print(f"## {which}")
    try:
        for type in types:
            for N, layer in SETS[which]:
                L = Layer(tab, torch, type, N, layer, seed=1, on_device=True)
                t = {s: [] for s in shapes}
                for rnd in range(4):  # the first round warms up
                    for s in shapes:
                        tab.set_conv_kernel(tab.CONV_MATRIX, s)
                        ms = graph_time_ms(torch, L.conv_kernel_only, 6 if N > 16 else 20, replays=3)
                        if rnd:
                            t[s].append(ms)
                print(f"type {type} {layer_name(N, layer):38s} | " + " ".join(f"{s}:{statistics.median(t[s]) * 1e3:.1f}" for s in shapes),
                      flush=True)
                del L
    finally:
        tab.set_conv_kernel(tab.CONV_AUTO, -1)


if __name__ == "__main__":
    main()
