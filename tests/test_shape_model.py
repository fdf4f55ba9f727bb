"""The cost model that picks the matrix-core workgroup shape (tab_conv_shape_model.h, conv_mfma_shape), on the host:
over a wide grid of geometries, far outside what it was fitted on, every choice is a shape the launch can run and every
predicted duration is positive, finite and no smaller when K grows."""
import ctypes
import itertools
import math

from tab_amd import _capi

TILE = {0: (128, 128), 1: (128, 64), 2: (64, 64), 3: (32, 32), 4: (256, 64), 5: (256, 128), 6: (128, 256), 8: (64, 64), 9: (128, 128), 10: (128, 128), 11: (128, 256)}


def _hook():
    lib = ctypes.CDLL(_capi.LIB_PATH)
    f = lib.tab_internal_conv_shape
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_int] * 6 + [ctypes.POINTER(ctypes.c_float)]
    return f


def _choose(f, type, M, KN, G, PC, packed):
    cost = ctypes.c_float(-1.0)
    return f(type, M, KN, G, PC, packed, ctypes.byref(cost)), cost.value


def test_every_choice_is_legal_and_priced_positive():
    f = _hook()
    Ms = [1, 31, 1024, 12544, 50176, 200704, 1605632, 4096 * 56 * 56, 2**31 - 600]
    KNs = [1, 63, 64, 100, 512, 1000, 2048, 4096]
    Ks = [(1, 1), (2, 2), (9, 1), (18, 2), (27, 3), (72, 8), (144, 16), (4096, 64), (65535, 65535)]  # (G, PC)
    for type, M, KN, (G, PC), packed in itertools.product(range(6), Ms, KNs, Ks, (0, 1)):
        if packed and type > 3:
            continue
        shape, cost = _choose(f, type, M, KN, G, PC, packed)
        what = (type, M, KN, G, PC, packed, shape, cost)
        if shape == 7:
            assert type <= 3 and G <= 9 and packed, what
            continue
        assert shape in TILE, what
        bn = TILE[shape][1]
        assert bn < 2 * ((KN + 63) // 64 * 64), what          # a filter tile under twice the filters
        assert not (packed and shape == 3), what              # packed output needs 64-filter tiles
        assert not (shape >= 8 and PC % 2), what              # split-K shapes: an even number of words per pixel
        assert not (shape in (10, 11) and (G <= 9 or M * KN < 128 * 128 * 2)), what
        assert not (shape == 11 and PC % 4), what   # the mixed launch: a long K, more than a round
        assert math.isfinite(cost) and cost > 0.9, what       # never below a launch


def test_predicted_duration_grows_with_k():
    f = _hook()
    for type, M, KN in itertools.product((0, 3), (784, 50176, 1605632, 10**8), (64, 512, 4096)):
        last = 0.0
        for taps in (1, 4, 9, 25, 49, 400, 4000):
            _, cost = _choose(f, type, M, KN, taps * 8, 8, 0)
            assert cost >= last, (type, M, KN, taps, cost, last)
            last = cost


def test_choice_on_the_training_cases_stays_within_the_stated_regret():
    """The compiled chooser (256 compute units where no device is present, as on the box the timings come from) on the model's
    own training cases: summed over them, the measured duration of its choice is within 2 % of the best measured candidate
    (the fit script reports 1.4 %), and no single choice is more than 25 % off."""
    import importlib.util
    import os

    here = os.path.dirname(os.path.abspath(__file__))
    tuning = os.path.join(os.path.dirname(here), "tab_amd", "tuning")
    spec = importlib.util.spec_from_file_location("fit_conv_shape_model", os.path.join(tuning, "fit_conv_shape_model.py"))
    fit = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(fit)
    rows = fit.parse(os.path.join(tuning, "conv_shape_training_timings.txt"))
    assert len(rows) >= 280
    f = _hook()
    chosen = best = 0.0
    for r in rows:
        shape, _ = _choose(f, r["type"], r["M"], r["KN"], r["G"], r["PC"], 0)
        assert shape in r["times"], (r["name"], shape)
        assert fit.eligible(r, shape), (r["name"], shape)      # the fit script and the chooser agree on the candidates
        b = fit.best_time(r)
        assert r["times"][shape] <= 1.25 * b, (r["type"], r["name"], shape, r["times"][shape], b)
        chosen += r["times"][shape]
        best += b
    assert chosen <= 1.02 * best, (chosen, best)
