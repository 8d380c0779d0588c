"""Fit the latency model's calibration constants to a measured tile sweep.

    python -m tdc_amd.fit_model sweep.csv [more.csv ...]

Reads the CSV rows written by ``python -m tdc_amd.sweep --out`` and searches the constants
(``tdc_model_set_constants``) for the smallest average selection loss — how much slower the tile
with the lowest PREDICTED time is than the fastest MEASURED tile of each layer, the reference's
``loss`` (2080Ti-evaluation/TDC-LAYERS-MODELING/model.py:237-254) — with the mean absolute
log-error of the prediction as a tie-breaker.  Host-only: no GPU is needed.  Prints the constants in
the order of ``tile_model.cpp``'s ModelConst.
"""
from __future__ import annotations

import collections
import csv
import math
import random
import sys

from . import _lib


def load(paths):
    layers = collections.defaultdict(list)
    for path in paths:
        for r in csv.DictReader(open(path)):
            key = tuple(int(r[k]) for k in ("C", "N", "H", "W", "K", "stride"))
            tile = _lib.Tile(*[int(r[k]) for k in ("mf", "mb", "nb", "wm", "wn", "wk", "cch", "tw")],
                             ks=int(r.get("ks") or 1), wl=int(r.get("wl") or 0), alg=int(r.get("alg") or r.get("wino") or 0))
            layers[key].append((tile, float(r["time_us"])))
    return layers


def score(layers):
    loss, logerr, n = 0.0, 0.0, 0
    for (C, N, H, W, K, stride), rows in layers.items():
        desc = _lib.conv_desc(1, C, N, H, W, K, K, stride, K // 2)
        best_meas = min(t for _, t in rows)
        preds = []
        for tile, t in rows:
            try:
                preds.append((_lib.model_evaluate(desc, tile).pred_us, t))
            except _lib.TdcError:
                pass    # a tile of an older sweep that the present geometry rules no longer admit
        if not preds:
            continue
        best_meas = min(t for _, t in preds)
        pick = min(preds)[1]
        loss += pick / best_meas - 1.0
        # prediction accuracy only matters near the top of the ranking
        near = [(p, t) for p, t in preds if t <= 1.5 * best_meas]
        logerr += sum(abs(math.log(p / t)) for p, t in near) / len(near)
        n += 1
    return loss / n, logerr / n


def fit(layers, rounds=6, seed=0):
    rng = random.Random(seed)
    cur = _lib.model_get_constants()
    best = score(layers)
    print("start: loss %.2f%%  log-err %.3f" % (100 * best[0], best[1]), flush=True)
    obj = lambda s: s[0] + 0.3 * s[1]
    for rnd in range(rounds):
        order = list(range(len(cur)))
        rng.shuffle(order)
        for i in order:
            for f in (0.5, 0.7, 0.85, 1.2, 1.5, 2.0):
                trial = list(cur)
                trial[i] = cur[i] * f
                _lib.model_set_constants(trial)
                sc = score(layers)
                if obj(sc) < obj(best) - 1e-6:
                    best, cur = sc, trial
            _lib.model_set_constants(cur)
        print("round %d: loss %.2f%%  log-err %.3f" % (rnd, 100 * best[0], best[1]), flush=True)
    return cur, best


def main(argv=None):
    paths = (argv or sys.argv[1:])
    if not paths:
        sys.exit(__doc__)
    layers = load(paths)
    cur, best = fit(layers)
    for name, v in zip(_lib.MODEL_CONSTANT_NAMES, cur):
        print("    double %s = %.6g;" % (name, v))
    print("average selection loss %.2f%% over %d layers" % (100 * best[0], len(layers)))


if __name__ == "__main__":
    main()
