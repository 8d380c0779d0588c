"""Measured tile sweep and model-loss report.

For every shape, time every launchable tile through the C ABI, record
``C,N,H,W,K,stride,mf,mb,nb,wm,wn,wk,cch,tw,ks,wl,alg,pred_us,time_us`` rows, and report how
much slower the analytic model's pick is than the measured best
(``loss = t(model pick) / t(best) - 1``).  This is the gfx950 counterpart of the
reference's brute-force occupancy/timing sweep
(2080Ti-evaluation/Gen-occupancy/gen.py:61-103), its oracle pick
(2080Ti-evaluation/TDC-LAYERS-ORACLE/gen_from_occupancy.py:51-66) and its
model-vs-oracle loss (2080Ti-evaluation/TDC-LAYERS-MODELING/model.py:237-254) —
without generating or compiling a source file per candidate.

    python -m tdc_amd.sweep --out sweep.csv            # the 28-shape core-conv sweep
"""
from __future__ import annotations

import argparse
import math
import sys
import time

import torch

from . import _lib
from .conv import Conv2dPlan

SWEEP_HW = (7, 14, 28, 56)
SWEEP_RANKS = ((16, 16), (32, 32), (64, 64), (96, 96), (128, 128), (32, 64), (64, 128))


def time_plan(plan, x, out, iters=50, warmup=5, reps=5):
    """Median over `reps` of the device time per launch (hipEvents around `iters` launches issued from C)."""
    plan.time_us(x, out, iters=warmup)
    samples = sorted(plan.time_us(x, out, iters=iters) for _ in range(reps))
    return samples[len(samples) // 2]


def sweep_shape(C, N, H, W, K=3, stride=1, pad=1, batch=1, iters=20, every=1, log=None, max_tiles=0, offset=0):
    desc = _lib.conv_desc(batch, C, N, H, W, K, K, stride, pad)
    tiles = _lib.model_enumerate(desc)
    if max_tiles and len(tiles) > max_tiles * every:
        every = -(-len(tiles) // max_tiles)
    tiles = tiles[offset % every::every]
    pick = _lib.model_select(desc)
    g = torch.Generator().manual_seed(H * 1_000_000 + C * 1_000 + N)
    x = (torch.rand(batch, C, H, W, generator=g) * 2 - 1).cuda()
    w = torch.empty(N, C, K, K).normal_(0, math.sqrt(2.0 / (C * K * K)), generator=g)
    rows = []
    if pick.tile.astuple() not in [t.astuple() for t in tiles]:
        tiles.append(pick.tile)
    for t in tiles:
        info = _lib.model_evaluate(desc, t)
        plan = Conv2dPlan(batch, C, N, H, W, K, K, stride, pad, tile=t).set_weights(w)
        out = torch.empty((batch, N, plan.Ho, plan.Wo), device="cuda")
        us = time_plan(plan, x, out, iters=iters)
        plan.close()
        row = (C, N, H, W, K, stride) + t.astuple() + (info.pred_us, us)
        rows.append(row)
        if log:
            log.write(",".join(f"{v:.3f}" if isinstance(v, float) else str(v) for v in row) + "\n")
            log.flush()
    best = min(rows, key=lambda r: r[-1])
    mine = next(r for r in rows if r[6:17] == pick.tile.astuple())
    return {"shape": (C, N, H, W, K, stride), "best": best, "model": mine, "loss": mine[-1] / best[-1] - 1,
            "roof_us": pick.roof_us, "n": len(rows)}


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=None, help="CSV of every (shape, tile) timing")
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--every", type=int, default=1, help="time every k-th candidate only")
    ap.add_argument("--max-tiles", type=int, default=0, help="thin the candidates of a shape to about this many")
    ap.add_argument("--offset", type=int, default=0, help="first candidate of the thinned list")
    ap.add_argument("--net", choices=("resnet18", "densenet121"), default=None,
                    help="sweep the distinct convolution shapes of a whole network instead of the core-conv layers")
    ap.add_argument("--shapes", nargs="*", default=None, metavar="C,N,H,W,K,stride,pad",
                    help="sweep these convolution shapes instead")
    ap.add_argument("--hw", type=int, nargs="*", default=list(SWEEP_HW))
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("tdc_amd.sweep needs a GPU")
    log = open(a.out, "w") if a.out else None
    if log:
        log.write("C,N,H,W,K,stride,mf,mb,nb,wm,wn,wk,cch,tw,ks,wl,alg,pred_us,time_us\n")
    total = 0.0
    n = 0
    t0 = time.time()
    if a.shapes:
        shapes = [tuple(int(v) for v in sh.split(",")) for sh in a.shapes]
        if any(len(sh) != 7 for sh in shapes):
            sys.exit("--shapes: every shape is C,N,H,W,K,stride,pad")
    elif a.net:
        from . import nets
        if a.net == "resnet18":
            net = nets.build_tucker_resnet18(nets.resnet18_params())
        else:
            net = nets.build_tucker_densenet121(nets.densenet121_params())
        shapes = sorted(set(net.conv_shapes))
        net.close()
    else:
        shapes = [(r1, r2, hw, hw, 3, 1, 1) for hw in a.hw for r1, r2 in SWEEP_RANKS]
    for (C, N, H, W, K, stride, pad) in shapes:
        r = sweep_shape(C, N, H, W, K=K, stride=stride, pad=pad, iters=a.iters, every=a.every, log=log,
                        max_tiles=a.max_tiles, offset=a.offset)
        total += r["loss"]
        n += 1
        print("shape %s roof %.3f us | best %s %.2f us | model %s %.2f us (pred %.2f) | loss %+.1f%% | %d tiles | %.0fs"
              % (r["shape"], r["roof_us"], r["best"][6:17], r["best"][-1], r["model"][6:17], r["model"][-1],
                 r["model"][-2], 100 * r["loss"], r["n"], time.time() - t0), flush=True)
    print("average loss %.1f%% over %d shapes" % (100 * total / max(n, 1), n))


if __name__ == "__main__":
    main()
