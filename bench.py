#!/usr/bin/env python3
"""Benchmark of the Tucker core-conv hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one pass over the 28-shape core-conv sweep (batch 1, fp32 NCHW, 3x3,
stride 1, pad 1; H=W in {7,14,28,56} x (R1,R2) in {(16,16),(32,32),(64,64),(96,96),
(128,128),(32,64),(64,128)}), one kernel launch per layer, inputs and packed
weights resident in HBM.  Prints ONE JSON line: the mean device time per layer
(us/layer), a per-layer table with each layer's fraction of its fp32/HBM
roofline, the roofline of the dominant kernel (the 128->128 @56 layer) from HIP
events on the launch stream, and the CPU baseline (the PyTorch-CPU convolution
the reference operator executes) timed on this host's cores.
"""
import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ppopp23-tdc_amd"))
sys.path.insert(0, ROOT)

PEAK_FP32_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PEAK_HBM_TBPS = 8.0
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "core_conv_128x128_56_hbm_traffic.txt")


def measured_traffic(tile):
    """HBM bytes per launch of the dominant kernel from the committed rocprofv3 --pmc summary
    (FETCH_SIZE + WRITE_SIZE, scaled by a copy kernel of known size); None if it was taken with another tile."""
    try:
        for line in open(TRAFFIC_FILE):
            if line.startswith("traffic_bytes_per_launch:"):
                parts = line.split()
                if [int(v) for v in parts[3].split(",")] == list(tile):
                    return int(parts[1])
    except (OSError, ValueError, IndexError):
        pass
    return None


KERNEL_ONLY_FILE = os.path.join(ROOT, "profiles", "core_conv_layers_kernel_only_durations.txt")

# (R1 = input channels, R2 = output channels, H = W, best recorded time in ms on RTX 2080Ti and on A100) of the 18 layer
# shapes the reference benchmarks: 2080Ti-evaluation/TDC-LAYERS-ORACLE/compile_run.py:21-38, times from the minimum
# over its recorded tile sweeps (2080Ti-occupancy-unrolled, a100-occupancy-unrolled).
REFERENCE_LAYERS = (
    (64, 32, 224, 0.410112, 0.258144), (64, 32, 112, 0.090464, 0.08416), (32, 32, 56, 0.021952, 0.025728),
    (64, 32, 56, 0.031936, 0.035616), (64, 64, 56, 0.053504, 0.054848), (32, 32, 28, 0.012608, 0.014336),
    (64, 32, 28, 0.016864, 0.01792), (96, 64, 28, 0.028384, 0.023296), (160, 96, 28, 0.055584, 0.038752),
    (192, 96, 28, 0.055616, 0.041152), (32, 32, 14, 0.00912, 0.011264), (64, 32, 14, 0.011904, 0.013568),
    (128, 96, 14, 0.022528, 0.022592), (192, 96, 14, 0.027296, 0.02464), (32, 32, 7, 0.00864, 0.009216),
    (64, 32, 7, 0.008928, 0.011488), (96, 64, 7, 0.011584, 0.01232), (192, 160, 7, 0.01872, 0.022176),
)


def cpu_model():
    """The host processor's name as /proc/cpuinfo gives it (reported beside the CPU baseline)."""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def kernel_only_durations():
    """{(R1, R2, H): (median us, p10 us, tile)} of isolated launches from the committed rocprofv3 kernel-trace summary
    (lines `kernel_only_us: R1 R2 H tile median p10`)."""
    out = {}
    try:
        for line in open(KERNEL_ONLY_FILE):
            if line.startswith("kernel_only_us:"):
                f = line.split()
                out[(int(f[1]), int(f[2]), int(f[3]))] = (float(f[5]), float(f[6]), [int(v) for v in f[4].split(",")])
    except (OSError, ValueError, IndexError):
        pass
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-miopen", action="store_true", help="skip timing the same layers with MIOpen (through torch)")
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end Tucker ResNet-18 forward")
    ap.add_argument("--no-graph", action="store_true", help="issue launches on a plain stream instead of a HIP graph")
    ap.add_argument("--only-dominant", action="store_true",
                    help="profiling aid: launch only the dominant layer (128->128 @56), `steps` times, and exit")
    ap.add_argument("--only-launch-floor", action="store_true",
                    help="time only the launch path (empty and spinning kernels, stream launches and graph replay), for profiling")
    ap.add_argument("--only-e2e", action="store_true",
                    help="profiling aid: run only the end-to-end Tucker ResNet-18 forward, `steps` times, and exit")
    ap.add_argument("--e2e-batch", type=int, default=1, help="with --only-e2e: images per forward")
    ap.add_argument("--e2e-net", choices=["resnet18", "densenet121"], default="resnet18",
                    help="which Tucker network --only-e2e runs (batch 1)")
    ap.add_argument("--only-conv", default=None, metavar="C,N,H,K[,stride]",
                    help="profiling aid: launch only this convolution (C -> N channels at HxH, KxK, pad (K-1)/2, batch 1), "
                         "`steps` times, and exit")
    ap.add_argument("--isolated-layers", action="store_true",
                    help="profiling aid: launch every layer of the sweep (and of the reference's 18 shapes) `steps` times, "
                         "each launch followed by a stream synchronisation, and exit; under rocprofv3 --kernel-trace the "
                         "kernel durations are then those of isolated launches, not launch-to-launch times")
    ap.add_argument("--tiles-from", default=None, metavar="FILE",
                    help="profiling aid: force the tiles recorded in this file, the output of a plain run of this benchmark")
    ap.add_argument("--tile", default=None, metavar="mf,mb,nb,wm,wn,wk,cch,tw,ks,wl,alg",
                    help="with --only-dominant / --only-conv: force this tile instead of selecting one")
    ap.add_argument("--tune", type=int, default=16, metavar="CLASSES",
                    help="measured tile selection at plan creation: time the model's favourite tile of this many tile "
                         "classes and keep the fastest (0 = the analytic model's pick alone)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="BYTES",
                    help="profiling aid: run a plain device copy of BYTES bytes a few times (reference reading for "
                         "the FETCH_SIZE / WRITE_SIZE counters) before anything else")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (single-GPU hot path, "
                 "no collectives)." % a.gpus)

    import torch
    import tdc_amd
    from tdc_amd.conv import Conv2dPlan, launch_floor_us, time_many_ms
    from oracle import ref   # checker + cpu_baseline leg only

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    torch.cuda.set_device(0)
    graph = not a.no_graph
    tdc_amd.set_autotune(a.tune)

    if a.calibrate_copy:
        src = torch.empty(a.calibrate_copy // 4, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    def floor_leg(as_graph):
        best = lambda **kw: min(launch_floor_us(launches=300, graph=as_graph, **kw) for _ in range(3))
        empty = best(grid=256, block=512)
        spins = {sp: best(grid=256, block=512, spin_us=sp) for sp in (1.0, 2.0, 4.0)}
        return {"empty_kernel_us": round(empty, 3), "empty_kernel_1_workgroup_us": round(best(grid=1, block=64), 3),
                "busy_1us": round(spins[1.0], 3), "busy_2us": round(spins[2.0], 3), "busy_4us": round(spins[4.0], 3),
                # what a launch adds to a kernel long enough not to hide under the launch path
                "overhead_beyond_duration_us": round(spins[4.0] - 4.0, 3)}
    if a.only_launch_floor:
        print(json.dumps({"only_launch_floor": True, "stream_launches": floor_leg(False), "graph_replay": floor_leg(True)}))
        return

    if a.only_e2e:
        from tdc_amd import nets
        if a.e2e_net == "densenet121":
            net = nets.build_tucker_densenet121(nets.densenet121_params(seed=121), batch=a.e2e_batch)
        else:
            net = nets.build_tucker_resnet18(nets.resnet18_params(seed=18), batch=a.e2e_batch)
        ms = net.time_ms(iters=a.steps, graph=graph)
        print(json.dumps({"only_e2e": True, "net": a.e2e_net, "batch": a.e2e_batch, "forwards": a.steps, "ms": ms,
                          "kernels": net.num_kernels}))
        return

    if a.only_dominant or a.only_conv:
        cv = [int(t) for t in a.only_conv.split(",")] if a.only_conv else [128, 128, 56, 3]
        C, N, hw, K = cv[:4]
        stride = cv[4] if len(cv) > 4 else 1
        if K == 3 and stride == 1:
            x, w = ref.make_core_case(hw, C, N)
        else:
            gq = torch.Generator().manual_seed(hw * 1_000_000 + C * 1_000 + N)
            x = torch.rand(1, C, hw, hw, generator=gq) * 2 - 1
            w = torch.empty(N, C, K, K).normal_(0, (2.0 / (C * K * K)) ** 0.5, generator=gq)
        forced = None
        if a.tile:
            v = [int(t) for t in a.tile.split(",")]
            forced = tdc_amd.Tile(*v[:8], ks=v[8], wl=v[9], alg=v[10] if len(v) > 10 else 0)
        plan = Conv2dPlan(1, C, N, hw, hw, K, K, stride, (K - 1) // 2, tile=forced).set_weights(w)
        xd, out = x.cuda(), torch.empty(1, N, plan.Ho, plan.Wo, device="cuda")
        got = plan.forward(xd).cpu()
        if not torch.allclose(got, ref.conv2d_torch(x, w, stride=stride, pad=(K - 1) // 2), rtol=1e-4, atol=1e-5):
            sys.exit("bench.py: parity check failed for --only-conv %s" % (cv,))
        # the same back-to-back launches as the timed region of the full run (one graph of `steps` launches)
        if a.warmup > 0:
            plan.time_us(xd, out, iters=a.warmup, graph=graph)
        us = plan.time_us(xd, out, iters=a.steps, graph=graph)
        info = plan.info
        print(json.dumps({"only_conv": [C, N, hw, K, stride], "launches": a.steps, "us_per_launch": round(us, 3),
                          "tile": list(info.tile.astuple()), "flops": info.flops, "bytes": info.bytes,
                          "roof_us": round(info.roof_us, 4), "timing": "hipEvents around the launches of this run"}))
        return

    # --tiles-from: the tiles a plain run of this benchmark timed (its JSON line), so that a profiled run launches
    # the same kernels (measured selection under a profiler times the candidates with the profiler's overhead).
    forced_tiles = {}
    if a.tiles_from:
        prev = json.loads(open(a.tiles_from).read().strip().splitlines()[-1])
        for row in prev["layers"] + prev["reference_layer_shapes"]["layers"]:
            forced_tiles[(row["R1"], row["R2"], row["H"])] = tdc_amd.Tile(*row["tile"])

    def make_layer(hw, r1, r2):
        x, w = ref.make_core_case(hw, r1, r2)
        plan = Conv2dPlan(1, r1, r2, hw, hw, 3, 3, 1, 1, tile=forced_tiles.get((r1, r2, hw))).set_weights(w)
        return {"hw": hw, "r1": r1, "r2": r2, "plan": plan, "x": x.cuda(), "out": torch.empty(1, r2, hw, hw, device="cuda"),
                "xc": x, "wc": w}

    def check_parity(l):
        """The plan that is about to be timed (its measured or modelled tile) against the reference operator's own
        arithmetic, torch.nn.functional.conv2d fp32 on the host: rel 1e-4, abs 1e-5.  Returns the largest share of
        that tolerance any element uses."""
        l["out"].fill_(float("nan"))
        l["plan"].forward(l["x"], out=l["out"])
        torch.cuda.synchronize()
        want = ref.conv2d_torch(l["xc"], l["wc"], pad=1)
        share = float(((l["out"].cpu() - want).abs() / (1e-5 + 1e-4 * want.abs())).max())
        if not share <= 1.0:   # (NaN fails too)
            sys.exit("bench.py: parity check failed for layer %s with tile %s: %.3g of the tolerance"
                     % ((l["hw"], l["r1"], l["r2"]), l["plan"].info.tile.astuple(), share))
        return share

    t_plans0 = time.perf_counter()
    layers = [make_layer(hw, r1, r2) for hw in ref.SWEEP_HW for r1, r2 in ref.SWEEP_RANKS]
    plan_creation_s = time.perf_counter() - t_plans0   # tile selection (measured, when --tune > 0), packing, upload
    # the reference's own 18 layer shapes (2080Ti-evaluation/TDC-LAYERS-ORACLE/compile_run.py:21-38), a secondary table
    ref_layers = [make_layer(hw, c, n) for (c, n, hw, _, _) in REFERENCE_LAYERS]
    plans = [l["plan"] for l in layers]
    xs = [l["x"] for l in layers]
    outs = [l["out"] for l in layers]

    # -- parity of EVERY plan that is timed below, with the tile it is timed with (outside every timed region) ------
    for l in layers + ref_layers:
        l["parity"] = check_parity(l)

    if a.isolated_layers:
        stream = torch.cuda.current_stream()
        for l in layers + ref_layers:
            for _ in range(a.steps):
                l["plan"].forward(l["x"], out=l["out"])
                stream.synchronize()
        print(json.dumps({"isolated_layers": True, "launches_per_layer": a.steps + 1,
                          "layers": [[l["r1"], l["r2"], l["hw"], list(l["plan"].info.tile.astuple())] for l in layers + ref_layers]}))
        return

    # -- the timed region: W warm-up steps, then exactly K steps ------------------
    # Two ways to issue the same launches: one HIP graph holding the 28 launches, replayed per step, and the 28 plain
    # tdc_conv_forward launches on a stream (what a caller of the library does; it needs a host that issues a launch
    # in under ~4 us).  Which one the timed region uses is decided BEFORE it, from the warm-up steps of both; the
    # other is timed afterwards and reported beside it.
    # (spin-up, untimed and not counted as warm-up steps: the same step for ~0.2 s, so that the W warm-up steps and the K
    #  timed steps run at the clocks of a busy GPU; the parity checks above leave it idle for hundreds of milliseconds,
    #  and with the driver's K = 20 the timed region is only 2.5 ms long)
    t_spin = time.perf_counter()
    while time.perf_counter() - t_spin < 0.2:
        time_many_ms(plans, xs, outs, iters=50, graph=False)
    warm = {}
    for mode in ([True, False] if graph else [False]):
        time_many_ms(plans, xs, outs, iters=2, graph=mode)
        warm[mode] = time_many_ms(plans, xs, outs, iters=max(a.warmup, 1), graph=mode) / max(a.warmup, 1)
    step_graph = min(warm, key=lambda m: warm[m])
    torch.cuda.synchronize()
    t_wall0 = time.perf_counter()
    total_ms = time_many_ms(plans, xs, outs, iters=a.steps, graph=step_graph)   # syncs before and after
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t_wall0) * 1e3
    ms_per_step = total_ms / a.steps
    us_per_layer = ms_per_step * 1e3 / len(layers)
    per_mode = {step_graph: total_ms}
    for mode in warm:
        if mode != step_graph:
            per_mode[mode] = time_many_ms(plans, xs, outs, iters=a.steps, graph=mode)

    # -- the same step with the analytic model's picks alone (reported beside `value`) -------------
    model_only_us = None
    if a.tune > 0:
        tdc_amd.set_autotune(0)
        mplans = [Conv2dPlan(1, l["r1"], l["r2"], l["hw"], l["hw"], 3, 3, 1, 1).set_weights(l["wc"]) for l in layers]
        tdc_amd.set_autotune(a.tune)
        time_many_ms(mplans, xs, outs, iters=max(a.warmup, 1), graph=step_graph)
        model_only_us = time_many_ms(mplans, xs, outs, iters=a.steps, graph=step_graph) / a.steps * 1e3 / len(layers)
        for l, mp in zip(layers, mplans):
            l["model_tile"] = list(mp.info.tile.astuple())
            mp.close()

    # -- per-layer device time and roofline fraction ------------------------------
    # `us` = launch-to-launch time (median of three runs of 100 graph-replayed launches: what a layer costs inside a
    # stream of work); `kernel_us_from_committed_trace` = begin-to-end duration of the kernel alone from the committed rocprofv3 trace of
    # isolated launches (every launch followed by a stream synchronisation; median, p10).  An isolated launch starts
    # on an idle, cold chip and pays its whole dispatch ramp and drain, which back-to-back launches overlap with their
    # neighbours: it is the LARGER of the two figures for every layer.
    kernel_only = kernel_only_durations()

    # -- the launch path by itself (tdc_launch_floor_time): dependent launches of a kernel with the same argument block
    #    that touches no memory, empty or with every wave busy for a set time; as stream launches (how the timed step is
    #    issued) and as one graph replay (how the per-layer `us` below are issued) -----------------------------------
    floor_stream, floor_graph = floor_leg(False), floor_leg(True)
    layer_floor = (floor_graph if graph else floor_stream)["empty_kernel_us"]   # same launch mode as the per-layer `us`

    def layer_row(l):
        info = l["plan"].info
        us = sorted(l["plan"].time_us(l["x"], l["out"], iters=100, graph=graph) for _ in range(3))[1]
        row = {"H": l["hw"], "R1": l["r1"], "R2": l["r2"], "us": round(us, 3),
               "roof_us": round(info.roof_us, 4), "frac": round(info.roof_us / us, 4),
               # the share of the roofline left once the launch floor (an empty kernel, same launch mode) is taken off
               "frac_attainable": round(info.roof_us / max(us - layer_floor, info.roof_us), 4),
               "gflops": round(info.flops / us * 1e-3, 1), "tile": list(info.tile.astuple()),
               "parity_share_of_tolerance": round(l["parity"], 4)}
        ko = kernel_only.get((l["r1"], l["r2"], l["hw"]))
        if ko and ko[2] == row["tile"]:   # (only when that trace was taken with the tile timed here)
            row["kernel_us_from_committed_trace"] = {"median": ko[0], "p10": ko[1]}
        return row

    table = []
    for l in layers:
        table.append(layer_row(l))
        if l.get("model_tile") and l["model_tile"] != table[-1]["tile"]:
            table[-1]["model_tile"] = l["model_tile"]
    ref_table = []
    for l, (c, n, hw, ms_2080ti, ms_a100) in zip(ref_layers, REFERENCE_LAYERS):
        row = layer_row(l)
        row["reference_best_us"] = {"rtx2080ti": round(ms_2080ti * 1e3, 2), "a100": round(ms_a100 * 1e3, 2)}
        ref_table.append(row)

    # -- comparator: MIOpen's convolution for the same layers (what torch.nn.functional.conv2d dispatches to on
    #    ROCm), graph-replayed the same way; the reference compares against cuDNN the same way
    #    (template_benchmark_cudnn.template:455-475).  Reported next to each layer, not part of `value`.
    if not a.no_miopen:
        import torch.nn.functional as F
        torch.backends.cudnn.benchmark = True     # let MIOpen search its algorithms
        for l, row in zip(layers, table):
            wd = l["wc"].cuda()
            for _ in range(5):
                F.conv2d(l["x"], wd, None, 1, 1)
            torch.cuda.synchronize()
            side = torch.cuda.Stream()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                F.conv2d(l["x"], wd, None, 1, 1)
                side.synchronize()
                with torch.cuda.graph(g, stream=side):
                    for _ in range(20):
                        F.conv2d(l["x"], wd, None, 1, 1)
            g.replay()
            torch.cuda.synchronize()
            best = float("inf")
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(5):
                    g.replay()
                e1.record()
                e1.synchronize()
                best = min(best, e0.elapsed_time(e1) * 1e3 / 100)
            row["miopen_us"] = round(best, 3)
            row["speedup_vs_miopen"] = round(best / row["us"], 2)

    # -- dominant kernel: the largest layer of the sweep --------------------------
    dom = max(range(len(layers)), key=lambda i: table[i]["us"])
    dl, dinfo = layers[dom], layers[dom]["plan"].info
    dom_us = sum(dl["plan"].time_us(dl["x"], dl["out"], iters=200, graph=graph) for _ in range(3)) / 3
    mfma_bound = dinfo.flops / (PEAK_FP32_TFLOPS * 1e6) >= dinfo.bytes / (PEAK_HBM_TBPS * 1e6)
    if mfma_bound:
        achieved = dinfo.flops / dom_us * 1e-6     # TFLOP/s
        roofline = {"bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(achieved / PEAK_FP32_TFLOPS, 4), "traffic": None}
    else:
        achieved = dinfo.bytes / dom_us * 1e-3     # GB/s
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_TBPS * 1e3, "unit": "GB/s",
                    "frac": round(achieved / (PEAK_HBM_TBPS * 1e3), 4), "traffic": None}
    roofline["traffic"] = measured_traffic(dinfo.tile.astuple())
    roofline["traffic_source"] = ("profiles/core_conv_128x128_56_hbm_traffic.txt (committed rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                                  "run with this tile; not measured in this run)" if roofline["traffic"] is not None else
                                  "none: the committed counter run used another tile")
    # the whole timed step against the sum of its layers' rooflines (time-weighted, unlike the dominant kernel's frac)
    roofline["sweep_sum_roof_us"] = round(sum(t["roof_us"] for t in table), 3)
    roofline["sweep_time_weighted_frac"] = round(sum(t["roof_us"] for t in table) / (ms_per_step * 1e3), 4)
    roofline["launch_floor_us"] = floor_stream["empty_kernel_us"] if not step_graph else floor_graph["empty_kernel_us"]
    # the same kernel as isolated launches (one hipEvent pair around ONE eager launch, 200 times): includes the
    # start-up of an idle queue, so it is reported next to the back-to-back figure, not used for `achieved`
    singles = sorted(dl["plan"].time_us(dl["x"], dl["out"], iters=1, graph=False) for _ in range(200))
    roofline["single_launch_us"] = {"median": round(singles[len(singles) // 2], 3), "p10": round(singles[20], 3)}
    roofline.update({"kernel": "core conv %d->%d @%dx%d" % (dl["r1"], dl["r2"], dl["hw"], dl["hw"]),
                     "avg_launch_us": round(dom_us, 3), "flops_per_launch": dinfo.flops,
                     "bytes_per_launch": dinfo.bytes, "timing": "hipEvents around 200 graph-replayed launches"})

    out = {
        "metric": "core_conv_us_per_layer", "value": round(us_per_layer, 4), "unit": "us/layer",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "core-conv sweep: 28 layers, batch 1, fp32 NCHW, 3x3 s1 p1, H=W in {7,14,28,56} x "
                               "7 rank pairs; one step = one pass over all 28 layers",
                   "launch": "HIP graph replay" if step_graph else "stream launches", "layers_per_step": len(layers),
                   "tile_selection": ("measured at plan creation: the model's favourite tile of each of the %d most "
                                      "promising tile classes is timed, the fastest kept" % a.tune) if a.tune > 0
                   else "analytic model"},
        "model_only_us_per_layer": None if model_only_us is None else round(model_only_us, 4),
        "roofline": roofline,
        "geomean_frac": round(float(torch.tensor([t["frac"] for t in table]).log().mean().exp()), 4),
        "layers_at_or_above_40_percent": sum(1 for t in table if t["frac"] >= 0.40),
        "launch_floor": {"what": "tdc_launch_floor_time: 300 dependent launches of a kernel with the convolution kernels' argument "
                                 "block (256 workgroups x 512 threads, no memory access), empty or with every wave busy for "
                                 "1 / 2 / 4 us; us per launch, best of 3",
                         "stream_launches": floor_stream, "graph_replay": floor_graph,
                         "per_layer_us_measured_as": "graph replay" if graph else "stream launches"},
        "tiles_sha": hashlib.sha1(json.dumps([t["tile"] for t in table]).encode()).hexdigest()[:16],
        "plan_creation_s": round(plan_creation_s, 2),
        "kernel_us_from_committed_trace": "profiles/core_conv_layers_kernel_only_durations.txt: rocprofv3 kernel-trace durations of "
                                          "isolated launches (each followed by a synchronisation); shown only for rows whose "
                                          "tile is the one that trace was taken with; NOT measured in this run",
        "layers": table,
        "reference_layer_shapes": {
            "what": "the 18 core-conv shapes the reference itself times (2080Ti-evaluation/TDC-LAYERS-ORACLE/compile_run.py:21-38), "
                    "same treatment as `layers`; reference_best_us = its recorded best tile on other hardware "
                    "(single cold launch between cudaEvents), context and not a same-machine comparison",
            "us_per_layer": round(sum(r["us"] for r in ref_table) / len(ref_table), 4), "layers": ref_table},
        "layers_faster_than_miopen": (sum(1 for t in table if t.get("speedup_vs_miopen", 0) > 1.0) if not a.no_miopen
                                      else None),
        "host_wall_ms_timed_region": round(wall_ms, 3),
        "us_per_layer_by_launch": {("HIP graph replay" if m else "stream launches"): round(v / a.steps * 1e3 / len(layers), 4)
                                   for m, v in per_mode.items()},
        "launch_mode_chosen_from": "warm-up steps of both modes, before the timed region",
    }

    # -- end-to-end Tucker ResNet-18, batch 1, 3x224x224 (one HIP-graph launch per forward) ---------
    e2e_params = e2e_x = None
    if not a.no_e2e:
        from tdc_amd import nets
        from oracle import nets_ref
        e2e_params = nets.resnet18_params(seed=18)
        e2e_x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(18))
        net = nets.build_tucker_resnet18(e2e_params, batch=1)
        def net_parity(got, want, what):
            """Per element |got - want| <= 1e-4 |want| + max(1e-5, 1e-6 max|want|) (activations of the synthetic nets
            are of order 1 to 30); returns the largest absolute error."""
            err = (got - want).abs()
            bound = 1e-4 * want.abs() + max(1e-5, 1e-6 * float(want.abs().max()))
            if not bool((err <= bound).all()):
                sys.exit("bench.py: %s parity check failed (max err %g at max|ref| %g)" % (what, float(err.max()), float(want.abs().max())))
            return float(err.max())

        logits = net(e2e_x.cuda()).cpu().reshape(1, -1)
        want, feats = nets_ref.tucker_resnet18_forward(e2e_params, e2e_x, return_features=True)
        err = net_parity(logits, want, "Tucker ResNet-18 logits")
        for name, tid in net.feature_ids.items():
            net_parity(net.read(tid), feats[name], "Tucker ResNet-18 " + name)
        net.time_ms(iters=20)
        e2e_ms = min(net.time_ms(iters=100) for _ in range(3))
        out["tucker_resnet18_b1"] = {"ms": round(e2e_ms, 4), "kernels_per_forward": net.num_kernels,
                                     "ms_eager_launches": round(net.time_ms(iters=50, graph=False), 4),
                                     "max_abs_err_vs_cpu": err, "launch": "one HIP graph replay per forward",
                                     "config": "ResNet-18 [2,2,2,2], every 3x3 conv = TKConv with R1=R2=planes/2, "
                                               "BN folded, batch 1, fp32 3x224x224, random init seed 18"}
        net.close()
        # Tucker DenseNet-121 (configuration 5), batch 1 and batch 8, same treatment
        dparams = nets.densenet121_params(seed=121)
        dres = {}
        for b in (1, 8):
            dx = torch.randn(b, 3, 224, 224, generator=torch.Generator().manual_seed(121))
            dnet = nets.build_tucker_densenet121(dparams, batch=b)
            dlog = dnet(dx.cuda()).cpu().reshape(b, -1)
            dwant, dfeats = nets_ref.tucker_densenet121_forward(dparams, dx, return_features=True)
            dres["b%d_max_abs_err_vs_cpu" % b] = net_parity(dlog, dwant, "Tucker DenseNet-121 batch %d logits" % b)
            for name, tid in dnet.feature_ids.items():
                net_parity(dnet.read(tid), dfeats[name], "Tucker DenseNet-121 batch %d %s" % (b, name))
            dnet.time_ms(iters=5)
            dres["b%d_ms" % b] = round(min(dnet.time_ms(iters=20) for _ in range(3)), 4)
            dres["b%d_kernels_per_forward" % b] = dnet.num_kernels
            dnet.close()
        out["tucker_densenet121"] = dres
        # The four full Tucker blocks (configuration 3): 1x1 C->R1, 3x3 R1->R2, 1x1 R2->N as three launches in a graph.
        # roof_us is the FUSED block's roofline: every flop, but input, output and weights moved once.
        blocks = []
        for (C, R1, R2, N, hw) in ref.BLOCKS:
            bx, first, core, last = ref.make_block_case(C, R1, R2, N, hw)
            bnet = nets.Net(1, C, hw, hw)
            y = bnet.tkconv(0, first, core, last, pad=1)
            bnet.finalize(y)
            got = bnet(bx.cuda()).cpu()
            want = ref.tkconv_torch(bx, first, core, last, pad=1)
            if not torch.allclose(got, want, rtol=1e-4, atol=1e-5):
                sys.exit("bench.py: Tucker block parity check failed (max err %g)" % float((got - want).abs().max()))
            bnet.time_ms(iters=20)
            us = min(bnet.time_ms(iters=200) for _ in range(3)) * 1e3
            us_stream = min(bnet.time_ms(iters=200, graph=False) for _ in range(3)) * 1e3   # the same launches, not from a graph
            flops = 2.0 * hw * hw * (C * R1 + 9 * R1 * R2 + R2 * N)
            nbytes = 4.0 * (hw * hw * (C + N) + C * R1 + 9 * R1 * R2 + R2 * N)
            roof = max(nbytes / 8e6, flops / 157.3e6)
            blocks.append({"C": C, "R1": R1, "R2": R2, "N": N, "H": hw, "us": round(us, 3), "roof_us": round(roof, 3),
                           "frac": round(roof / min(us, us_stream), 4), "kernels": bnet.num_kernels,
                           "us_stream_launches": round(us_stream, 3)})   # us: one graph replay per block (a replay costs ~5 us by itself)
            bnet.close()
        out["tucker_blocks_b1"] = blocks

    # -- CPU baseline: the reference operator's CPU path (F.conv2d), same layers --
    if not a.no_cpu_baseline:
        torch.set_num_threads(os.cpu_count() or 1)
        import torch.nn.functional as F
        with torch.no_grad():
            for l in layers:
                F.conv2d(l["xc"], l["wc"], None, 1, 1)
            passes, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < 10.0:
                for l in layers:
                    ref.conv2d_torch(l["xc"], l["wc"], pad=1)
                passes += 1
            cpu_s = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(cpu_s * 1e6 / (passes * len(layers)), 2), "unit": "us/layer",
                               "cores": torch.get_num_threads(), "cpu_model": cpu_model(), "kind": "port",
                               "sample": "%d passes over the same 28 layers with torch.nn.functional.conv2d fp32 on "
                                         "the host (the call the reference operator makes on CPU), ~10 s" % passes}
        if e2e_params is not None:
            from oracle import nets_ref
            for _ in range(3):
                nets_ref.tucker_resnet18_forward(e2e_params, e2e_x)
            n, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < 5.0:
                nets_ref.tucker_resnet18_forward(e2e_params, e2e_x)
                n += 1
            out["tucker_resnet18_b1"]["cpu_ms"] = round((time.perf_counter() - t0) * 1e3 / n, 3)
            out["tucker_resnet18_b1"]["cpu_cores"] = torch.get_num_threads()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
