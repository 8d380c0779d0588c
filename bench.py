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
    ap.add_argument("--only-e2e", action="store_true",
                    help="profiling aid: run only the end-to-end Tucker ResNet-18 forward, `steps` times, and exit")
    ap.add_argument("--e2e-net", choices=["resnet18", "densenet121"], default="resnet18",
                    help="which Tucker network --only-e2e runs (batch 1)")
    ap.add_argument("--tile", default=None, metavar="mf,mb,nb,wm,wn,wk,cch,tw,ks,wl,alg",
                    help="with --only-dominant: force this tile instead of selecting one")
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
    from tdc_amd.conv import Conv2dPlan, time_many_ms
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

    if a.only_e2e:
        from tdc_amd import nets
        if a.e2e_net == "densenet121":
            net = nets.build_tucker_densenet121(nets.densenet121_params(seed=121), batch=1)
        else:
            net = nets.build_tucker_resnet18(nets.resnet18_params(seed=18), batch=1)
        ms = net.time_ms(iters=a.steps, graph=graph)
        print(json.dumps({"only_e2e": True, "net": a.e2e_net, "forwards": a.steps, "ms": ms,
                          "kernels": net.num_kernels}))
        return

    if a.only_dominant:
        x, w = ref.make_core_case(56, 128, 128)
        forced = None
        if a.tile:
            v = [int(t) for t in a.tile.split(",")]
            forced = tdc_amd.Tile(*v[:8], ks=v[8], wl=v[9], alg=v[10] if len(v) > 10 else 0)
        plan = Conv2dPlan(1, 128, 128, 56, 56, 3, 3, 1, 1, tile=forced).set_weights(w)
        xd, out = x.cuda(), torch.empty(1, 128, 56, 56, device="cuda")
        # the same back-to-back launches as the timed region of the full run (one graph of `steps` launches)
        if a.warmup > 0:
            plan.time_us(xd, out, iters=a.warmup, graph=graph)
        us = plan.time_us(xd, out, iters=a.steps, graph=graph)
        print(json.dumps({"only_dominant": True, "launches": a.steps, "us_per_launch": round(us, 3),
                          "tile": list(plan.info.tile.astuple())}))
        return

    layers = []
    for hw in ref.SWEEP_HW:
        for r1, r2 in ref.SWEEP_RANKS:
            x, w = ref.make_core_case(hw, r1, r2)
            plan = Conv2dPlan(1, r1, r2, hw, hw, 3, 3, 1, 1).set_weights(w)
            xd = x.cuda()
            out = torch.empty(1, r2, hw, hw, device="cuda")
            layers.append({"hw": hw, "r1": r1, "r2": r2, "plan": plan, "x": xd, "out": out, "xc": x, "wc": w})
    plans = [l["plan"] for l in layers]
    xs = [l["x"] for l in layers]
    outs = [l["out"] for l in layers]

    # -- parity spot check (outside every timed region) -------------------------
    for l in (layers[1], layers[-4]):
        l["plan"].forward(l["x"], out=l["out"])
        torch.cuda.synchronize()
        want = ref.conv2d_torch(l["xc"], l["wc"], pad=1)
        if not torch.allclose(l["out"].cpu(), want, rtol=1e-4, atol=1e-5):
            sys.exit("bench.py: parity check failed for layer %s" % ((l["hw"], l["r1"], l["r2"]),))

    # -- the timed region: W warm-up steps, then exactly K steps ------------------
    # Two ways to issue the same launches, each timed over its own W + K steps: one HIP graph holding the 28 launches,
    # replayed per step, and the 28 plain tdc_conv_forward launches on a stream (what a caller of the library does).
    # `value` is the faster one on this machine (stream launches need a host that issues a launch in under ~4 us);
    # both are reported.
    per_mode = {}
    for mode in ([True, False] if graph else [False]):
        if a.warmup > 0:
            time_many_ms(plans, xs, outs, iters=a.warmup, graph=mode)
        torch.cuda.synchronize()
        t_wall0 = time.perf_counter()
        mode_ms = time_many_ms(plans, xs, outs, iters=a.steps, graph=mode)   # syncs before and after
        torch.cuda.synchronize()
        per_mode[mode] = (mode_ms, (time.perf_counter() - t_wall0) * 1e3)
    step_graph = min(per_mode, key=lambda m: per_mode[m][0])
    total_ms, wall_ms = per_mode[step_graph]
    ms_per_step = total_ms / a.steps
    us_per_layer = ms_per_step * 1e3 / len(layers)

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
    table = []
    for l in layers:
        info = l["plan"].info
        us = min(l["plan"].time_us(l["x"], l["out"], iters=100, graph=graph) for _ in range(3))
        table.append({"H": l["hw"], "R1": l["r1"], "R2": l["r2"], "us": round(us, 3),
                      "roof_us": round(info.roof_us, 4), "frac": round(info.roof_us / us, 4),
                      "gflops": round(info.flops / us * 1e-3, 1), "tile": list(info.tile.astuple())})
        if l.get("model_tile") and l["model_tile"] != table[-1]["tile"]:
            table[-1]["model_tile"] = l["model_tile"]

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
        "layers": table,
        "layers_faster_than_miopen": (sum(1 for t in table if t.get("speedup_vs_miopen", 0) > 1.0) if not a.no_miopen
                                      else None),
        "host_wall_ms_timed_region": round(wall_ms, 3),
        "us_per_layer_by_launch": {("HIP graph replay" if m else "stream launches"): round(v[0] / a.steps * 1e3 / len(layers), 4)
                                   for m, v in per_mode.items()},
    }

    # -- end-to-end Tucker ResNet-18, batch 1, 3x224x224 (one HIP-graph launch per forward) ---------
    e2e_params = e2e_x = None
    if not a.no_e2e:
        from tdc_amd import nets
        from oracle import nets_ref
        e2e_params = nets.resnet18_params(seed=18)
        e2e_x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(18))
        net = nets.build_tucker_resnet18(e2e_params, batch=1)
        logits = net(e2e_x.cuda()).cpu().reshape(1, -1)
        want = nets_ref.tucker_resnet18_forward(e2e_params, e2e_x)
        err = float((logits - want).abs().max())
        if not err <= 1e-5 + 1e-4 * float(want.abs().max()):
            sys.exit("bench.py: end-to-end parity check failed (max err %g)" % err)
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
            if b == 1:
                dwant = nets_ref.tucker_densenet121_forward(dparams, dx)
                derr = float((dlog - dwant).abs().max())
                if not derr <= 1e-5 + 1e-4 * float(dwant.abs().max()):
                    sys.exit("bench.py: DenseNet-121 parity check failed (max err %g)" % derr)
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
            berr = float((got - want).abs().max())
            if not berr <= 1e-5 + 1e-4 * float(want.abs().max()):
                sys.exit("bench.py: Tucker block parity check failed (max err %g)" % berr)
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
                               "cores": torch.get_num_threads(), "kind": "port",
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
