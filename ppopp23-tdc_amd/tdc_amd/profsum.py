"""Summarise rocprofv3 CSV output per (kernel, launch geometry).

rocprofv3's own ``--stats`` table aggregates by kernel NAME, and one template
instantiation of the convolution kernel serves many layer shapes; the launch
geometry (grid, workgroup, LDS) is what tells the layers apart.

    python -m tdc_amd.profsum kernel <dir-with-*_kernel_trace.csv>
    python -m tdc_amd.profsum pmc    <dir-with-*_counter_collection.csv> [--copy-bytes N]
    python -m tdc_amd.profsum timeline <dir-with-*_kernel_trace.csv> --last N
    python -m tdc_amd.profsum durations <dir-with-*_kernel_trace.csv>
    python -m tdc_amd.profsum isolated <dir-with-*_kernel_trace.csv> --layers <output of bench.py --isolated-layers>
    python -m tdc_amd.profsum isolated-pmc <dir,dir,...> --layers <output of bench.py --isolated-layers> [--copy-bytes N]

``kernel``: count / mean / min / max duration in microseconds per (kernel, grid, workgroup, LDS).
``pmc``: mean counter value per (kernel, grid, workgroup); with ``--copy-bytes N`` the FETCH_SIZE /
WRITE_SIZE readings (KiB) of every kernel are also shown scaled by the reading of the largest
copy kernel in the same run, which is known to read and write N bytes.
``timeline``: the last N dispatches of the trace in launch order (one forward of a network of N kernels):
start offset, duration, and the idle gap since the previous kernel ended.
``durations``: dispatches per kernel, launch geometry and duration class (nearest 0.5 us): launches, duration
statistics and the median start-to-start interval under the tracer.
``isolated``: median / p10 kernel duration per benchmark layer from a trace of ``bench.py --isolated-layers``.
``isolated-pmc``: counters per benchmark layer from ``--pmc`` runs of the same command (one directory per counter set).
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import os
import sys


def _short(name):
    name = name.replace("void tdc::", "").replace("(tdc::ConvKParams)", "")
    return name if len(name) <= 60 else name[:57] + "..."


def _is_conv(name):
    """A dispatch of one of the convolution kernels (staged, streamed, streamed Winograd)."""
    return "tdc_conv" in name or "tdc_wino" in name


def kernel_summary(path, out=sys.stdout):
    files = sorted(glob.glob(os.path.join(path, "**", "*kernel_trace.csv"), recursive=True))
    if not files:
        raise SystemExit(f"no *kernel_trace.csv under {path}")
    acc = collections.defaultdict(list)
    for f in files:
        for r in csv.DictReader(open(f)):
            key = (_short(r["Kernel_Name"]), int(r["Grid_Size_X"]), int(r["Grid_Size_Y"]), int(r["Workgroup_Size_X"]),
                   int(r.get("LDS_Block_Size", 0) or 0))
            acc[key].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) * 1e-3)
    rows = sorted(acc.items(), key=lambda kv: -sum(kv[1]))
    out.write("%-60s %9s %6s %5s %7s %7s %9s %9s %9s\n" % ("kernel", "grid_x", "grid_y", "wg", "lds", "calls", "mean_us",
                                                       "min_us", "max_us"))
    for (name, gx, gy, wg, lds), v in rows:
        out.write("%-60s %9d %6d %5d %7d %7d %9.3f %9.3f %9.3f\n" % (name, gx, gy, wg, lds, len(v), sum(v) / len(v), min(v),
                                                                   max(v)))
    return rows


def pmc_summary(path, copy_bytes=None, out=sys.stdout):
    files = sorted(glob.glob(os.path.join(path, "**", "*counter_collection.csv"), recursive=True))
    if not files:
        raise SystemExit(f"no *counter_collection.csv under {path}")
    acc = collections.defaultdict(lambda: collections.defaultdict(list))
    for f in files:
        for r in csv.DictReader(open(f)):
            key = (_short(r["Kernel_Name"]), int(r["Grid_Size"]), int(r["Workgroup_Size"]))
            acc[key][r["Counter_Name"]].append(float(r["Counter_Value"]))
    scale = {}
    if copy_bytes:
        # the biggest copy-like kernel of the run is the calibration copy
        for cname in ("FETCH_SIZE", "WRITE_SIZE"):
            best = 0.0
            for (name, _, _), ctrs in acc.items():
                if cname in ctrs and ("copy" in name.lower() or "elementwise" in name.lower()):
                    best = max(best, max(ctrs[cname]))
            if best > 0:
                scale[cname] = copy_bytes / (best * 1024.0)
                out.write("# %s of the %d-byte copy kernel: %.1f KiB -> 1 counted KiB = %.4f KiB moved\n" % (
                    cname, copy_bytes, best, scale[cname]))
    for (name, grid, wg), ctrs in sorted(acc.items(), key=lambda kv: -kv[0][1]):
        for cname, v in sorted(ctrs.items()):
            mean = sum(v) / len(v)
            line = "%-60s grid %9d wg %5d  %-28s n=%5d mean=%16.2f" % (name, grid, wg, cname, len(v), mean)
            if cname in scale:
                line += "   scaled bytes/launch = %.0f" % (mean * 1024.0 * scale[cname])
            out.write(line + "\n")


def timeline(path, last, out=sys.stdout):
    files = sorted(glob.glob(os.path.join(path, "**", "*kernel_trace.csv"), recursive=True))
    if not files:
        raise SystemExit(f"no *kernel_trace.csv under {path}")
    rows = []
    for f in files:
        rows += list(csv.DictReader(open(f)))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    rows = rows[-last:]
    t0 = int(rows[0]["Start_Timestamp"])
    prev_end, busy, idle = None, 0.0, 0.0
    out.write("%3s %-58s %8s %5s %9s %8s %7s\n" % ("#", "kernel", "grid_x", "wg", "start_us", "dur_us", "gap_us"))
    for i, r in enumerate(rows):
        b, e = int(r["Start_Timestamp"]), int(r["End_Timestamp"])
        gap = 0.0 if prev_end is None else (b - prev_end) * 1e-3
        busy += (e - b) * 1e-3
        idle += max(gap, 0.0)
        out.write("%3d %-58s %8d %5d %9.2f %8.2f %7.2f\n" % (i, _short(r["Kernel_Name"])[:58], int(r["Grid_Size_X"]),
                                                            int(r["Workgroup_Size_X"]), (b - t0) * 1e-3, (e - b) * 1e-3, gap))
        prev_end = e
    out.write("# %d kernels: first start to last end %.2f us; sum of durations %.2f us; idle between kernels %.2f us\n" % (
        len(rows), (prev_end - t0) * 1e-3, busy, idle))


def duration_classes(path, out=sys.stdout, min_len=20):
    """Dispatches grouped by kernel, launch geometry and duration class (nearest half microsecond): what loops of
    dependent launches of one kernel with different run times (the launch probe with its spin times) look like in a
    trace.  The duration is the kernel alone; the start-to-start interval (median over the class, to the previous
    dispatch in the trace) is the launch-to-launch time UNDER THE TRACER, which serialises dispatches."""
    files = sorted(glob.glob(os.path.join(path, "**", "*kernel_trace.csv"), recursive=True))
    if not files:
        raise SystemExit(f"no *kernel_trace.csv under {path}")
    rows = []
    for f in files:
        rows += list(csv.DictReader(open(f)))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    acc = collections.defaultdict(lambda: ([], []))
    prev = None
    for r in rows:
        d = (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) * 1e-3
        key = (_short(r["Kernel_Name"]), int(r["Grid_Size_X"]), int(r["Workgroup_Size_X"]), round(d * 2.0) / 2.0)
        acc[key][0].append(d)
        if prev is not None:
            acc[key][1].append((int(r["Start_Timestamp"]) - prev) * 1e-3)
        prev = int(r["Start_Timestamp"])
    out.write("%-52s %9s %5s %6s %8s %9s %9s %9s %9s %15s\n" % ("kernel", "grid_x", "wg", "class", "launches", "mean_dur",
                                                               "p10_dur", "median", "p90_dur", "start_to_start"))
    for (name, gx, wg, cls), (d, gaps) in sorted(acc.items()):
        if len(d) < min_len:
            continue
        d.sort()
        gaps.sort()
        out.write("%-52s %9d %5d %6.1f %8d %9.3f %9.3f %9.3f %9.3f %15.3f\n" % (
            name[:52], gx, wg, cls, len(d), sum(d) / len(d), d[len(d) // 10], d[len(d) // 2], d[(9 * len(d)) // 10],
            gaps[len(gaps) // 2] if gaps else float("nan")))


def isolated(path, layers_json, out=sys.stdout):
    """Kernel-only durations per layer from a trace of ``bench.py --isolated-layers`` (every launch followed by a stream
    synchronisation, so a kernel's start-to-end time contains no other kernel): the last (layers x launches)
    convolution dispatches of the trace, in launch order, against the layer list that run printed."""
    import json
    info = None
    for line in open(layers_json):
        line = line.strip()
        if line.startswith("{") and "isolated_layers" in line:
            info = json.loads(line)
    if info is None:
        raise SystemExit(f"no --isolated-layers result line in {layers_json}")
    per = info["launches_per_layer"] - 1          # (the first launch of each layer was its parity check, earlier in the trace)
    files = sorted(glob.glob(os.path.join(path, "**", "*kernel_trace.csv"), recursive=True))
    rows = []
    for f in files:
        rows += [r for r in csv.DictReader(open(f)) if _is_conv(r["Kernel_Name"])]
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    need = per * len(info["layers"])
    if len(rows) < need:
        raise SystemExit(f"trace holds {len(rows)} convolution dispatches, expected at least {need}")
    rows = rows[-need:]
    out.write("# columns: R1 (input channels) R2 (output channels) H=W tile(mf,mb,nb,wm,wn,wk,cch,tw,ks,wl,alg) median_us p10_us"
              "   | kernel, launches, min_us, max_us\n")
    for i, (r1, r2, hw, tile) in enumerate(info["layers"]):
        chunk = rows[i * per:(i + 1) * per]
        names = {_short(r["Kernel_Name"]) for r in chunk}
        if len(names) != 1:
            raise SystemExit(f"layer {i}: the dispatches do not line up with the layer list ({names})")
        d = sorted((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) * 1e-3 for r in chunk)
        out.write("kernel_only_us: %d %d %d %s %.3f %.3f   | %s n=%d min %.3f max %.3f\n" % (
            r1, r2, hw, ",".join(str(v) for v in tile), d[len(d) // 2], d[len(d) // 10], names.pop(), len(d), d[0], d[-1]))


def isolated_pmc(paths, layers_json, copy_bytes=None, out=sys.stdout):
    """Counters per benchmark layer from ``rocprofv3 --pmc`` runs of ``bench.py --isolated-layers`` (one run per counter
    set; `paths` = their output directories): the last (layers x launches) convolution dispatches of each run, in
    dispatch order, against the layer list the run printed; mean over the launches of a layer.  FETCH_SIZE and
    WRITE_SIZE are scaled by what the run's calibration copy of `copy_bytes` bytes reads."""
    import json
    info = None
    for line in open(layers_json):
        line = line.strip()
        if line.startswith("{") and "isolated_layers" in line:
            info = json.loads(line)
    if info is None:
        raise SystemExit(f"no --isolated-layers result line in {layers_json}")
    per = info["launches_per_layer"]      # (one of them is the layer's parity launch, which comes before all isolated launches)
    nl = len(info["layers"])
    means = [dict() for _ in range(nl)]
    kernels = [None] * nl
    scale = {}
    for path in paths:
        files = sorted(glob.glob(os.path.join(path, "**", "*counter_collection.csv"), recursive=True))
        if not files:
            raise SystemExit(f"no *counter_collection.csv under {path}")
        disp = collections.OrderedDict()
        copies = collections.defaultdict(float)
        for f in files:
            for r in csv.DictReader(open(f)):
                name = _short(r["Kernel_Name"])
                if _is_conv(name):
                    disp.setdefault(int(r["Dispatch_Id"]), (name, {}))[1][r["Counter_Name"]] = float(r["Counter_Value"])
                elif "copy" in name.lower() and r["Counter_Name"] in ("FETCH_SIZE", "WRITE_SIZE"):
                    copies[r["Counter_Name"]] = max(copies[r["Counter_Name"]], float(r["Counter_Value"]))
        if copy_bytes:
            for cname, best in copies.items():
                if best > 0:
                    scale[cname] = copy_bytes / (best * 1024.0)
        ids = sorted(disp)
        # every layer: one parity launch (all of them first), then `per - 1` isolated launches, layer after layer
        need = (per - 1) * nl
        if len(ids) < need:
            raise SystemExit(f"{path}: {len(ids)} convolution dispatches, expected at least {need}")
        ids = ids[-need:]
        for i in range(nl):
            chunk = [disp[d] for d in ids[i * (per - 1):(i + 1) * (per - 1)]]
            names = {c[0] for c in chunk}
            if len(names) != 1:
                raise SystemExit(f"{path}: layer {i}: the dispatches do not line up with the layer list ({names})")
            kernels[i] = names.pop()
            for cname in chunk[0][1]:
                means[i][cname] = sum(c[1][cname] for c in chunk) / len(chunk)
    for cname, sc in sorted(scale.items()):
        out.write("# %s: 1 counted KiB = %.4f KiB moved (from the calibration copy of %d bytes)\n" % (cname, sc, copy_bytes))
    out.write("# per layer: R1 R2 H=W tile | kernel | waves, MFMA instructions, MFMA-busy cycles per SIMD (1024 SIMDs), share of wave "
              "cycles waiting on any instruction, LDS bank-conflict share of LDS-active cycles | L2 read bytes (sectors x 32) "
              "and their ratio to the algorithmic bytes, L2 hit rate | HBM traffic (FETCH_SIZE + WRITE_SIZE, scaled) and its ratio\n")
    for i, (r1, r2, hw, tile) in enumerate(info["layers"]):
        m = means[i]
        alg = 4.0 * (r1 * hw * hw + r2 * hw * hw + 9 * r1 * r2)
        g = lambda k: m.get(k, float("nan"))
        l2 = g("TCC_READ_SECTORS_sum") * 32.0
        hbm = g("FETCH_SIZE") * 1024.0 * scale.get("FETCH_SIZE", 1.0) + g("WRITE_SIZE") * 1024.0 * scale.get("WRITE_SIZE", 1.0)
        out.write("layer_counters: %d %d %d %s | %s | waves %d mfma %d busy/simd %.0f wait %.0f%% lds_conflict %.0f%% | "
                  "l2_read %.2f MB x%.1f hit %.0f%% | hbm %.2f MB x%.2f\n" % (
                      r1, r2, hw, ",".join(str(v) for v in tile), kernels[i], g("SQ_WAVES"), g("SQ_INSTS_MFMA"),
                      g("SQ_VALU_MFMA_BUSY_CYCLES") / 1024.0, 100.0 * g("SQ_WAIT_INST_ANY") / max(g("SQ_WAVE_CYCLES"), 1.0),
                      100.0 * g("SQ_LDS_BANK_CONFLICT") / max(g("SQ_LDS_IDX_ACTIVE"), 1.0) if g("SQ_LDS_IDX_ACTIVE") > 0 else 0.0,
                      l2 * 1e-6, l2 / alg, 100.0 * g("TCC_HIT_sum") / max(g("TCC_REQ_sum"), 1.0), hbm * 1e-6, hbm / alg))


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("mode", choices=["kernel", "pmc", "timeline", "durations", "isolated", "isolated-pmc"])
    ap.add_argument("path")
    ap.add_argument("--copy-bytes", type=int, default=None)
    ap.add_argument("--layers", default=None, help="isolated: file holding the JSON line bench.py --isolated-layers printed")
    ap.add_argument("--last", type=int, default=64, help="timeline: how many dispatches from the end of the trace")
    a = ap.parse_args(argv)
    if a.mode == "isolated-pmc":
        if not a.layers:
            raise SystemExit("isolated-pmc: --layers <file with the output of bench.py --isolated-layers> is required")
        isolated_pmc(a.path.split(","), a.layers, a.copy_bytes)
    elif a.mode == "isolated":
        if not a.layers:
            raise SystemExit("isolated: --layers <file with the output of bench.py --isolated-layers> is required")
        isolated(a.path, a.layers)
    elif a.mode == "kernel":
        kernel_summary(a.path)
    elif a.mode == "timeline":
        timeline(a.path, a.last)
    elif a.mode == "durations":
        duration_classes(a.path)
    else:
        pmc_summary(a.path, a.copy_bytes)


if __name__ == "__main__":
    main()
