"""Per-wave time line of one convolution launch, from the time stamps of the PROFILING build of the library.

    make -C ppopp23-tdc_amd/csrc STAMPS=1 OUT=/tmp/tdc_stamps/libtdc_amd.so OBJDIR=/tmp/tdc_stamps/build RESOURCES=/dev/null all
    TDC_AMD_LIBRARY=/tmp/tdc_stamps/libtdc_amd.so python -m tdc_amd.stamps C,N,HW[,K] mf,mb,nb,wm,wn,wk,cch,tw,ks,wl,alg [tile ...]

(from ppopp23-tdc_amd, or with it on PYTHONPATH; K = 3 (default: 3x3, pad 1) or 1 (1x1, pad 0)).  The profiling build
compiles s_memrealtime reads (the 100 MHz constant clock: 10 ns per tick) into the staged kernel's Winograd path and into
the streamed kernels (1x1, 3x3, 3x3 with several pixel blocks per wave, Winograd; these have no pass loop and take stamps
0, 1, 4, 5, 6, 7 only), at the phase boundaries

    0 entry   1 every operand request of the first pass issued   2 this wave's copies landed   3 barrier: all landed
    4 multiply loop done   5 partial results parked in LDS, barrier   6 output stores issued   7 kernel arguments cached

and exports tdc_debug_read_stamps.  Each tile is timed back to back first (the stamps cost ~0.5 us per launch), then
launched alone five times, and the stamps of the last launch are summarised: when the phases end relative to the
first wave's entry, how long each takes per wave (mean, p10, p50, p90, max), and the same by wave index of the
workgroup (waves 0-3 and 4-7 of an 8-wave workgroup share the four SIMDs in pairs).  The reference times its candidate
kernels from outside only (2080Ti-evaluation/TDC-LAYERS-ORACLE/template_benchmark_cudnn.template:455-496)."""
import ctypes
import sys

import numpy as np
import torch

import tdc_amd
from tdc_amd.conv import Conv2dPlan

PHASES = ["entry -> requests issued", "issued -> mine landed", "mine landed -> barrier", "multiply loop",
          "park in LDS + barrier", "store issue"]


def timeline(c, n, hw, tile_text, k=3):
    v = [int(a) for a in tile_text.split(",")]
    tile = tdc_amd.Tile(*v[:8], ks=v[8], wl=v[9], alg=v[10])
    gen = torch.Generator().manual_seed(7)
    x = torch.randn(1, c, hw, hw, generator=gen)
    w = torch.randn(n, c, k, k, generator=gen) * (2.0 / (k * k * c)) ** 0.5
    xd = x.cuda()
    out = torch.empty(1, n, hw, hw, device="cuda")
    lib = tdc_amd.lib()
    if not hasattr(lib, "tdc_debug_read_stamps"):
        sys.exit("this library has no time stamps: build it with STAMPS=1 and point TDC_AMD_LIBRARY at it")
    lib.tdc_debug_read_stamps.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64,
                                          ctypes.POINTER(ctypes.c_uint64)]
    plan = Conv2dPlan(1, c, n, hw, hw, k, k, 1, k // 2, tile=tile).set_weights(w)
    us = min(plan.time_us(xd, out, iters=100) for _ in range(3))
    for _ in range(5):   # isolated launches; the stamps of the last one are read
        plan.forward(xd, out=out)
        torch.cuda.synchronize()
    words = plan.info.grid_x * plan.info.grid_y * plan.info.grid_z * 16 * 8
    buf = np.zeros(words, dtype=np.uint64)
    got = ctypes.c_uint64(0)
    if lib.tdc_debug_read_stamps(plan._h, buf.ctypes.data_as(ctypes.c_void_p), words, ctypes.byref(got)) != 0:
        sys.exit("tdc_debug_read_stamps failed")
    s = buf.reshape(-1, 16, 8).astype(np.int64)
    live = s[:, :, 0] > 0
    st = s[live]                       # [waves, 8]
    t0 = st[:, 0].min()
    rel = (st - t0) * 0.01             # microseconds
    print("== %d->%d @%d %s tile %s: %.2f us back to back; %d waves of %d workgroups stamped"
          % (c, n, hw, "1x1" if k == 1 else "3x3", tile_text, us, int(live.sum()), s.shape[0]))
    print("   kernel span (first entry -> last store issue): %.2f us; entries spread over %.2f us"
          % (rel[:, 6].max(), rel[:, 0].max()))
    for i, name in enumerate(PHASES):
        ok = (st[:, i] > 0) & (st[:, i + 1] > 0)
        if not ok.any():
            continue
        d = (rel[:, i + 1] - rel[:, i])[ok]
        end = rel[:, i + 1][ok]
        print("   %-26s mean %.2f  p10 %.2f  p50 %.2f  p90 %.2f  max %.2f   (phase ends at: mean %.2f max %.2f)"
              % (name, d.mean(), np.percentile(d, 10), np.percentile(d, 50), np.percentile(d, 90), d.max(),
                 end.mean(), end.max()))
    if (st[:, 7] > 0).any():
        ka = (st[:, 7] - st[:, 0]) * 0.01
        print("   kernel arguments in the scalar cache after: mean %.2f p10 %.2f p90 %.2f max %.2f"
              % (ka.mean(), np.percentile(ka, 10), np.percentile(ka, 90), ka.max()))
    nwv = int(live[0].sum())
    ent = (s[:, :, 0] - t0) * 0.01
    pro = (s[:, :, 1] - s[:, :, 0]) * 0.01
    cols = []
    have_loop = bool(((s[:, :, 3] > 0) & (s[:, :, 4] > 0))[live].all())
    loop = (s[:, :, 4] - s[:, :, 3]) * 0.01
    for wv in range(nwv):
        m = live[:, wv]
        text = "w%d entry %.2f prologue %.2f" % (wv, ent[:, wv][m].mean(), pro[:, wv][m].mean())
        if have_loop:
            text += " loop %.2f" % loop[:, wv][m].mean()
        cols.append(text)
    print("   by wave index:  " + "  ".join(cols))
    plan.close()


def main():
    if len(sys.argv) < 3:
        sys.exit(__doc__)
    shape = [int(v) for v in sys.argv[1].split(",")]
    c, n, hw = shape[:3]
    k = shape[3] if len(shape) > 3 else 3
    if k not in (1, 3):
        sys.exit("K must be 1 or 3")
    for tile_text in sys.argv[2:]:
        timeline(c, n, hw, tile_text, k)


if __name__ == "__main__":
    main()
