"""TEST INFRASTRUCTURE — restatement of the reference's analytic tile model
(2080Ti-evaluation/TDC-LAYERS-MODELING/model.py), used only to document what the
gfx950 model replaces and to check the volumes it reasons about.

Everything is integer arithmetic on (C, N, H, W, th, tw, tc) with a 3x3 filter.
"""
import math


def compute_latency(C, N, H, W, th, tw, tc, r, s, sms, ths_sm, occupancy):
    """model.py:136-144.  `occupancy` is the measured CUDA-occupancy-API value the
    reference looks up in its recorded table (model.py:141)."""
    flops = (th + r - 1) * (tw + s - 1) * tc * r * s
    bnum = math.ceil(H / th) * math.ceil(C / tc)
    bdim = math.ceil(W / tw) * N
    bnums_one_wave = math.floor((sms * ths_sm * occupancy) / bdim)
    waves = math.ceil(bnum / bnums_one_wave)
    return flops * waves, bnum, bdim


def compute_input_vol(C, N, H, W, th, tw, tc):
    """model.py:146-148"""
    return math.ceil(H / th) * (th + 2) * (W + 2) * C


def compute_out_vol(C, N, H, W, th, tw, tc):
    """model.py:149-152 (counts the partial-sum writes of every channel slab)"""
    bnum = math.ceil(H / th) * math.ceil(W / tw) * math.ceil(C / tc)
    return th * tw * N * bnum


def compute_kernel_vol(C, N, H, W, th, tw, tc):
    """model.py:153-156"""
    bnum = math.ceil(H / th) * math.ceil(W / tw) * math.ceil(C / tc)
    return 3 * 3 * tc * N * bnum


def launch_shape(C, N, H, W, th, tw, tc):
    """Grid, block and dynamic shared memory of the reference kernel
    (TDC-LAYERS-ORACLE/template_benchmark_cudnn.template:490-492)."""
    ths, tws, tcs = math.ceil(H / th), math.ceil(W / tw), math.ceil(C / tc)
    return tcs * ths, N * tws, tc * (th + 2) * (tws * tw + 2) * 4
