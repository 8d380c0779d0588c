"""TEST INFRASTRUCTURE — CPU oracle (never imported by the product package).

Three independent statements of the same convolution, used to check each other
and then the HIP kernels:

* ``conv2d_c`` / ``tkconv_c`` / ``tdc_tiled_c`` — the C restatement in
  ``conv_ref.c`` (double accumulation; plus the reference's own tiled kernel run
  sequentially), loaded through ctypes.
* ``conv2d_numpy`` — an explicit-loop numpy version for tiny shapes.
* ``conv2d_torch`` / ``tkconv_torch`` — ``torch.nn.functional.conv2d`` composed
  exactly as ``TKConv2dC.forward`` composes it
  (reference inference/TKConv.py:90-95).  This is the library routine the
  reference's CPU path executes, so it is also what bench.py times as the CPU
  baseline.

``make_core_case`` / ``make_block_case`` generate the seeded synthetic inputs of
the benchmark configurations.
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def _lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "libtdc_oracle.so")
        if not os.path.exists(so):
            subprocess.check_call(["make", "-C", _HERE, "libtdc_oracle.so"])
        _LIB = ctypes.CDLL(so)
    return _LIB


def _fp(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float)) if a is not None else None


def out_dim(n, k, stride, pad, dil):
    return (n + 2 * pad - dil * (k - 1) - 1) // stride + 1


def _c32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def conv2d_c(x, w, bias=None, resid=None, stride=1, pad=0, dil=1, relu=False):
    """x [B,C,H,W], w [N,C,KH,KW] float32 numpy -> [B,N,Ho,Wo] (conv_ref.c ref_conv2d)."""
    x, w, bias, resid = _c32(x), _c32(w), _c32(bias), _c32(resid)
    B, C, H, W = x.shape
    N, C2, KH, KW = w.shape
    assert C == C2
    Ho, Wo = out_dim(H, KH, stride, pad, dil), out_dim(W, KW, stride, pad, dil)
    out = np.empty((B, N, Ho, Wo), np.float32)
    rc = _lib().ref_conv2d(_fp(x), _fp(w), _fp(bias), _fp(resid), _fp(out), B, C, N, H, W, KH, KW,
                           stride, pad, dil, int(relu))
    if rc:
        raise ValueError("ref_conv2d rejected the shape")
    return out


def tkconv_c(x, first, core, last, bias=None, stride=1, pad=0, dil=1):
    """Returns (out, f1, f2) as float32 numpy (conv_ref.c ref_tkconv)."""
    x, first, core, last, bias = _c32(x), _c32(first), _c32(core), _c32(last), _c32(bias)
    B, C, H, W = x.shape
    R1, R2, N, K = first.shape[0], core.shape[0], last.shape[0], core.shape[2]
    Ho, Wo = out_dim(H, K, stride, pad, dil), out_dim(W, K, stride, pad, dil)
    f1 = np.empty((B, R1, H, W), np.float32)
    f2 = np.empty((B, R2, Ho, Wo), np.float32)
    out = np.empty((B, N, Ho, Wo), np.float32)
    rc = _lib().ref_tkconv(_fp(x), _fp(first), _fp(core), _fp(last), _fp(bias), _fp(f1), _fp(f2), _fp(out),
                           B, C, R1, R2, N, H, W, K, stride, pad, dil)
    if rc:
        raise ValueError("ref_tkconv rejected the shape")
    return out, f1, f2


def tdc_tiled_c(x, w, TH, TW, TC):
    """The reference kernel run sequentially: x [C,H,W], w [N,C,3,3] -> [N,H,W]."""
    x, w = _c32(x), _c32(w)
    C, H, W = x.shape
    N = w.shape[0]
    out = np.empty((N, H, W), np.float32)
    rc = _lib().ref_tdc_tiled(_fp(x), _fp(w), _fp(out), C, N, H, W, TH, TW, TC)
    if rc:
        raise ValueError("ref_tdc_tiled rejected the tiling (TC must divide C)")
    return out


def conv2d_numpy(x, w, bias=None, stride=1, pad=0, dil=1):
    """Explicit loops in float64; tiny shapes only."""
    x = np.asarray(x, np.float64)
    w = np.asarray(w, np.float64)
    B, C, H, W = x.shape
    N, _, KH, KW = w.shape
    Ho, Wo = out_dim(H, KH, stride, pad, dil), out_dim(W, KW, stride, pad, dil)
    xp = np.zeros((B, C, H + 2 * pad, W + 2 * pad))
    xp[:, :, pad:pad + H, pad:pad + W] = x
    out = np.zeros((B, N, Ho, Wo))
    for oy in range(Ho):
        for ox in range(Wo):
            for r in range(KH):
                for s in range(KW):
                    out[:, :, oy, ox] += xp[:, :, oy * stride + r * dil, ox * stride + s * dil] @ w[:, :, r, s].T
    if bias is not None:
        out += np.asarray(bias, np.float64)[None, :, None, None]
    return out


def conv2d_torch(x, w, bias=None, stride=1, pad=0, dil=1):
    import torch.nn.functional as F
    return F.conv2d(x, w, bias, stride, pad, dil, 1)


def tkconv_torch(x, first, core, last, bias=None, stride=1, pad=0, dil=1):
    """TKConv2dC.forward (reference inference/TKConv.py:90-95)."""
    import torch.nn.functional as F
    out = F.conv2d(x, first)
    out = F.conv2d(out, core, None, stride, pad, dil, 1)
    return F.conv2d(out, last, bias)


# --------------------------------------------------------------------------
# Seeded synthetic inputs of the benchmark configurations (generated on CPU).
# --------------------------------------------------------------------------
SWEEP_HW = (7, 14, 28, 56)
SWEEP_RANKS = ((16, 16), (32, 32), (64, 64), (96, 96), (128, 128), (32, 64), (64, 128))
BLOCKS = ((256, 64, 64, 256, 56), (512, 128, 128, 512, 28), (1024, 192, 192, 1024, 14), (2048, 256, 256, 2048, 7))


def core_seed(hw, r1, r2):
    return hw * 1_000_000 + r1 * 1_000 + r2


def make_core_case(hw, r1, r2, seed=None, batch=1):
    """x ~ U[-1,1] [batch,r1,hw,hw]; w ~ N(0, 2/(9 r1)) [r2,r1,3,3] (Kaiming-normal, fan_in)."""
    import torch
    g = torch.Generator().manual_seed(core_seed(hw, r1, r2) if seed is None else seed)
    x = torch.rand(batch, r1, hw, hw, generator=g) * 2 - 1
    w = torch.empty(r2, r1, 3, 3).normal_(0, math.sqrt(2.0 / (r1 * 9)), generator=g)
    return x, w


def make_block_case(C, R1, R2, N, hw, batch=1):
    """Full Tucker block: x ~ N(0,1); factors with orthonormal columns (QR of Gaussian); core ~ N(0, 0.02^2)."""
    import torch
    g = torch.Generator().manual_seed(C)
    x = torch.randn(batch, C, hw, hw, generator=g)
    q1, _ = torch.linalg.qr(torch.randn(C, R1, generator=g))
    first = q1.t().contiguous().reshape(R1, C, 1, 1)
    q2, _ = torch.linalg.qr(torch.randn(N, R2, generator=g))
    last = q2.contiguous().reshape(N, R2, 1, 1)
    core = torch.randn(R2, R1, 3, 3, generator=g) * 0.02
    return x, first, core, last
