"""Host objects over the C ABI.  torch is used for device memory and streams only."""
from __future__ import annotations

from ctypes import byref, c_void_p

import torch

from . import _lib
from ._lib import ConvDesc, Tile, TileInfo, TKConvDesc, check, lib


def _stream_ptr():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _host_f32(t):
    if t is None:
        return None
    return t.detach().to(device="cpu", dtype=torch.float32).contiguous()


def _dev_check(t, shape, what):
    if not t.is_cuda:
        raise ValueError(f"{what} must be a device tensor")
    if t.dtype != torch.float32:
        raise TypeError(f"{what} must be float32")
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{what} has shape {tuple(t.shape)}, expected {tuple(shape)}")
    if not t.is_contiguous():
        raise ValueError(f"{what} must be contiguous NCHW")


class Conv2dPlan:
    """One convolution (optionally + bias, + residual, ReLU) on the GPU.

    Counterpart of the reference's native ``Conv`` object
    (2080Ti-evaluation/EndToEnd/resnet18-tk/inc/common.h:38-69): ``initialize``
    = constructor + ``set_weights``; ``forward`` takes/returns device tensors.
    """

    def __init__(self, batch, C, N, H, W, KH, KW, stride=1, pad=0, dilation=1, bias=False, relu=False, tile=None,
                 tail=None):
        """``tail=(tail_N, tail_bias, tail_relu)`` fuses a 1x1 convolution with tail_N outputs behind this one
        (``bias`` / ``relu`` then act between the two); the output has tail_N channels."""
        self.desc = _lib.conv_desc(batch, C, N, H, W, KH, KW, stride, pad, dilation, bias, relu)
        self._h = c_void_p()
        tptr = byref(tile) if tile is not None else None
        self.tail = tail
        if tail is None:
            check(lib().tdc_conv_plan_create(byref(self.desc), tptr, byref(self._h)))
        else:
            check(lib().tdc_conv_plan_create_with_tail(byref(self.desc), int(tail[0]), int(bool(tail[1])),
                                                       int(bool(tail[2])), tptr, byref(self._h)))
        self.info = TileInfo()
        check(lib().tdc_conv_plan_query(self._h, byref(self.info)))
        self.Ho = _out_dim(H, KH, stride, pad, dilation)
        self.Wo = _out_dim(W, KW, stride, pad, dilation)

    def set_weights(self, weight, bias=None):
        d = self.desc
        w = _host_f32(weight)
        if tuple(w.shape) != (d.N, d.C, d.KH, d.KW):
            raise ValueError(f"weight has shape {tuple(w.shape)}, expected {(d.N, d.C, d.KH, d.KW)}")
        b = _host_f32(bias)
        if b is not None and tuple(b.shape) != (d.N,):
            raise ValueError("bias must have shape [N]")
        check(lib().tdc_conv_plan_set_weights(self._h, c_void_p(w.data_ptr()),
                                              c_void_p(b.data_ptr()) if b is not None else None))
        return self

    def set_tail_weights(self, weight, bias=None):
        """Weights [tail_N, N] (or [tail_N, N, 1, 1]) and bias [tail_N] of the fused 1x1 tail."""
        w, b = _host_f32(weight), _host_f32(bias)
        if self.tail is None or w.numel() != self.tail[0] * self.desc.N:
            raise ValueError("tail weight must be [tail_N, N]")
        check(lib().tdc_conv_plan_set_tail_weights(self._h, c_void_p(w.data_ptr()),
                                                   c_void_p(b.data_ptr()) if b is not None else None))
        return self

    def set_head(self, weight):
        """Fuse a 1x1 convolution [C, head_C] (or [C, head_C, 1, 1]) in front of a streamed 3x3 plan with a fused tail:
        with the tail, a whole TKConv in one launch.  The plan's input then has head_C channels."""
        w = _host_f32(weight)
        if w.dim() not in (2, 4) or w.shape[0] != self.desc.C or w.numel() != w.shape[0] * w.shape[1]:
            raise ValueError("head weight must be [C, head_C]")
        check(lib().tdc_conv_plan_set_head(self._h, int(w.shape[1]), c_void_p(w.data_ptr())))
        self.head_C = int(w.shape[1])
        return self

    def set_input_affine(self, scale, shift, relu=True):
        """y = conv(relu?(x * scale[c] + shift[c])) in one kernel (1x1 convolutions without padding only)."""
        sc, sh = _host_f32(scale), _host_f32(shift)
        if sc.numel() != self.desc.C or sh.numel() != self.desc.C:
            raise ValueError(f"scale and shift must have {self.desc.C} elements")
        check(lib().tdc_conv_plan_set_input_affine(self._h, c_void_p(sc.data_ptr()), c_void_p(sh.data_ptr()), int(relu)))
        return self

    def forward(self, x, residual=None, out=None):
        d = self.desc
        _dev_check(x, (d.batch, getattr(self, "head_C", None) or d.C, d.H, d.W), "input")
        oshape = (d.batch, self.tail[0] if self.tail else d.N, self.Ho, self.Wo)
        if out is None:
            out = torch.empty(oshape, device=x.device, dtype=torch.float32)
        else:
            _dev_check(out, oshape, "out")
        rp = None
        if residual is not None:
            _dev_check(residual, oshape, "residual")
            rp = c_void_p(residual.data_ptr())
        check(lib().tdc_conv_forward(self._h, c_void_p(x.data_ptr()), rp, c_void_p(out.data_ptr()), _stream_ptr()))
        return out

    __call__ = forward

    def forward_static_ws(self, x, residual=None, out=None):
        """``forward`` through tdc_conv_forward_static_ws: the partial tiles and counters of a split across workgroups
        live in the library's static device array instead of plan-owned buffers (for callers that cannot allocate)."""
        d = self.desc
        _dev_check(x, (d.batch, getattr(self, "head_C", None) or d.C, d.H, d.W), "input")
        oshape = (d.batch, self.tail[0] if self.tail else d.N, self.Ho, self.Wo)
        if out is None:
            out = torch.empty(oshape, device=x.device, dtype=torch.float32)
        else:
            _dev_check(out, oshape, "out")
        rp = None
        if residual is not None:
            _dev_check(residual, oshape, "residual")
            rp = c_void_p(residual.data_ptr())
        check(lib().tdc_conv_forward_static_ws(self._h, c_void_p(x.data_ptr()), rp, c_void_p(out.data_ptr()), _stream_ptr()))
        return out

    def occupancy(self):
        """What the compiled kernel of this plan uses (registers per lane, resident workgroups per compute unit as the
        HIP runtime computes them) next to the tile model's assumptions: a ``_lib.KernelOccupancy``."""
        occ = _lib.KernelOccupancy()
        check(lib().tdc_conv_plan_occupancy(self._h, byref(occ)))
        return occ

    def time_us(self, x, out, residual=None, iters=100, graph=True):
        """Device microseconds per launch: hipEvents around `iters` back-to-back launches issued from C
        (replayed from one HIP graph when `graph`)."""
        import ctypes
        ms = ctypes.c_float(0.0)
        rp = c_void_p(residual.data_ptr()) if residual is not None else None
        check(lib().tdc_conv_time(self._h, c_void_p(x.data_ptr()), rp, c_void_p(out.data_ptr()), iters,
                                  int(graph), byref(ms)))
        return ms.value * 1e3 / iters

    def close(self):
        if self._h:
            lib().tdc_conv_plan_destroy(self._h)
            self._h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def time_many_ms(plans, xs, outs, iters=1, graph=True):
    """Device milliseconds of `iters` passes over the list of (plan, input, output), launched from C."""
    import ctypes
    n = len(plans)
    P = (c_void_p * n)(*[p._h for p in plans])
    X = (c_void_p * n)(*[c_void_p(x.data_ptr()) for x in xs])
    O = (c_void_p * n)(*[c_void_p(o.data_ptr()) for o in outs])
    ms = ctypes.c_float(0.0)
    check(lib().tdc_conv_time_many(P, X, O, n, iters, int(graph), byref(ms)))
    return ms.value


def launch_floor_us(launches=300, graph=False, grid=256, block=512, spin_us=0.0):
    """Device microseconds per launch of `launches` dependent probe kernels (the convolution kernels' argument block,
    no memory access, every wave busy for `spin_us`): the launch floor with spin_us = 0."""
    import ctypes
    ms = ctypes.c_float(0.0)
    check(lib().tdc_launch_floor_time(launches, int(graph), grid, block, float(spin_us), byref(ms)))
    return ms.value * 1e3 / launches


def _out_dim(n, k, stride, pad, dil):
    return (n + 2 * pad - dil * (k - 1) - 1) // stride + 1


class TKConvOp:
    """Handle on a native tdc_tkconv (1x1 -> KxK core -> 1x1) for a fixed input shape."""

    def __init__(self, batch, C, R1, R2, N, H, W, K, stride=1, pad=0, dilation=1, bias=False, relu=False):
        self.desc = TKConvDesc(batch, C, R1, R2, N, H, W, K, stride, pad, dilation, int(bias), int(relu))
        self._h = c_void_p()
        check(lib().tdc_tkconv_create(byref(self.desc), byref(self._h)))
        self.Ho = _out_dim(H, K, stride, pad, dilation)
        self.Wo = _out_dim(W, K, stride, pad, dilation)

    def set_weights(self, first, core, last, bias=None):
        d = self.desc
        f, c, l, b = _host_f32(first), _host_f32(core), _host_f32(last), _host_f32(bias)
        if tuple(f.shape) != (d.R1, d.C, 1, 1) or tuple(c.shape) != (d.R2, d.R1, d.K, d.K) \
                or tuple(l.shape) != (d.N, d.R2, 1, 1):
            raise ValueError("factor/core kernel shapes do not match the descriptor")
        check(lib().tdc_tkconv_set_weights(self._h, c_void_p(f.data_ptr()), c_void_p(c.data_ptr()),
                                           c_void_p(l.data_ptr()),
                                           c_void_p(b.data_ptr()) if b is not None else None))
        return self

    def forward(self, x, residual=None, out=None):
        d = self.desc
        _dev_check(x, (d.batch, d.C, d.H, d.W), "input")
        oshape = (d.batch, d.N, self.Ho, self.Wo)
        if out is None:
            out = torch.empty(oshape, device=x.device, dtype=torch.float32)
        else:
            _dev_check(out, oshape, "out")
        rp = None
        if residual is not None:
            _dev_check(residual, oshape, "residual")
            rp = c_void_p(residual.data_ptr())
        check(lib().tdc_tkconv_forward(self._h, c_void_p(x.data_ptr()), rp, c_void_p(out.data_ptr()), _stream_ptr()))
        return out

    def forward_features(self, x):
        d = self.desc
        _dev_check(x, (d.batch, d.C, d.H, d.W), "input")
        f1 = torch.empty((d.batch, d.R1, d.H, d.W), device=x.device, dtype=torch.float32)
        f2 = torch.empty((d.batch, d.R2, self.Ho, self.Wo), device=x.device, dtype=torch.float32)
        out = torch.empty((d.batch, d.N, self.Ho, self.Wo), device=x.device, dtype=torch.float32)
        check(lib().tdc_tkconv_forward_features(self._h, c_void_p(x.data_ptr()), c_void_p(f1.data_ptr()),
                                                c_void_p(f2.data_ptr()), c_void_p(out.data_ptr()), _stream_ptr()))
        return out, [f1, f2, out]

    def core_forward(self, x, out=None):
        d = self.desc
        _dev_check(x, (d.batch, d.R1, d.H, d.W), "core input")
        if out is None:
            out = torch.empty((d.batch, d.R2, self.Ho, self.Wo), device=x.device, dtype=torch.float32)
        check(lib().tdc_tkconv_core_forward(self._h, c_void_p(x.data_ptr()), c_void_p(out.data_ptr()), _stream_ptr()))
        return out

    @property
    def num_kernels(self):
        """Launches per forward: 3, 2 (core + last factor fused) or 1 (the first factor fused in front as well)."""
        return int(lib().tdc_tkconv_num_kernels(self._h))

    def query(self, which):
        info = TileInfo()
        check(lib().tdc_tkconv_query(self._h, which, byref(info)))
        return info

    def close(self):
        if self._h:
            lib().tdc_tkconv_destroy(self._h)
            self._h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
