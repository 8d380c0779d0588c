"""``TKConv2dC`` on the MI355X library — same constructor, parameters and
``forward`` / ``forward_features`` contract as the reference operator
(inference/TKConv.py:23-141), with the three ``F.conv2d`` calls of its forward
(:90-95) replaced by the native 1x1 -> KxK core -> 1x1 kernels.

Not carried over: initialisation from a dense weight (``dense_w``), which the
reference does with ``tensorly.partial_tucker`` at construction time (:75-80) —
it is init-time work off the inference path; pass already-decomposed kernels
with ``load_kernels`` or a state dict instead.
"""
from __future__ import annotations

import math
from types import SimpleNamespace

import torch
from torch import nn

from .conv import TKConvOp


def _pair(v):
    return tuple(v) if isinstance(v, (tuple, list)) else (v, v)


class TKConv2dC(nn.Module):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, padding_mode="zeros", hp_dict=None, name=None, dense_w=None, dense_b=None):
        if groups != 1:
            raise ValueError("groups must be 1 in this mode")
        if padding_mode != "zeros":
            raise ValueError("padding_mode must be zero in this mode")
        if dense_w is not None:
            raise NotImplementedError(
                "construction from a dense weight (partial Tucker decomposition) is init-time work "
                "outside this library; decompose offline and call load_kernels()")
        super().__init__()
        kernel_size, stride, padding, dilation = _pair(kernel_size), _pair(stride), _pair(padding), _pair(dilation)
        for what, v in (("kernel_size", kernel_size), ("stride", stride), ("padding", padding), ("dilation", dilation)):
            if v[0] != v[1]:
                raise ValueError(f"{what} must be square for the native core conv")
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.ranks = hp_dict.ranks[name]
        self.in_rank = self.ranks[1]
        self.out_rank = self.ranks[0]
        self.kernel_size, self.stride, self.padding, self.dilation = kernel_size, stride, padding, dilation
        self.groups = groups
        self.padding_mode = padding_mode
        self.first_kernel = nn.Parameter(torch.empty(self.in_rank, in_channels, 1, 1))
        self.core_kernel = nn.Parameter(torch.empty(self.out_rank, self.in_rank, *kernel_size))
        self.last_kernel = nn.Parameter(torch.empty(out_channels, self.out_rank, 1, 1))
        if bias:
            self.bias = nn.Parameter(torch.zeros(out_channels))
            if dense_b is not None:
                self.bias.data = dense_b
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()
        self._ops = {}       # (batch, H, W) -> TKConvOp
        self._stamp = None   # parameter versions the native copies were packed from

    def reset_parameters(self):
        nn.init.xavier_uniform_(self.first_kernel)
        nn.init.xavier_uniform_(self.core_kernel)
        nn.init.xavier_uniform_(self.last_kernel)

    def load_kernels(self, first, core, last, bias=None):
        with torch.no_grad():
            self.first_kernel.copy_(first)
            self.core_kernel.copy_(core)
            self.last_kernel.copy_(last)
            if bias is not None:
                self.bias.copy_(bias)
        return self

    def _versions(self):
        ps = [self.first_kernel, self.core_kernel, self.last_kernel] + ([self.bias] if self.bias is not None else [])
        return tuple((p.data_ptr(), p._version) for p in ps)

    def _op_for(self, x):
        if x.dim() != 4 or x.shape[1] != self.in_channels:
            raise ValueError(f"expected input [B,{self.in_channels},H,W], got {tuple(x.shape)}")
        stamp = self._versions()
        if stamp != self._stamp:      # parameters changed: re-pack on next use
            for op in self._ops.values():
                op.close()
            self._ops.clear()
            self._stamp = stamp
        key = (x.shape[0], x.shape[2], x.shape[3])
        op = self._ops.get(key)
        if op is None:
            op = TKConvOp(x.shape[0], self.in_channels, self.in_rank, self.out_rank, self.out_channels,
                          x.shape[2], x.shape[3], self.kernel_size[0], self.stride[0], self.padding[0],
                          self.dilation[0], bias=self.bias is not None)
            op.set_weights(self.first_kernel, self.core_kernel, self.last_kernel, self.bias)
            self._ops[key] = op
        return op

    @torch.no_grad()
    def forward(self, x):
        return self._op_for(x).forward(x.contiguous())

    @torch.no_grad()
    def forward_features(self, x):
        return self._op_for(x).forward_features(x.contiguous())

    def extra_repr(self):
        return ("first_conv(in={}, out={}, kernel_size=(1, 1), bias=False), "
                "core_conv(in={}, out={}, kernel_size={}, stride={}, padding={}, bias={}), "
                "last_conv(in={}, out={}, kernel_size=(1, 1), bias=False)").format(
            self.in_channels, self.in_rank, self.in_rank, self.out_rank, self.kernel_size, self.stride,
            self.padding, self.bias is None, self.out_rank, self.out_channels)


def ranks_dict(**ranks):
    """Minimal stand-in for the reference's hp_dict objects: ``ranks_dict(conv1=[out_rank, in_rank]).ranks``."""
    return SimpleNamespace(ranks=dict(ranks))
