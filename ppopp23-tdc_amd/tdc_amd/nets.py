"""Whole-network forward graphs on the native library (tdc_net_*).

``Net`` wraps the C handle.  ``build_tucker_resnet18`` lays out the reference's
Tucker-compressed ResNet-18 (inference/resnet_inet_tt.py:53-117 ``TTBasicBlock``,
:287-394 ``TTResNet`` with ``[2,2,2,2]`` blocks; every 3x3 convolution a
``TKConv2dC``) from a state-dict-style parameter dictionary whose keys are the
reference's (``layer1.0.conv1.first_kernel`` ...).  BatchNorm (inference mode) is
folded into the weights and bias of the convolution in front of it at build time;
ReLU and the residual add run in the convolution epilogues; the whole forward is
one HIP-graph launch.
"""
from __future__ import annotations

import ctypes
import math
from ctypes import byref, c_int32, c_void_p

import torch

from . import _lib
from ._lib import check, lib

BN_EPS = 1e-5


def _h(t):
    return None if t is None else t.detach().to(device="cpu", dtype=torch.float32).contiguous()


def _p(t):
    return None if t is None else c_void_p(t.data_ptr())


class Net:
    def __init__(self, batch, C, H, W):
        self._h = c_void_p()
        check(lib().tdc_net_create(batch, C, H, W, byref(self._h)))
        self.batch = batch
        self.input_id = 0
        self.output_id = None
        self._keep = []
        self.conv_shapes = []   # (C, N, H, W, K, stride, pad) of every convolution launched per forward, in order

    def tensor(self, C, H, W):
        out = c_int32()
        check(lib().tdc_net_tensor(self._h, C, H, W, byref(out)))
        return out.value

    def view(self, tid, c0, C):
        out = c_int32()
        check(lib().tdc_net_view(self._h, tid, c0, C, byref(out)))
        return out.value

    def conv(self, x, weight, bias=None, stride=1, pad=0, residual=-1, relu=False, dst=-1):
        w, b = _h(weight), _h(bias)
        out = c_int32()
        _, C, H, W = self.shape(x)
        self.conv_shapes.append((C, w.shape[0], H, W, w.shape[2], stride, pad))
        check(lib().tdc_net_conv(self._h, x, w.shape[0], w.shape[2], w.shape[3], stride, pad, _p(w), _p(b), residual,
                                 int(relu), dst, byref(out)))
        return out.value

    def conv_tail(self, x, weight, tail_weight, bias=None, relu=False, tail_bias=None, stride=1, pad=0, residual=-1,
                  tail_relu=False, dst=-1, in_affine=None):
        """Convolution with a 1x1 convolution fused behind it (one kernel); ``in_affine=(scale, shift, relu)`` adds
        a per-channel affine on the input (1x1 convolutions without padding only)."""
        w, b, w2, b2 = _h(weight), _h(bias), _h(tail_weight), _h(tail_bias)
        out = c_int32()
        _, C, H, W = self.shape(x)
        self.conv_shapes.append((C, w.shape[0], H, W, w.shape[2], stride, pad))
        check(lib().tdc_net_conv_tail(self._h, x, w.shape[0], w.shape[2], w.shape[3], stride, pad, _p(w), _p(b), int(relu),
                                      w2.shape[0], _p(w2), _p(b2), residual, int(tail_relu), dst, byref(out)))
        if in_affine is not None:
            sc, sh = _h(in_affine[0]), _h(in_affine[1])
            check(lib().tdc_net_set_input_affine(self._h, _p(sc), _p(sh), int(in_affine[2])))
        return out.value

    def affine_conv(self, x, scale, shift, weight, bias=None, affine_relu=True, residual=-1, relu=False, dst=-1):
        """relu?(x*scale+shift) followed by a 1x1 convolution, in one kernel."""
        sc, sh, w, b = _h(scale), _h(shift), _h(weight), _h(bias)
        out = c_int32()
        _, C, H, W = self.shape(x)
        self.conv_shapes.append((C, w.shape[0], H, W, 1, 1, 0))
        check(lib().tdc_net_affine_conv(self._h, x, _p(sc), _p(sh), int(affine_relu), w.shape[0], _p(w), _p(b), residual,
                                        int(relu), dst, byref(out)))
        return out.value

    def tkconv(self, x, first, core, last, bias=None, stride=1, pad=0, residual=-1, relu=False, dst=-1):
        f, c, l, b = _h(first), _h(core), _h(last), _h(bias)
        out = c_int32()
        _, C, H, W = self.shape(x)
        K = c.shape[2]
        Ho, Wo = (H + 2 * pad - K) // stride + 1, (W + 2 * pad - K) // stride + 1
        self.conv_shapes += [(C, f.shape[0], H, W, 1, 1, 0), (f.shape[0], c.shape[0], H, W, K, stride, pad),
                             (c.shape[0], l.shape[0], Ho, Wo, 1, 1, 0)]
        check(lib().tdc_net_tkconv(self._h, x, f.shape[0], c.shape[0], l.shape[0], c.shape[2], stride, pad, _p(f), _p(c),
                                   _p(l), _p(b), residual, int(relu), dst, byref(out)))
        return out.value

    def pool(self, x, mode, k, stride, pad=0, dst=-1):
        out = c_int32()
        check(lib().tdc_net_pool(self._h, x, {"max": 0, "avg": 1}[mode], k, stride, pad, dst, byref(out)))
        return out.value

    def affine(self, x, scale, shift, relu=True, dst=-1):
        s, t = _h(scale), _h(shift)
        out = c_int32()
        check(lib().tdc_net_affine(self._h, x, _p(s), _p(t), int(relu), dst, byref(out)))
        return out.value

    def global_avgpool(self, x):
        out = c_int32()
        check(lib().tdc_net_global_avgpool(self._h, x, byref(out)))
        return out.value

    def concat(self, ids):
        arr = (c_int32 * len(ids))(*ids)
        out = c_int32()
        check(lib().tdc_net_concat(self._h, arr, len(ids), byref(out)))
        return out.value

    def shape(self, tid):
        c, h, w = c_int32(), c_int32(), c_int32()
        check(lib().tdc_net_tensor_shape(self._h, tid, byref(c), byref(h), byref(w)))
        return (self.batch, c.value, h.value, w.value)

    def finalize(self, output_id):
        check(lib().tdc_net_finalize(self._h, output_id))
        self.output_id = output_id
        return self

    @property
    def num_kernels(self):
        return lib().tdc_net_num_kernels(self._h)

    def forward(self, x):
        """x: device tensor [B,C,H,W]; returns a new device tensor with the output."""
        if not x.is_cuda or x.dtype != torch.float32 or tuple(x.shape) != self.shape(0) or not x.is_contiguous():
            raise ValueError(f"input must be a contiguous float32 device tensor of shape {self.shape(0)}")
        out = torch.empty(self.shape(self.output_id), device=x.device, dtype=torch.float32)
        s = c_void_p(torch.cuda.current_stream().cuda_stream)
        check(lib().tdc_net_forward(self._h, c_void_p(x.data_ptr()), c_void_p(out.data_ptr()), s))
        return out

    __call__ = forward

    def time_ms(self, iters=100, graph=True):
        ms = ctypes.c_float(0.0)
        check(lib().tdc_net_time(self._h, iters, int(graph), byref(ms)))
        return ms.value / iters

    def read(self, tid):
        out = torch.empty(self.shape(tid), dtype=torch.float32)
        check(lib().tdc_net_read_tensor(self._h, tid, c_void_p(out.data_ptr())))
        return out

    def close(self):
        if self._h:
            lib().tdc_net_destroy(self._h)
            self._h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


# ---------------------------------------------------------------------------------------------------
def bn_scale_shift(p, prefix):
    """Inference-mode BatchNorm as y = x*scale + shift."""
    scale = p[prefix + ".weight"] / torch.sqrt(p[prefix + ".running_var"] + BN_EPS)
    shift = p[prefix + ".bias"] - p[prefix + ".running_mean"] * scale
    return scale, shift


def fold_dense(weight, scale):
    return weight * scale.reshape(-1, 1, 1, 1)


RESNET18_STAGES = ((64, 1), (128, 2), (256, 2), (512, 2))   # (planes, stride of the first block)


def resnet18_params(seed=18, num_classes=1000, rank_ratio=0.5):
    """Random-init Tucker ResNet-18 with the reference's state-dict key names: Kaiming-normal convolutions,
    non-trivial BatchNorm statistics (so that the folding is exercised), ranks R1 = R2 = planes * rank_ratio.
    The Kaiming gain of 2 is applied once per ReLU, not once per convolution: a Tucker convolution is three linear
    maps in a row with a single ReLU behind them (first factor and core get gain 1, the last factor gain 2), and the
    BatchNorm that closes a residual branch is scaled by 0.3, so activations stay of order one through all eight
    blocks instead of growing by orders of magnitude, and element-wise tolerances mean something."""
    g = torch.Generator().manual_seed(seed)

    def kaiming(*shape, gain=2.0):
        fan_in = shape[1] * shape[2] * shape[3]
        return torch.empty(*shape).normal_(0, math.sqrt(gain / fan_in), generator=g)

    def bn(prefix, n, p, scale=1.0):
        p[prefix + ".weight"] = (torch.rand(n, generator=g) * 0.5 + 0.75) * scale
        p[prefix + ".bias"] = torch.randn(n, generator=g) * 0.1
        p[prefix + ".running_mean"] = torch.randn(n, generator=g) * 0.1
        p[prefix + ".running_var"] = torch.rand(n, generator=g) * 0.5 + 0.75

    p = {"conv1.weight": kaiming(64, 3, 7, 7)}
    bn("bn1", 64, p)
    inplanes = 64
    for s, (planes, stride) in enumerate(RESNET18_STAGES, start=1):
        r = int(planes * rank_ratio)
        for b in range(2):
            cin = inplanes if b == 0 else planes
            for k, c in (("conv1", cin), ("conv2", planes)):
                pre = f"layer{s}.{b}.{k}"
                p[pre + ".first_kernel"] = kaiming(r, c, 1, 1, gain=1.0)
                p[pre + ".core_kernel"] = kaiming(r, r, 3, 3, gain=1.0)
                p[pre + ".last_kernel"] = kaiming(planes, r, 1, 1)
                bn(f"layer{s}.{b}.bn{k[-1]}", planes, p, scale=0.3 if k == "conv2" else 1.0)
            if b == 0 and (stride != 1 or inplanes != planes):
                p[f"layer{s}.0.downsample.0.weight"] = kaiming(planes, inplanes, 1, 1)
                bn(f"layer{s}.0.downsample.1", planes, p)
        inplanes = planes
    p["fc.weight"] = torch.empty(num_classes, 512).normal_(0, 0.01, generator=g)
    p["fc.bias"] = torch.randn(num_classes, generator=g) * 0.01
    return p


def _basic_block(net, x, p, pre, blk_stride, fused_middle):
    """One TTBasicBlock (inference/resnet_inet_tt.py:53-117): conv1 (TKConv) + bn1 + ReLU, conv2 (TKConv) + bn2,
    + identity (through the 1x1 downsample convolution + BatchNorm where the block has one), ReLU.  With
    `fused_middle` the last factor of conv1 (with bn1 folded in, + ReLU) and the first factor of conv2 run as ONE kernel
    (a 1x1 convolution with a 1x1 tail): the block's middle tensor of `planes` channels never reaches memory and a
    launch disappears; the two cores and the outer factors are separate launches then."""
    identity = x
    if pre + ".downsample.0.weight" in p:
        ds, dt = bn_scale_shift(p, pre + ".downsample.1")
        identity = net.conv(x, fold_dense(p[pre + ".downsample.0.weight"], ds), dt, stride=blk_stride)
    s1, t1 = bn_scale_shift(p, pre + ".bn1")
    s2, t2 = bn_scale_shift(p, pre + ".bn2")
    last1 = fold_dense(p[pre + ".conv1.last_kernel"], s1)
    last2 = fold_dense(p[pre + ".conv2.last_kernel"], s2)
    if not fused_middle:
        y = net.tkconv(x, p[pre + ".conv1.first_kernel"], p[pre + ".conv1.core_kernel"], last1, t1, stride=blk_stride, pad=1,
                       relu=True)
        return net.tkconv(y, p[pre + ".conv2.first_kernel"], p[pre + ".conv2.core_kernel"], last2, t2, stride=1, pad=1,
                          residual=identity, relu=True)
    y = net.conv(x, p[pre + ".conv1.first_kernel"])
    y = net.conv(y, p[pre + ".conv1.core_kernel"], stride=blk_stride, pad=1)
    y = net.conv_tail(y, last1, p[pre + ".conv2.first_kernel"], bias=t1, relu=True)
    y = net.conv(y, p[pre + ".conv2.core_kernel"], stride=1, pad=1)
    return net.conv(y, last2, t2, residual=identity, relu=True)


_BASIC_BLOCK_FUSES = {}


def _basic_block_fuses(batch, cin, h, w, p, pre, blk_stride):
    """Whether a block runs faster with the middle pair of 1x1 factors fused (see _basic_block).  The fused kernel needs
    every channel of the block's middle tensor in one workgroup, which the kernels offer up to 256 channels.  Without
    measured tile selection the tile model decides (the fused kernel predicted at 0.7 of the two launches or less: timed
    at batch 1 it takes 1.4-3.7x of what two launches take — 64 -> 128 -> 64 @28x28: 7.9 us against 2.7 + 2.8;
    128 -> 256 -> 128 @14x14: 22.9 against 2.9 + 3.1 — because one workgroup per 16-64 pixels owns every channel).  With
    it, both layouts of the block are built as networks of their own and timed (remembered per shape)."""
    planes = p[pre + ".conv1.last_kernel"].shape[0]
    r2 = p[pre + ".conv1.last_kernel"].shape[1]
    if planes > 256:
        return False
    if _lib.get_autotune() <= 0:
        ho, wo = (h + 2 - 3) // blk_stride + 1, (w + 2 - 3) // blk_stride + 1
        d1 = _lib.conv_desc(batch, r2, planes, ho, wo, 1, 1, 1, 0, 1, True, True)
        return _lib.fused_tail_pays(d1, p[pre + ".conv2.first_kernel"].shape[0], margin=0.7)
    key = (batch, cin, h, w, planes, p[pre + ".conv1.first_kernel"].shape[0], blk_stride, pre + ".downsample.0.weight" in p,
           _lib.get_autotune() > 0)
    if key not in _BASIC_BLOCK_FUSES:
        nets, ok = [], True
        for fused in (False, True):
            m = Net(batch, cin, h, w)
            try:
                m.finalize(_basic_block(m, 0, p, pre, blk_stride, fused))
            except _lib.TdcError:      # (no tile carries this tail)
                m.close()
                ok = False
                break
            nets.append(m)
        if not ok:
            _BASIC_BLOCK_FUSES[key] = False
        else:
            x = torch.randn(batch, cin, h, w, device="cuda")
            t = []
            for m in nets:
                m.forward(x)
                m.time_ms(iters=10)
                t.append(min(m.time_ms(iters=30) for _ in range(3)))
            _BASIC_BLOCK_FUSES[key] = t[1] < 0.98 * t[0]
        for m in nets:
            m.close()
    return _BASIC_BLOCK_FUSES[key]


def build_tucker_resnet18(params, batch=1, H=224, W=224):
    """Returns a finalized Net computing the logits [batch, num_classes, 1, 1]."""
    p = params
    net = Net(batch, 3, H, W)
    s, t = bn_scale_shift(p, "bn1")
    net.feature_ids = {}    # tensor ids of the stage outputs, by the names oracle/nets_ref.py uses
    x = net.conv(0, fold_dense(p["conv1.weight"], s), t, stride=2, pad=3, relu=True)      # conv1 + bn1 + relu
    net.feature_ids["stem"] = x
    x = net.pool(x, "max", 3, 2, 1)
    net.feature_ids["maxpool"] = x
    for st, (planes, stride) in enumerate(RESNET18_STAGES, start=1):
        for b in range(2):
            pre = f"layer{st}.{b}"
            blk_stride = stride if b == 0 else 1
            _, cin, h, w = net.shape(x)
            x = _basic_block(net, x, p, pre, blk_stride, _basic_block_fuses(batch, cin, h, w, p, pre, blk_stride))
            net.feature_ids[pre] = x
    x = net.global_avgpool(x)
    x = net.conv(x, p["fc.weight"].reshape(p["fc.weight"].shape[0], -1, 1, 1), p["fc.bias"])
    return net.finalize(x)


# ---------------------------------------------------------------------------------------------------
# Tucker DenseNet-121 (inference/densenet_inet_tt.py:36-158 TenDenseLayer / TenDenseBlock /
# TenDenseTransition; growth 32, bn_size 4, blocks (6, 12, 24, 16)); every 3x3 convolution 128->32 a
# TKConv2dC with ranks (R1, R2) = (64, 16).
DENSENET121_BLOCKS = (6, 12, 24, 16)


def densenet121_params(seed=121, num_classes=1000, growth=32, bn_size=4, ranks=(64, 16)):
    """Random-init Tucker DenseNet-121 with the reference's state-dict key names.  As in ``resnet18_params`` the
    Kaiming gain of 2 goes to the convolutions that read a ReLU's output (conv0, conv1, the first factor, the
    transitions); core and last factor read a linear map's output and get gain 1, so activations stay of order one."""
    g = torch.Generator().manual_seed(seed)

    def kaiming(*shape, gain=2.0):
        fan_in = shape[1] * shape[2] * shape[3]
        return torch.empty(*shape).normal_(0, math.sqrt(gain / fan_in), generator=g)

    def bn(prefix, n, p):
        p[prefix + ".weight"] = torch.rand(n, generator=g) * 0.5 + 0.75
        p[prefix + ".bias"] = torch.randn(n, generator=g) * 0.1
        p[prefix + ".running_mean"] = torch.randn(n, generator=g) * 0.1
        p[prefix + ".running_var"] = torch.rand(n, generator=g) * 0.5 + 0.75

    r1, r2 = ranks
    mid = bn_size * growth
    p = {"features.conv0.weight": kaiming(64, 3, 7, 7)}
    bn("features.norm0", 64, p)
    c = 64
    for b, nl in enumerate(DENSENET121_BLOCKS, start=1):
        for l in range(1, nl + 1):
            pre = f"features.denseblock{b}.denselayer{l}"
            bn(pre + ".norm1", c, p)
            p[pre + ".conv1.weight"] = kaiming(mid, c, 1, 1)
            bn(pre + ".norm2", mid, p)
            p[pre + ".conv2.first_kernel"] = kaiming(r1, mid, 1, 1)
            p[pre + ".conv2.core_kernel"] = kaiming(r2, r1, 3, 3, gain=1.0)
            p[pre + ".conv2.last_kernel"] = kaiming(growth, r2, 1, 1, gain=1.0)
            c += growth
        if b < len(DENSENET121_BLOCKS):
            pre = f"features.transition{b}"
            bn(pre + ".norm", c, p)
            p[pre + ".conv.weight"] = kaiming(c // 2, c, 1, 1)
            c //= 2
    bn("features.norm5", c, p)
    p["classifier.weight"] = torch.empty(num_classes, c).normal_(0, 0.01, generator=g)
    p["classifier.bias"] = torch.randn(num_classes, generator=g) * 0.01
    return p


def _dense_layer(net, src, dst, fused, s1, t1, w1, t2, first, core, last):
    if fused:
        # norm1 + relu, conv1, norm2 + relu and the first Tucker factor in one kernel; core + last in another
        y = net.conv_tail(src, w1, first, bias=t2, relu=True, in_affine=(s1, t1, True))
        return net.conv_tail(y, core, last, pad=1, dst=dst)
    # norm1 + relu on the concatenation, conv1, norm2 + relu: one kernel; then the Tucker convolution
    y = net.affine_conv(src, s1, t1, w1, t2, relu=True)
    return net.tkconv(y, first, core, last, pad=1, dst=dst)


_DENSE_LAYER_FUSES = {}


def _dense_layer_fuses(batch, c, h, w, d1, layer):
    """Whether a dense layer runs faster with its bottleneck convolution and first Tucker factor fused into one kernel
    (and core + last into another) or as bottleneck + Tucker convolution: the model's answer, checked, when the measured
    tile selection is switched on, against a measurement (both variants of the layer are built as a network of their
    own and timed; remembered per shape)."""
    first = layer[4]
    if _lib.model_select_with_tail(d1, first.shape[0]) is None:
        return False
    # (timed at batch 1, the fused kernel with the input affine in front takes 1.5-1.7x what the model predicts: 13.9 us
    #  where the two launches take 9-10; at batch 8 the prediction holds)
    model_fuses = _lib.fused_tail_pays(d1, first.shape[0], margin=0.7 if batch == 1 else 0.9)
    if _lib.get_autotune() <= 0:
        return model_fuses
    key = (batch, c, h, w, tuple(layer[2].shape), tuple(first.shape), tuple(layer[5].shape), tuple(layer[6].shape))
    if key not in _DENSE_LAYER_FUSES:
        x = torch.randn(batch, c, h, w, device="cuda")
        t = []
        for fused in (True, False):
            m = Net(batch, c, h, w)
            m.finalize(_dense_layer(m, 0, -1, fused, *layer))
            m.forward(x)
            m.time_ms(iters=10)
            t.append(min(m.time_ms(iters=30) for _ in range(3)))
            m.close()
        # (a layer timed alone sees warmer caches than inside the network: the model's answer is only overruled by 5 %)
        _DENSE_LAYER_FUSES[key] = (t[0] < 1.05 * t[1]) if model_fuses else (t[0] < 0.95 * t[1])
    return _DENSE_LAYER_FUSES[key]


def build_tucker_densenet121(params, batch=1, H=224, W=224, growth=32):
    """Finalized Net for the logits [batch, num_classes, 1, 1].  The concatenation of a dense block is one
    buffer; every layer's Tucker convolution writes its 32 new channels straight into its slice."""
    p = params
    net = Net(batch, 3, H, W)
    s, t = bn_scale_shift(p, "features.norm0")
    x = net.conv(0, fold_dense(p["features.conv0.weight"], s), t, stride=2, pad=3, relu=True)
    c = 64
    h, w = net.shape(x)[2], net.shape(x)[3]
    h, w = (h + 2 - 3) // 2 + 1, (w + 2 - 3) // 2 + 1
    cat = net.tensor(c + DENSENET121_BLOCKS[0] * growth, h, w)
    net.pool(x, "max", 3, 2, 1, dst=net.view(cat, 0, c))
    net.feature_ids = {"stem": x}    # tensor ids of the block outputs, by the names oracle/nets_ref.py uses
    for b, nl in enumerate(DENSENET121_BLOCKS, start=1):
        for l in range(1, nl + 1):
            pre = f"features.denseblock{b}.denselayer{l}"
            s1, t1 = bn_scale_shift(p, pre + ".norm1")
            s2, t2 = bn_scale_shift(p, pre + ".norm2")
            w1 = fold_dense(p[pre + ".conv1.weight"], s2)
            first, core, last = (p[pre + ".conv2.first_kernel"], p[pre + ".conv2.core_kernel"],
                                 p[pre + ".conv2.last_kernel"])
            d1 = _lib.conv_desc(batch, c, w1.shape[0], h, w, 1, 1, 1, 0, 1, True, True)
            layer = (s1, t1, w1, t2, first, core, last)
            if _dense_layer_fuses(batch, c, h, w, d1, layer):
                _dense_layer(net, net.view(cat, 0, c), net.view(cat, c, growth), True, *layer)
            else:
                _dense_layer(net, net.view(cat, 0, c), net.view(cat, c, growth), False, *layer)
            c += growth
        net.feature_ids[f"denseblock{b}"] = cat
        if b < len(DENSENET121_BLOCKS):
            pre = f"features.transition{b}"
            st, tt = bn_scale_shift(p, pre + ".norm")
            y = net.affine_conv(cat, st, tt, p[pre + ".conv.weight"])
            c //= 2
            h, w = h // 2, w // 2
            cat = net.tensor(c + DENSENET121_BLOCKS[b] * growth, h, w)
            net.pool(y, "avg", 2, 2, 0, dst=net.view(cat, 0, c))
    s5, t5 = bn_scale_shift(p, "features.norm5")
    y = net.affine(cat, s5, t5, relu=True)
    y = net.global_avgpool(y)
    y = net.conv(y, p["classifier.weight"].reshape(p["classifier.weight"].shape[0], -1, 1, 1), p["classifier.bias"])
    return net.finalize(y)
