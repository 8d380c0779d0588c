"""Pins the WIRING of oracle/nets_ref.py (which BatchNorm follows which convolution, where the residual enters, where
the stride sits, in which order a dense block concatenates) with special parameter settings for which the mathematics
fixes the answer, so that a plausible wiring mistake fails one of them.  The convolution / TKConv pieces themselves are
pinned in test_oracle.py.  Block structure as read from the reference: inference/resnet_inet_tt.py:102-117
(TTBasicBlock.forward), :380-394 (TTResNet.forward), inference/densenet_inet_tt.py:96-112, 132-158.  CPU only."""
import torch
import torch.nn.functional as F

from oracle import nets_ref
from tdc_amd import nets


class Recording(dict):
    """A parameter dictionary that remembers which keys were read."""

    def __init__(self, *a):
        super().__init__(*a)
        self.read = set()

    def __getitem__(self, k):
        self.read.add(k)
        return super().__getitem__(k)


def identity_bn(p):
    """Every BatchNorm becomes the identity up to 1 / sqrt(1 + eps)."""
    for k in p:
        if k.endswith(".running_mean") or (k.endswith(".bias") and (".bn" in k or "norm" in k or "downsample.1" in k or k == "bn1.bias")):
            p[k] = torch.zeros_like(p[k])
        if k.endswith(".running_var") or (k.endswith(".weight") and k[:-7] + ".running_var" in p):
            p[k] = torch.ones_like(p[k])
    return p


BN_GAIN = 1.0 / (1.0 + nets_ref.BN_EPS) ** 0.5


def bn_shift(p, prefix):
    scale = p[prefix + ".weight"] / torch.sqrt(p[prefix + ".running_var"] + nets_ref.BN_EPS)
    return scale, p[prefix + ".bias"] - p[prefix + ".running_mean"] * scale


def resnet_case(seed=18):
    p = nets.resnet18_params(seed=seed)
    x = torch.randn(1, 3, 64, 64, generator=torch.Generator().manual_seed(seed))
    return p, x


def test_resnet_parameter_names_and_stage_shapes():
    """The key set is the reference's module tree (conv1, bn1, layerS.B.{conv1,bn1,conv2,bn2}, layerS.0.downsample.{0,1}
    from stage 2 on, fc; Tucker convolutions hold first_kernel / core_kernel / last_kernel, inference/TKConv.py:64-66),
    the oracle reads every key and no other, and the stages have the shapes of a ResNet-18."""
    p, x = resnet_case()
    bn = lambda pre: {pre + s for s in (".weight", ".bias", ".running_mean", ".running_var")}
    want = {"conv1.weight", "fc.weight", "fc.bias"} | bn("bn1")
    for s in range(1, 5):
        for b in range(2):
            for c in ("conv1", "conv2"):
                want |= {f"layer{s}.{b}.{c}.{k}" for k in ("first_kernel", "core_kernel", "last_kernel")}
            want |= bn(f"layer{s}.{b}.bn1") | bn(f"layer{s}.{b}.bn2")
        if s > 1:
            want |= {f"layer{s}.0.downsample.0.weight"} | bn(f"layer{s}.0.downsample.1")
    assert set(p) == want
    rec = Recording(p)
    logits, feats = nets_ref.tucker_resnet18_forward(rec, x, return_features=True)
    assert rec.read == want
    assert tuple(logits.shape) == (1, 1000)
    assert tuple(feats["stem"].shape) == (1, 64, 32, 32) and tuple(feats["maxpool"].shape) == (1, 64, 16, 16)
    for s, (planes, hw) in enumerate(((64, 16), (128, 8), (256, 4), (512, 2)), start=1):
        for b in range(2):
            assert tuple(feats[f"layer{s}.{b}"].shape) == (1, planes, hw, hw)


def test_resnet_block_with_a_dead_second_branch_returns_its_identity():
    """Identity BatchNorms and conv2.last_kernel = 0 in every block: the residual branch contributes exactly zero, so a
    block returns relu(identity) — its input where it has no downsample path, else the stride-2 1x1 convolution of its
    INPUT (not of the branch) through the downsample BatchNorm."""
    p, x = resnet_case()
    identity_bn(p)
    for s in range(1, 5):
        for b in range(2):
            p[f"layer{s}.{b}.conv2.last_kernel"].zero_()
    _, feats = nets_ref.tucker_resnet18_forward(p, x, return_features=True)
    prev = feats["maxpool"]
    assert float(prev.min()) >= 0.0
    for s in range(1, 5):
        for b in range(2):
            name = f"layer{s}.{b}"
            want = prev
            if s > 1 and b == 0:
                want = F.relu(F.conv2d(prev, p[name + ".downsample.0.weight"], None, 2) * BN_GAIN)
            torch.testing.assert_close(feats[name], want, rtol=1e-6, atol=1e-7)
            prev = feats[name]


def test_resnet_block_with_all_convolutions_dead_shows_bn2_last_and_the_add_before_the_relu():
    """All six Tucker factors of a block zero, BatchNorms as generated: the branch is the per-channel constant
    bn2(0) = shift2 (bn1's constants never reach the output), and the block returns relu(shift2 + identity)."""
    p, x = resnet_case()
    name = "layer1.1"
    for c in ("conv1", "conv2"):
        for k in ("first_kernel", "core_kernel", "last_kernel"):
            p[f"{name}.{c}.{k}"].zero_()
    _, feats = nets_ref.tucker_resnet18_forward(p, x, return_features=True)
    _, shift2 = bn_shift(p, name + ".bn2")
    assert float(shift2.abs().max()) > 0.01 and float((shift2 < 0).sum()) > 0
    want = F.relu(shift2.view(1, -1, 1, 1) + feats["layer1.0"])
    torch.testing.assert_close(feats[name], want, rtol=1e-6, atol=1e-7)


def test_resnet_block_with_a_dead_first_convolution_shows_bn1_and_relu_between_the_convolutions():
    """conv1 zero: the second Tucker convolution sees the constant image relu(shift1) (bn1's constants, rectified —
    negative entries must vanish), so the block returns relu(bn2(conv2(that image)) + identity).  A stride-2 block, so
    the constant image has the HALVED size and the identity comes through the downsample path."""
    p, x = resnet_case()
    name = "layer2.0"
    p[name + ".conv1.last_kernel"].zero_()
    _, feats = nets_ref.tucker_resnet18_forward(p, x, return_features=True)
    xin = feats["layer1.1"]
    _, shift1 = bn_shift(p, name + ".bn1")
    assert float((shift1 < 0).sum()) > 0
    const = F.relu(shift1).view(1, -1, 1, 1).expand(1, -1, xin.shape[2] // 2, xin.shape[3] // 2)
    branch = F.conv2d(F.conv2d(F.conv2d(const, p[name + ".conv2.first_kernel"]), p[name + ".conv2.core_kernel"], None, 1, 1),
                      p[name + ".conv2.last_kernel"])
    s2, t2 = bn_shift(p, name + ".bn2")
    sd, td = bn_shift(p, name + ".downsample.1")
    ident = F.conv2d(xin, p[name + ".downsample.0.weight"], None, 2) * sd.view(1, -1, 1, 1) + td.view(1, -1, 1, 1)
    want = F.relu(branch * s2.view(1, -1, 1, 1) + t2.view(1, -1, 1, 1) + ident)
    torch.testing.assert_close(feats[name], want, rtol=1e-4, atol=2e-5)


def test_resnet_stride_sits_on_the_core_convolution_of_conv1():
    """The first factor of a stride-2 block runs at the INPUT resolution and the core convolution carries the stride
    (inference/TKConv.py:91-93); the block's output equals the explicit composition on its input, with the downsample
    path reading that same input at stride 2."""
    p, x = resnet_case()
    identity_bn(p)
    name = "layer3.0"
    _, feats = nets_ref.tucker_resnet18_forward(p, x, return_features=True)
    xin = feats["layer2.1"]
    y = F.conv2d(xin, p[name + ".conv1.first_kernel"])
    assert y.shape[2] == xin.shape[2]
    y = F.conv2d(y, p[name + ".conv1.core_kernel"], None, 2, 1)
    assert y.shape[2] == xin.shape[2] // 2
    y = F.relu(F.conv2d(y, p[name + ".conv1.last_kernel"]) * BN_GAIN)
    y = F.conv2d(F.conv2d(F.conv2d(y, p[name + ".conv2.first_kernel"]), p[name + ".conv2.core_kernel"], None, 1, 1),
                 p[name + ".conv2.last_kernel"]) * BN_GAIN
    ident = F.conv2d(xin, p[name + ".downsample.0.weight"], None, 2) * BN_GAIN
    torch.testing.assert_close(feats[name], F.relu(y + ident), rtol=1e-4, atol=2e-5)


def test_resnet_head_is_global_average_then_the_linear_layer():
    p, x = resnet_case()
    p["fc.weight"] = torch.eye(1000, 512)
    p["fc.bias"] = torch.arange(1000, dtype=torch.float32)
    logits, feats = nets_ref.tucker_resnet18_forward(p, x, return_features=True)
    want = torch.zeros(1, 1000)
    want[:, :512] = feats["layer4.1"].mean((2, 3))
    torch.testing.assert_close(logits, want + p["fc.bias"], rtol=1e-6, atol=1e-6)


# ---- Tucker DenseNet-121 ---------------------------------------------------------------------------------------------
def densenet_case(seed=121):
    p = nets.densenet121_params(seed=seed)
    x = torch.randn(1, 3, 64, 64, generator=torch.Generator().manual_seed(seed))
    return p, x


def test_densenet_parameter_names_and_block_shapes():
    p, x = densenet_case()
    bn = lambda pre: {pre + s for s in (".weight", ".bias", ".running_mean", ".running_var")}
    want = {"features.conv0.weight", "classifier.weight", "classifier.bias"} | bn("features.norm0") | bn("features.norm5")
    for b, nl in enumerate((6, 12, 24, 16), start=1):
        for l in range(1, nl + 1):
            pre = f"features.denseblock{b}.denselayer{l}"
            want |= bn(pre + ".norm1") | bn(pre + ".norm2") | {pre + ".conv1.weight"}
            want |= {pre + ".conv2." + k for k in ("first_kernel", "core_kernel", "last_kernel")}
        if b < 4:
            want |= bn(f"features.transition{b}.norm") | {f"features.transition{b}.conv.weight"}
    assert set(p) == want
    rec = Recording(p)
    logits, feats = nets_ref.tucker_densenet121_forward(rec, x, return_features=True)
    assert rec.read == want and tuple(logits.shape) == (1, 1000)
    assert tuple(feats["stem"].shape) == (1, 64, 32, 32)
    for b, (c, hw) in enumerate(((256, 16), (512, 8), (1024, 4), (1024, 2)), start=1):
        assert tuple(feats[f"denseblock{b}"].shape) == (1, c, hw, hw)


def test_densenet_block_with_dead_layers_is_its_input_followed_by_zeros():
    """Every last factor zero: each layer appends 32 zero channels, so a block's output is its input in the first
    channels and zero elsewhere; the first block's input is the 3x3 / stride 2 / pad 1 max pool of the stem."""
    p, x = densenet_case()
    for k in p:
        if k.endswith("conv2.last_kernel"):
            p[k].zero_()
    _, feats = nets_ref.tucker_densenet121_forward(p, x, return_features=True)
    b1 = feats["denseblock1"]
    torch.testing.assert_close(b1[:, :64], F.max_pool2d(feats["stem"], 3, 2, 1), rtol=0, atol=0)
    assert float(b1[:, 64:].abs().max()) == 0.0
    # transition: norm + ReLU, 1x1 convolution to half the channels, THEN the 2x2 average pool
    s, t = bn_shift(p, "features.transition1.norm")
    y = F.relu(b1 * s.view(1, -1, 1, 1) + t.view(1, -1, 1, 1))
    y = F.avg_pool2d(F.conv2d(y, p["features.transition1.conv.weight"]), 2, 2)
    b2 = feats["denseblock2"]
    torch.testing.assert_close(b2[:, :128], y, rtol=1e-4, atol=2e-5)
    assert float(b2[:, 128:].abs().max()) == 0.0


def test_densenet_layers_append_in_order_and_read_everything_before_them():
    """Only layer 3 of the first block alive: its 32 channels sit at offset 64 + 2 * 32.  With layer 1 alive as well,
    layer 3's channels change (it reads layer 1's output) while layer 1's own slice does not depend on layer 3."""
    p, x = densenet_case()
    saved = {k: p[k].clone() for k in p if k.endswith("conv2.last_kernel")}
    for k in saved:
        p[k].zero_()
    k1 = "features.denseblock1.denselayer1.conv2.last_kernel"
    k3 = "features.denseblock1.denselayer3.conv2.last_kernel"
    p[k3] = saved[k3].clone()
    _, f3 = nets_ref.tucker_densenet121_forward(p, x, return_features=True)
    b = f3["denseblock1"]
    alive = (b[:, 64:].abs().amax((0, 2, 3)) > 0).nonzero().flatten() + 64    # (the first 64 channels are the block's input)
    assert int(alive.min()) >= 128 and int(alive.max()) < 160 and len(alive) > 16
    p[k1] = saved[k1].clone()
    _, f13 = nets_ref.tucker_densenet121_forward(p, x, return_features=True)
    b13 = f13["denseblock1"]
    assert float((b13[:, 128:160] - b[:, 128:160]).abs().max()) > 1e-4
    p[k3].zero_()
    _, f1 = nets_ref.tucker_densenet121_forward(p, x, return_features=True)
    torch.testing.assert_close(f1["denseblock1"][:, 64:96], b13[:, 64:96], rtol=0, atol=0)
    # inside a layer: norm1 + ReLU on the concatenation, 1x1 bottleneck, norm2 + ReLU, then the Tucker convolution
    cat = b13[:, :64]
    pre = "features.denseblock1.denselayer1"
    s1, t1 = bn_shift(p, pre + ".norm1")
    s2, t2 = bn_shift(p, pre + ".norm2")
    y = F.conv2d(F.relu(cat * s1.view(1, -1, 1, 1) + t1.view(1, -1, 1, 1)), p[pre + ".conv1.weight"])
    y = F.relu(y * s2.view(1, -1, 1, 1) + t2.view(1, -1, 1, 1))
    y = F.conv2d(F.conv2d(F.conv2d(y, p[pre + ".conv2.first_kernel"]), p[pre + ".conv2.core_kernel"], None, 1, 1),
                 p[pre + ".conv2.last_kernel"])
    torch.testing.assert_close(b13[:, 64:96], y, rtol=1e-4, atol=2e-5)


def test_densenet_head_is_norm5_relu_global_average_classifier():
    p, x = densenet_case()
    p["classifier.weight"] = torch.eye(1000, 1024)
    p["classifier.bias"] = torch.zeros(1000)
    logits, feats = nets_ref.tucker_densenet121_forward(p, x, return_features=True)
    s, t = bn_shift(p, "features.norm5")
    want = torch.zeros(1, 1000)
    want[:, :1000] = F.relu(feats["denseblock4"] * s.view(1, -1, 1, 1) + t.view(1, -1, 1, 1)).mean((2, 3))[:, :1000]
    torch.testing.assert_close(logits, want, rtol=1e-4, atol=2e-5)
