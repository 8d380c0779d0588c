"""End-to-end Tucker ResNet-18 (benchmark configuration 4) on the GPU against the CPU restatement."""
import sys

import numpy as np
import pytest
import torch

import tdc_amd
from tdc_amd import nets
from oracle import nets_ref
from util import ATOL, RTOL

pytestmark = pytest.mark.gpu


def net_close(got, ref, what):
    """Per element: |got - ref| <= RTOL * |ref| + max(ATOL, 1e-6 * max|ref|).  The layer tolerance (1e-4 relative,
    1e-5 absolute), with the absolute part following the tensor's scale once that exceeds ten: the rounding errors of
    the ~55 stacked fp32 layers in front of an element are proportional to the size of the summands, not to the
    element itself.  The synthetic initialisation keeps every stage of both networks at max|x| of 7 to 30, so the
    absolute part is at most 3e-5."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.shape == ref.shape, what
    err = np.abs(got - ref)
    bound = RTOL * np.abs(ref) + max(ATOL, 1e-6 * np.abs(ref).max())
    bad = ~(err <= bound)
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(f"{what}: {bad.sum()} of {bad.size} outside tolerance; worst at {i}: got {got[i]!r} "
                             f"ref {ref[i]!r} err {err[i]:.3e} (max|ref| {np.abs(ref).max():.3g})")


def check_features(net, feats, what):
    """Every stage output the oracle returns against the network's own tensor of that name."""
    assert set(net.feature_ids) == set(feats), (sorted(net.feature_ids), sorted(feats))
    for name, tid in net.feature_ids.items():
        ref = feats[name].numpy()
        assert 1.0 < np.abs(ref).max() < 100.0, f"{what} {name}: synthetic activations left the range the tolerance assumes"
        net_close(net.read(tid).numpy(), ref, f"{what} {name}")


def test_pool_and_concat_ops():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 6, 13, 11, generator=g)
    net = nets.Net(2, 6, 13, 11)
    a = net.pool(0, "max", 3, 2, 1)
    b = net.pool(0, "avg", 2, 2, 0)
    c = net.global_avgpool(0)
    d = net.concat([0, 0])
    w = torch.randn(4, 12, 1, 1, generator=g)
    e = net.conv(d, w)
    # in-place concatenation: two producers write channel slices of one buffer, a consumer reads a prefix
    cat = net.tensor(10, 13, 11)
    scale, shift = torch.randn(6, generator=g), torch.randn(6, generator=g)
    net.affine(0, scale, shift, relu=True, dst=net.view(cat, 0, 6))
    w2 = torch.randn(4, 6, 3, 3, generator=g) * 0.2
    net.conv(net.view(cat, 0, 6), w2, pad=1, dst=net.view(cat, 6, 4))
    net.finalize(e)
    out = net(x.cuda()).cpu()
    F = torch.nn.functional
    assert torch.equal(net.read(a), F.max_pool2d(x, 3, 2, 1))
    assert torch.allclose(net.read(b), F.avg_pool2d(x, 2, 2), atol=1e-6)
    assert torch.allclose(net.read(c), F.adaptive_avg_pool2d(x, 1), atol=1e-6)
    assert torch.equal(net.read(d), torch.cat([x, x], 1))
    assert torch.allclose(out, F.conv2d(torch.cat([x, x], 1), w), rtol=1e-4, atol=1e-5)
    aff = torch.relu(x * scale.reshape(1, -1, 1, 1) + shift.reshape(1, -1, 1, 1))
    got_cat = net.read(cat)
    assert torch.allclose(got_cat[:, :6], aff, atol=1e-6)
    assert torch.allclose(got_cat[:, 6:], F.conv2d(aff, w2, None, 1, 1), rtol=1e-4, atol=1e-5)
    assert net.num_kernels == 8
    net.close()


def test_tucker_resnet18_logits_and_features():
    p = nets.resnet18_params(seed=18)
    x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(18))
    want, feats = nets_ref.tucker_resnet18_forward(p, x, return_features=True)
    net = nets.build_tucker_resnet18(p, batch=1)
    print("kernels per forward:", net.num_kernels, flush=True)
    sys.stdout.flush()
    got = net(x.cuda())
    torch.cuda.synchronize()
    assert tuple(got.shape) == (1, 1000, 1, 1)
    net_close(got.cpu().numpy().reshape(1, 1000), want.numpy(), "logits")
    # stem, max-pool and the output of each of the eight residual blocks
    check_features(net, feats, "resnet18")
    # graph replays are repeatable and do not depend on what ran in between
    again = net(x.cuda())
    other = net(torch.randn(1, 3, 224, 224).cuda())
    third = net(x.cuda())
    torch.cuda.synchronize()
    assert torch.equal(got, again) and torch.equal(got, third) and not torch.equal(got, other)
    net.close()


def test_resnet18_batch2_small_resolution():
    p = nets.resnet18_params(seed=5, num_classes=10)
    x = torch.randn(2, 3, 64, 64, generator=torch.Generator().manual_seed(6))
    want = nets_ref.tucker_resnet18_forward(p, x)
    net = nets.build_tucker_resnet18(p, batch=2, H=64, W=64)
    got = net(x.cuda()).cpu().numpy().reshape(2, 10)
    net_close(got, want.numpy(), "logits b2")
    net.close()


def test_resnet18_with_measured_tile_selection():
    """The same network with every tile choice (and every core + last fusion) measured at build time: the picks
    may be Winograd or global-weight tiles, the logits must not move beyond the tolerance."""
    import tdc_amd
    p = nets.resnet18_params(seed=18)
    x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(18))
    want = nets_ref.tucker_resnet18_forward(p, x)
    prev = tdc_amd.set_autotune(8)
    try:
        net = nets.build_tucker_resnet18(p, batch=1)
    finally:
        tdc_amd.set_autotune(prev)
    print("kernels per forward:", net.num_kernels, flush=True)
    got = net(x.cuda())
    torch.cuda.synchronize()
    net_close(got.cpu().numpy().reshape(1, 1000), want.numpy(), "logits, measured selection")
    net.close()


@pytest.mark.parametrize("batch,res", [(1, 224), (8, 224), (8, 64)])
def test_tucker_densenet121(batch, res):
    """Benchmark configuration 5: batch 1 and batch 8 at 3x224x224 (plus batch 8 at a reduced resolution, whose small
    images take other tiles), logits and the output of every dense block against the CPU restatement."""
    p = nets.densenet121_params(seed=121)
    x = torch.randn(batch, 3, res, res, generator=torch.Generator().manual_seed(121))
    want, feats = nets_ref.tucker_densenet121_forward(p, x, return_features=True)
    net = nets.build_tucker_densenet121(p, batch=batch, H=res, W=res)
    print("densenet kernels per forward:", net.num_kernels, flush=True)
    got = net(x.cuda()).cpu().numpy().reshape(batch, 1000)
    net_close(got, want.numpy(), f"densenet logits b{batch} @{res}")
    check_features(net, feats, f"densenet b{batch} @{res}")
    net.close()
