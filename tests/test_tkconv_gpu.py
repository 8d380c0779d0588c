"""GPU parity of the TKConv operator (tdc_tkconv_* and the TKConv2dC module) against the CPU oracle."""
import sys

import numpy as np
import pytest
import torch

import tdc_amd
from oracle import ref
from util import assert_close, seeded

pytestmark = pytest.mark.gpu


def announce(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("blk", ref.BLOCKS, ids=lambda b: "C%d_R%d_%d_N%d_H%d" % b)
def test_full_tucker_block_matches_reference_composition(blk):
    """Benchmark configuration 3: 1x1 C->R1, 3x3 R1->R2 pad 1, 1x1 R2->N; orthonormal factors, Gaussian core."""
    C, R1, R2, N, hw = blk
    announce("block", blk)
    x, first, core, last = ref.make_block_case(C, R1, R2, N, hw)
    op = tdc_amd.TKConvOp(1, C, R1, R2, N, hw, hw, 3, 1, 1, 1).set_weights(first, core, last)
    out, feats = op.forward_features(x.cuda())
    torch.cuda.synchronize()
    want = ref.tkconv_torch(x, first, core, last, None, 1, 1, 1)
    assert_close(out.cpu().numpy(), want.numpy(), f"block {blk}")
    f1 = ref.conv2d_torch(x, first)
    f2 = ref.conv2d_torch(f1, core, pad=1)
    assert_close(feats[0].cpu().numpy(), f1.numpy(), "first feature")
    assert_close(feats[1].cpu().numpy(), f2.numpy(), "core feature")
    assert feats[2] is out
    # the core conv alone, on the reference's intermediate
    got_core = op.core_forward(f1.cuda()).cpu().numpy()
    assert_close(got_core, f2.numpy(), "core_forward")
    for which in range(3):
        assert op.query(which).pred_us > 0
    op.close()


def test_block_against_c_oracle_small():
    g = seeded(77)
    x = torch.randn(2, 20, 9, 11, generator=g)
    first = torch.randn(6, 20, 1, 1, generator=g) * 0.3
    core = torch.randn(10, 6, 3, 3, generator=g) * 0.2
    last = torch.randn(14, 10, 1, 1, generator=g) * 0.3
    bias = torch.randn(14, generator=g)
    for stride in (1, 2):
        announce("small block stride", stride)
        op = tdc_amd.TKConvOp(2, 20, 6, 10, 14, 9, 11, 3, stride, 1, 1, bias=True).set_weights(first, core, last, bias)
        got = op.forward(x.cuda()).cpu().numpy()
        want, _, _ = ref.tkconv_c(x.numpy(), first.numpy(), core.numpy(), last.numpy(), bias.numpy(), stride, 1, 1)
        assert_close(got, want, f"small block stride {stride}")
        op.close()


@pytest.mark.parametrize("shape", [(1, 32, 16, 16, 32, 14, 14), (2, 64, 32, 32, 64, 28, 28), (1, 64, 32, 32, 64, 56, 56), (3, 20, 6, 10, 14, 9, 11)])
@pytest.mark.parametrize("measured", [False, True])
def test_whole_operator_in_one_launch(shape, measured):
    """Small first factors are fused in front of core + last factor (one launch per TKConv): same answer as the
    oracle's three convolutions with bias, residual and ReLU on the last one, whether the choice is the model's or
    measured, and the feature maps of forward_features still come from the three separate plans."""
    B, C, R1, R2, N, H, W = shape
    g = seeded(880 + C + H)
    x = torch.rand(B, C, H, W, generator=g) * 2 - 1
    first = torch.randn(R1, C, 1, 1, generator=g) / C ** 0.5
    core = torch.randn(R2, R1, 3, 3, generator=g) * (2.0 / (9 * R1)) ** 0.5
    last = torch.randn(N, R2, 1, 1, generator=g) / R2 ** 0.5
    bias = torch.randn(N, generator=g)
    resid = torch.randn(B, N, H, W, generator=g)
    want, f1, f2 = ref.tkconv_c(x.numpy(), first.numpy(), core.numpy(), last.numpy(), bias.numpy(), 1, 1, 1)
    want = np.maximum(want + resid.numpy(), 0.0)
    prev = tdc_amd.set_autotune(4 if measured else 0)
    try:
        op = tdc_amd.TKConvOp(B, C, R1, R2, N, H, W, 3, 1, 1, 1, bias=True, relu=True).set_weights(first, core, last, bias)
    finally:
        tdc_amd.set_autotune(prev)
    announce("whole TKConv", shape, "measured" if measured else "model", "kernels", op.num_kernels)
    if not measured:
        assert op.num_kernels == 1
    got = op.forward(x.cuda(), resid.cuda()).cpu().numpy()
    assert_close(got, want, f"one-launch TKConv {shape}")
    _, feats = op.forward_features(x.cuda())
    assert_close(feats[0].cpu().numpy(), f1, "first feature")
    assert_close(feats[1].cpu().numpy(), f2, "core feature")
    op.close()


def test_module_forward_matches_reference_forward():
    """TKConv2dC.forward(x) == F.conv2d(F.conv2d(F.conv2d(x, first), core, None, stride, padding, dilation), last, bias)."""
    torch.manual_seed(5)
    hp = tdc_amd.ranks_dict(layer1=[24, 16])
    m = tdc_amd.TKConv2dC(40, 48, 3, stride=1, padding=1, bias=True, hp_dict=hp, name="layer1")
    with torch.no_grad():
        m.bias.copy_(torch.randn(48))
    x = torch.randn(1, 40, 28, 28)
    want = ref.tkconv_torch(x, m.first_kernel.detach(), m.core_kernel.detach(), m.last_kernel.detach(), m.bias.detach(),
                            1, 1, 1)
    got = m(x.cuda())
    assert got.is_cuda and tuple(got.shape) == (1, 48, 28, 28)
    assert_close(got.cpu().numpy(), want.numpy(), "module forward")
    out, feats = m.forward_features(x.cuda())
    assert len(feats) == 3 and tuple(feats[0].shape) == (1, 16, 28, 28) and tuple(feats[1].shape) == (1, 24, 28, 28)
    assert_close(out.cpu().numpy(), want.numpy(), "module forward_features")
    # a second input shape and a parameter update are both picked up
    x2 = torch.randn(2, 40, 14, 14)
    with torch.no_grad():
        m.core_kernel.mul_(0.5)
    want2 = ref.tkconv_torch(x2, m.first_kernel.detach(), m.core_kernel.detach(), m.last_kernel.detach(), m.bias.detach(),
                             1, 1, 1)
    assert_close(m(x2.cuda()).cpu().numpy(), want2.numpy(), "module after update")
    # writes through .data do not bump the version counter: invalidate() (or load_state_dict / load_kernels) re-packs
    m.last_kernel.data[1:-1].mul_(-2.0)          # (the stamp — storage address and version counter — cannot see it)
    m.invalidate()
    want3 = ref.tkconv_torch(x2, m.first_kernel.detach(), m.core_kernel.detach(), m.last_kernel.detach(), m.bias.detach(),
                             1, 1, 1)
    assert_close(m(x2.cuda()).cpu().numpy(), want3.numpy(), "module after invalidate()")
    sd = {k: v.clone() * 0.5 for k, v in m.state_dict().items()}
    m.load_state_dict(sd)
    want4 = ref.tkconv_torch(x2, sd["first_kernel"], sd["core_kernel"], sd["last_kernel"], sd["bias"], 1, 1, 1)
    assert_close(m(x2.cuda()).cpu().numpy(), want4.numpy(), "module after load_state_dict")
    # a module moved to the device works too, and a forward with unchanged parameters reads no parameter element
    # (the stamp is addresses and version counters only), so it can run with the device's copy engines busy or idle alike
    m.cuda()
    assert_close(m(x2.cuda()).cpu().numpy(), want4.numpy(), "module after .cuda()")
    assert all(isinstance(v, int) for pair in m._versions() for v in pair)
    m.cpu()
    # the per-shape operator cache is bounded
    for hw in range(5, 5 + m.MAX_CACHED_SHAPES + 3):
        m(torch.randn(1, 40, hw, hw).cuda())
    assert len(m._ops) == m.MAX_CACHED_SHAPES


def test_module_stride2_no_bias_and_load_kernels():
    hp = tdc_amd.ranks_dict(down=[32, 32])
    m = tdc_amd.TKConv2dC(64, 64, 3, stride=2, padding=1, bias=False, hp_dict=hp, name="down")
    g = seeded(9)
    first, core, last = (torch.randn(32, 64, 1, 1, generator=g) * .1, torch.randn(32, 32, 3, 3, generator=g) * .1,
                         torch.randn(64, 32, 1, 1, generator=g) * .1)
    m.load_kernels(first, core, last)
    x = torch.randn(1, 64, 56, 56, generator=g)
    got = m(x.cuda()).cpu().numpy()
    assert got.shape == (1, 64, 28, 28)
    assert_close(got, ref.tkconv_torch(x, first, core, last, None, 2, 1, 1).numpy(), "stride-2 module")


def test_densenet_style_batch8_layer():
    """Configuration 5's Tucker layer: 1x1 128->64, core 64->16, 1x1 16->32, batch 8."""
    g = seeded(121)
    x = torch.randn(8, 128, 14, 14, generator=g)
    first = torch.randn(64, 128, 1, 1, generator=g) * 0.1
    core = torch.randn(16, 64, 3, 3, generator=g) * 0.1
    last = torch.randn(32, 16, 1, 1, generator=g) * 0.2
    op = tdc_amd.TKConvOp(8, 128, 64, 16, 32, 14, 14, 3, 1, 1, 1).set_weights(first, core, last)
    got = op.forward(x.cuda()).cpu().numpy()
    assert_close(got, ref.tkconv_torch(x, first, core, last, None, 1, 1, 1).numpy(), "densenet layer b8")
    op.close()


def test_fused_residual_and_relu_on_the_last_factor():
    g = seeded(31)
    x = torch.randn(1, 16, 10, 10, generator=g)
    first, core, last = (torch.randn(8, 16, 1, 1, generator=g) * .3, torch.randn(8, 8, 3, 3, generator=g) * .2,
                         torch.randn(16, 8, 1, 1, generator=g) * .3)
    bias = torch.randn(16, generator=g)
    op = tdc_amd.TKConvOp(1, 16, 8, 8, 16, 10, 10, 3, 1, 1, 1, bias=True, relu=True).set_weights(first, core, last, bias)
    got = op.forward(x.cuda(), residual=x.cuda()).cpu().numpy()
    want = torch.relu(ref.tkconv_torch(x, first, core, last, bias, 1, 1, 1) + x).numpy()
    assert_close(got, want, "residual + relu")
    op.close()
