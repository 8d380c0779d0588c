"""GPU parity of the single-convolution entry points (tdc_conv_*) against the CPU oracle."""
import math
import sys

import numpy as np
import pytest
import torch

import tdc_amd
from oracle import ref
from util import assert_close, seeded

pytestmark = pytest.mark.gpu


def run_conv(x, w, bias=None, resid=None, stride=1, pad=0, dil=1, relu=False, tile=None):
    B, C, H, W = x.shape
    N, _, KH, KW = w.shape
    plan = tdc_amd.Conv2dPlan(B, C, N, H, W, KH, KW, stride, pad, dil, bias is not None, relu, tile=tile)
    plan.set_weights(w, bias)
    out = torch.full((B, N, plan.Ho, plan.Wo), float("nan"), device="cuda")  # never pre-zeroed
    plan.forward(x.cuda(), None if resid is None else resid.cuda(), out=out)
    torch.cuda.synchronize()
    res = out.cpu().numpy()
    plan.close()
    return res


def case(seed, B, C, N, H, W, K):
    g = seeded(seed)
    x = torch.rand(B, C, H, W, generator=g) * 2 - 1
    w = torch.empty(N, C, K, K).normal_(0, math.sqrt(2.0 / (C * K * K)), generator=g)
    return x, w


def announce(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def test_config1_core_conv_model_tile():
    """Benchmark configuration 1: 1x32x56x56, 32x32x3x3, stride 1, pad 1, seed 0."""
    x, w = ref.make_core_case(56, 32, 32, seed=0)
    got = run_conv(x, w, pad=1)
    assert_close(got, ref.conv2d_c(x.numpy(), w.numpy(), pad=1), "config 1 vs C oracle")
    assert_close(got, ref.conv2d_torch(x, w, pad=1).numpy(), "config 1 vs F.conv2d")


@pytest.mark.parametrize("hw", ref.SWEEP_HW)
@pytest.mark.parametrize("r1,r2", ref.SWEEP_RANKS)
def test_sweep_shapes_model_tile(hw, r1, r2):
    """Every shape of the core-conv sweep with the model's tile, against F.conv2d (and the C oracle when small)."""
    announce("sweep", hw, r1, r2)
    x, w = ref.make_core_case(hw, r1, r2)
    got = run_conv(x, w, pad=1)
    assert_close(got, ref.conv2d_torch(x, w, pad=1).numpy(), f"sweep {hw} {r1}->{r2} vs F.conv2d")
    if hw * hw * r1 * r2 <= 28 * 28 * 64 * 64:
        assert_close(got, ref.conv2d_c(x.numpy(), w.numpy(), pad=1), f"sweep {hw} {r1}->{r2} vs C oracle")


@pytest.mark.parametrize("shape", [(1, 8, 8, 5, 5), (1, 5, 3, 4, 7), (2, 3, 17, 9, 6), (1, 40, 24, 14, 14),
                                   (1, 32, 32, 7, 7), (1, 20, 33, 13, 11)])
def test_every_tile_3x3(shape):
    """All launchable tiles give the oracle's answer (the reference's recorded sweeps show diff = 0 for every tile)."""
    B, C, N, H, W = shape
    x, w = case(1000 + C * N + H, B, C, N, H, W, 3)
    want = ref.conv2d_c(x.numpy(), w.numpy(), pad=1)
    tiles = tdc_amd.model_enumerate(tdc_amd.conv_desc(B, C, N, H, W, 3, 3, 1, 1))
    assert tiles
    for t in tiles[::max(1, len(tiles) // 150)]:
        announce("tile3x3", shape, t)
        assert_close(run_conv(x, w, pad=1, tile=t), want, f"{shape} {t}")


@pytest.mark.parametrize("shape,pad", [((1, 8, 16, 8, 8), 1), ((2, 13, 20, 9, 11), 1), ((1, 7, 5, 5, 7), 0),
                                       ((1, 16, 16, 12, 12), 2), ((1, 40, 24, 14, 14), 1), ((1, 3, 2, 2, 2), 1),
                                       ((1, 4, 4, 1, 9), 1)])
def test_every_winograd_tile(shape, pad):
    """The Winograd F(2x2,3x3) path (tile.alg = 1) with every launchable tile: odd image sizes (the last tile row
    and column are half outside), paddings 0..2, several passes, splits over waves and workgroups, loader waves."""
    B, C, N, H, W = shape
    x, w = case(1500 + C * N + H, B, C, N, H, W, 3)
    want = ref.conv2d_c(x.numpy(), w.numpy(), pad=pad)
    tiles = [t for t in tdc_amd.model_enumerate(tdc_amd.conv_desc(B, C, N, H, W, 3, 3, 1, pad)) if t.alg == 1]
    assert tiles
    for t in tiles[::max(1, len(tiles) // 100)]:
        announce("winograd", shape, pad, t)
        assert_close(run_conv(x, w, pad=pad, tile=t), want, f"{shape} pad {pad} {t}")


@pytest.mark.parametrize("shape,stride,pad", [((1, 8, 16, 8, 8), 1, 1), ((2, 13, 20, 9, 11), 1, 1), ((1, 40, 24, 13, 13), 2, 1),
                                              ((1, 16, 16, 12, 12), 1, 2), ((1, 128, 48, 7, 7), 1, 1)])
def test_every_global_weight_tile(shape, stride, pad):
    """The direct 3x3 path that reads its weights from global memory into registers (tile.alg = 2), every launchable
    tile: both MFMA shapes, stride 2, ragged channel counts (zero-filled channel groups), several passes."""
    B, C, N, H, W = shape
    x, w = case(1700 + C * N + H, B, C, N, H, W, 3)
    want = ref.conv2d_c(x.numpy(), w.numpy(), stride=stride, pad=pad)
    tiles = [t for t in tdc_amd.model_enumerate(tdc_amd.conv_desc(B, C, N, H, W, 3, 3, stride, pad)) if t.alg == 2]
    assert tiles and {t.mf for t in tiles} == {16, 32}
    for t in tiles[::max(1, len(tiles) // 100)]:
        announce("global weights", shape, stride, pad, t)
        assert_close(run_conv(x, w, stride=stride, pad=pad, tile=t), want, f"{shape} s{stride} p{pad} {t}")


@pytest.mark.parametrize("shape", [(1, 64, 16, 7, 7), (2, 100, 40, 5, 6), (1, 288, 128, 14, 14), (1, 1024, 128, 7, 7),
                                   (1, 512, 1000, 1, 1), (3, 19, 5, 3, 3), (1, 256, 64, 20, 20)])
def test_every_streamed_1x1_tile(shape):
    """The 1x1 path that streams both operands from global memory into registers (tile.alg = 3): every launchable
    tile (1, 2, 4 or 8 runs of 16 channels per wave, 1 to 16 waves), ragged channel and pixel counts, a single pixel,
    batches; plain, with bias + residual + ReLU written into a channel slice of a wider buffer, and with the input
    affine (+ReLU) in front."""
    from ctypes import c_void_p
    B, C, N, H, W = shape
    x, w = case(2300 + C + N + H, B, C, N, H, W, 1)
    g = seeded(2301)
    bias = torch.randn(N, generator=g)
    resid = torch.randn(B, N, H, W, generator=g)
    scale = torch.rand(C, generator=g) * 2 - 0.5
    shift = torch.randn(C, generator=g) * 0.3
    want_plain = ref.conv2d_c(x.numpy(), w.numpy())
    want_full = (ref.conv2d_torch(x, w) + bias.view(1, -1, 1, 1) + resid).clamp_min(0).numpy()
    xt = (x * scale.view(1, C, 1, 1) + shift.view(1, C, 1, 1)).clamp_min(0)
    want_aff = ref.conv2d_c(xt.numpy(), w.numpy(), bias.numpy(), relu=True)
    tiles = [t for t in tdc_amd.model_enumerate(tdc_amd.conv_desc(B, C, N, H, W, 1, 1, 1, 0)) if t.alg == 3]
    assert tiles
    P = H * W
    for t in tiles:
        announce("streamed 1x1", shape, t)
        assert_close(run_conv(x, w, tile=t), want_plain, f"{shape} {t}")
        # bias + residual + ReLU, input and output as channel slices of wider buffers
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 1, 1, 1, 0, 1, True, True, tile=t).set_weights(w, bias)
        xin = torch.zeros(B, C + 3, H, W, device="cuda"); xin[:, 1:1 + C] = x.cuda()
        rbuf = torch.zeros(B, N + 2, H, W, device="cuda"); rbuf[:, 2:] = resid.cuda()
        obuf = torch.full((B, N + 5, H, W), 7.0, device="cuda")
        tdc_amd._lib.check(tdc_amd.lib().tdc_conv_forward_strided(
            plan._h, c_void_p(xin[:, 1:].data_ptr()), (C + 3) * P, c_void_p(rbuf[:, 2:].data_ptr()), (N + 2) * P,
            c_void_p(obuf[:, 4:].data_ptr()), (N + 5) * P, c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        got = obuf.cpu()
        assert_close(got[:, 4:4 + N].numpy(), want_full, f"slices {shape} {t}")
        assert (got[:, :4] == 7.0).all() and (got[:, 4 + N:] == 7.0).all()
        # the input affine in front
        plan.set_input_affine(scale, shift, relu=True)
        out = torch.full((B, N, H, W), float("nan"), device="cuda")
        plan.forward(x.cuda(), out=out)
        torch.cuda.synchronize()
        plan.close()
        assert_close(out.cpu().numpy(), want_aff, f"input affine {shape} {t}")


@pytest.mark.parametrize("shape,stride", [((1, 64, 128, 56, 56), 2), ((2, 100, 40, 9, 11), 2), ((1, 256, 512, 14, 14), 2),
                                          ((3, 19, 5, 7, 5), 3), ((1, 128, 256, 28, 28), 2), ((1, 33, 17, 1, 9), 2)])
def test_streamed_1x1_with_stride(shape, stride):
    """The streamed 1x1 kernel on stride > 1 (ResNet's downsampling shortcuts): output pixel (oy, ox) reads input pixel
    (oy * stride, ox * stride); every launchable tile, odd image sizes, batches, with bias + ReLU, and with the input
    affine in front."""
    B, C, N, H, W = shape
    x, w = case(2400 + C + N + H, B, C, N, H, W, 1)
    g = seeded(2401)
    bias = torch.randn(N, generator=g)
    scale = torch.rand(C, generator=g) * 2 - 0.5
    shift = torch.randn(C, generator=g) * 0.3
    want = ref.conv2d_c(x.numpy(), w.numpy(), bias.numpy(), stride=stride, relu=True)
    xt = (x * scale.view(1, C, 1, 1) + shift.view(1, C, 1, 1)).clamp_min(0)
    want_aff = ref.conv2d_c(xt.numpy(), w.numpy(), bias.numpy(), stride=stride, relu=True)
    tiles = [t for t in tdc_amd.model_enumerate(tdc_amd.conv_desc(B, C, N, H, W, 1, 1, stride, 0)) if t.alg == 3]
    assert tiles
    for t in tiles:
        announce("streamed 1x1 stride", shape, stride, t)
        assert_close(run_conv(x, w, bias, stride=stride, relu=True, tile=t), want, f"{shape} s{stride} {t}")
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 1, 1, stride, 0, 1, True, True, tile=t).set_weights(w, bias)
        plan.set_input_affine(scale, shift, relu=True)
        out = torch.full((B, N, plan.Ho, plan.Wo), float("nan"), device="cuda")
        plan.forward(x.cuda(), out=out)
        torch.cuda.synchronize()
        plan.close()
        assert_close(out.cpu().numpy(), want_aff, f"input affine {shape} s{stride} {t}")


@pytest.mark.parametrize("shape,stride,pad", [((1, 16, 16, 7, 7), 1, 1), ((2, 13, 20, 9, 11), 1, 1), ((1, 40, 24, 13, 13), 2, 1),
                                              ((1, 16, 16, 12, 12), 1, 2), ((1, 128, 48, 7, 7), 1, 1), ((1, 64, 32, 28, 28), 1, 1),
                                              ((3, 5, 3, 4, 3), 1, 0), ((1, 250, 17, 5, 5), 2, 1), ((2, 20, 33, 9, 58), 1, 1),
                                              ((1, 96, 40, 6, 30), 1, 1), ((1, 64, 48, 5, 56), 1, 0), ((1, 16, 20, 4, 44), 1, 1)])
def test_every_streamed_3x3_tile(shape, stride, pad):
    """The 3x3 path that streams both operands from global memory into registers (tile.alg = 4, and 6 with the input
    window loaded in 128-bit pieces and passed through LDS): every launchable tile
    (1, 2 or 4 channel groups per wave, 1 to 16 waves, every shape of the 16-pixel tile; 2 or 4 neighbouring 14-pixel row
    tiles per workgroup where the rows are wide enough, including rows whose last workgroup has blocks past the image),
    stride 2, wide and no padding, ragged channel counts, batches; plain, and with bias + residual + ReLU written into a
    channel slice."""
    from ctypes import c_void_p
    B, C, N, H, W = shape
    x, w = case(2500 + C * N + H, B, C, N, H, W, 3)
    g = seeded(2501)
    bias = torch.randn(N, generator=g)
    want = ref.conv2d_c(x.numpy(), w.numpy(), stride=stride, pad=pad)
    Ho, Wo = want.shape[2], want.shape[3]
    resid = torch.randn(B, N, Ho, Wo, generator=g)
    want_full = (torch.from_numpy(want) + bias.view(1, -1, 1, 1) + resid).clamp_min(0).numpy()
    tiles = [t for t in tdc_amd.model_enumerate(tdc_amd.conv_desc(B, C, N, H, W, 3, 3, stride, pad)) if t.alg in (4, 6)]
    assert tiles
    if stride == 1 and Wo > 14:
        assert {t.nb for t in tiles} == ({1, 2, 4} if Wo > 42 else {1, 2})
    # (tile.alg = 6, the input window in 128-bit pieces through LDS, wherever padding and stride allow it and the image has four columns)
    assert any(t.alg == 6 for t in tiles) == (pad <= 1 and W >= 4)
    for t in tiles:
        announce("streamed 3x3", shape, stride, pad, t)
        assert_close(run_conv(x, w, stride=stride, pad=pad, tile=t), want, f"{shape} s{stride} p{pad} {t}")
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 3, 3, stride, pad, 1, True, True, tile=t).set_weights(w, bias)
        xin = torch.zeros(B, C + 3, H, W, device="cuda"); xin[:, 1:1 + C] = x.cuda()
        rbuf = torch.zeros(B, N + 2, Ho, Wo, device="cuda"); rbuf[:, 2:] = resid.cuda()
        obuf = torch.full((B, N + 5, Ho, Wo), 7.0, device="cuda")
        tdc_amd._lib.check(tdc_amd.lib().tdc_conv_forward_strided(
            plan._h, c_void_p(xin[:, 1:].data_ptr()), (C + 3) * H * W, c_void_p(rbuf[:, 2:].data_ptr()), (N + 2) * Ho * Wo,
            c_void_p(obuf[:, 4:].data_ptr()), (N + 5) * Ho * Wo, c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        plan.close()
        got = obuf.cpu()
        assert_close(got[:, 4:4 + N].numpy(), want_full, f"slices {shape} {t}")
        assert (got[:, :4] == 7.0).all() and (got[:, 4 + N:] == 7.0).all()


@pytest.mark.parametrize("shape", [(1, 16, 16, 7, 8), (2, 13, 20, 9, 12), (1, 64, 32, 28, 28), (1, 40, 24, 13, 30),
                                   (2, 20, 33, 9, 58), (1, 96, 40, 6, 30), (1, 130, 48, 5, 56), (1, 16, 20, 4, 44),
                                   (1, 180, 17, 3, 14), (3, 5, 3, 2, 2), (1, 48, 96, 11, 84)])
def test_every_streamed_winograd_tile(shape):
    """The Winograd path that streams both operands from global memory into registers (tile.alg = 5): every launchable
    tile (1 to 4 channel groups per wave, one or two channel blocks per workgroup) on images whose rows have one, two or
    three 28-column blocks, the last one partial; odd heights (a tile row with one output row), ragged channel counts,
    batches; plain, and with bias + residual + ReLU written into a channel slice whose addresses are only 4-byte aligned."""
    from ctypes import c_void_p
    B, C, N, H, W = shape
    x, w = case(2700 + C * N + H, B, C, N, H, W, 3)
    g = seeded(2701)
    bias = torch.randn(N, generator=g)
    want = ref.conv2d_c(x.numpy(), w.numpy(), stride=1, pad=1)
    resid = torch.randn(B, N, H, W, generator=g)
    want_full = (torch.from_numpy(want) + bias.view(1, -1, 1, 1) + resid).clamp_min(0).numpy()
    # (the enumeration offers these tiles for single images; forced, they run any batch)
    tiles = [t for t in tdc_amd.model_enumerate(tdc_amd.conv_desc(1, C, N, H, W, 3, 3, 1, 1)) if t.alg == 5]
    assert tiles and not any(t.alg == 5 for t in tdc_amd.model_enumerate(tdc_amd.conv_desc(2, C, N, H, W, 3, 3, 1, 1)))
    if C >= 16:
        assert len({t.cch // (4 * t.wk) for t in tiles}) >= 2
    for t in tiles:
        announce("streamed winograd", shape, t)
        assert_close(run_conv(x, w, pad=1, tile=t), want, f"{shape} {t}")
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 3, 3, 1, 1, 1, True, True, tile=t).set_weights(w, bias)
        for shift in (0, 1):   # shift 1: the output and residual images start on an odd float
            xin = torch.zeros(B * (C + 3) * H * W + 1, device="cuda")
            xv = xin[shift:shift + B * (C + 3) * H * W].view(B, C + 3, H, W); xv[:, 1:1 + C] = x.cuda()
            rbuf = torch.zeros(B * (N + 2) * H * W + 1, device="cuda")
            rv = rbuf[shift:shift + B * (N + 2) * H * W].view(B, N + 2, H, W); rv[:, 2:] = resid.cuda()
            obuf = torch.full((B * (N + 5) * H * W + 1,), 7.0, device="cuda")
            ov = obuf[shift:shift + B * (N + 5) * H * W].view(B, N + 5, H, W)
            tdc_amd._lib.check(tdc_amd.lib().tdc_conv_forward_strided(
                plan._h, c_void_p(xv[:, 1:].data_ptr()), (C + 3) * H * W, c_void_p(rv[:, 2:].data_ptr()), (N + 2) * H * W,
                c_void_p(ov[:, 4:].data_ptr()), (N + 5) * H * W, c_void_p(torch.cuda.current_stream().cuda_stream)))
            torch.cuda.synchronize()
            got = ov.cpu()
            assert_close(got[:, 4:4 + N].numpy(), want_full, f"slices {shape} {t} shift {shift}")
            assert (got[:, :4] == 7.0).all() and (got[:, 4 + N:] == 7.0).all()
        plan.close()


@pytest.mark.parametrize("W,c0", [(16, 0), (16, 3), (14, 3), (13, 1)])
def test_winograd_into_channel_slices(W, c0):
    """A Winograd tile reading from, adding a residual from, and writing into channel slices of wider buffers (the
    strided entry point): the wide epilogue stores must respect the batch strides and fall back to narrower stores
    when width or slice offset break their alignment."""
    from ctypes import c_void_p
    B, C, N, H = 2, 16, 24, 12
    x, w = case(1900 + W + c0, B, C, N, H, W, 3)
    g = seeded(1901)
    bias = torch.randn(N, generator=g)
    resid = torch.randn(B, N, H, W, generator=g)
    want = (ref.conv2d_torch(x, w, pad=1) + bias.view(1, -1, 1, 1) + resid).clamp_min(0)
    tile = tdc_amd.Tile(16, 1, 1, 1, 1, 2, 8, min(8, (W + 1) // 2), 1, 0, 1)
    plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 3, 3, 1, 1, 1, True, True, tile=tile).set_weights(w, bias)
    xin = torch.zeros(B, C + 5, H, W, device="cuda"); xin[:, 2:2 + C] = x.cuda()
    rbuf = torch.zeros(B, N + 7, H, W, device="cuda"); rbuf[:, c0:c0 + N] = resid.cuda()
    obuf = torch.full((B, N + 9, H, W), 7.0, device="cuda")
    P = H * W
    tdc_amd._lib.check(tdc_amd.lib().tdc_conv_forward_strided(
        plan._h, c_void_p(xin[:, 2:].data_ptr()), (C + 5) * P, c_void_p(rbuf[:, c0:].data_ptr()), (N + 7) * P,
        c_void_p(obuf[:, c0:].data_ptr()), (N + 9) * P, c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = obuf.cpu()
    assert_close(got[:, c0:c0 + N].numpy(), want.numpy(), f"winograd slices W={W} c0={c0}")
    assert (got[:, :c0] == 7.0).all() and (got[:, c0 + N:] == 7.0).all()      # nothing written outside the slice
    plan.close()


def test_winograd_epilogue_exactness_and_determinism():
    """Winograd tiles on a benchmark layer: bias + residual + ReLU, the same bits on every launch, and the
    reference's integer known-answer test stays exact (the transformed weights 1, 3/2, 1/2, 9/4, 3/4, 1/4 and all
    partial sums are exactly representable)."""
    tiles = [tdc_amd.Tile(16, 1, 1, 1, 2, 2, 32, 14, 1, 4, 1), tdc_amd.Tile(16, 1, 1, 2, 1, 4, 16, 7, 2, 0, 1)]
    x, w = ref.make_core_case(56, 64, 64)
    g = seeded(77)
    bias = torch.randn(64, generator=g)
    resid = torch.randn(1, 64, 56, 56, generator=g)
    want = (ref.conv2d_torch(x, w, pad=1) + bias.view(1, -1, 1, 1) + resid).clamp_min(0).numpy()
    rng = np.random.default_rng(8)
    xi = torch.from_numpy(rng.integers(0, 10, size=(1, 64, 56, 56)).astype(np.float32))
    s = np.pad(xi.numpy().sum(axis=1)[0].astype(np.float64), 1)
    box = sum(s[r:r + 56, c:c + 56] for r in range(3) for c in range(3))
    for t in tiles:
        announce("winograd epilogue", t)
        a = run_conv(x, w, bias, resid, pad=1, relu=True, tile=t)
        b = run_conv(x, w, bias, resid, pad=1, relu=True, tile=t)
        assert_close(a, want, f"winograd epilogue {t}")
        assert np.array_equal(a, b)
        got = run_conv(xi, torch.ones(64, 64, 3, 3), pad=1, tile=t)
        assert np.abs(got - box[None, None]).sum() == 0.0


@pytest.mark.parametrize("shape", [(1, 16, 8, 5, 5), (1, 7, 5, 9, 4), (2, 64, 48, 7, 7), (1, 100, 36, 14, 14)])
def test_every_tile_1x1(shape):
    B, C, N, H, W = shape
    x, w = case(2000 + C * N + H, B, C, N, H, W, 1)
    want = ref.conv2d_c(x.numpy(), w.numpy())
    tiles = tdc_amd.model_enumerate(tdc_amd.conv_desc(B, C, N, H, W, 1, 1, 1, 0))
    assert tiles
    for t in tiles[::max(1, len(tiles) // 150)]:
        announce("tile1x1", shape, t)
        assert_close(run_conv(x, w, tile=t), want, f"{shape} {t}")


@pytest.mark.parametrize("K,stride,pad,dil", [(3, 2, 1, 1), (3, 1, 0, 1), (3, 1, 2, 2), (5, 1, 2, 1), (7, 2, 3, 1),
                                              (1, 2, 0, 1), (2, 1, 1, 1), (3, 3, 1, 1)])
def test_general_filters(K, stride, pad, dil):
    """Stride, padding, dilation and filter sizes beyond the 3x3/s1/p1 core conv."""
    x, w = case(3000 + K * 10 + stride, 1, 6, 10, 15, 12, K)
    want = ref.conv2d_c(x.numpy(), w.numpy(), stride=stride, pad=pad, dil=dil)
    tiles = tdc_amd.model_enumerate(tdc_amd.conv_desc(1, 6, 10, 15, 12, K, K, stride, pad, dil))
    for t in tiles[::3]:
        announce("general", K, stride, pad, dil, t)
        assert_close(run_conv(x, w, stride=stride, pad=pad, dil=dil, tile=t), want, f"K{K} s{stride} p{pad} d{dil} {t}")


@pytest.mark.parametrize("C,stride", [(3, 2), (9, 1)])
def test_seven_by_seven_instantiations(C, stride):
    """The unrolled 7x7 loop (the network stems) in all its register-block variants: 16- and 32-row MFMAs, one or two
    channel and pixel blocks per wave, one and three channel groups, stride 1 and 2; and the same filter with a
    dilation, which falls back to the run-time tap walker."""
    N, H, W = 64, 30, 27
    x, w = case(3100 + C, 1, C, N, H, W, 7)
    want = ref.conv2d_c(x.numpy(), w.numpy(), stride=stride, pad=3)
    d = tdc_amd.conv_desc(1, C, N, H, W, 7, 7, stride, 3, 1)
    seen = set()
    for t in tdc_amd.model_enumerate(d):
        key = (t.mf, t.mb, t.nb)
        if t.alg != 0 or key in seen:
            continue
        seen.add(key)
        name, _, _ = tdc_amd._lib.model_kernel_info(d, t)
        assert ", 49, " in name, name
        announce("7x7", C, stride, t)
        assert_close(run_conv(x, w, stride=stride, pad=3, tile=t), want, f"7x7 C{C} s{stride} {t}")
    assert len(seen) >= 6, seen
    dd = tdc_amd.conv_desc(1, C, N, H, W, 7, 7, stride, 6, 2)
    t = tdc_amd.model_select(dd).tile
    assert ", 0, " in tdc_amd._lib.model_kernel_info(dd, t)[0]
    want = ref.conv2d_c(x.numpy(), w.numpy(), stride=stride, pad=6, dil=2)
    assert_close(run_conv(x, w, stride=stride, pad=6, dil=2, tile=t), want, f"7x7 dilated C{C} s{stride}")


def _epilogue_tiles(d):
    """One tile of every kernel family the enumeration offers for `d` (staged direct with one and several register
    blocks, Winograd, global weights, streamed with 1 / 2 / 4 row blocks, and the variants split across workgroups)."""
    seen, out = set(), []
    for t in tdc_amd.model_enumerate(d):
        key = (t.alg, t.mf, t.mb, t.nb, t.wk > 1, t.ks > 1)
        if key not in seen:
            seen.add(key)
            out.append(t)
    return out


@pytest.mark.parametrize("shape,K", [((2, 24, 40, 10, 30), 3), ((1, 64, 48, 9, 56), 3), ((2, 96, 40, 6, 7), 1), ((1, 16, 20, 11, 13), 5)])
def test_epilogue_on_every_kernel_family(shape, K):
    """+ bias, + residual, ReLU on one tile of every kernel family: against the oracle, with the residual in its own
    buffer and IN PLACE (the residual buffer is the output buffer), where every lane must have read its residual
    values before it stores."""
    B, C, N, H, W = shape
    x, w = case(8800 + C + N, B, C, N, H, W, K)
    g = seeded(8801 + H)
    bias = torch.randn(N, generator=g)
    resid = torch.randn(B, N, H, W, generator=g)
    want = ref.conv2d_c(x.numpy(), w.numpy(), bias.numpy(), resid.numpy(), pad=K // 2, relu=True)
    d = tdc_amd.conv_desc(B, C, N, H, W, K, K, 1, K // 2)
    tiles = _epilogue_tiles(d)
    assert len({t.alg for t in tiles}) >= (2 if K in (1, 3) else 1)
    xd = x.cuda()
    for t in tiles:
        announce("epilogue", shape, K, t)
        assert_close(run_conv(x, w, bias, resid, pad=K // 2, relu=True, tile=t), want, f"epilogue {shape} {t}")
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, K, K, 1, K // 2, 1, True, True, tile=t).set_weights(w, bias)
        buf = resid.cuda().clone()
        plan.forward(xd, buf, out=buf)
        torch.cuda.synchronize()
        plan.close()
        assert_close(buf.cpu().numpy(), want, f"in-place epilogue {shape} {t}")


@pytest.mark.parametrize("shape,K", [((1, 24, 32, 12, 16), 3), ((2, 40, 20, 8, 28), 3), ((1, 48, 16, 6, 8), 1), ((1, 12, 16, 9, 12), 5)])
def test_input_not_aligned_to_16_bytes(shape, K):
    """Image rows that are a multiple of four floats are staged with 16-byte copy elements; an input pointer that is
    only 4-byte aligned (a view one float into its buffer) makes the launch fall back to 4-byte elements, four times
    as many copy blocks.  One tile of every kernel family, input and output both one float off."""
    B, C, N, H, W = shape
    x, w = case(8900 + C + N, B, C, N, H, W, K)
    want = ref.conv2d_c(x.numpy(), w.numpy(), pad=K // 2)
    d = tdc_amd.conv_desc(B, C, N, H, W, K, K, 1, K // 2)
    xbuf = torch.zeros(x.numel() + 1, device="cuda")
    xv = xbuf[1:].view(B, C, H, W)
    xv.copy_(x)
    assert xv.data_ptr() % 16 == 4
    for t in _epilogue_tiles(d):
        announce("unaligned input", shape, K, t)
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, K, K, 1, K // 2, tile=t).set_weights(w)
        obuf = torch.full((B * N * H * W + 1,), float("nan"), device="cuda")
        ov = obuf[1:].view(B, N, H, W)
        plan.forward(xv, out=ov)
        torch.cuda.synchronize()
        plan.close()
        assert_close(ov.cpu().numpy(), want, f"unaligned input {shape} {t}")


def test_random_shapes_model_tile():
    """Forty seeded random problems (ragged sizes, batch, stride, padding, dilation, rectangular images, every
    epilogue combination) with the tile the model picks, against F.conv2d on the host."""
    rng = np.random.default_rng(20240607)
    done = 0
    while done < 40:
        B = int(rng.integers(1, 4)); C = int(rng.integers(1, 70)); N = int(rng.integers(1, 70))
        H = int(rng.integers(1, 40)); W = int(rng.integers(1, 40))
        K = int(rng.choice([1, 1, 3, 3, 3, 5, 2, 7])); stride = int(rng.integers(1, 4)); dil = int(rng.integers(1, 3))
        pad = int(rng.integers(0, K + 1))
        if H + 2 * pad < dil * (K - 1) + 1 or W + 2 * pad < dil * (K - 1) + 1:
            continue
        use_bias, use_res, relu = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        announce("random", done, B, C, N, H, W, K, stride, pad, dil, use_bias, use_res, relu)
        x, w = case(int(rng.integers(1, 1 << 30)), B, C, N, H, W, K)
        g = seeded(done)
        bias = torch.randn(N, generator=g) if use_bias else None
        want = ref.conv2d_torch(x, w, stride=stride, pad=pad, dil=dil)
        if use_bias:
            want = want + bias.view(1, N, 1, 1)
        resid = torch.randn(want.shape, generator=g) if use_res else None
        if use_res:
            want = want + resid
        if relu:
            want = want.clamp_min(0)
        got = run_conv(x, w, bias, resid, stride=stride, pad=pad, dil=dil, relu=relu)
        assert_close(got, want.numpy(), f"random case {done}")
        done += 1


@pytest.mark.parametrize("B,C,N,H,W,K,stride,pad", [
    (1, 3, 5, 1030, 770, 3, 1, 1),      # a large ragged image, few channels
    (1, 2, 3, 64, 4100, 1, 1, 0),       # 1x1 on a 262 400-pixel flattened image
    (1, 520, 24, 9, 9, 3, 1, 1),        # many input channels (several passes, ragged last pass)
    (1, 24, 520, 9, 9, 3, 1, 1),        # many output channels (many channel tiles)
    (37, 5, 7, 11, 13, 3, 2, 1),        # a long batch
    (1, 4, 4, 1, 1, 1, 1, 0),           # a single pixel
    (2, 1, 1, 1, 300, 3, 1, 1),         # one row
    (2, 1, 1, 300, 1, 3, 1, 1),         # one column
])
def test_extreme_shapes_model_tile(B, C, N, H, W, K, stride, pad):
    """Shapes at the edges of what the layers of the networks use: very large and degenerate images, long
    batches, channel counts far above the tile sizes; model-picked tile, against F.conv2d on the host."""
    announce("extreme", B, C, N, H, W, K, stride, pad)
    x, w = case(7000 + C + N + H, B, C, N, H, W, K)
    got = run_conv(x, w, stride=stride, pad=pad)
    assert_close(got, ref.conv2d_torch(x, w, stride=stride, pad=pad).numpy(), f"extreme {(B, C, N, H, W, K)}")


def test_measured_tile_selection():
    """With tuning on, a plan without a forced tile gets a measured pick: results stay within tolerance, the pick
    is one of the launchable tiles, a second plan of the same problem reuses it, and a forced tile is still obeyed."""
    prev = tdc_amd.set_autotune(6)
    try:
        assert tdc_amd.lib().tdc_get_autotune() == 6
        for (C, N, hw, K, stride, pad) in ((64, 64, 28, 3, 1, 1), (48, 200, 14, 1, 1, 0), (3, 16, 40, 7, 2, 3)):
            announce("tuned", C, N, hw, K, stride, pad)
            x, w = case(8100 + C, 1, C, N, hw, hw, K)
            want = ref.conv2d_torch(x, w, stride=stride, pad=pad).numpy()
            picks = []
            for _ in range(2):
                plan = tdc_amd.Conv2dPlan(1, C, N, hw, hw, K, K, stride, pad).set_weights(w)
                out = torch.full((1, N, plan.Ho, plan.Wo), float("nan"), device="cuda")
                plan.forward(x.cuda(), out=out)
                torch.cuda.synchronize()
                assert_close(out.cpu().numpy(), want, f"tuned {(C, N, hw, K)}")
                picks.append(plan.info.tile.astuple())
                plan.close()
            assert picks[0] == picks[1]
            desc = tdc_amd.conv_desc(1, C, N, hw, hw, K, K, stride, pad)
            assert picks[0] in [t.astuple() for t in tdc_amd.model_enumerate(desc)]
            forced = tdc_amd.model_select(desc).tile
            plan = tdc_amd.Conv2dPlan(1, C, N, hw, hw, K, K, stride, pad, tile=forced)
            assert plan.info.tile.astuple() == forced.astuple()
            plan.close()
    finally:
        tdc_amd.set_autotune(prev)
    with pytest.raises(tdc_amd.TdcError):
        tdc_amd.set_autotune(-1)


def test_stride2_resnet_core_shapes():
    """The three stride-2 core convs of Tucker ResNet-18 (64->64 56->28, 128->128 28->14, 256->256 14->7)."""
    for r, hw in ((64, 56), (128, 28), (256, 14)):
        announce("stride2", r, hw)
        x, w = case(4000 + r, 1, r, r, hw, hw, 3)
        got = run_conv(x, w, stride=2, pad=1)
        want = ref.conv2d_torch(x, w, stride=2, pad=1).numpy()
        assert got.shape == (1, r, hw // 2, hw // 2)
        assert_close(got, want, f"stride-2 {r}@{hw}")
        # conv_s2(x) == conv_s1(x)[::2, ::2]
        full = run_conv(x, w, stride=1, pad=1)
        assert_close(got, full[:, :, ::2, ::2], "stride-2 subsampling identity")


def test_epilogue_bias_residual_relu():
    x, w = case(5000, 2, 12, 20, 9, 9, 3)
    g = seeded(5001)
    bias = torch.randn(20, generator=g)
    resid = torch.randn(2, 20, 9, 9, generator=g)
    want = ref.conv2d_c(x.numpy(), w.numpy(), bias.numpy(), resid.numpy(), pad=1, relu=True)
    for t in tdc_amd.model_enumerate(tdc_amd.conv_desc(2, 12, 20, 9, 9, 3, 3, 1, 1))[::5]:
        announce("epilogue", t)
        assert_close(run_conv(x, w, bias, resid, pad=1, relu=True, tile=t), want, f"epilogue {t}")
    assert (want == 0).any() and (want > 0).any()


def test_reference_known_answer_integers_all_ones():
    """The reference harness's own check: integer inputs 0..9, all-ones weights -> exact integers, diff == 0
    (2080Ti-evaluation/TDC-LAYERS-ORACLE/template_benchmark_cudnn.template:418-428,509)."""
    rng = np.random.default_rng(7)
    for (C, N, H, W) in ((32, 32, 56, 56), (64, 32, 28, 28), (96, 64, 7, 7), (192, 160, 7, 7), (32, 32, 14, 14)):
        announce("kat", C, N, H, W)
        x = torch.from_numpy(rng.integers(0, 10, size=(1, C, H, W)).astype(np.float32))
        w = torch.ones(N, C, 3, 3)
        got = run_conv(x, w, pad=1)
        # closed form: 3x3 box sum of the channel-summed image, identical for every output channel
        s = np.pad(x.numpy().sum(axis=1)[0].astype(np.float64), 1)
        box = sum(s[r:r + H, c:c + W] for r in range(3) for c in range(3))
        assert np.abs(got - box[None, None]).sum() == 0.0


def test_deterministic_bitwise():
    x, w = ref.make_core_case(28, 64, 64)
    a = run_conv(x, w, pad=1)
    b = run_conv(x, w, pad=1)
    assert np.array_equal(a, b)


def _split_rounds(plan, B, C, N, H, W, K, pad, seed, what, reupload_weights=False):
    """One plan, four launches whose data CHANGES between launches (input x, a new input, x again; optionally new
    weights for a fourth), each into a NaN-filled output and each checked against the oracle; the first and third
    must agree bit for bit.  With unchanged data a partial tile left over from the previous launch, or read before
    its writer had stored it, would still hold the right value and go unseen."""
    g = seeded(seed)
    bias = torch.randn(N, generator=g)
    resid = torch.randn(B, N, plan.Ho, plan.Wo, generator=g)
    xs = [torch.rand(B, C, H, W, generator=g) * 2 - 1 for _ in range(2)]
    ws = [torch.empty(N, C, K, K).normal_(0, math.sqrt(2.0 / (C * K * K)), generator=g) for _ in range(2)]
    plan.set_weights(ws[0], bias)
    rd = resid.cuda()
    outs = []
    rounds = [(0, 0), (1, 0), (0, 0)] + ([(1, 1)] if reupload_weights else [])
    for xi, wi in rounds:
        if wi != 0:
            plan.set_weights(ws[wi], bias)
        out = torch.full((B, N, plan.Ho, plan.Wo), float("nan"), device="cuda")
        plan.forward(xs[xi].cuda(), rd, out=out)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        want = ref.conv2d_c(xs[xi].numpy(), ws[wi].numpy(), bias.numpy(), resid.numpy(), pad=pad, relu=True)
        assert_close(got, want, f"{what}, launch {len(outs)} (input {xi}, weights {wi})")
        outs.append(got)
    assert np.array_equal(outs[0], outs[2]), f"{what}: the same input gave different bits after another launch in between"
    assert not np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("tile", [tdc_amd.Tile(16, 1, 1, 1, 1, 1, 8, 8, ks=5),      # 5 slices of one pass each
                                  tdc_amd.Tile(16, 1, 1, 2, 1, 2, 16, 8, ks=2),     # 3 passes over 2 slices: 2 + 1
                                  tdc_amd.Tile(32, 1, 2, 1, 1, 4, 8, 9, ks=3),
                                  tdc_amd.Tile(16, 1, 1, 1, 1, 1, 4, 8, ks=4),
                                  tdc_amd.Tile(32, 2, 2, 1, 1, 1, 4, 9, ks=10)])
def test_split_across_workgroups(tile):
    """Input-channel passes dealt to several workgroups (tile.ks > 1; here 2, 3, 4, 5 and 10 slices at batch 2): the
    oracle's answer with the whole epilogue on every launch while inputs and weights change between launches, the same
    bits for the same input, and the ticket counters back at zero for the next launch."""
    announce("ksplit", tile)
    B, C, N, H, W = 2, 40, 37, 9, 9
    plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 3, 3, 1, 1, 1, True, True, tile=tile)
    assert plan.info.grid_z == B * tile.ks
    _split_rounds(plan, B, C, N, H, W, 3, 1, 6000, f"split-K {tile}", reupload_weights=tile.ks == 5)
    plan.close()


@pytest.mark.parametrize("shape,K,pad", [((1, 256, 256, 7, 7), 3, 1), ((2, 130, 40, 5, 6), 3, 1), ((1, 2048, 256, 7, 7), 1, 0),
                                         ((2, 300, 24, 3, 5), 1, 0)])
def test_streamed_tiles_split_across_workgroups(shape, K, pad):
    """Streamed kernels with the input channels dealt to several workgroups (tile.alg = 3 / 4 with tile.ks > 1): the
    enumeration offers such tiles for layers with few workgroups; every one matches the oracle with the whole epilogue
    on every launch while the input changes between launches (the partial blocks are added in slice order by whichever
    workgroup comes last), gives the same bits for the same input, and leaves the ticket counters at zero."""
    B, C, N, H, W = shape
    tiles = [t for t in tdc_amd.model_enumerate(tdc_amd.conv_desc(B, C, N, H, W, K, K, 1, pad)) if t.alg >= 3 and t.ks > 1]
    assert tiles and {t.ks for t in tiles} >= {2, 4}
    for i, t in enumerate(tiles):
        announce("streamed split", shape, K, t)
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, K, K, 1, pad, 1, True, True, tile=t)
        assert plan.info.grid_z == B * t.ks
        _split_rounds(plan, B, C, N, H, W, K, pad, 6100 + C + N, f"streamed split {shape} {t}", reupload_weights=i == 0)
        plan.close()


@pytest.mark.parametrize("C,K,pad,alg", [(256, 3, 1, 0), (256, 3, 1, 4), (2048, 1, 0, 0), (2048, 1, 0, 3)])
def test_split_hand_over_many_launches(C, K, pad, alg):
    """The hand-over between the workgroups of a split (partials through the workspace, a ticket per tile) over 2000
    back-to-back launches of one plan on the two layers that rely on it (256 -> 256 @7x7 3x3, 2048 -> 256 @7x7 1x1),
    staged and streamed kernels.  The input alternates between x and -x: with no bias and no ReLU the two results are
    exact negations of each other, so a partial tile that is read stale (the previous launch's) or too early flips a
    sign and cannot hide.  Every launch is compared bit for bit on the device; the test stops at the first mismatch."""
    N, H, W = 256, 7, 7
    desc = tdc_amd.conv_desc(1, C, N, H, W, K, K, 1, pad)
    tiles = [t for t in tdc_amd.model_enumerate(desc) if t.alg == alg and t.ks > 1]
    assert tiles
    # the model's favourite among the split tiles of this kernel family
    tile = min(tiles, key=lambda t: tdc_amd.model_evaluate(desc, t).pred_us)
    announce("hand-over soak", C, K, tile)
    x, w = case(6200 + C + alg, 1, C, N, H, W, K)
    plan = tdc_amd.Conv2dPlan(1, C, N, H, W, K, K, 1, pad, tile=tile).set_weights(w)
    xp, xn = x.cuda(), (-x).cuda()
    first = plan.forward(xp)
    torch.cuda.synchronize()
    assert_close(first.cpu().numpy(), ref.conv2d_c(x.numpy(), w.numpy(), pad=pad), f"soak reference {tile}")
    neg = -first
    out = torch.empty_like(first)
    for i in range(2000):
        flip = i & 1
        out.fill_(float("nan"))
        plan.forward(xn if flip else xp, out=out)
        same = torch.equal(out, neg if flip else first)     # (synchronises)
        assert same, f"launch {i} of {tile}: result differs from the first launch"
    plan.close()


@pytest.mark.parametrize("order", ["0", "1"])
def test_both_logical_workgroup_orders(order, monkeypatch):
    """The launch is one-dimensional and decoded in the kernel; both decode orders (channel tile fastest / pixel
    tile fastest) must give the oracle's answer, also when the number of workgroups is not a multiple of 8."""
    monkeypatch.setenv("TDC_EXPERIMENT_XCD_ORDER", order)
    for (B, C, N, H, W, K, stride) in ((1, 12, 40, 13, 11, 3, 1), (3, 8, 24, 9, 10, 3, 2), (2, 20, 18, 7, 7, 1, 1)):
        announce("order", order, B, C, N, H, W, K, stride)
        x, w = case(7000 + C + N, B, C, N, H, W, K)
        want = ref.conv2d_c(x.numpy(), w.numpy(), stride=stride, pad=K // 2)
        tiles = tdc_amd.model_enumerate(tdc_amd.conv_desc(B, C, N, H, W, K, K, stride, K // 2))
        for t in tiles[::max(1, len(tiles) // 40)]:
            assert_close(run_conv(x, w, stride=stride, pad=K // 2, tile=t), want, f"order {order} {t}")


@pytest.mark.parametrize("shape", [(1, 40, 24, 9, 9, 1), (2, 100, 36, 14, 14, 1), (1, 7, 5, 5, 6, 1), (2, 16, 8, 9, 9, 2)])
@pytest.mark.parametrize("relu_in", [True, False])
def test_input_affine_fused_into_1x1(shape, relu_in):
    """conv1x1(relu?(x*scale[c] + shift[c])): the norm -> relu -> conv order of the reference's DenseNet layers,
    as one kernel; every tile (multi-pass ones, loaders, split-K) against the C oracle on the transformed input."""
    B, C, N, H, W, stride = shape
    x, w = case(9000 + C + N, B, C, N, H, W, 1)
    g = seeded(9001)
    scale = torch.rand(C, generator=g) * 2 - 0.5
    shift = torch.randn(C, generator=g) * 0.3
    bias = torch.randn(N, generator=g)
    xt = x * scale.view(1, C, 1, 1) + shift.view(1, C, 1, 1)
    if relu_in:
        xt = xt.clamp_min(0)
    want = ref.conv2d_c(xt.numpy(), w.numpy(), bias.numpy(), stride=stride, relu=True)
    tiles = tdc_amd.model_enumerate(tdc_amd.conv_desc(B, C, N, H, W, 1, 1, stride, 0))
    xd = x.cuda()
    for t in tiles[::max(1, len(tiles) // 60)]:
        announce("affine-in", shape, relu_in, t)
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 1, 1, stride, 0, 1, True, True, tile=t).set_weights(w, bias)
        plan.set_input_affine(scale, shift, relu=relu_in)
        out = torch.full((B, N, plan.Ho, plan.Wo), float("nan"), device="cuda")
        plan.forward(xd, out=out)
        torch.cuda.synchronize()
        plan.close()
        assert_close(out.cpu().numpy(), want, f"input affine {shape} {t}")


@pytest.mark.parametrize("shape", [(1, 24, 16, 40, 9, 9, 3, 1), (2, 40, 10, 33, 14, 14, 3, 1), (1, 64, 32, 64, 13, 11, 3, 2),
                                   (2, 50, 64, 24, 7, 7, 1, 1), (1, 20, 128, 64, 9, 9, 1, 1), (1, 12, 7, 5, 6, 5, 5, 1)])
def test_fused_1x1_tail(shape):
    """relu(W_tail * relu(conv(x) + b1) + b2 + residual) in one kernel, every tile that can hold all output
    channels of the convolution in one workgroup, against the two convolutions done one after the other."""
    B, C, N, N2, H, W, K, stride = shape
    x, w = case(9500 + C + N, B, C, N, H, W, K)
    g = seeded(9501 + N2)
    b1 = torch.randn(N, generator=g) * 0.5
    w2 = torch.randn(N2, N, 1, 1, generator=g) / math.sqrt(N)
    b2 = torch.randn(N2, generator=g)
    mid = ref.conv2d_torch(x, w, b1, stride=stride, pad=K // 2).clamp_min(0)
    resid = torch.randn(B, N2, mid.shape[2], mid.shape[3], generator=g)
    want = (ref.conv2d_torch(mid, w2, b2) + resid).clamp_min(0).numpy()
    want_c = ref.conv2d_c(ref.conv2d_c(x.numpy(), w.numpy(), b1.numpy(), stride=stride, pad=K // 2, relu=True),
                          w2.numpy(), b2.numpy(), resid.numpy(), relu=True)
    assert_close(want, want_c, "host references agree")
    desc = tdc_amd.conv_desc(B, C, N, H, W, K, K, stride, K // 2, 1, True, True)
    ok = []
    for t in tdc_amd.model_enumerate(desc):
        if t.ks == 1 and t.mf * t.mb * t.wm >= N and not t.alg:    # (the Winograd path carries no tail)
            ok.append(t)
    assert ok
    xd, rd = x.cuda(), resid.cuda()
    ran = 0
    for t in ok[::max(1, len(ok) // 50)] + [None]:
        announce("tail", shape, t)
        try:
            plan = tdc_amd.Conv2dPlan(B, C, N, H, W, K, K, stride, K // 2, 1, True, True, tile=t, tail=(N2, True, True))
        except tdc_amd.TdcError as e:     # the parked tile can push a candidate over the LDS limit
            assert t is not None and "LDS" in str(e), str(e)
            continue
        ran += 1
        plan.set_weights(w, b1).set_tail_weights(w2, b2)
        out = torch.full((B, N2, plan.Ho, plan.Wo), float("nan"), device="cuda")
        plan.forward(xd, rd, out=out)
        torch.cuda.synchronize()
        plan.close()
        assert_close(out.cpu().numpy(), want_c, f"fused tail {shape} {t}")
    assert ran >= 10


@pytest.mark.parametrize("shape", [(1, 24, 16, 40, 9, 9, 1), (2, 40, 10, 33, 14, 14, 1), (1, 32, 32, 64, 28, 28, 1), (1, 64, 64, 128, 13, 11, 2),
                                   (1, 16, 128, 64, 7, 7, 1), (1, 13, 37, 5, 6, 5, 1)])
def test_fused_tail_on_streamed_3x3(shape):
    """The same fusion behind the streamed 3x3 kernel (tile.alg = 4 with one wave per block of 16 output channels and
    channel slice): relu(W_tail * relu(conv(x) + b1) + b2 + residual), every admissible split of the waves and a few
    tile widths, and whatever the model picks when a tail is asked for."""
    B, C, N, N2, H, W, stride = shape
    x, w = case(9700 + C + N, B, C, N, H, W, 3)
    g = seeded(9701 + N2)
    b1 = torch.randn(N, generator=g) * 0.5
    w2 = torch.randn(N2, N, 1, 1, generator=g) / math.sqrt(N)
    b2 = torch.randn(N2, generator=g)
    want_mid = ref.conv2d_c(x.numpy(), w.numpy(), b1.numpy(), stride=stride, pad=1, relu=True)
    resid = torch.randn(B, N2, want_mid.shape[2], want_mid.shape[3], generator=g)
    want = ref.conv2d_c(want_mid, w2.numpy(), b2.numpy(), resid.numpy(), relu=True)
    Wo = want.shape[3]
    wm, groups = -(-N // 16), -(-C // 4)
    tiles = []
    for per_wave in (4, 2, 1):
        wk = -(-groups // per_wave)
        if per_wave <= groups and wm * wk <= 16:
            for tw in sorted({min(16, Wo), min(14, Wo), min(7, Wo), min(4, Wo)}):
                tiles.append(tdc_amd.Tile(16, 1, 1, wm, 1, wk, 4 * per_wave * wk, tw, 1, 0, 4))
    assert tiles
    xd, rd = x.cuda(), resid.cuda()
    for t in tiles + [None]:
        announce("streamed tail", shape, t)
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 3, 3, stride, 1, 1, True, True, tile=t, tail=(N2, True, True))
        plan.set_weights(w, b1).set_tail_weights(w2, b2)
        out = torch.full((B, N2, plan.Ho, plan.Wo), float("nan"), device="cuda")
        plan.forward(xd, rd, out=out)
        torch.cuda.synchronize()
        plan.close()
        assert_close(out.cpu().numpy(), want, f"streamed fused tail {shape} {t}")


@pytest.mark.parametrize("shape", [(1, 40, 24, 16, 40, 9, 9), (2, 100, 40, 10, 33, 14, 14), (1, 128, 64, 16, 32, 14, 14),
                                   (1, 128, 64, 16, 32, 7, 7), (1, 64, 32, 32, 64, 28, 28), (1, 300, 64, 64, 70, 13, 11),
                                   (3, 5, 3, 4, 6, 4, 3), (1, 128, 64, 64, 128, 56, 56)])
def test_fused_head_and_tail_on_streamed_3x3(shape):
    """A whole Tucker convolution in one launch: 1x1 head (no bias) -> 3x3 core (pad 1, + bias, ReLU) -> 1x1 tail
    (+ bias, + residual, ReLU) on the streamed 3x3 kernel.  The head is recomputed on every tile's window, where pixels
    outside the image must read as the core's zero padding; ragged channel counts, every tile shape, batches."""
    B, C0, C, N, N2, H, W = shape
    g = seeded(9800 + C0 + N2)
    x = torch.rand(B, C0, H, W, generator=g) * 2 - 1
    w0 = torch.randn(C, C0, 1, 1, generator=g) / math.sqrt(C0)
    w = torch.randn(N, C, 3, 3, generator=g) * math.sqrt(2.0 / (9 * C))
    b1 = torch.randn(N, generator=g) * 0.5
    w2 = torch.randn(N2, N, 1, 1, generator=g) / math.sqrt(N)
    b2 = torch.randn(N2, generator=g)
    resid = torch.randn(B, N2, H, W, generator=g)
    f1 = ref.conv2d_c(x.numpy(), w0.numpy())
    mid = ref.conv2d_c(f1, w.numpy(), b1.numpy(), pad=1, relu=True)
    want = ref.conv2d_c(mid, w2.numpy(), b2.numpy(), resid.numpy(), relu=True)
    wm, groups = -(-N // 16), -(-C // 4)
    tiles = []
    for per_wave in (4, 2, 1):
        wk = -(-groups // per_wave)
        if per_wave <= groups and wm * wk <= 16:
            for tw in sorted({min(16, W), min(14, W), min(7, W), min(4, W)}):
                tiles.append(tdc_amd.Tile(16, 1, 1, wm, 1, wk, 4 * per_wave * wk, tw, 1, 0, 4))
    assert tiles
    xd, rd = x.cuda(), resid.cuda()
    for t in tiles:
        announce("streamed head + tail", shape, t)
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 3, 3, 1, 1, 1, True, True, tile=t, tail=(N2, True, True))
        plan.set_weights(w, b1).set_tail_weights(w2, b2).set_head(w0)
        outs = []
        for rep in range(2):
            out = torch.full((B, N2, H, W), float("nan"), device="cuda")
            plan.forward(xd, rd, out=out)
            torch.cuda.synchronize()
            outs.append(out.cpu().numpy())
        plan.close()
        assert_close(outs[0], want, f"streamed fused head + tail {shape} {t}")
        assert np.array_equal(outs[0], outs[1])


def test_fused_head_is_refused_where_it_does_not_apply():
    plan = tdc_amd.Conv2dPlan(1, 8, 16, 9, 9, 3, 3, 1, 1, tile=tdc_amd.Tile(16, 1, 1, 1, 1, 2, 8, 9, 1, 0, 4)).set_weights(torch.randn(16, 8, 3, 3))
    with pytest.raises(tdc_amd.TdcError) as e:   # no fused tail
        plan.set_head(torch.randn(8, 20))
    assert e.value.status == tdc_amd._lib.TDC_ERR_UNSUPPORTED
    plan.close()
    plan = tdc_amd.Conv2dPlan(1, 8, 16, 9, 9, 3, 3, 2, 1, tile=tdc_amd.Tile(16, 1, 1, 1, 1, 2, 8, 5, 1, 0, 4), tail=(8, False, False))
    with pytest.raises(tdc_amd.TdcError):        # stride 2
        plan.set_head(torch.randn(8, 20))
    plan.close()


def test_fused_tail_needs_one_channel_tile():
    with pytest.raises(tdc_amd.TdcError):   # 40 output channels cannot sit in a 16-channel tile
        tdc_amd.Conv2dPlan(1, 8, 40, 9, 9, 3, 3, 1, 1, tile=tdc_amd.Tile(16, 1, 1, 1, 1, 1, 8, 8), tail=(8, False, False))
    plan = tdc_amd.Conv2dPlan(1, 8, 16, 9, 9, 3, 3, 1, 1, tail=(8, False, False)).set_weights(torch.randn(16, 8, 3, 3))
    with pytest.raises(tdc_amd.TdcError) as e:   # tail weights missing
        plan.forward(torch.randn(1, 8, 9, 9).cuda())
    assert e.value.status == tdc_amd._lib.TDC_ERR_STATE
    plan.close()


def test_input_affine_is_refused_where_padding_would_have_to_stay_zero():
    plan = tdc_amd.Conv2dPlan(1, 8, 8, 9, 9, 3, 3, 1, 1)
    with pytest.raises(tdc_amd.TdcError) as e:
        plan.set_input_affine(torch.ones(8), torch.zeros(8))
    assert e.value.status == tdc_amd._lib.TDC_ERR_UNSUPPORTED
    plan.close()


def test_plans_sharing_a_kernel_keep_their_large_lds_requests():
    """Two plans on the same kernel instantiation, both above the 64 KiB default of dynamic LDS, the second asking
    for less: the first must still launch (the opt-in attribute is per function, not per plan)."""
    B, C, N, H, W = 1, 128, 32, 28, 28
    desc = tdc_amd.conv_desc(B, C, N, H, W, 3, 3, 1, 1)
    cands = [(tdc_amd.model_evaluate(desc, t).lds_bytes, t) for t in tdc_amd.model_enumerate(desc)
             if (t.mf, t.mb, t.nb, t.ks) == (16, 1, 1, 1)]
    big = max(cands, key=lambda c: c[0])
    mid = min((c for c in cands if c[0] > 70 * 1024), key=lambda c: c[0])
    assert big[0] > 120 * 1024 and mid[0] < big[0] - 16 * 1024
    announce("lds", big, mid)
    x, w = case(8000, B, C, N, H, W, 3)
    want = ref.conv2d_torch(x, w, pad=1).numpy()
    pa = tdc_amd.Conv2dPlan(B, C, N, H, W, 3, 3, 1, 1, tile=big[1]).set_weights(w)
    pb = tdc_amd.Conv2dPlan(B, C, N, H, W, 3, 3, 1, 1, tile=mid[1]).set_weights(w)
    xd = x.cuda()
    for plan in (pb, pa, pb, pa):
        out = torch.full((B, N, H, W), float("nan"), device="cuda")
        plan.forward(xd, out=out)
        torch.cuda.synchronize()
        assert_close(out.cpu().numpy(), want, "shared kernel, different LDS sizes")
    pa.close()
    pb.close()


def test_split_across_workgroups_rejects_empty_slices():
    with pytest.raises(tdc_amd.TdcError):   # 40 channels in passes of 8 = 5 passes: 4 slices take 2,2,1,0
        tdc_amd.model_evaluate(tdc_amd.conv_desc(1, 40, 16, 9, 9, 3, 3, 1, 1), tdc_amd.Tile(16, 1, 1, 1, 1, 1, 8, 8, ks=4))
    with pytest.raises(tdc_amd.TdcError):
        tdc_amd.model_evaluate(tdc_amd.conv_desc(1, 40, 16, 9, 9, 3, 3, 1, 1), tdc_amd.Tile(16, 1, 1, 1, 1, 1, 8, 8, ks=0))


def test_linearity_full_size():
    """Size-independent property at the largest sweep shape: conv(a*x1 + x2) == a*conv(x1) + conv(x2)."""
    x1, w = ref.make_core_case(56, 128, 128)
    x2, _ = ref.make_core_case(56, 128, 128, seed=99)
    y1 = run_conv(x1, w, pad=1)
    y2 = run_conv(x2, w, pad=1)
    y = run_conv(0.5 * x1 + x2, w, pad=1)
    np.testing.assert_allclose(y, 0.5 * y1 + y2, rtol=1e-4, atol=2e-5)


def test_launch_floor_probe():
    """The launch-path probe: an empty kernel costs something, a kernel that keeps every wave busy for 5 us costs at
    least those 5 us per launch and not much more, on a stream and inside a graph."""
    from tdc_amd.conv import launch_floor_us
    for graph in (False, True):
        empty = min(launch_floor_us(launches=200, graph=graph) for _ in range(3))
        busy = min(launch_floor_us(launches=200, graph=graph, spin_us=5.0) for _ in range(3))
        assert 0.3 < empty < 20.0, (graph, empty)
        assert 5.0 <= busy < 5.0 + max(4.0, 2.0 * empty), (graph, empty, busy)


def test_errors():
    with pytest.raises(tdc_amd.TdcError):
        tdc_amd.Conv2dPlan(1, 4, 4, 2, 2, 5, 5, 1, 0)  # filter larger than input
    plan = tdc_amd.Conv2dPlan(1, 4, 4, 6, 6, 3, 3, 1, 1)
    with pytest.raises(tdc_amd.TdcError):  # forward before weights
        plan.forward(torch.zeros(1, 4, 6, 6, device="cuda"))
    with pytest.raises(ValueError):
        plan.set_weights(torch.zeros(4, 4, 1, 1))
    bad = tdc_amd.Tile(32, 1, 1, 1, 1, 1, 3, 4)  # cch not a multiple of kc
    with pytest.raises(tdc_amd.TdcError):
        tdc_amd.Conv2dPlan(1, 4, 4, 6, 6, 3, 3, 1, 1, tile=bad)
