"""The entry point that allocates nothing (tdc_conv_forward_static_ws): partial tiles and ticket counters of a split
across workgroups live in the library's static device array.  Checked against tdc_conv_forward, bit for bit, on two
calls in a row, the second on a smaller problem (so the array still holds the first call's partials and its counter
region is larger than the second call's)."""
import math

import numpy as np
import pytest
import torch

import tdc_amd
from tdc_amd import _lib
from oracle import ref
from util import assert_close, seeded

pytestmark = pytest.mark.gpu


def _case(seed, B, C, N, H, W, K):
    g = seeded(seed)
    x = torch.rand(B, C, H, W, generator=g) * 2 - 1
    w = torch.empty(N, C, K, K).normal_(0, math.sqrt(2.0 / (C * K * K)), generator=g)
    bias = torch.randn(N, generator=g)
    resid = torch.randn(B, N, H, W, generator=g)
    return x, w, bias, resid


def _split_tile(desc, alg):
    tiles = [t for t in tdc_amd.model_enumerate(desc) if t.alg == alg and t.ks > 1]
    assert tiles, "no tile with a split across workgroups for this shape"
    return max(tiles, key=lambda t: t.ks)


def test_static_workspace_entry_point_matches_the_allocating_one():
    # first call: 256 -> 256 @7x7, 3x3, streamed kernel with its input channels dealt to several workgroups;
    # second call: a smaller, ragged problem on the staged kernel with five slices; third: a 1x1 layer, batch 2
    cases = [((1, 256, 256, 7, 7), 3, 1, None, 4), ((2, 40, 37, 9, 9), 3, 1, tdc_amd.Tile(16, 1, 1, 1, 1, 1, 8, 8, ks=5), 0),
             ((2, 300, 24, 3, 5), 1, 0, None, 3)]
    for i, (shape, K, pad, tile, alg) in enumerate(cases):
        B, C, N, H, W = shape
        print("static ws case", i, shape, K, flush=True)
        x, w, bias, resid = _case(7000 + i, B, C, N, H, W, K)
        desc = tdc_amd.conv_desc(B, C, N, H, W, K, K, 1, pad)
        tile = tile or _split_tile(desc, alg)
        plan = tdc_amd.Conv2dPlan(B, C, N, H, W, K, K, 1, pad, 1, True, True, tile=tile).set_weights(w, bias)
        assert plan.info.tile.ks > 1
        xd, rd = x.cuda(), resid.cuda()
        want = torch.full((B, N, H, W), float("nan"), device="cuda")
        plan.forward(xd, rd, out=want)
        torch.cuda.synchronize()
        for rep in range(2):
            got = torch.full((B, N, H, W), float("nan"), device="cuda")
            plan.forward_static_ws(xd, rd, out=got)
            torch.cuda.synchronize()
            assert torch.equal(got, want), f"case {i} rep {rep}: static-workspace result differs from tdc_conv_forward"
        assert_close(want.cpu().numpy(), ref.conv2d_c(x.numpy(), w.numpy(), bias.numpy(), resid.numpy(), pad=pad, relu=True),
                     f"case {i} vs oracle")
        plan.close()


def test_static_workspace_rejects_plans_beyond_its_size():
    # 64 images x 8 slices x 256 channels x 49 pixels x 4 bytes = 25.7 MB of partial tiles: more than the 4 MiB array
    B, C, N, H, W = 64, 2048, 256, 7, 7
    desc = tdc_amd.conv_desc(B, C, N, H, W, 1, 1, 1, 0)
    tile = _split_tile(desc, 0)
    plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 1, 1, 1, 0, tile=tile)
    plan.set_weights(torch.zeros(N, C, 1, 1))
    x = torch.zeros(B, C, H, W, device="cuda")
    with pytest.raises(tdc_amd.TdcError) as e:
        plan.forward_static_ws(x)
    assert e.value.status == _lib.TDC_ERR_UNSUPPORTED and "static scratch" in str(e.value)
    plan.close()


def test_plans_without_a_split_need_no_scratch():
    x, w = ref.make_core_case(14, 32, 32)
    plan = tdc_amd.Conv2dPlan(1, 32, 32, 14, 14, 3, 3, 1, 1).set_weights(w)
    assert plan.info.tile.ks == 1
    a = plan.forward(x.cuda())
    b = plan.forward_static_ws(x.cuda())
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    plan.close()


def test_static_workspace_entry_point_allocates_nothing_and_replays_from_a_graph():
    """The two properties the entry point exists for: no device allocation per call (free device memory as the driver
    reports it does not move over many calls), and usable under stream capture — the captured graph is replayed several
    times with the program's own eager work and synchronisations in between and inputs that change between replays, and
    every replay is compared bit for bit with the eager entry point.  The symbol address of the static array is resolved
    by the eager call in front of the capture."""
    B, C, N, H, W = 1, 256, 256, 7, 7
    x, w, bias, resid = _case(7100, B, C, N, H, W, 3)
    tile = _split_tile(tdc_amd.conv_desc(B, C, N, H, W, 3, 3, 1, 1), 4)
    plan = tdc_amd.Conv2dPlan(B, C, N, H, W, 3, 3, 1, 1, 1, True, True, tile=tile).set_weights(w, bias)
    xd, rd = x.cuda(), resid.cuda()
    got = torch.empty(B, N, H, W, device="cuda")
    want = torch.empty(B, N, H, W, device="cuda")
    plan.forward_static_ws(xd, rd, out=got)      # eager: also resolves the address of this device's copy of the array
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(50):
        plan.forward_static_ws(xd, rd, out=got)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "free device memory moved across 50 calls"
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            plan.forward_static_ws(xd, rd, out=got)
    g = seeded(7101)
    for rep in range(4):
        xd.copy_((torch.rand(B, C, H, W, generator=g) * 2 - 1).cuda())     # eager work between the replays
        plan.forward(xd, rd, out=want)
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {rep}: graph-replayed static-workspace result differs from tdc_conv_forward"
    del graph
    plan.close()
