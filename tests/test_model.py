"""Host-side checks of the launch geometry and the analytic gfx950 tile model (no GPU needed)."""
import math

import pytest

import tdc_amd
from oracle import ref

LDS_BYTES = 160 * 1024


def conv3(c, n, hw, stride=1):
    return tdc_amd.conv_desc(1, c, n, hw, hw, 3, 3, stride, 1)


@pytest.mark.parametrize("hw", ref.SWEEP_HW)
@pytest.mark.parametrize("r1,r2", ref.SWEEP_RANKS)
def test_every_candidate_is_launchable_and_covers_the_output(hw, r1, r2):
    d = conv3(r1, r2, hw)
    tiles = tdc_amd.model_enumerate(d)
    assert tiles, "no tile for a sweep shape"
    for t in tiles[:: max(1, len(tiles) // 60)]:
        i = tdc_amd.model_evaluate(d, t)
        lanes = t.mf * t.nb * t.wn
        # a Winograd lane stands for a 2x2-pixel tile and tw counts those
        tw_px, lane_px = (2 * t.tw, 4) if t.alg == 1 else (t.tw, 1)
        assert 1 <= i.th and i.th * tw_px <= lanes * lane_px
        ntx, nty = math.ceil(hw / tw_px), math.ceil(hw / i.th)
        assert i.grid_x == ntx * nty and ntx * tw_px >= hw and nty * i.th >= hw     # tiles cover the image
        assert i.grid_y * t.mf * t.mb * t.wm >= r2                                   # ... and all channels
        assert i.nchunks * t.cch >= r1 and t.cch % ((2 if t.mf == 32 else 4) * t.wk) == 0
        assert i.block_threads == 64 * (t.wm * t.wn * t.wk + t.wl) <= 1024      # computing waves + loader waves
        # (the streamed paths stage nothing: their LDS only holds the partial sums of a split over waves)
        assert (0 if t.alg >= 3 else 1) <= i.lds_bytes <= LDS_BYTES
        assert i.wg_per_cu >= 1 and i.pred_us > 0


def test_streamed_tiles_only_where_they_apply():
    """tile.alg = 3 (1x1) and 4 (3x3) read both operands from global memory: one 16x16 block per workgroup, every
    input channel in one pass, 1/2/4/8 runs of 16 channels (alg 3) or 1/2/4 groups of 4 channels (alg 4) per wave."""
    d1 = tdc_amd.conv_desc(1, 256, 64, 14, 14, 1, 1, 1, 0)
    ok = tdc_amd.model_evaluate(d1, tdc_amd.Tile(16, 1, 1, 1, 1, 4, 256, 16, 1, 0, 3))
    assert (ok.grid_x, ok.grid_y, ok.block_threads, ok.lds_bytes, ok.nchunks) == (13, 4, 256, 4096, 1)
    split = tdc_amd.model_evaluate(d1, tdc_amd.Tile(16, 1, 1, 1, 1, 4, 128, 16, 2, 0, 3))   # two workgroups, 128 channels each
    assert (split.grid_x, split.grid_y, split.grid_z, split.nchunks) == (13, 4, 2, 2)
    # stride 2: runs of 16 consecutive output pixels (7 x 7 = 49 of them), whatever the rows of the image are
    s2 = tdc_amd.model_evaluate(tdc_amd.conv_desc(1, 256, 64, 14, 14, 1, 1, 2, 0), tdc_amd.Tile(16, 1, 1, 1, 1, 4, 256, 16, 1, 0, 3))
    assert (s2.grid_x, s2.grid_y) == (4, 4)
    for d, t in [(d1, tdc_amd.Tile(16, 1, 1, 1, 1, 1, 256, 16, 1, 0, 3)),      # 16 runs per wave
                 (d1, tdc_amd.Tile(16, 1, 1, 1, 1, 4, 128, 16, 1, 0, 3)),      # not all channels in one pass
                 (d1, tdc_amd.Tile(16, 1, 1, 1, 1, 4, 256, 16, 2, 0, 3)),      # two slices of which one is empty
                 (d1, tdc_amd.Tile(16, 1, 1, 1, 2, 4, 256, 16, 1, 0, 3)),      # more than one block
                 (d1, tdc_amd.Tile(32, 1, 1, 1, 1, 4, 256, 16, 1, 0, 3)),
                 (d1, tdc_amd.Tile(16, 1, 1, 1, 1, 4, 256, 8, 1, 0, 3)),       # tw must be 16 (or all pixels)
                 (tdc_amd.conv_desc(1, 2048, 64, 7, 7, 1, 1, 1, 0), tdc_amd.Tile(16, 1, 1, 1, 1, 16, 2048, 16, 1, 0, 3)),  # 8 runs x 16 waves
                 (tdc_amd.conv_desc(1, 256, 64, 14, 14, 1, 1, 2, 0), tdc_amd.Tile(16, 1, 1, 1, 1, 4, 128, 16, 2, 0, 3)),   # stride 2 and a split across workgroups
                 (conv3(64, 64, 14), tdc_amd.Tile(16, 1, 1, 1, 1, 4, 64, 14, 1, 0, 3))]:
        with pytest.raises(tdc_amd.TdcError):
            tdc_amd.model_evaluate(d, t)
    d3 = conv3(64, 64, 14)
    ok = tdc_amd.model_evaluate(d3, tdc_amd.Tile(16, 1, 1, 1, 1, 4, 64, 14, 1, 0, 4))
    assert (ok.grid_x, ok.grid_y, ok.th, ok.block_threads) == (14, 4, 1, 256)
    assert tdc_amd.model_evaluate(conv3(64, 64, 14, stride=2), tdc_amd.Tile(16, 1, 1, 1, 1, 4, 64, 7, 1, 0, 4)).th == 2
    wide = tdc_amd.model_evaluate(d3, tdc_amd.Tile(16, 1, 1, 2, 1, 4, 64, 14, 1, 0, 4))   # two blocks of 16 channels per workgroup
    assert (wide.grid_x, wide.grid_y, wide.block_threads) == (14, 2, 512)
    for d, t in [(d3, tdc_amd.Tile(16, 1, 1, 1, 1, 2, 64, 14, 1, 0, 4)),       # 8 groups per wave
                 (d3, tdc_amd.Tile(16, 1, 1, 1, 1, 4, 32, 14, 1, 0, 4)),       # not all channels in one pass
                 (d3, tdc_amd.Tile(16, 1, 1, 1, 1, 4, 64, 14, 1, 2, 4)),       # loader waves
                 (d3, tdc_amd.Tile(16, 1, 1, 8, 1, 4, 64, 14, 1, 0, 4)),       # 32 waves
                 (d3, tdc_amd.Tile(16, 1, 2, 1, 1, 4, 64, 14, 1, 0, 4)),       # two pixel blocks per wave, one 14-pixel tile per row
                 (conv3(64, 64, 56), tdc_amd.Tile(16, 1, 2, 1, 1, 4, 64, 16, 1, 0, 4)),   # several blocks need rows of 14 pixels
                 (conv3(64, 64, 56), tdc_amd.Tile(16, 1, 2, 1, 1, 4, 32, 14, 2, 0, 4)),   # ... and no split across workgroups
                 (conv3(64, 64, 56, stride=2), tdc_amd.Tile(16, 1, 2, 1, 1, 4, 64, 14, 1, 0, 4)),   # ... and stride 1
                 (tdc_amd.conv_desc(1, 64, 64, 14, 14, 3, 3, 1, 2, 2), tdc_amd.Tile(16, 1, 1, 1, 1, 4, 64, 14, 1, 0, 4)),  # dilation 2
                 (d1, tdc_amd.Tile(16, 1, 1, 1, 1, 4, 256, 16, 1, 0, 4))]:
        with pytest.raises(tdc_amd.TdcError):
            tdc_amd.model_evaluate(d, t)
    # nb = 2 or 4 neighbouring 14-pixel row tiles per workgroup (the weights a wave holds feed nb MFMAs each)
    nb4 = tdc_amd.model_evaluate(conv3(64, 64, 56), tdc_amd.Tile(16, 1, 4, 1, 1, 8, 64, 14, 1, 0, 4))
    assert (nb4.grid_x, nb4.grid_y, nb4.th, nb4.block_threads, nb4.lds_bytes) == (56, 4, 1, 512, 8 * 4 * 1024)
    nb2 = tdc_amd.model_evaluate(conv3(64, 64, 28), tdc_amd.Tile(16, 1, 2, 1, 1, 16, 64, 14, 1, 0, 4))
    assert (nb2.grid_x, nb2.grid_y, nb2.block_threads) == (28, 4, 1024)
    assert any(t.alg == 4 and t.nb == 4 for t in tdc_amd.model_enumerate(conv3(64, 64, 56)))
    assert not any(t.alg == 4 and t.nb > 1 for t in tdc_amd.model_enumerate(conv3(64, 64, 14)))
    # the enumeration offers them for every 1x1 / 3x3 shape they fit, and only there
    assert any(t.alg == 3 for t in tdc_amd.model_enumerate(d1)) and not any(t.alg == 4 for t in tdc_amd.model_enumerate(d1))
    assert any(t.alg == 4 for t in tdc_amd.model_enumerate(d3)) and not any(t.alg == 3 for t in tdc_amd.model_enumerate(d3))
    assert not any(t.alg >= 3 for t in tdc_amd.model_enumerate(tdc_amd.conv_desc(1, 3, 64, 32, 32, 7, 7, 2, 3)))


def test_streamed_winograd_tiles_only_where_they_apply():
    """tile.alg = 5: Winograd F(2x2,3x3) with both operands read from global memory; 3x3 / stride 1 / pad 1 / even width,
    a tile-row block of 2 x 28 pixels per workgroup, every input channel in one pass, 1 to 4 groups of four per wave."""
    d = conv3(64, 64, 56)
    ok = tdc_amd.model_evaluate(d, tdc_amd.Tile(16, 1, 1, 1, 1, 8, 64, 28, 1, 0, 5))
    assert (ok.grid_x, ok.grid_y, ok.th, ok.block_threads, ok.lds_bytes, ok.nchunks) == (56, 4, 2, 512, 8 * 16 * 64 * 4, 1)
    from tdc_amd import _lib
    name, regs, waves = _lib.model_kernel_info(d, ok.tile, False)
    assert name == "tdc_wino3x3_stream_kernel<2, 16>" and regs <= 128 and waves >= 4
    wide = tdc_amd.model_evaluate(d, tdc_amd.Tile(16, 1, 1, 2, 1, 4, 64, 28, 1, 0, 5))     # two blocks of 16 channels, four groups per wave
    assert (wide.grid_x, wide.grid_y, wide.block_threads) == (56, 2, 512)
    ragged = tdc_amd.model_evaluate(conv3(50, 20, 30), tdc_amd.Tile(16, 1, 1, 1, 1, 13, 52, 28, 1, 0, 5))   # 13 groups, one per wave
    assert (ragged.grid_x, ragged.grid_y) == (2 * 15, 2)
    for dd, t in [(d, tdc_amd.Tile(16, 1, 1, 1, 1, 2, 64, 28, 1, 0, 5)),        # eight groups per wave
                  (d, tdc_amd.Tile(16, 1, 1, 1, 1, 8, 32, 28, 1, 0, 5)),        # not all channels in one pass
                  (d, tdc_amd.Tile(16, 1, 1, 1, 1, 16, 128, 28, 1, 0, 5)),      # half of the waves without channels
                  (d, tdc_amd.Tile(16, 1, 1, 1, 1, 8, 64, 14, 1, 0, 5)),        # tw must be 28
                  (d, tdc_amd.Tile(16, 1, 1, 1, 1, 8, 64, 28, 2, 0, 5)),        # no split across workgroups
                  (d, tdc_amd.Tile(16, 1, 1, 1, 1, 8, 64, 28, 1, 2, 5)),        # no loader waves
                  (d, tdc_amd.Tile(16, 1, 1, 1, 2, 8, 64, 28, 1, 0, 5)),        # one block per wave set
                  (d, tdc_amd.Tile(16, 1, 1, 8, 1, 4, 64, 28, 1, 0, 5)),        # 32 waves
                  (conv3(64, 64, 7), tdc_amd.Tile(16, 1, 1, 1, 1, 8, 64, 28, 1, 0, 5)),                 # odd width
                  (conv3(64, 64, 56, stride=2), tdc_amd.Tile(16, 1, 1, 1, 1, 8, 64, 28, 1, 0, 5)),      # stride 2
                  (tdc_amd.conv_desc(1, 64, 64, 56, 56, 3, 3, 1, 0), tdc_amd.Tile(16, 1, 1, 1, 1, 8, 64, 28, 1, 0, 5)),     # pad 0
                  (tdc_amd.conv_desc(1, 64, 64, 56, 56, 3, 3, 1, 2, 2), tdc_amd.Tile(16, 1, 1, 1, 1, 8, 64, 28, 1, 0, 5)),  # dilation
                  (tdc_amd.conv_desc(1, 64, 64, 56, 56, 1, 1, 1, 0), tdc_amd.Tile(16, 1, 1, 1, 1, 8, 64, 28, 1, 0, 5))]:
        with pytest.raises(tdc_amd.TdcError):
            tdc_amd.model_evaluate(dd, t)
    assert any(t.alg == 5 for t in tdc_amd.model_enumerate(d))
    assert not any(t.alg == 5 for t in tdc_amd.model_enumerate(conv3(64, 64, 7)))
    assert not any(t.alg == 5 for t in tdc_amd.model_enumerate(conv3(64, 64, 56, stride=2)))
    assert not any(t.alg == 5 for t in tdc_amd.model_enumerate(d, ) if t.ks != 1 or t.wl != 0)
    # the model takes it where it was measured faster: the mid-size 56 x 56 layers
    assert tdc_amd.model_select(d).tile.alg == 5 and tdc_amd.model_select(conv3(64, 128, 56)).tile.alg == 5
    assert tdc_amd.model_select(conv3(16, 16, 56)).tile.alg == 4 and tdc_amd.model_select(conv3(128, 128, 28)).tile.alg == 4


def test_winograd_tiles_only_where_the_algorithm_applies():
    """tile.alg needs a 3x3 / stride 1 / dilation 1 convolution and one 16x16 block per wave; the model hands the
    large 56x56 layers to it and keeps the small ones on the direct path."""
    w = tdc_amd.Tile(16, 1, 1, 1, 2, 2, 32, 14, 1, 0, 1)
    assert tdc_amd.model_evaluate(conv3(128, 128, 56), w).th == 4           # 2 tile rows of 14 tiles = 4 x 28 pixels
    for d, t in [(conv3(64, 64, 56, stride=2), w),
                 (tdc_amd.conv_desc(1, 64, 64, 56, 56, 1, 1, 1, 0), w),
                 (tdc_amd.conv_desc(1, 64, 64, 56, 56, 3, 3, 1, 2, 2), w),      # dilation 2
                 (conv3(128, 128, 56), tdc_amd.Tile(32, 1, 1, 1, 2, 2, 32, 14, 1, 0, 1)),
                 (conv3(128, 128, 56), tdc_amd.Tile(16, 1, 2, 1, 2, 2, 32, 14, 1, 0, 1)),
                 (conv3(128, 128, 56), tdc_amd.Tile(16, 1, 1, 1, 2, 2, 32, 29, 1, 0, 1)),   # wider than the image in tiles
                 (conv3(128, 128, 56), tdc_amd.Tile(16, 1, 1, 2, 4, 2, 32, 14, 1, 0, 1))]:   # 16 waves: over the budget of 8
        with pytest.raises(tdc_amd.TdcError):
            tdc_amd.model_evaluate(d, t)
    # alg = 2 (weights from global memory): 3x3 only, one block per wave, an even number of channel groups per wave
    assert tdc_amd.model_evaluate(conv3(64, 64, 28), tdc_amd.Tile(16, 1, 1, 1, 1, 4, 64, 7, 1, 0, 2)).lds_bytes < \
        tdc_amd.model_evaluate(conv3(64, 64, 28), tdc_amd.Tile(16, 1, 1, 1, 1, 4, 64, 7, 1, 0, 0)).lds_bytes
    for d, t in [(tdc_amd.conv_desc(1, 64, 64, 56, 56, 1, 1, 1, 0), tdc_amd.Tile(16, 1, 1, 1, 1, 4, 64, 7, 1, 0, 2)),
                 (conv3(64, 64, 28), tdc_amd.Tile(16, 2, 1, 1, 1, 4, 64, 7, 1, 0, 2)),
                 (conv3(64, 64, 28), tdc_amd.Tile(16, 1, 1, 1, 1, 4, 16, 7, 1, 0, 2)),      # one channel group per wave
                 (conv3(64, 64, 28), tdc_amd.Tile(16, 1, 1, 1, 1, 4, 64, 7, 1, 0, 3))]:
        with pytest.raises(tdc_amd.TdcError):
            tdc_amd.model_evaluate(d, t)
    # (the staged Winograd tiles keep the large layers where the streamed one does not apply: batches, 112 x 112 images)
    assert tdc_amd.model_select(tdc_amd.conv_desc(4, 128, 128, 56, 56, 3, 3, 1, 1)).tile.alg == 1
    assert tdc_amd.model_select(conv3(128, 128, 56)).tile.alg == 5
    assert tdc_amd.model_select(conv3(32, 32, 14)).tile.alg != 1
    assert not any(t.alg == 1 for t in tdc_amd.model_enumerate(conv3(64, 64, 56, stride=2)))


def test_algorithmic_work_and_roofline_of_config1():
    i = tdc_amd.model_select(conv3(32, 32, 56))
    assert i.flops == 2 * 56 * 56 * 32 * 32 * 9 == 57802752
    assert i.bytes == 4 * (32 * 56 * 56 + 32 * 56 * 56 + 9 * 32 * 32) == 839680
    assert abs(i.roof_us - 57802752 / 157.3e6) < 1e-9          # fp32-bound: 0.367 us
    big = tdc_amd.model_select(conv3(128, 128, 56))
    assert abs(big.roof_us - 5.8795) < 1e-3
    tiny = tdc_amd.model_select(conv3(16, 16, 7))
    assert abs(tiny.roof_us - 15488 / 8e6) < 1e-9               # HBM-bound: 0.0019 us


def test_select_is_argmin_of_the_enumeration():
    d = conv3(64, 64, 28)
    best = tdc_amd.model_select(d)
    preds = [tdc_amd.model_evaluate(d, t).pred_us for t in tdc_amd.model_enumerate(d)]
    assert best.pred_us == min(preds)


def test_model_prefers_split_k_waves_for_tiny_layers_and_more_tiles_for_big_ones():
    small = tdc_amd.model_select(conv3(128, 128, 7))
    big = tdc_amd.model_select(conv3(128, 128, 56))
    assert small.tile.wk >= 2                       # few pixels: parallelism has to come from input channels
    assert big.grid_x * big.grid_y >= 128           # enough workgroups to spread over the 256 CUs
    assert big.pred_us > small.pred_us


def test_one_by_one_convolutions_run_on_the_flattened_image():
    d = tdc_amd.conv_desc(1, 256, 64, 56, 56, 1, 1, 1, 0)
    i = tdc_amd.model_select(d)
    assert i.th == 1 and i.tile.tw == i.tile.mf * i.tile.nb * i.tile.wn     # a tile is a run of consecutive pixels
    assert i.flops == 2 * 56 * 56 * 256 * 64


def test_invalid_tiles_are_rejected():
    d = conv3(32, 32, 14)
    for t in [tdc_amd.Tile(8, 1, 1, 1, 1, 1, 32, 4),      # mf
              tdc_amd.Tile(16, 3, 1, 1, 1, 1, 32, 4),     # mb
              tdc_amd.Tile(16, 1, 1, 4, 4, 4, 32, 4),     # 64 waves
              tdc_amd.Tile(16, 1, 1, 1, 1, 1, 30, 4),     # cch not a multiple of 4
              tdc_amd.Tile(16, 1, 1, 1, 1, 1, 32, 15),    # tw wider than the image
              tdc_amd.Tile(16, 1, 1, 1, 1, 1, 32, 0)]:
        with pytest.raises(tdc_amd.TdcError):
            tdc_amd.model_evaluate(d, t)
    with pytest.raises(tdc_amd.TdcError):                  # LDS overflow
        tdc_amd.model_evaluate(conv3(2048, 256, 56), tdc_amd.Tile(32, 2, 2, 2, 2, 1, 2048, 56))


def test_stride2_and_stem_shapes_have_tiles():
    for d in (conv3(64, 64, 56, 2), conv3(256, 256, 14, 2), tdc_amd.conv_desc(1, 3, 64, 224, 224, 7, 7, 2, 3),
              tdc_amd.conv_desc(8, 64, 16, 56, 56, 3, 3, 1, 1)):
        i = tdc_amd.model_select(d)
        assert i.grid_x > 0 and i.lds_bytes <= LDS_BYTES


def test_model_register_table_matches_the_compiled_kernels():
    """Occupancy probe, host side: for every kernel instantiation that any candidate tile of a spread of layers maps
    to, the registers per lane the model's occupancy term assumes equal what hipcc reports for the build at hand
    (VGPRs + AGPRs, rounded up to the allocation granule of 8), and no kernel spills to scratch.  The reference
    measures occupancy per candidate by compiling and probing each one
    (2080Ti-evaluation/Gen-occupancy/template.cu:277-284)."""
    from tdc_amd import _lib
    compiled = _lib.kernel_resources()
    assert len(compiled) >= 90
    assert all(r["scratch"] == 0 for r in compiled.values()), "a kernel spills registers to scratch memory"
    seen = {}
    descs = [conv3(64, 64, 56), conv3(128, 128, 56), conv3(16, 16, 7), conv3(256, 256, 7), conv3(40, 24, 13, stride=2),
             tdc_amd.conv_desc(1, 256, 64, 56, 56, 1, 1, 1, 0), tdc_amd.conv_desc(1, 2048, 256, 7, 7, 1, 1, 1, 0),
             tdc_amd.conv_desc(1, 64, 128, 56, 56, 1, 1, 2, 0), tdc_amd.conv_desc(1, 3, 64, 224, 224, 7, 7, 2, 3),
             tdc_amd.conv_desc(2, 100, 36, 14, 14, 1, 1, 1, 0)]
    for d in descs:
        for t in tdc_amd.model_enumerate(d):
            for extras in (False, True):
                try:
                    name, regs, waves = _lib.model_kernel_info(d, t, extras)
                except tdc_amd.TdcError:
                    continue   # (no instantiation with extras for this path)
                seen[name] = (regs, waves)
                if not extras:
                    assert tdc_amd.model_evaluate(d, t).vgpr_estimate == regs
    assert len(seen) >= 60, sorted(seen)
    for name, (regs, waves) in sorted(seen.items()):
        assert name in compiled, f"{name}: the model names a kernel the build does not contain"
        real = compiled[name]["vgprs"] + compiled[name]["agprs"]
        assert regs == (real + 7) // 8 * 8, f"{name}: model assumes {regs} registers per lane, compiled kernel uses {real}"
        # the compiler's own waves-per-SIMD figure (vector and scalar register limits) is the model's
        assert compiled[name]["waves_per_simd"] == waves, f"{name}: {compiled[name]} against the model's {waves} waves per SIMD"
