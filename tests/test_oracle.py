"""Pins the CPU oracle (oracle/) before it is trusted as the arbiter of the GPU kernels.

Each statement of the convolution — the C restatement (double accumulation), the sequential run of
the reference's own tiled kernel, and torch.nn.functional.conv2d (the call the reference operator
makes) — is checked against facts none of them was written from: exact integer golden vectors
computed with Python integers, closed forms, shift/delta kernels that pin tap orientation and
padding, the stride-2 subsampling identity, and brute-force loops on tiny shapes.
"""
import hashlib
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import ref, tdc_model_ref
from util import assert_close

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def load(name):
    with open(os.path.join(GOLD, name)) as f:
        return json.load(f)


# ---- golden vectors ----------------------------------------------------------------------------
@pytest.mark.parametrize("case", load("small_cases.json"), ids=lambda c: "C%dN%dH%dW%dK%ds%dp%dd%d" % (
    c["C"], c["N"], c["H"], c["W"], c["K"], c["stride"], c["pad"], c["dil"]))
def test_golden_integer_cases_exact(case):
    x = np.array(case["x"], np.float32)[None]
    w = np.array(case["w"], np.float32)
    want = np.array(case["out"], np.float32)[None]
    got_c = ref.conv2d_c(x, w, stride=case["stride"], pad=case["pad"], dil=case["dil"])
    assert np.array_equal(got_c, want)
    got_np = ref.conv2d_numpy(x, w, stride=case["stride"], pad=case["pad"], dil=case["dil"])
    assert np.array_equal(got_np, want)
    got_t = ref.conv2d_torch(torch.from_numpy(x), torch.from_numpy(w), stride=case["stride"], pad=case["pad"],
                             dil=case["dil"]).numpy()
    assert np.array_equal(got_t, want)


def test_seeded_generator_has_not_drifted():
    rec = load("seeded_inputs.json")
    for r in rec["core"]:
        x, w = ref.make_core_case(r["hw"], r["r1"], r["r2"], seed=r["seed"])
        assert hashlib.sha256(x.numpy().tobytes()).hexdigest() == r["x_sha256"]
        assert hashlib.sha256(w.numpy().tobytes()).hexdigest() == r["w_sha256"]
        y = ref.conv2d_torch(x, w, pad=1).flatten()[r["sample_index"]].numpy()
        np.testing.assert_allclose(y, np.array(r["sample_out"], np.float32), rtol=1e-5, atol=1e-6)
    for b in rec["blocks"][:2]:
        x, first, core, last = ref.make_block_case(b["C"], b["R1"], b["R2"], b["N"], b["hw"])
        assert hashlib.sha256(x.numpy().tobytes()).hexdigest() == b["x_sha256"]
        assert hashlib.sha256(core.numpy().tobytes()).hexdigest() == b["core_sha256"]


def test_input_distributions_match_the_benchmark_recipe():
    x, w = ref.make_core_case(56, 32, 32, seed=0)
    assert x.shape == (1, 32, 56, 56) and w.shape == (32, 32, 3, 3)
    assert -1 <= float(x.min()) < -0.99 and 0.99 < float(x.max()) <= 1
    assert abs(float(w.std()) - math.sqrt(2 / (32 * 9))) < 2e-3
    x, first, core, last = ref.make_block_case(256, 64, 64, 256, 56)
    f = first.reshape(64, 256)
    assert torch.allclose(f @ f.t(), torch.eye(64), atol=1e-5)       # orthonormal rows = columns of Q
    l = last.reshape(256, 64)
    assert torch.allclose(l.t() @ l, torch.eye(64), atol=1e-5)
    assert abs(float(core.std()) - 0.02) < 1e-3


# ---- closed forms and invariants ------------------------------------------------------------------
def test_centre_delta_identity_and_single_tap_shift():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1, 3, 6, 7)).astype(np.float32)
    w = np.zeros((3, 3, 3, 3), np.float32)
    for c in range(3):
        w[c, c, 1, 1] = 1
    assert np.array_equal(ref.conv2d_c(x, w, pad=1), x)
    # one off-centre tap: out[oy,ox] = in[oy-1+r, ox-1+s]  (cross-correlation, not flipped)
    for (r, s) in [(0, 0), (0, 2), (2, 1), (1, 0)]:
        w = np.zeros((1, 3, 3, 3), np.float32)
        w[0, 1, r, s] = 1
        want = np.zeros((1, 1, 6, 7), np.float32)
        for oy in range(6):
            for ox in range(7):
                iy, ix = oy - 1 + r, ox - 1 + s
                if 0 <= iy < 6 and 0 <= ix < 7:
                    want[0, 0, oy, ox] = x[0, 1, iy, ix]
        assert np.array_equal(ref.conv2d_c(x, w, pad=1), want)
        assert np.array_equal(ref.conv2d_torch(torch.from_numpy(x), torch.from_numpy(w), pad=1).numpy(), want)


def box_sum_closed_form(x):
    """All-ones 3x3 weights: every output channel = 3x3 box sum of the channel-summed image."""
    C, H, W = x.shape
    s = np.pad(x.sum(axis=0).astype(np.float64), 1)
    return sum(s[r:r + H, c:c + W] for r in range(3) for c in range(3))


@pytest.mark.parametrize("shape", [(32, 32, 14, 14), (64, 32, 7, 7), (96, 64, 7, 7), (32, 32, 28, 28)])
def test_reference_known_answer_closed_form(shape):
    """Integers 0..9 x all-ones weights (template_benchmark_cudnn.template:418-428): exact in fp32."""
    C, N, H, W = shape
    x = np.random.default_rng(C + H).integers(0, 10, size=(C, H, W)).astype(np.float32)
    w = np.ones((N, C, 3, 3), np.float32)
    want = box_sum_closed_form(x)
    got = ref.conv2d_c(x[None], w, pad=1)[0]
    assert np.abs(got - want[None]).sum() == 0.0


def test_stride2_is_subsampled_stride1():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 5, 12, 10)).astype(np.float32)
    w = rng.standard_normal((4, 5, 3, 3)).astype(np.float32)
    full = ref.conv2d_c(x, w, pad=1)
    assert np.array_equal(ref.conv2d_c(x, w, stride=2, pad=1), full[:, :, ::2, ::2])


def test_linearity_and_channel_permutation():
    rng = np.random.default_rng(3)
    x1 = rng.standard_normal((1, 6, 9, 9)).astype(np.float32)
    x2 = rng.standard_normal((1, 6, 9, 9)).astype(np.float32)
    w = rng.standard_normal((5, 6, 3, 3)).astype(np.float32)
    y = ref.conv2d_c(2 * x1 + x2, w, pad=1)
    np.testing.assert_allclose(y, 2 * ref.conv2d_c(x1, w, pad=1) + ref.conv2d_c(x2, w, pad=1), rtol=1e-5, atol=1e-5)
    perm = rng.permutation(6)
    np.testing.assert_allclose(ref.conv2d_c(x1[:, perm], w[:, perm], pad=1), ref.conv2d_c(x1, w, pad=1), rtol=1e-6, atol=1e-6)
    operm = rng.permutation(5)
    assert np.array_equal(ref.conv2d_c(x1, w[operm], pad=1), ref.conv2d_c(x1, w, pad=1)[:, operm])


@pytest.mark.parametrize("cfg", [(1, 3, 4, 5, 5, 3, 1, 1, 1), (2, 4, 3, 5, 4, 3, 2, 1, 1), (1, 2, 2, 7, 6, 3, 1, 2, 2),
                                 (1, 3, 2, 6, 6, 5, 1, 2, 1), (1, 4, 4, 3, 3, 1, 1, 0, 1), (1, 1, 1, 9, 9, 7, 2, 3, 1)])
def test_c_oracle_vs_bruteforce_and_torch(cfg):
    B, C, N, H, W, K, stride, pad, dil = cfg
    rng = np.random.default_rng(sum(cfg))
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    w = rng.standard_normal((N, C, K, K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    c = ref.conv2d_c(x, w, b, stride=stride, pad=pad, dil=dil)
    n = ref.conv2d_numpy(x, w, b, stride=stride, pad=pad, dil=dil)
    t = ref.conv2d_torch(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(b), stride, pad, dil).numpy()
    np.testing.assert_allclose(c, n, rtol=1e-6, atol=1e-6)
    assert_close(t, c, "F.conv2d vs C oracle")


def test_epilogue_order_bias_residual_relu():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((1, 3, 5, 5)).astype(np.float32)
    w = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    b = rng.standard_normal(4).astype(np.float32)
    r = rng.standard_normal((1, 4, 5, 5)).astype(np.float32)
    base = ref.conv2d_c(x, w, pad=1).astype(np.float64)
    want = np.maximum(base + b[None, :, None, None] + r, 0)
    np.testing.assert_allclose(ref.conv2d_c(x, w, b, r, pad=1, relu=True), want, rtol=1e-6, atol=1e-6)


def test_torch_vs_c_oracle_on_a_sweep_shape():
    x, w = ref.make_core_case(14, 64, 64)
    assert_close(ref.conv2d_torch(x, w, pad=1).numpy(), ref.conv2d_c(x.numpy(), w.numpy(), pad=1), "14/64/64")


# ---- TKConv composition -------------------------------------------------------------------------
def test_tkconv_composition_matches_three_convs():
    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, 10, 8, 8, generator=g)
    first = torch.randn(4, 10, 1, 1, generator=g)
    core = torch.randn(6, 4, 3, 3, generator=g)
    last = torch.randn(12, 6, 1, 1, generator=g)
    bias = torch.randn(12, generator=g)
    for stride in (1, 2):
        out_c, f1, f2 = ref.tkconv_c(x.numpy(), first.numpy(), core.numpy(), last.numpy(), bias.numpy(), stride, 1, 1)
        out_t = ref.tkconv_torch(x, first, core, last, bias, stride, 1, 1).numpy()
        assert_close(out_t, out_c, "tkconv torch vs C")
        # the first factor is a per-pixel matrix product
        want_f1 = np.einsum("rc,bchw->brhw", first.reshape(4, 10).numpy().astype(np.float64), x.numpy().astype(np.float64))
        np.testing.assert_allclose(f1, want_f1, rtol=1e-5, atol=1e-5)
        assert f2.shape == (2, 6, 8 // stride, 8 // stride)


def test_orthonormal_first_factor_cannot_grow_pixel_norm():
    x, first, core, last = ref.make_block_case(256, 64, 64, 256, 56)
    xs = x[:, :, :8, :8]
    f1 = ref.conv2d_torch(xs, first)
    assert bool((f1.norm(dim=1) <= xs.norm(dim=1) * (1 + 1e-5)).all())


# ---- the reference kernel, run sequentially ---------------------------------------------------------
def test_reference_tiled_kernel_reproduces_direct_result_exactly():
    """Column 9 (`diff`) of every row of the reference's recorded sweeps is 0: each legal tiling gives
    exactly the direct result on integer inputs with all-ones weights.  Same statement, on the CPU."""
    picks = load("reference_tile_picks.json")
    rng = np.random.default_rng(9)
    for key in ("32_32_14_14", "64_32_7_7", "96_64_7_7", "32_32_7_7", "64_32_14_14"):
        C, N, H, W = (int(v) for v in key.split("_"))
        x = rng.integers(0, 10, size=(C, H, W)).astype(np.float32)
        w = np.ones((N, C, 3, 3), np.float32)
        direct = ref.conv2d_c(x[None], w, pad=1)[0]
        for th, tw, tc in picks[key]:
            assert np.array_equal(ref.tdc_tiled_c(x, w, th, tw, tc), direct), (key, th, tw, tc)


def test_reference_tiled_kernel_weight_order_and_ragged_tiles():
    """Asymmetric weights (which the reference's own check cannot see) and tiles that do not divide H, W."""
    rng = np.random.default_rng(10)
    x = rng.integers(-3, 4, size=(8, 7, 10)).astype(np.float32)
    w = rng.integers(-2, 3, size=(5, 8, 3, 3)).astype(np.float32)
    direct = ref.conv2d_c(x[None], w, pad=1)[0]
    for (th, tw, tc) in [(1, 1, 1), (2, 3, 4), (3, 4, 8), (7, 10, 2), (4, 7, 1), (12, 12, 8)]:
        assert np.array_equal(ref.tdc_tiled_c(x, w, th, tw, tc), direct), (th, tw, tc)
    with pytest.raises(ValueError):
        ref.tdc_tiled_c(x, w, 2, 2, 3)      # TC must divide C, as in the reference


# ---- the reference's analytic model (what the gfx950 model replaces) ----------------------------------
def test_reference_model_volumes_hand_computed():
    C, N, H, W, th, tw, tc = 32, 32, 56, 56, 1, 4, 32
    assert tdc_model_ref.compute_input_vol(C, N, H, W, th, tw, tc) == 56 * 3 * 58 * 32 == 311808
    assert tdc_model_ref.compute_out_vol(C, N, H, W, th, tw, tc) == 1 * 4 * 32 * 56 * 14 * 1 == 100352
    assert tdc_model_ref.compute_kernel_vol(C, N, H, W, th, tw, tc) == 9 * 32 * 32 * 784 == 7225344
    lat, bnum, bdim = tdc_model_ref.compute_latency(C, N, H, W, th, tw, tc, 3, 3, 68, 1024, 0.4375)
    assert (bnum, bdim) == (56, 448)
    # 68 SMs * 1024 threads * 0.4375 / 448 = 68 blocks per wave -> 1 wave
    assert lat == (1 + 2) * (4 + 2) * 32 * 9 * 1
    # launch shape of the shipped 2080Ti kernel for this layer: 56 blocks x 448 threads x 22272 bytes
    assert tdc_model_ref.launch_shape(C, N, H, W, th, tw, tc) == (56, 448, 22272)
    assert tdc_model_ref.launch_shape(192, 160, 7, 7, 2, 2, 16) == (48, 640, 16 * 4 * 10 * 4)
