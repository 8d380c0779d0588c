"""Writes the committed golden fixtures (run from the repo root: python tests/golden/make_golden.py).

* ``small_cases.json`` — tiny convolutions with asymmetric integer weights whose outputs are exact
  integers, computed by explicit loops in Python integers (no floating point, no library) and
  cross-checked against torch.nn.functional.conv2d before being written.
* ``seeded_inputs.json`` — SHA-256 of the seeded synthetic inputs of the benchmark configurations
  plus 16 sampled outputs of the fp32 CPU convolution, so that a drift of the input generator (or a
  different torch build) is detected on the GPU box without shipping megabytes.
* ``reference_tile_picks.json`` — the (TH, TW, TC) the reference ships per layer on its two GPUs
  (the ``#define TH/TW/TC`` lines of its generated kernels), data only.
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import ref  # noqa: E402


def int_conv(x, w, stride, pad, dil):
    """Pure Python integer loops: x [C][H][W], w [N][C][KH][KW] nested lists."""
    C, H, W = len(x), len(x[0]), len(x[0][0])
    N, KH, KW = len(w), len(w[0][0]), len(w[0][0][0])
    Ho = (H + 2 * pad - dil * (KH - 1) - 1) // stride + 1
    Wo = (W + 2 * pad - dil * (KW - 1) - 1) // stride + 1
    out = [[[0] * Wo for _ in range(Ho)] for _ in range(N)]
    for n in range(N):
        for oy in range(Ho):
            for ox in range(Wo):
                acc = 0
                for c in range(C):
                    for r in range(KH):
                        iy = oy * stride - pad + r * dil
                        if not 0 <= iy < H:
                            continue
                        for s in range(KW):
                            ix = ox * stride - pad + s * dil
                            if 0 <= ix < W:
                                acc += w[n][c][r][s] * x[c][iy][ix]
                out[n][oy][ox] = acc
    return out


def small_cases():
    rng = np.random.default_rng(20231)
    cases = []
    for (C, N, H, W, K, stride, pad, dil) in [(2, 2, 4, 4, 3, 1, 1, 1), (3, 2, 5, 5, 3, 1, 1, 1), (1, 1, 3, 3, 3, 1, 1, 1),
                                              (2, 3, 5, 4, 3, 2, 1, 1), (3, 4, 6, 5, 1, 1, 0, 1), (2, 2, 7, 7, 3, 1, 2, 2),
                                              (4, 1, 2, 9, 3, 1, 1, 1), (1, 5, 6, 6, 5, 1, 2, 1), (5, 3, 4, 6, 1, 2, 0, 1)]:
        x = rng.integers(-4, 10, size=(C, H, W))
        w = rng.integers(-3, 4, size=(N, C, K, K))
        out = int_conv(x.tolist(), w.tolist(), stride, pad, dil)
        chk = F.conv2d(torch.tensor(x, dtype=torch.float32)[None], torch.tensor(w, dtype=torch.float32), None, stride, pad,
                       dil)[0]
        assert torch.equal(chk, torch.tensor(out, dtype=torch.float32)), "loop result disagrees with F.conv2d"
        cases.append({"C": C, "N": N, "H": H, "W": W, "K": K, "stride": stride, "pad": pad, "dil": dil,
                      "x": x.tolist(), "w": w.tolist(), "out": out})
    return cases


def digest(t):
    return hashlib.sha256(t.contiguous().numpy().tobytes()).hexdigest()


def seeded_inputs():
    recs = []
    for (hw, r1, r2, seed) in [(56, 32, 32, 0), (7, 16, 16, None), (14, 64, 64, None), (28, 96, 96, None), (56, 128, 128, None),
                               (56, 64, 128, None)]:
        x, w = ref.make_core_case(hw, r1, r2, seed=seed)
        y = F.conv2d(x, w, None, 1, 1)
        idx = np.linspace(0, y.numel() - 1, 16).astype(np.int64)
        recs.append({"hw": hw, "r1": r1, "r2": r2, "seed": seed, "x_sha256": digest(x), "w_sha256": digest(w),
                     "sample_index": idx.tolist(), "sample_out": [float(v) for v in y.flatten()[idx]]})
    blocks = []
    for (C, R1, R2, N, hw) in ref.BLOCKS:
        x, first, core, last = ref.make_block_case(C, R1, R2, N, hw)
        blocks.append({"C": C, "R1": R1, "R2": R2, "N": N, "hw": hw, "x_sha256": digest(x), "first_sha256": digest(first),
                       "core_sha256": digest(core), "last_sha256": digest(last)})
    return {"torch": torch.__version__, "core": recs, "blocks": blocks}


# shape "C_N_H_W" -> [2080Ti oracle, 2080Ti model, A100 oracle, A100 model], each (TH, TW, TC)
REFERENCE_TILE_PICKS = {
    "64_32_224_224": [[2, 12, 16], [1, 7, 16], [1, 7, 32], [1, 7, 8]],
    "64_32_112_112": [[2, 6, 32], [2, 4, 16], [3, 5, 32], [1, 4, 16]],
    "32_32_56_56": [[1, 4, 32], [2, 2, 16], [2, 6, 16], [1, 2, 16]],
    "64_32_56_56": [[2, 4, 32], [2, 2, 16], [1, 8, 16], [1, 2, 16]],
    "64_64_56_56": [[2, 6, 32], [2, 4, 16], [1, 8, 16], [1, 4, 16]],
    "32_32_28_28": [[1, 3, 16], [2, 1, 16], [1, 2, 8], [1, 1, 16]],
    "64_32_28_28": [[1, 5, 16], [2, 1, 16], [1, 2, 16], [1, 1, 16]],
    "96_64_28_28": [[3, 2, 16], [2, 2, 16], [2, 4, 16], [1, 2, 16]],
    "160_96_28_28": [[5, 4, 16], [2, 4, 16], [2, 6, 32], [1, 4, 16]],
    "192_96_28_28": [[3, 4, 32], [2, 4, 16], [1, 4, 32], [1, 4, 16]],
    "32_32_14_14": [[2, 3, 4], [2, 1, 16], [1, 1, 8], [1, 1, 16]],
    "64_32_14_14": [[1, 2, 16], [2, 1, 16], [1, 1, 16], [1, 1, 16]],
    "128_96_14_14": [[1, 4, 16], [2, 2, 16], [1, 2, 32], [1, 2, 16]],
    "192_96_14_14": [[3, 4, 16], [2, 2, 16], [1, 6, 16], [1, 2, 16]],
    "32_32_7_7": [[1, 1, 8], [1, 1, 16], [1, 2, 4], [1, 1, 16]],
    "64_32_7_7": [[4, 1, 4], [1, 1, 16], [2, 1, 4], [1, 1, 16]],
    "96_64_7_7": [[2, 1, 8], [1, 1, 16], [4, 1, 8], [1, 1, 16]],
    "192_160_7_7": [[2, 2, 16], [1, 2, 16], [2, 2, 16], [1, 2, 16]],
}


if __name__ == "__main__":
    with open(os.path.join(HERE, "small_cases.json"), "w") as f:
        json.dump(small_cases(), f)
    with open(os.path.join(HERE, "seeded_inputs.json"), "w") as f:
        json.dump(seeded_inputs(), f, indent=1)
    with open(os.path.join(HERE, "reference_tile_picks.json"), "w") as f:
        json.dump(REFERENCE_TILE_PICKS, f, indent=1)
    print("golden fixtures written")
