"""Shared helpers for the parity tests."""
import numpy as np
import torch

# Tolerance of the parity contract against the fp32 reference convolution.
RTOL = 1e-4
ATOL = 1e-5


def assert_close(got, ref, what=""):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    err = np.abs(got - ref)
    bound = ATOL + RTOL * np.abs(ref)
    bad = ~(err <= bound)  # NaN counts as a mismatch
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(f"{what}: {bad.sum()} of {bad.size} outside tolerance; worst at {i}: "
                             f"got {got[i]!r} ref {ref[i]!r} err {err[i]:.3e}")


def seeded(seed):
    return torch.Generator().manual_seed(seed)
