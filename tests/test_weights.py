"""Weight files: raw little-endian float32 (the reference's load_input format) and the state-dict directory."""
import os
import struct

import numpy as np
import pytest
import torch

import tdc_amd
from tdc_amd import weights


def test_bin_is_raw_little_endian_float32(tmp_path):
    t = torch.tensor([[1.0, -2.5], [3.25, 1e-3]])
    path = os.path.join(tmp_path, "w.bin")
    weights.save_bin(path, t)
    raw = open(path, "rb").read()
    assert raw == struct.pack("<4f", 1.0, -2.5, 3.25, 1e-3)                 # no header, row-major, LE
    assert torch.equal(weights.load_bin(path, (2, 2)), t)
    np.testing.assert_array_equal(np.fromfile(path, dtype="<f4"), t.numpy().ravel())


def test_wrong_length_and_missing_file_are_errors(tmp_path):
    path = os.path.join(tmp_path, "w.bin")
    weights.save_bin(path, torch.arange(6, dtype=torch.float32))
    for shape in ((5,), (7,)):
        with pytest.raises(tdc_amd.TdcError, match="exactly"):
            weights.load_bin(path, shape)
    with pytest.raises(tdc_amd.TdcError, match="cannot open"):
        weights.load_bin(os.path.join(tmp_path, "nope.bin"), (1,))


def test_state_dict_round_trip_with_reference_keys(tmp_path):
    from tdc_amd import nets
    p = nets.resnet18_params(seed=3, num_classes=7)
    p["bn1.num_batches_tracked"] = torch.tensor(5)        # integer entries are skipped like non-parameters
    n = weights.export_state_dict(p, tmp_path)
    q = weights.import_state_dict(tmp_path)
    assert n == len(q) == len(p) - 1
    assert "layer2.0.conv1.first_kernel" in q and "layer4.1.conv2.core_kernel" in q and "fc.bias" in q
    for k, v in q.items():
        assert torch.equal(v, p[k]) and v.shape == p[k].shape
