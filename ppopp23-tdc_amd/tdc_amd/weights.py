"""Weight I/O for the Tucker networks.

* ``save_bin`` / ``load_bin`` — one tensor per file, raw little-endian float32 without a header, the format
  the reference's native layer library reads (``load_input``,
  2080Ti-evaluation/EndToEnd/resnet18-tk/src/common.cpp:2-19).
* ``export_state_dict`` / ``import_state_dict`` — a whole parameter dictionary as a directory of such files
  plus ``manifest.json`` (key, shape, file).  Keys are the reference's state-dict keys
  (``layer1.0.conv1.first_kernel`` ..., inference/TKConv.py:64-66), so a checkpoint of the reference's
  Tucker models can be exported once with ``export_state_dict(torch.load(path, weights_only=True), dir)``
  and then loaded without torch pickles.
"""
from __future__ import annotations

import json
import os
from ctypes import c_void_p

import torch

from ._lib import check, lib


def save_bin(path, tensor):
    t = tensor.detach().to(device="cpu", dtype=torch.float32).contiguous()
    check(lib().tdc_save_bin(os.fsencode(path), c_void_p(t.data_ptr()), t.numel()))


def load_bin(path, shape):
    t = torch.empty(tuple(shape), dtype=torch.float32)
    check(lib().tdc_load_bin(os.fsencode(path), c_void_p(t.data_ptr()), t.numel()))
    return t


def export_state_dict(state, directory):
    os.makedirs(directory, exist_ok=True)
    manifest = []
    for i, (key, value) in enumerate(state.items()):
        if not torch.is_tensor(value) or not value.dtype.is_floating_point:
            continue                                     # e.g. BatchNorm's num_batches_tracked
        fname = "%04d.bin" % i
        save_bin(os.path.join(directory, fname), value)
        manifest.append({"key": key, "shape": list(value.shape), "file": fname})
    with open(os.path.join(directory, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1)
    return len(manifest)


def import_state_dict(directory):
    with open(os.path.join(directory, "manifest.json")) as f:
        manifest = json.load(f)
    return {m["key"]: load_bin(os.path.join(directory, m["file"]), m["shape"]) for m in manifest}
