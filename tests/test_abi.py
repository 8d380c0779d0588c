"""The C-ABI library loads, exports every symbol include/tdc.h declares, and its host-only entry
points (the tile model) work without a GPU.  No convolution is computed here."""
import ctypes
import os
import re

import pytest

import tdc_amd
from tdc_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "tdc.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tdc_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 18
    L = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(L, n), f"{n} is declared in include/tdc.h but not exported"
    assert set(names) == set(_lib.EXPORTS), "Python binding list and header disagree"


def test_version_and_error_string():
    L = tdc_amd.lib()
    assert b"gfx950" in L.tdc_version()
    assert L.tdc_model_select(None, None) == _lib.TDC_ERR_INVALID
    assert b"null" in L.tdc_last_error_string()


def test_struct_layouts_match_the_header():
    assert ctypes.sizeof(_lib.ConvDesc) == 12 * 4
    assert ctypes.sizeof(_lib.Tile) == 11 * 4
    assert ctypes.sizeof(_lib.TKConvDesc) == 13 * 4
    # tile (11 ints) + 10 ints + 4 bytes of padding + 5 doubles
    assert ctypes.sizeof(_lib.TileInfo) == 11 * 4 + 10 * 4 + 4 + 5 * 8
    assert _lib.TileInfo.flops.offset == 88


def test_invalid_descriptors_are_rejected_with_a_reason():
    bad = [
        tdc_amd.conv_desc(1, 0, 4, 8, 8, 3, 3, 1, 1),       # no input channels
        tdc_amd.conv_desc(1, 4, 4, 2, 2, 5, 5, 1, 0),       # filter larger than the input
        tdc_amd.conv_desc(1, 4, 4, 8, 8, 3, 3, 0, 1),       # stride 0
        tdc_amd.conv_desc(1, 4, 4, 8, 8, 3, 3, 1, -1),      # negative padding
    ]
    for d in bad:
        with pytest.raises(tdc_amd.TdcError) as e:
            tdc_amd.model_select(d)
        assert e.value.status == _lib.TDC_ERR_INVALID and len(str(e.value)) > 20


def test_shapes_beyond_the_addressing_limits_are_rejected_not_truncated():
    """One image is addressed with 32-bit byte offsets and 24-bit index products; anything larger must be
    refused with a reason instead of wrapping around."""
    too_big = [
        (tdc_amd.conv_desc(1, 2048, 8, 1024, 1024, 3, 3, 1, 1), "2^29"),    # 2^31 input elements per image
        (tdc_amd.conv_desc(1, 8, 2048, 1024, 1024, 3, 3, 1, 1), "2^29"),    # ... output elements per image
        (tdc_amd.conv_desc(1, 20000, 20000, 8, 8, 3, 3, 1, 1), "2^28"),     # 3.6e9 weights
        (tdc_amd.conv_desc(1, 4096, 4, 4096, 16, 3, 3, 1, 1), "too large"),  # (C+1)*H beyond 24 bits
    ]
    for d, reason in too_big:
        with pytest.raises(tdc_amd.TdcError) as e:
            tdc_amd.model_select(d)
        assert reason in str(e.value), str(e.value)
    # just inside the limits a tile is found
    assert tdc_amd.model_select(tdc_amd.conv_desc(1, 4000, 4, 4000, 16, 3, 3, 1, 1)).pred_us > 0


def test_plan_creation_without_a_gpu_fails_loudly():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    d = tdc_amd.conv_desc(1, 8, 8, 8, 8, 3, 3, 1, 1)
    h = ctypes.c_void_p()
    st = tdc_amd.lib().tdc_conv_plan_create(ctypes.byref(d), None, ctypes.byref(h))
    assert st == _lib.TDC_ERR_HIP and not h.value
    assert b"HIP device" in tdc_amd.lib().tdc_last_error_string()


def test_launch_floor_probe_rejects_bad_arguments():
    """tdc_launch_floor_time checks its arguments before it touches the device."""
    import ctypes
    L = tdc_amd.lib()
    ms = ctypes.c_float(-1.0)
    for launches, graph, grid, block, spin in ((0, 0, 256, 512, 0.0), (300, 0, 0, 512, 0.0), (300, 0, 70000, 512, 0.0),
                                                (300, 0, 256, 100, 0.0), (300, 0, 256, 2048, 0.0), (300, 1, 256, 512, -1.0),
                                                (300, 0, 256, 512, 1000.0), (300, 0, 256, 512, float("nan"))):
        st = L.tdc_launch_floor_time(launches, graph, grid, block, ctypes.c_float(spin), ctypes.byref(ms))
        assert st == tdc_amd._lib.TDC_ERR_INVALID, (launches, graph, grid, block, spin, st)
    assert L.tdc_launch_floor_time(300, 0, 256, 512, ctypes.c_float(0.0), None) == tdc_amd._lib.TDC_ERR_INVALID
    assert ms.value == -1.0


def test_python_operator_argument_errors_match_the_reference():
    """groups != 1 and non-zero padding modes are rejected like TKConv2dC.__init__ (inference/TKConv.py:39-42)."""
    hp = tdc_amd.ranks_dict(conv=[4, 3])
    with pytest.raises(ValueError, match="groups must be 1"):
        tdc_amd.TKConv2dC(8, 8, 3, groups=2, hp_dict=hp, name="conv")
    with pytest.raises(ValueError, match="padding_mode"):
        tdc_amd.TKConv2dC(8, 8, 3, padding_mode="reflect", hp_dict=hp, name="conv")
    m = tdc_amd.TKConv2dC(8, 10, 3, stride=2, padding=1, hp_dict=hp, name="conv")
    assert (m.in_rank, m.out_rank) == (3, 4)                      # ranks[name] = [out_rank, in_rank]
    assert tuple(m.first_kernel.shape) == (3, 8, 1, 1)
    assert tuple(m.core_kernel.shape) == (4, 3, 3, 3)
    assert tuple(m.last_kernel.shape) == (10, 4, 1, 1)
    assert tuple(m.bias.shape) == (10,)
    assert set(m.state_dict()) == {"first_kernel", "core_kernel", "last_kernel", "bias"}
    assert tdc_amd.TKConv2dC(8, 10, 3, bias=False, hp_dict=hp, name="conv").bias is None
