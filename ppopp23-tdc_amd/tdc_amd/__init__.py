"""MI355X-native Tucker convolution (TDC hot path) — Python host layer over libtdc_amd.so."""
from ._lib import (LIB_PATH, ConvDesc, TdcError, Tile, TileInfo, conv_desc, lib, model_enumerate, model_evaluate,
                   model_select, set_autotune)

__all__ = ["LIB_PATH", "ConvDesc", "TdcError", "Tile", "TileInfo", "conv_desc", "lib", "model_enumerate",
           "model_evaluate", "model_select", "set_autotune", "Conv2dPlan", "TKConvOp", "TKConv2dC", "ranks_dict", "partial_tucker2"]


def __getattr__(name):
    # torch-dependent classes are imported lazily so the model API works without torch.
    if name in ("Conv2dPlan", "TKConvOp"):
        from . import conv
        return getattr(conv, name)
    if name in ("TKConv2dC", "ranks_dict", "partial_tucker2"):
        from . import TKConv
        return getattr(TKConv, name)
    raise AttributeError(name)
