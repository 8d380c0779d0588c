"""ctypes binding of libtdc_amd.so (the C ABI declared in include/tdc.h).

The library is built in-tree by ``ppopp23-tdc_amd/build.py``; nothing here falls
back to another implementation when it is missing.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, byref, c_char_p, c_double, c_int, c_int32, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
# (TDC_AMD_LIBRARY in the environment points at another build of the same library, e.g. the profiling build with time stamps)
LIB_PATH = os.environ.get("TDC_AMD_LIBRARY") or os.path.join(_HERE, "libtdc_amd.so")

TDC_OK, TDC_ERR_INVALID, TDC_ERR_UNSUPPORTED, TDC_ERR_HIP, TDC_ERR_NOMEM, TDC_ERR_STATE = range(6)

# Every symbol include/tdc.h declares.
EXPORTS = (
    "tdc_last_error_string", "tdc_version", "tdc_load_bin", "tdc_save_bin",
    "tdc_conv_plan_create", "tdc_conv_plan_create_with_tail", "tdc_conv_plan_set_tail_weights",
    "tdc_conv_plan_set_weights", "tdc_conv_plan_set_input_affine", "tdc_conv_plan_set_head", "tdc_conv_plan_query",
    "tdc_conv_forward", "tdc_conv_forward_static_ws", "tdc_conv_plan_occupancy",
    "tdc_conv_forward_strided", "tdc_tkconv_forward_strided",
    "tdc_conv_time", "tdc_conv_time_many", "tdc_launch_floor_time", "tdc_conv_plan_destroy",
    "tdc_tkconv_create", "tdc_tkconv_set_weights", "tdc_tkconv_forward", "tdc_tkconv_forward_features",
    "tdc_tkconv_core_forward", "tdc_tkconv_query", "tdc_tkconv_num_kernels", "tdc_tkconv_destroy",
    "tdc_model_evaluate", "tdc_model_kernel_info", "tdc_model_enumerate", "tdc_model_select", "tdc_model_select_with_tail", "tdc_model_get_constants",
    "tdc_model_set_constants", "tdc_set_autotune", "tdc_get_autotune",
    "tdc_net_create", "tdc_net_tensor", "tdc_net_view", "tdc_net_affine", "tdc_net_affine_conv", "tdc_net_conv", "tdc_net_conv_tail", "tdc_net_set_input_affine", "tdc_net_tkconv", "tdc_net_pool", "tdc_net_global_avgpool", "tdc_net_concat",
    "tdc_net_tensor_shape", "tdc_net_num_kernels", "tdc_net_finalize", "tdc_net_forward", "tdc_net_time",
    "tdc_net_read_tensor", "tdc_net_destroy",
)


class TdcError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"tdc status {status}: {message}")
        self.status = status


class ConvDesc(Structure):
    _fields_ = [(n, c_int32) for n in ("batch", "C", "N", "H", "W", "KH", "KW", "stride", "pad", "dilation",
                                       "has_bias", "relu")]


class Tile(Structure):
    _fields_ = [(n, c_int32) for n in ("mf", "mb", "nb", "wm", "wn", "wk", "cch", "tw", "ks", "wl", "alg")]

    def __init__(self, mf=0, mb=0, nb=0, wm=0, wn=0, wk=0, cch=0, tw=0, ks=1, wl=0, alg=0):
        super().__init__(mf, mb, nb, wm, wn, wk, cch, tw, ks, wl, alg)

    def astuple(self):
        return (self.mf, self.mb, self.nb, self.wm, self.wn, self.wk, self.cch, self.tw, self.ks, self.wl, self.alg)

    def __repr__(self):
        return "Tile(mf=%d, mb=%d, nb=%d, wm=%d, wn=%d, wk=%d, cch=%d, tw=%d, ks=%d, wl=%d, alg=%d)" % self.astuple()


class TileInfo(Structure):
    _fields_ = [("tile", Tile)] + [(n, c_int32) for n in (
        "grid_x", "grid_y", "grid_z", "block_threads", "lds_bytes", "vgpr_estimate", "waves_per_simd",
        "wg_per_cu", "nchunks", "th")] + [(n, c_double) for n in ("flops", "bytes", "roof_us", "pred_us",
                                                                 "pred_l2_bytes")]

    def asdict(self):
        d = {n: getattr(self, n) for n, _ in self._fields_ if n != "tile"}
        d["tile"] = self.tile.astuple()
        return d


class KernelOccupancy(Structure):
    _fields_ = [(n, c_int32) for n in ("kernel_vgprs", "kernel_static_lds_bytes", "kernel_max_threads", "runtime_wg_per_cu",
                                       "block_threads", "dynamic_lds_bytes", "model_vgprs", "model_wg_per_cu")]

    def asdict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


class TKConvDesc(Structure):
    _fields_ = [(n, c_int32) for n in ("batch", "C", "R1", "R2", "N", "H", "W", "K", "stride", "pad", "dilation",
                                       "has_bias", "relu")]


_lib = None


def lib():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python ppopp23-tdc_amd/build.py` "
            "(hipcc, gfx950). There is no fallback implementation.")
    L = ctypes.CDLL(LIB_PATH)
    fp = POINTER(ctypes.c_float)
    L.tdc_last_error_string.restype = c_char_p
    L.tdc_version.restype = c_char_p
    L.tdc_load_bin.argtypes = [c_char_p, c_void_p, ctypes.c_uint64]
    L.tdc_save_bin.argtypes = [c_char_p, c_void_p, ctypes.c_uint64]
    L.tdc_conv_plan_create.argtypes = [POINTER(ConvDesc), POINTER(Tile), POINTER(c_void_p)]
    L.tdc_conv_plan_set_weights.argtypes = [c_void_p, c_void_p, c_void_p]
    L.tdc_conv_plan_query.argtypes = [c_void_p, POINTER(TileInfo)]
    L.tdc_conv_forward.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    L.tdc_conv_forward_static_ws.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    L.tdc_conv_plan_occupancy.argtypes = [c_void_p, POINTER(KernelOccupancy)]
    L.tdc_conv_time.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, POINTER(ctypes.c_float)]
    L.tdc_launch_floor_time.argtypes = [c_int32, c_int32, c_int32, c_int32, ctypes.c_float, POINTER(ctypes.c_float)]
    L.tdc_conv_time_many.argtypes = [POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p), c_int32, c_int32, c_int32,
                                     POINTER(ctypes.c_float)]
    L.tdc_conv_plan_destroy.argtypes = [c_void_p]
    L.tdc_conv_plan_destroy.restype = None
    L.tdc_tkconv_create.argtypes = [POINTER(TKConvDesc), POINTER(c_void_p)]
    L.tdc_tkconv_set_weights.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    L.tdc_tkconv_forward.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    L.tdc_tkconv_forward_features.argtypes = [c_void_p] * 6
    L.tdc_tkconv_core_forward.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p]
    L.tdc_tkconv_query.argtypes = [c_void_p, c_int, POINTER(TileInfo)]
    L.tdc_tkconv_destroy.argtypes = [c_void_p]
    L.tdc_tkconv_destroy.restype = None
    L.tdc_model_evaluate.argtypes = [POINTER(ConvDesc), POINTER(Tile), POINTER(TileInfo)]
    L.tdc_model_enumerate.argtypes = [POINTER(ConvDesc), POINTER(Tile), c_int32, POINTER(c_int32)]
    L.tdc_model_select.argtypes = [POINTER(ConvDesc), POINTER(TileInfo)]
    L.tdc_model_kernel_info.argtypes = [POINTER(ConvDesc), POINTER(Tile), c_int32, c_char_p, c_int32, POINTER(c_int32),
                                        POINTER(c_int32)]
    L.tdc_model_get_constants.argtypes = [POINTER(c_double), c_int32, POINTER(c_int32)]
    L.tdc_model_set_constants.argtypes = [POINTER(c_double), c_int32]
    i32, i32p, fpv = c_int32, POINTER(c_int32), c_void_p
    L.tdc_net_create.argtypes = [i32, i32, i32, i32, POINTER(c_void_p)]
    i64 = ctypes.c_int64
    L.tdc_conv_forward_strided.argtypes = [c_void_p, c_void_p, i64, c_void_p, i64, c_void_p, i64, c_void_p]
    L.tdc_tkconv_forward_strided.argtypes = [c_void_p, c_void_p, i64, c_void_p, i64, c_void_p, i64, c_void_p]
    L.tdc_net_tensor.argtypes = [c_void_p, i32, i32, i32, i32p]
    L.tdc_net_view.argtypes = [c_void_p, i32, i32, i32, i32p]
    L.tdc_net_affine.argtypes = [c_void_p, i32, fpv, fpv, i32, i32, i32p]
    L.tdc_net_conv.argtypes = [c_void_p, i32, i32, i32, i32, i32, i32, fpv, fpv, i32, i32, i32, i32p]
    L.tdc_net_tkconv.argtypes = [c_void_p, i32, i32, i32, i32, i32, i32, i32, fpv, fpv, fpv, fpv, i32, i32, i32, i32p]
    L.tdc_net_pool.argtypes = [c_void_p, i32, i32, i32, i32, i32, i32, i32p]
    L.tdc_net_global_avgpool.argtypes = [c_void_p, i32, i32p]
    L.tdc_net_concat.argtypes = [c_void_p, i32p, i32, i32p]
    L.tdc_net_tensor_shape.argtypes = [c_void_p, i32, i32p, i32p, i32p]
    L.tdc_net_num_kernels.argtypes = [c_void_p]
    L.tdc_net_finalize.argtypes = [c_void_p, i32]
    L.tdc_net_forward.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p]
    L.tdc_net_time.argtypes = [c_void_p, i32, i32, POINTER(ctypes.c_float)]
    L.tdc_net_read_tensor.argtypes = [c_void_p, i32, c_void_p]
    L.tdc_net_destroy.argtypes = [c_void_p]
    L.tdc_net_destroy.restype = None
    L.tdc_set_autotune.argtypes = [i32]
    L.tdc_get_autotune.argtypes = []
    for name in EXPORTS:
        fn = getattr(L, name)
        if fn.restype is c_int:  # default restype: status code
            fn.restype = c_int
    _lib = L
    return L


def check(status):
    if status != TDC_OK:
        raise TdcError(status, lib().tdc_last_error_string().decode())


def conv_desc(batch, C, N, H, W, KH, KW, stride=1, pad=0, dilation=1, has_bias=False, relu=False):
    return ConvDesc(batch, C, N, H, W, KH, KW, stride, pad, dilation, int(has_bias), int(relu))


# ---- analytic model (host only) ---------------------------------------------
def model_select(desc: ConvDesc) -> TileInfo:
    info = TileInfo()
    check(lib().tdc_model_select(byref(desc), byref(info)))
    return info


def model_evaluate(desc: ConvDesc, tile: Tile) -> TileInfo:
    info = TileInfo()
    check(lib().tdc_model_evaluate(byref(desc), byref(tile), byref(info)))
    return info


def model_kernel_info(desc: ConvDesc, tile: Tile, extras: bool = False):
    """(name of the compiled kernel that serves `tile`, registers per lane the model assumes for it, waves of it per
    SIMD by the model's register arithmetic)."""
    buf = ctypes.create_string_buffer(128)
    regs, waves = c_int32(0), c_int32(0)
    check(lib().tdc_model_kernel_info(byref(desc), byref(tile), int(extras), buf, 128, byref(regs), byref(waves)))
    return buf.value.decode(), regs.value, waves.value


def kernel_resources():
    """The compiler's resource report of the built kernels: {name: dict(vgprs, agprs, sgprs, scratch, waves_per_simd,
    static_lds)} from kernel_resources.txt, which the build writes next to the library."""
    path = os.path.join(_HERE, "kernel_resources.txt")
    out = {}
    for line in open(path):
        if line.startswith("#") or not line.strip():
            continue
        f = [x.strip() for x in line.split("|")]
        out[f[0]] = dict(zip(("vgprs", "agprs", "sgprs", "scratch", "waves_per_simd", "static_lds"), map(int, f[1:])))
    return out


MODEL_CONSTANT_NAMES = ("launch_us", "setup_clk", "copy_latency_clk", "copy_bytes_per_clk", "l2_bytes_per_clk",
                        "lds_bytes_per_clk", "sync_clk", "store_bytes_per_clk", "kstep_issue_clk", "pass_overhead_clk",
                        "wave_setup_clk", "ksplit_clk", "copy_issue_clk", "lds_read_clk", "wino_kstep_clk", "gw_latency_clk",
                        "stream_setup_clk", "stream_latency_clk")


def model_select_with_tail(desc: ConvDesc, tail_N: int):
    """The model's pick for `desc` with a 1x1 convolution of tail_N outputs fused behind it, or None if no tile can
    hold all output channels in one workgroup."""
    info = TileInfo()
    if lib().tdc_model_select_with_tail(byref(desc), int(tail_N), byref(info)) != TDC_OK:
        return None
    return info


def fused_tail_pays(desc: ConvDesc, tail_N: int, margin: float = 0.9):
    """True if the model predicts conv + fused 1x1 tail faster than the two convolutions launched separately
    (by at least 10 %: measured, the model is that much too kind to the fused kernel at batch 1)."""
    fused = model_select_with_tail(desc, tail_N)
    if fused is None:
        return False
    Ho = (desc.H + 2 * desc.pad - desc.dilation * (desc.KH - 1) - 1) // desc.stride + 1
    Wo = (desc.W + 2 * desc.pad - desc.dilation * (desc.KW - 1) - 1) // desc.stride + 1
    tail = conv_desc(desc.batch, desc.N, tail_N, Ho, Wo, 1, 1, 1, 0)
    return fused.pred_us < margin * (model_select(desc).pred_us + model_select(tail).pred_us)


def model_get_constants():
    n = c_int32(0)
    buf = (c_double * 64)()
    check(lib().tdc_model_get_constants(buf, 64, byref(n)))
    return [buf[i] for i in range(n.value)]


def model_set_constants(values):
    arr = (c_double * len(values))(*values)
    check(lib().tdc_model_set_constants(arr, len(values)))


def get_autotune() -> int:
    """The current setting of the measured tile selection (0 = off)."""
    return int(lib().tdc_get_autotune())


def set_autotune(classes: int):
    """Measured tile selection for every plan created from now on without a forced tile: time the model's
    favourite of each of the `classes` most promising tile classes on the device and keep the fastest
    (0 = the model's pick alone, the default).  Returns the previous setting."""
    prev = lib().tdc_get_autotune()
    check(lib().tdc_set_autotune(int(classes)))
    return prev


def model_enumerate(desc: ConvDesc, cap: int = 1 << 17):
    arr = (Tile * cap)()
    n = c_int32(0)
    check(lib().tdc_model_enumerate(byref(desc), arr, cap, byref(n)))
    return [Tile(*arr[i].astuple()) for i in range(n.value)]
