"""ctypes binding of libmie_hip.so (the C ABI declared in include/mie.h).

The library is the only compute path of this package: there is no eager /
CPU fallback.  If the shared object is missing, `lib()` raises.
"""
import ctypes
import os

# torch must be imported before the library is loaded: the PyTorch-ROCm wheel ships its own
# HIP runtime (soname libamdhip64.so.7); once it is mapped, the loader binds libmie_hip.so to
# that same runtime, so both share one device context and one set of streams.  In the other
# order the process ends up with two HIP runtimes and the second one finds no device.
import torch  # noqa: F401  (import order matters, see above)

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# MIE_HIP_LIB points at another build of the same library (kernel experiments)
LIB_PATH = os.environ.get("MIE_HIP_LIB") or os.path.join(_PKG_DIR, "lib", "libmie_hip.so")

MIE_OK = 0
MIE_TILE = 8
NOALLOC_WS_BYTES = 8 * 1024 * 1024

ACT_NONE, ACT_RELU, ACT_LEAKY_RELU, ACT_SIGMOID, ACT_TANH = 0, 1, 2, 3, 4
FOOT_CONV, FOOT_UP2X, FOOT_TCONV = 0, 1, 2
EVENTS_VOXEL, EVENTS_HISTOGRAM = 0, 1
DTYPE_F32, DTYPE_BF16, DTYPE_F32_BF16X3 = 0, 1, 2
PATH_AUTO, PATH_VALU, PATH_MFMA = 0, 1, 2
FLAG_KEEP_RESERVOIR = 1
CNT_ACTIVE, CNT_STALE, CNT_TICKET, CNT_WORDS = 0, 1, 2, 4

# every symbol include/mie.h declares
EXPORTS = (
    "mie_version", "mie_last_error_string", "mie_tile_capacity", "mie_mask_from_delta", "mie_build_mask_tiles_thresholded",
    "mie_build_mask_tiles", "mie_conv_masked", "mie_act_incr", "mie_mul_incr", "mie_add_incr",
    "mie_upsample2x_incr", "mie_convlstm_gates_incr", "mie_tconv_masked", "mie_conv_refresh",
    "mie_pack_filter", "mie_kfence_incr", "mie_events_to_frame", "mie_events_to_frame_bf16", "mie_tconv_refresh", "mie_conv_gates_masked", "mie_conv_gates_masked_ws",
    "mie_maxpool_incr", "mie_accumulate", "mie_scale_incr", "mie_avgpool_incr", "mie_linear_incr", "mie_upconv_masked", "mie_upconv_masked_ws", "mie_upconv_pred_masked",
    "mie_conv_masked_ws", "mie_convgru_gates_incr", "mie_upsample2x_pair_incr", "mie_conv_masked_noalloc",
    "mie_convlstm_gates_refresh", "mie_convgru_gates_refresh", "mie_mul_dense", "mie_tconv2x_masked",
    "mie_tconv2x_refresh", "mie_conv_f32x3_takes", "mie_build_mask_plan", "mie_build_mask_plan_wgs",
)
PLAN_MAX_STEPS = 40


class MieTileSet(ctypes.Structure):
    """struct mie_tileset of include/mie.h."""
    _fields_ = [
        ("n", ctypes.c_int32), ("h", ctypes.c_int32), ("w", ctypes.c_int32),
        ("pixmask", ctypes.c_void_p), ("tiles", ctypes.c_void_p), ("stale", ctypes.c_void_p),
        ("counts", ctypes.c_void_p), ("flags", ctypes.c_void_p),
    ]


class MiePlanOp(ctypes.Structure):
    """struct mie_plan_op of include/mie.h: the arguments of one mie_build_mask_tiles call."""
    _fields_ = [
        ("in_mask", ctypes.c_void_p), ("in_mask2", ctypes.c_void_p),
        ("h_in", ctypes.c_int32), ("w_in", ctypes.c_int32),
        ("foot", ctypes.c_int32), ("k", ctypes.c_int32), ("stride", ctypes.c_int32), ("pad", ctypes.c_int32),
        ("out", MieTileSet),
    ]


class MieError(RuntimeError):
    """A libmie_hip.so entry point returned a negative status."""

    def __init__(self, code, message):
        super().__init__("libmie_hip status %d: %s" % (code, message))
        self.code = code


_lib = None


def _declare(l):
    vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    tsp = ctypes.POINTER(MieTileSet)
    l.mie_version.restype = ci
    l.mie_version.argtypes = []
    l.mie_last_error_string.restype = ctypes.c_char_p
    l.mie_last_error_string.argtypes = []
    l.mie_tile_capacity.restype = ci
    l.mie_tile_capacity.argtypes = [ci, ci, ci]
    l.mie_mask_from_delta.restype = ci
    l.mie_mask_from_delta.argtypes = [vp, ci, ci, ci, ci, cf, vp, ci, vp]
    l.mie_build_mask_tiles_thresholded.restype = ci
    l.mie_build_mask_tiles_thresholded.argtypes = [vp, ci, ci, cf, vp, vp, ci, ci, ci, ci, ci, tsp, vp]
    l.mie_build_mask_tiles.restype = ci
    l.mie_build_mask_tiles.argtypes = [vp, vp, ci, ci, ci, ci, ci, ci, tsp, vp]
    l.mie_build_mask_plan.restype = ci
    l.mie_build_mask_plan.argtypes = [ctypes.POINTER(MiePlanOp), ci, vp]
    l.mie_build_mask_plan_wgs.restype = ci
    l.mie_build_mask_plan_wgs.argtypes = [ctypes.POINTER(MiePlanOp), ci, ci, vp]
    l.mie_conv_masked.restype = ci
    l.mie_conv_masked.argtypes = [vp, vp, ci, vp, vp, ci, ci, ci, vp, vp, ci, ci, ci, ci, ci, tsp, vp,
                                  vp, vp, ci, cf, ci, ci, vp]
    l.mie_convlstm_gates_refresh.restype = ci
    l.mie_convlstm_gates_refresh.argtypes = [vp, ci, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    l.mie_convgru_gates_refresh.restype = ci
    l.mie_convgru_gates_refresh.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
    l.mie_mul_dense.restype = ci
    l.mie_mul_dense.argtypes = [vp, vp, vp, ctypes.c_longlong, ci, vp]
    l.mie_tconv2x_masked.restype = ci
    l.mie_tconv2x_masked.argtypes = [vp, vp, ci, vp, vp, ci, ci, ci, vp, vp, ci, ci, ci, tsp, tsp, vp, vp, vp, ci, cf, ci,
                                     vp, ctypes.c_longlong, vp]
    l.mie_tconv2x_refresh.restype = ci
    l.mie_tconv2x_refresh.argtypes = [vp, ci, vp, ci, ci, ci, vp, vp, ci, ci, ci, vp, tsp, tsp, vp, vp, vp, ci, cf, ci, vp]
    l.mie_conv_masked_noalloc.restype = ci
    l.mie_conv_masked_noalloc.argtypes = list(l.mie_conv_masked.argtypes)
    l.mie_conv_masked_ws.restype = ci
    l.mie_conv_masked_ws.argtypes = [vp, vp, ci, vp, vp, ci, ci, ci, vp, vp, ci, ci, ci, ci, ci, tsp, vp,
                                     vp, vp, ci, cf, ci, ci, vp, ctypes.c_longlong, vp]
    l.mie_upsample2x_pair_incr.restype = ci
    l.mie_upsample2x_pair_incr.argtypes = [vp, vp, tsp, vp, vp, vp, tsp, vp, ci, ci, ci, ci, vp]
    l.mie_convgru_gates_incr.restype = ci
    l.mie_convgru_gates_incr.argtypes = [vp, vp, vp, vp, ci, tsp, ci, vp]
    l.mie_kfence_incr.restype = ci
    l.mie_kfence_incr.argtypes = [vp, vp, vp, cf, vp, ci, tsp, vp, ci, vp]
    l.mie_events_to_frame.restype = ci
    cd = ctypes.c_double
    l.mie_events_to_frame.argtypes = [vp, ci, ci, ci, ci, ci, ci, ci, ci, ci, cd, cd, cd, cd, ci, vp, vp, vp]
    l.mie_events_to_frame_bf16.restype = ci
    l.mie_events_to_frame_bf16.argtypes = [vp, ci, ci, ci, ci, ci, ci, ci, ci, ci, cd, cd, cd, cd, ci, vp, vp, vp, vp]
    l.mie_conv_f32x3_takes.restype = ci
    l.mie_conv_f32x3_takes.argtypes = [ci, ci, ci, ci, ci]
    l.mie_pack_filter.restype = ci
    l.mie_pack_filter.argtypes = [vp, ci, ci, ci, vp, ci, vp]
    l.mie_conv_refresh.restype = ci
    l.mie_conv_refresh.argtypes = [vp, ci, vp, ci, ci, ci, vp, vp, ci, ci, ci, ci, ci, vp, tsp, vp, vp,
                                   vp, ci, cf, ci, ci, vp]
    l.mie_act_incr.restype = ci
    l.mie_act_incr.argtypes = [ci, cf, vp, vp, vp, ci, tsp, vp, ci, ci, vp]
    l.mie_mul_incr.restype = ci
    l.mie_mul_incr.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, tsp, ci, ci, vp]
    l.mie_add_incr.restype = ci
    l.mie_add_incr.argtypes = [vp, vp, vp, vp, vp, ci, tsp, ci, vp]
    l.mie_upsample2x_incr.restype = ci
    l.mie_upsample2x_incr.argtypes = [vp, vp, vp, vp, ci, ci, ci, tsp, vp, ci, vp]
    l.mie_convlstm_gates_incr.restype = ci
    l.mie_convlstm_gates_incr.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, ci, tsp, ci, vp]
    l.mie_conv_gates_masked.restype = ci
    l.mie_conv_gates_masked.argtypes = [vp, vp, ci, vp, vp, ci, ci, ci, vp, vp, ci, ci, tsp, vp, vp, vp, vp, vp,
                                        vp, vp, ci, vp]
    l.mie_conv_gates_masked_ws.restype = ci
    l.mie_conv_gates_masked_ws.argtypes = [vp, vp, ci, vp, vp, ci, ci, ci, vp, vp, ci, ci, tsp, vp, vp, vp, vp, vp,
                                           vp, vp, ci, vp, ctypes.c_longlong, vp]
    l.mie_maxpool_incr.restype = ci
    l.mie_maxpool_incr.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci, ci, tsp, vp, ci, vp]
    l.mie_accumulate.restype = ci
    l.mie_accumulate.argtypes = [vp, vp, ci, tsp, ci, vp]
    l.mie_scale_incr.restype = ci
    l.mie_scale_incr.argtypes = [vp, vp, vp, ci, tsp, ci, vp]
    l.mie_avgpool_incr.restype = ci
    l.mie_avgpool_incr.argtypes = [vp, vp, ci, ci, ci, ci, ci, ci, vp, ci, vp]
    l.mie_linear_incr.restype = ci
    l.mie_linear_incr.argtypes = [vp, ci, ci, vp, ci, vp, ci, vp]
    l.mie_upconv_masked.restype = ci
    l.mie_upconv_masked.argtypes = [vp, vp, vp, vp, ci, ci, ci, vp, vp, ci, ci, ci, ci, tsp, vp, vp, vp, ci, cf, ci, vp]
    l.mie_upconv_pred_masked.restype = ci
    l.mie_upconv_pred_masked.argtypes = [vp, vp, vp, vp, ci, ci, ci, vp, vp, ci, ci, tsp, vp, ci, cf, vp, vp, vp, vp, ci, cf,
                                         vp, ci, vp]
    l.mie_upconv_masked_ws.restype = ci
    l.mie_upconv_masked_ws.argtypes = [vp, vp, vp, vp, ci, ci, ci, vp, vp, ci, ci, ci, ci, tsp, vp, vp, vp, ci, cf, ci, vp,
                                       ctypes.c_longlong, vp]
    l.mie_tconv_refresh.restype = ci
    l.mie_tconv_refresh.argtypes = [vp, ci, ci, ci, vp, ci, ci, ci, ci, vp, tsp, vp, vp, ci, cf, ci, vp]
    l.mie_tconv_masked.restype = ci
    l.mie_tconv_masked.argtypes = [vp, vp, ci, ci, ci, vp, ci, ci, ci, ci, tsp, vp, vp, ci, cf, ci, vp]


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libmie_hip.so not found at %s -- build it with "
                "`python -m maskedincrementeval_amd.build` (there is no fallback path)" % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        _declare(l)
        _lib = l
    return _lib


def check(status):
    """Raise MieError for a negative status code."""
    if status != MIE_OK:
        msg = lib().mie_last_error_string()
        raise MieError(status, msg.decode("utf-8", "replace") if msg else "")


def tile_capacity(n, h, w):
    return ((h + MIE_TILE - 1) // MIE_TILE) * ((w + MIE_TILE - 1) // MIE_TILE) * n
