"""ctypes binding of libtorch_col_hip.so (the C ABI declared in include/*.h).

There is no fallback: if the shared library has not been built, importing the
handle raises, so no caller can silently run anything but the HIP path.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libtorch_col_hip.so")

_lib = None


class TorchColHipError(RuntimeError):
    pass


class KernelStat(ctypes.Structure):
    """Mirror of tch_kernel_stat (include/torch_col_hip.h)."""
    _fields_ = [("name", ctypes.c_char * 96), ("total_ms", ctypes.c_double), ("work", ctypes.c_double),
                ("launches", c_int64), ("work_is_bytes", c_int)]


def _declare(lib):
    vp, i, i64, f = c_void_p, c_int, c_int64, c_float
    sig = {
        "tch_last_error": (c_char_p, []),
        "tch_has_device_code": (i, []),
        "tch_context_create": (i, [vp, POINTER(vp)]),
        "tch_context_destroy": (None, [vp]),
        "tch_context_take_rejected": (c_uint64, [vp]),
        "tch_program_create": (i, [POINTER(vp)]),
        "tch_program_destroy": (None, [vp]),
        "tch_program_size": (i64, [vp]),
        "tch_program_begin_record": (i, [vp, vp]),
        "tch_program_end_record": (i, [vp]),
        "tch_program_run": (i, [vp, vp, i64, i64]),
        "tch_RegisterStream": (c_uint64, [c_uint64]),
        "tch_UnRegisterStream": (i, [c_uint64]),
        "tch_UnRegisterAllStreams": (None, []),
        "tch_GetXQueueSize": (c_size_t, [c_uint64]),
        "tch_GetXQueueSizeAllStreams": (c_size_t, []),
        "tch_GetTotalXQueueSize": (c_size_t, []),
        "tch_AbortStream": (c_size_t, [c_uint64]),
        "tch_AbortAllStreams": (c_size_t, []),
        "tch_SyncStream": (i, [c_uint64]),
        "tch_SyncAllStreams": (i, []),
        "tch_QueryRejectCudaCalls": (i, []),
        "tch_SetRejectCudaCalls": (None, [i]),
        "tch_SetXQueueShape": (None, [i, i]),
        "tch_GetXQueueInFlight": (c_size_t, [c_uint64]),
        "tch_program_profile": (i, [vp, vp, i, vp, i, POINTER(c_int)]),
        "tch_conv2d_fwd": (i, [vp, i, vp, vp, vp, vp, vp, vp, i] + [i] * 11),
        "tch_conv2d_dgrad": (i, [vp, i, vp, vp, vp, vp, vp] + [i] * 11),
        "tch_conv2d_wgrad_pick_splits": (i, [i] * 10),
        "tch_conv2d_wgrad_workspace_bytes": (i64, [i] * 6),
        "tch_conv2d_wgrad": (i, [vp, i, vp, vp, vp, vp, i, i] + [i] * 11),
        "tch_bn_workspace_bytes": (i64, [i, i64, i]),
        "tch_bn_fwd_train": (i, [vp, i, vp, vp, vp, i, i64, i, vp, vp, vp, vp, vp, vp, f, f, vp]),
        "tch_bn_bwd": (i, [vp, i, vp, vp, vp, vp, i64, i, vp, vp, vp, vp, vp, i, vp]),
        "tch_maxpool_fwd": (i, [vp, i, vp, vp, vp] + [i] * 7),
        "tch_maxpool_bwd": (i, [vp, i, vp, vp, vp] + [i] * 7),
        "tch_avgpool_fwd": (i, [vp, i, vp, vp, i, i, i]),
        "tch_avgpool_bwd": (i, [vp, i, vp, vp, i, i, i]),
        "tch_softmax_ce_fwd_bwd": (i, [vp, i, vp, vp, vp, vp, vp, i, i, i, f]),
        "tch_sgd_momentum_step": (i, [vp, vp, vp, vp, vp, i64, f, f, f]),
        "tch_grad_accumulate": (i, [vp, vp, vp, i64]),
        "tch_fill_zero": (i, [vp, vp, i64]),
        "tch_bias_grad": (i, [vp, i, vp, vp, i, i, i, i]),
        "tch_nchw_to_nhwc_pad": (i, [vp, i, vp, vp, i, i, i, i, i]),
        "tch_filter_transpose_batched": (i, [vp, i, vp, vp, vp, i, i64, i64]),
        "tch_cast_from_f32": (i, [vp, i, vp, vp, i64]),
        "tch_cast_to_f32": (i, [vp, i, vp, vp, i64]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return sig


DEVICE_SYMBOLS = None


def lib():
    """The loaded shared library; raises if it was never built."""
    global _lib, DEVICE_SYMBOLS
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TorchColHipError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C sirius_amd/csrc`. There is no CPU fallback for this path.")
        handle = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        DEVICE_SYMBOLS = _declare(handle)
        from . import _lib_host  # noqa: F401  (declares the host-runtime half of the ABI)
        _lib_host.declare(handle)
        _lib = handle
    return _lib


def check(rc, what=""):
    if rc < 0:
        msg = lib().tch_last_error()
        raise TorchColHipError(f"{what} failed ({rc}): {msg.decode() if msg else ''}")
    return rc
