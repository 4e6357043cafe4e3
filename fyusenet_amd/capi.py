"""ctypes binding of the C ABI declared in include/fynhip.h.

The shared library is required: there is no fallback.  Loading fails loudly when libfynhip.so has
not been built (python -m fyusenet_amd.build), and every failing call raises FynException with the
message the engine recorded.
"""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("FYNHIP_LIBRARY") or os.path.join(HERE, "libfynhip.so")  # override: alternative builds

FYN_MAX_CONCAT_INPUTS = 8
FYN_NAME_LEN = 64

# fyn_status
OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_STATE, ERR_DEVICE, ERR_NOTFOUND, ERR_DUPLICATE = 0, -1, -2, -3, -4, -5, -6
# fyn_storage
STORAGE_F32, STORAGE_F16 = 0, 1
# fyn_order
ORDER_CHANNELWISE, ORDER_GPU_SHALLOW, ORDER_GPU_DEEP = 0, 1, 2


class FynException(RuntimeError):
    """Counterpart of the reference's FynException (fyusenet/common/fynexception.h)."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


class _ConcatInput(ctypes.Structure):
    _fields_ = [("channels", ctypes.c_int32), ("padding", ctypes.c_int32), ("flags", ctypes.c_uint32)]


class LayerDesc(ctypes.Structure):
    """struct fyn_layer_desc."""
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("type", ctypes.c_int32),
        ("number", ctypes.c_int32),
        ("name", ctypes.c_char * FYN_NAME_LEN),
        ("flags", ctypes.c_uint32),
        ("width", ctypes.c_int32),
        ("height", ctypes.c_int32),
        ("in_channels", ctypes.c_int32),
        ("out_channels", ctypes.c_int32),
        ("input_padding", ctypes.c_int32),
        ("output_padding", ctypes.c_int32),
        ("residual_padding", ctypes.c_int32),
        ("downsample", ctypes.c_int32 * 2),
        ("upsample", ctypes.c_int32 * 2),
        ("leaky_relu", ctypes.c_float),
        ("clip_low", ctypes.c_float),
        ("clip_high", ctypes.c_float),
        ("kernel", ctypes.c_int32),
        ("dilation", ctypes.c_int32 * 2),
        ("group_size", ctypes.c_int32),
        ("pool_size", ctypes.c_int32 * 2),
        ("global_pool", ctypes.c_int32),
        ("num_inputs", ctypes.c_int32),
        ("inputs", _ConcatInput * FYN_MAX_CONCAT_INPUTS),
        ("transconv_crop", ctypes.c_int32),
        ("scale_type", ctypes.c_int32),
        ("arith_op", ctypes.c_int32),
        ("operand", ctypes.c_float),
        ("cast_target", ctypes.c_int32),
        ("window", ctypes.c_int32),
        ("blur_type", ctypes.c_int32),
        ("source_step", ctypes.c_float),
    ]


class TensorView(ctypes.Structure):
    """struct fyn_tensor_view."""
    _fields_ = [("data", ctypes.c_void_p), ("channels", ctypes.c_int32), ("height", ctypes.c_int32), ("width", ctypes.c_int32),
                ("padding", ctypes.c_int32), ("channel_pitch", ctypes.c_int32), ("storage", ctypes.c_int32)]


CUSTOM_SETUP_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(TensorView), ctypes.c_int, ctypes.POINTER(TensorView))
CUSTOM_FORWARD_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(TensorView), ctypes.c_int, ctypes.POINTER(TensorView),
                                     ctypes.c_void_p, ctypes.c_uint64)
CUSTOM_CLEANUP_FN = ctypes.CFUNCTYPE(None, ctypes.c_void_p)


class CustomLayer(ctypes.Structure):
    """struct fyn_custom_layer."""
    _fields_ = [("user", ctypes.c_void_p), ("setup", CUSTOM_SETUP_FN), ("forward", CUSTOM_FORWARD_FN), ("cleanup", CUSTOM_CLEANUP_FN)]


# every symbol include/fynhip.h declares: name -> (restype, argtypes)
_P = ctypes.c_void_p
_F = ctypes.POINTER(ctypes.c_float)
SYMBOLS = {
    "fyn_last_error": (ctypes.c_char_p, []),
    "fyn_device_info": (ctypes.c_int, [ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]),
    "fyn_net_create": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.POINTER(_P)]),
    "fyn_net_destroy": (ctypes.c_int, [_P]),
    "fyn_net_add_layer": (ctypes.c_int, [_P, ctypes.POINTER(LayerDesc)]),
    "fyn_net_add_custom_layer": (ctypes.c_int, [_P, ctypes.POINTER(LayerDesc), ctypes.POINTER(CustomLayer)]),
    "fyn_net_connect": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "fyn_layer_load_weights": (ctypes.c_int, [_P, ctypes.c_int, _F, ctypes.c_size_t]),
    "fyn_layer_load_scale_bias": (ctypes.c_int, [_P, ctypes.c_int, _F, ctypes.c_size_t]),
    "fyn_layer_weight_floats": (ctypes.c_int, [_P, ctypes.c_int, ctypes.POINTER(ctypes.c_size_t)]),
    "fyn_net_setup": (ctypes.c_int, [_P]),
    "fyn_net_set_input": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, _F, ctypes.c_int]),
    "fyn_net_forward": (ctypes.c_int, [_P, ctypes.POINTER(ctypes.c_uint64)]),
    "fyn_net_finish": (ctypes.c_int, [_P]),
    "fyn_layer_copy_result": (ctypes.c_int, [_P, ctypes.c_int, _F, ctypes.c_int]),
    "fyn_layer_copy_result_noalloc": (ctypes.c_int, [_P, ctypes.c_int, _F, ctypes.c_int]),
    "fyn_layer_output_shape": (ctypes.c_int, [_P, ctypes.c_int] + [ctypes.POINTER(ctypes.c_int)] * 4),
    "fyn_net_get_output": (ctypes.c_int, [_P, ctypes.c_int, _F, ctypes.c_int]),
    "fyn_layer_copy_argmax": (ctypes.c_int, [_P, ctypes.c_int, ctypes.POINTER(ctypes.c_int32), _F]),
    "fyn_net_enable_timings": (ctypes.c_int, [_P, ctypes.c_int]),
    "fyn_net_get_timing": (ctypes.c_int, [_P, ctypes.c_int, _F, ctypes.POINTER(ctypes.c_int)]),
    "fyn_net_enable_intermediate_output": (ctypes.c_int, [_P, ctypes.c_char_p]),
    "fyn_net_set_buffer_reuse": (ctypes.c_int, [_P, ctypes.c_int]),
    "fyn_net_use_graph": (ctypes.c_int, [_P, ctypes.c_int]),
    "fyn_net_time_forward": (ctypes.c_int, [_P, ctypes.c_int, _F]),
    "fyn_net_time_steps": (ctypes.c_int, [_P, ctypes.c_int, _F]),
    "fyn_net_input_floats": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_size_t)]),
    "fyn_net_async_sizes": (ctypes.c_int, [_P, ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]),
    "fyn_layer_time": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, _F]),
    "fyn_net_async_begin": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "fyn_net_async_submit": (ctypes.c_int, [_P, _F, _F, ctypes.POINTER(ctypes.c_uint64)]),
    "fyn_net_async_wait": (ctypes.c_int, [_P, ctypes.c_uint64]),
    "fyn_net_async_end": (ctypes.c_int, [_P]),
    "fyn_layer_kernel_info": (ctypes.c_int, [_P, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]),
    "fyn_net_device_allocations": (ctypes.c_int, [_P, ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]),
}

_lib = None


def lib():
    """Loads libfynhip.so (once) and declares all prototypes."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "fyusenet_amd: %s is missing; build it with `python -m fyusenet_amd.build` "
                "(there is no CPU fallback)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status):
    if status != OK:
        msg = lib().fyn_last_error()
        raise FynException(status, msg.decode("utf-8", "replace") if msg else "error %d" % status)


def fptr(arr):
    assert arr.dtype == np.float32 and arr.flags["C_CONTIGUOUS"]
    return arr.ctypes.data_as(_F)


def device_info(device=0):
    buf = ctypes.create_string_buffer(512)
    check(lib().fyn_device_info(device, buf, len(buf)))
    return buf.value.decode()
