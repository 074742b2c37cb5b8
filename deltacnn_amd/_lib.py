"""ctypes binding of libdeltacnn_hip.so (declared in include/deltacnn_hip.h).

The library is the only compute path of this package: if it is missing, loading
raises instead of falling back to anything else.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdeltacnn_hip.so")

DC_F32, DC_F16, DC_BF16 = 0, 1, 2
ERROR_NAMES = {0: "DC_OK", -1: "DC_ERR_DTYPE", -2: "DC_ERR_SHAPE", -3: "DC_ERR_UNSUPPORTED",
               -4: "DC_ERR_NULL", -5: "DC_ERR_ALIGN", -6: "DC_ERR_LAUNCH"}


class Geometry(ctypes.Structure):
    """struct dc_geometry."""
    _fields_ = [(n, c_int32) for n in (
        "batch", "in_h", "in_w", "in_c", "out_h", "out_w", "out_c", "kernel_h", "kernel_w",
        "stride_h", "stride_w", "dilation_h", "dilation_w", "pad_top", "pad_left", "pad_bottom",
        "pad_right", "groups")]


class BlockArgs(ctypes.Structure):
    """struct dc_block_args."""
    _fields_ = [
        ("input", c_void_p), ("mask", c_void_p), ("dw_filter", c_void_p), ("dw_prev_out", c_void_p),
        ("dw_truncated", c_void_p), ("dw_threshold", c_float), ("dw_activation", c_int32),
        ("dw_truncation_mode", c_int32),
        ("project_packed_filter", c_void_p), ("project_channels", c_int32), ("residual", c_void_p),
        ("residual_mask", c_void_p), ("weight_residual", c_float), ("weight_conv", c_float),
        ("out", c_void_p), ("out_mask", c_void_p),
        ("expand_packed_filter", c_void_p), ("expand_channels", c_int32), ("expand_prev_out", c_void_p),
        ("expand_truncated", c_void_p), ("expand_threshold", c_float), ("expand_activation", c_int32),
        ("expand_truncation_mode", c_int32), ("expand_out", c_void_p), ("expand_out_mask", c_void_p),
        ("flags", c_int32)]


class ExpandDwArgs(ctypes.Structure):
    """struct dc_expand_dw_args."""
    _fields_ = [
        ("input", c_void_p), ("mask", c_void_p), ("expand_packed_filter", c_void_p),
        ("expand_in_channels", c_int32), ("expand_prev_out", c_void_p), ("expand_truncated", c_void_p),
        ("expand_threshold", c_float), ("expand_activation", c_int32), ("expand_truncation_mode", c_int32),
        ("expand_out", c_void_p), ("expand_out_mask", c_void_p),
        ("dw_filter", c_void_p), ("dw_prev_out", c_void_p), ("dw_truncated", c_void_p),
        ("dw_threshold", c_float), ("dw_activation", c_int32), ("dw_truncation_mode", c_int32),
        ("out", c_void_p), ("out_mask", c_void_p)]


class ProjectExpandArgs(ctypes.Structure):
    """struct dc_project_expand_args."""
    _fields_ = [
        ("input", c_void_p), ("mask", c_void_p), ("project_packed_filter", c_void_p),
        ("residual", c_void_p), ("residual_mask", c_void_p), ("weight_residual", c_float), ("weight_conv", c_float),
        ("out", c_void_p), ("out_mask", c_void_p),
        ("expand_packed_filter", c_void_p), ("expand_channels", c_int32), ("expand_prev_out", c_void_p),
        ("expand_truncated", c_void_p), ("expand_activation", c_int32), ("expand_out", c_void_p),
        ("expand_out_mask", c_void_p),
        ("dw_geometry", POINTER(Geometry)), ("dw_activation", c_int32), ("dw_truncation_mode", c_int32)]


class ConvItem(ctypes.Structure):
    """struct dc_conv_item."""
    _fields_ = [
        ("geometry", Geometry), ("input", c_void_p), ("mask", c_void_p), ("packed_filter", c_void_p),
        ("bias", c_void_p), ("out", c_void_p), ("out_mask", c_void_p),
        ("residual", c_void_p), ("residual_mask", c_void_p), ("weight_residual", c_float), ("weight_conv", c_float),
        ("sum_prev_out", c_void_p), ("sum_activation", c_int32),
        ("prev_out", c_void_p), ("truncated", c_void_p), ("threshold", c_float), ("activation", c_int32),
        ("truncation_mode", c_int32)]


class AddItem(ctypes.Structure):
    """struct dc_add_item."""
    _fields_ = [
        ("a", c_void_p), ("b", c_void_p), ("prev_out", c_void_p), ("out", c_void_p),
        ("mask_a", c_void_p), ("mask_b", c_void_p), ("mask_out", c_void_p),
        ("weight_a", c_float), ("weight_b", c_float), ("activation", c_int32),
        ("batch", c_int32), ("height", c_int32), ("width", c_int32), ("channels", c_int32), ("scale", c_int32)]


CONV_GROUP_MAX = 8

_P = c_void_p
_G = POINTER(Geometry)
_SIGNATURES = {
    "dc_version": (c_char_p, []),
    "dc_last_error": (c_char_p, []),
    "dc_last_kernels": (ctypes.c_char_p, []),
    "dc_sparsify": (c_int, [_P, _P, _P, _P, c_float, c_int32, c_int32, c_int, _P]),
    "dc_activate_truncate": (c_int, [_P, _P, _P, _P, c_float, c_int, c_int, c_int32, c_int32, c_int, _P]),
    "dc_conv": (c_int, [_G, _P, _P, _P, _P, _P, _P, _P, c_int, _P]),
    "dc_conv_act": (c_int, [_G, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_float, c_int, c_int, c_int, _P]),
    "dc_conv_add": (c_int, [_G, _P, _P, _P, _P, _P, _P, _P, _P, c_float, c_float, _P, c_int, c_int, _P]),
    "dc_block": (c_int, [_G, POINTER(BlockArgs), c_int, _P]),
    "dc_expand_depthwise": (c_int, [_G, POINTER(ExpandDwArgs), c_int, _P]),
    "dc_project_expand": (c_int, [_G, POINTER(ProjectExpandArgs), c_int, _P]),
    "dc_conv_group": (c_int, [POINTER(ConvItem), c_int32, c_int, _P]),
    "dc_add_group": (c_int, [POINTER(AddItem), c_int32, c_int, _P]),
    "dc_packed_filter_bytes": (c_int64, [_G, c_int, c_int]),
    "dc_pack_filter": (c_int, [_G, _P, _P, c_int, c_int, _P]),
    "dc_deconv": (c_int, [_G, _P, _P, _P, _P, _P, _P, _P, c_int, _P]),
    "dc_deconv_add": (c_int, [_G, _P, _P, _P, _P, _P, _P, _P, c_float, c_float, c_int, _P]),
    "dc_pool": (c_int, [_G, _P, _P, _P, _P, _P, c_int, c_int, c_int, _P]),
    "dc_pool_update": (c_int, [_G, _P, _P, _P, _P, _P, c_int, _P]),
    "dc_concat_conv": (c_int, [_G, c_int, _P, _P, _P, _P, _P, _P, c_int, _P]),
    "dc_densify": (c_int, [_P, _P, _P, _P, c_int32, c_int32, c_int, _P]),
    "dc_pool_densify": (c_int, [_G, _P, _P, _P, _P, c_int, _P]),
    "dc_linear": (c_int, [_P, _P, _P, _P, c_int32, c_int32, c_int32, c_int, _P]),
    "dc_add": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_float, c_float, c_int, c_int, c_int32, c_int32, c_int, _P]),
    "dc_add_upsampled": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_float, c_float, c_int, c_int32, c_int32, c_int32, c_int32, c_int32, c_int, _P]),
    "dc_add_to_dense": (c_int, [_P, _P, _P, c_int, c_int32, c_int32, c_int, _P]),
    "dc_upsample": (c_int, [_P, _P, _P, _P, c_int32, c_int32, c_int32, c_int32, c_int32, c_int, _P]),
    "dc_concat": (c_int, [_P, _P, _P, _P, _P, _P, c_int32, c_int32, c_int32, c_int, _P]),
    "dc_mul_add": (c_int, [_P, _P, _P, _P, _P, _P, c_int32, c_int32, c_int, _P]),
}

_lib = None


class DeltaCNNError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"{ERROR_NAMES.get(code, code)}: {message}")
        self.code = code


def load() -> ctypes.CDLL:
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python deltacnn_amd/csrc/build.py` "
            "(hipcc --offload-arch=gfx950). There is no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int) -> None:
    if code != 0:
        raise DeltaCNNError(code, load().dc_last_error().decode())
