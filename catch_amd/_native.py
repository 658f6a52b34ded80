"""Loads the native libraries and exposes the C ABI of include/catchq.h through ctypes."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
KERNEL_LIB = os.path.join(LIB_DIR, "libcatchq.so")
TORCH_LIB = os.path.join(LIB_DIR, "_catchq_torch.so")

_lib = None
_torch_loaded = False


class CatchqError(RuntimeError):
    pass


class Epilogue(ctypes.Structure):
    """struct catchq_epilogue"""
    _fields_ = [("exp2", ctypes.c_int), ("chan_div", ctypes.c_void_p), ("chan_rcp", ctypes.c_void_p), ("bias", ctypes.c_void_p),
                ("resid", ctypes.c_void_p), ("act", ctypes.c_int), ("y", ctypes.c_void_p),
                ("y_dtype", ctypes.c_int), ("acc_out", ctypes.c_void_p), ("q", ctypes.c_void_p),
                ("q_bitwidth", ctypes.c_int), ("q_position", ctypes.c_int), ("q_scale", ctypes.c_float),
                ("act_slope", ctypes.c_float), ("resid_after_act", ctypes.c_int),
                ("exp2_dev", ctypes.c_void_p * 2), ("half_steps", ctypes.c_int), ("sharing", ctypes.c_int)]


class PointwiseHead(ctypes.Structure):
    """struct catchq_pointwise_head"""
    _fields_ = [("w", ctypes.c_void_p), ("ci", ctypes.c_int), ("exp2", ctypes.c_int), ("chan_div", ctypes.c_void_p),
                ("chan_rcp", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("q_position", ctypes.c_int)]


class RequantStage(ctypes.Structure):
    """struct catchq_requant_stage"""
    _fields_ = [("w", ctypes.c_void_p), ("exp2", ctypes.c_int), ("chan_div", ctypes.c_void_p),
                ("chan_rcp", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("act", ctypes.c_int),
                ("q_position", ctypes.c_int)]


class ConvDesc(ctypes.Structure):
    """struct catchq_conv_desc"""
    _fields_ = [(n, ctypes.c_int) for n in ("n", "h", "w", "ci", "co", "kh", "kw", "pad_h", "pad_w", "stride_h",
                                            "stride_w", "dil_h", "dil_w", "groups")]


class Shortcut(ctypes.Structure):
    """struct catchq_shortcut"""
    _fields_ = [("x", ctypes.c_void_p), ("w", ctypes.c_void_p), ("x_bits", ctypes.c_int), ("w_bits", ctypes.c_int),
                ("in_h", ctypes.c_int), ("in_w", ctypes.c_int), ("ci", ctypes.c_int), ("stride", ctypes.c_int),
                ("exp2", ctypes.c_int), ("chan_div", ctypes.c_void_p), ("chan_rcp", ctypes.c_void_p),
                ("bias", ctypes.c_void_p)]


class ChainLink(ctypes.Structure):
    """struct catchq_chain_link"""
    _fields_ = [("x", ctypes.c_void_p), ("w", ctypes.c_void_p), ("in_h", ctypes.c_int), ("in_w", ctypes.c_int),
                ("ci", ctypes.c_int), ("stride", ctypes.c_int), ("exp2", ctypes.c_int), ("chan_div", ctypes.c_void_p),
                ("chan_rcp", ctypes.c_void_p), ("bias", ctypes.c_void_p)]


# name -> (restype, argtypes); every symbol include/catchq.h declares
_I, _I64, _F, _P, _SZ = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t
SIGNATURES = {
    "catchq_version": (_I, []),
    "catchq_status_string": (ctypes.c_char_p, [_I]),
    "catchq_pos_from_scale": (_I, [_I, _F, ctypes.POINTER(_I)]),
    "catchq_quant_params": (_I, [_I, _F, ctypes.POINTER(_I), ctypes.POINTER(_F), ctypes.POINTER(_F)]),
    "catchq_per_channel_params": (_I, [_I, _P, _I, ctypes.POINTER(_I), _P, _P]),
    "catchq_quantize": (_I, [_P, _I, _P, _I, _I64, _I, _F, _P]),
    "catchq_quantize_devpos": (_I, [_P, _I, _P, _I, _I64, _P, _P, _P]),
    "catchq_quantize_nchw_to_nhwc": (_I, [_P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _F, _P]),
    "catchq_quantize_nchw_to_nhwc_frame": (_I, [_P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _F, _P]),
    "catchq_quantize_param_workspace_size": (_I, [_I64, ctypes.POINTER(_SZ)]),
    "catchq_quantize_param": (_I, [_P, _I, _I64, _I, _I, _P, _SZ, _P, _P, _P, _P, _P]),
    "catchq_quantize_param_noalloc": (_I, [_P, _I, _I64, _I, _I, _P, _P, _P, _P, _P]),
    "catchq_quantize_per_channel": (_I, [_P, _I, _P, _I, _I, _I64, _P, _P]),
    "catchq_quantize_per_channel_f16": (_I, [_P, _P, _I, _I, _I64, _P, _P]),
    "catchq_per_channel_params_f16": (_I, [_I, _P, _I, ctypes.POINTER(_I), _P, _P]),
    "catchq_dequantize": (_I, [_P, _I, _P, _I, _I64, _I, _F, _P]),
    "catchq_gemm_nt": (_I, [_P, _I, _P, _I, _I64, _I64, _I64, ctypes.POINTER(Epilogue), _P]),
    "catchq_conv_out_size": (_I, [_I] * 5),
    "catchq_conv2d_nhwc": (_I, [_P, _I, _P, _I, ctypes.POINTER(ConvDesc), ctypes.POINTER(Epilogue), _P]),
    "catchq_maxpool_nhwc": (_I, [_P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "catchq_global_avgpool_nhwc": (_I, [_P, _P, _I, _I, _I, _P]),
    "catchq_global_avgpool_quantize_nhwc": (_I, [_P, _P, _I, _I, _I, _I, _I, _F, _P]),
    "catchq_quantize_conv2d_workspace_size": (_I, [ctypes.POINTER(ConvDesc), _I, _I, ctypes.POINTER(_SZ)]),
    "catchq_quantize_conv2d_nhwc": (_I, [_P, _I, _P, _I, _P, _I, _P, _I, ctypes.POINTER(ConvDesc), _P, _P, _I, _P, _SZ, _P]),
    "catchq_conv2d_shortcut_workspace_size": (_I, [_I, _I, ctypes.POINTER(ConvDesc), ctypes.POINTER(Shortcut),
                                                   ctypes.POINTER(_SZ)]),
    "catchq_conv1x1_chain_nhwc": (_I, [ctypes.POINTER(ChainLink), _I, _I, _I, _I, _I, _P, _P, _I, _I, _P]),
    "catchq_conv2d_shortcut_nhwc": (_I, [_P, _I, _P, _I, ctypes.POINTER(ConvDesc), ctypes.POINTER(Epilogue),
                                         ctypes.POINTER(Shortcut), _P, _SZ, _P]),
    "catchq_conv1x1_conv3x3_workspace_size": (_I, [ctypes.POINTER(PointwiseHead), ctypes.POINTER(ConvDesc),
                                                   ctypes.POINTER(Epilogue), ctypes.POINTER(_SZ)]),
    "catchq_conv1x1_conv3x3_nhwc": (_I, [_P, ctypes.POINTER(PointwiseHead), _P, ctypes.POINTER(ConvDesc),
                                         ctypes.POINTER(Epilogue), _P, _SZ, _P]),
    "catchq_inverted_residual_workspace_size": (_I, [_I, _I, _I, _I, _I, _I, _I, ctypes.POINTER(RequantStage),
                                                     ctypes.POINTER(RequantStage), ctypes.POINTER(Epilogue),
                                                     ctypes.POINTER(_SZ)]),
    "catchq_inverted_residual_nhwc": (_I, [_P, _I, _I, _I, _I, _I, _I, _I, ctypes.POINTER(RequantStage),
                                           ctypes.POINTER(RequantStage), _P, ctypes.POINTER(Epilogue), _P, _SZ, _P]),
    "catchq_first_layers_workspace_size": (_I, [_I, _I, _I, _I, _I, _I, _I, _I, _I, ctypes.POINTER(RequantStage), _I, _I, _I,
                                                _I, ctypes.POINTER(_SZ)]),
    "catchq_first_layers_nchw": (_I, [_P, _I, _I, _I, _I, _I, ctypes.c_float, _I, _I, _I, _I, _I,
                                      ctypes.POINTER(RequantStage), _I, _I, _I, _P, _I, _P, _SZ, _P]),
    "catchq_conv1x1_avgpool_workspace_size": (_I, [_I, _I, _I, _I, ctypes.POINTER(Epilogue), ctypes.POINTER(_SZ)]),
    "catchq_conv1x1_avgpool_nhwc": (_I, [_P, _P, _I, _I, _I, _I, ctypes.POINTER(Epilogue), _P, _P, _I, _I, ctypes.c_float,
                                         _P, _SZ, _P]),
    "catchq_conv2d_route": (ctypes.c_char_p, [_I, _I, ctypes.POINTER(ConvDesc)]),
    "catchq_gemm_route": (ctypes.c_char_p, [_I, _I, _I64, _I64, _I64]),
    "catchq_diag_mfma_i8_loop": (_I, [_P, _I, _I, _P, _P]),
}

_BUILD_HINT = "build it with `python catch_amd/build.py` (hipcc cross-compiles gfx950 without a GPU)"


def kernel_lib():
    """ctypes handle of libcatchq.so with argument types set."""
    global _lib
    if _lib is None:
        if not os.path.exists(KERNEL_LIB):
            raise ImportError("catch_amd: %s is missing; %s" % (KERNEL_LIB, _BUILD_HINT))
        lib = ctypes.CDLL(KERNEL_LIB, mode=ctypes.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError here = header and library disagree
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def load():
    """Load libcatchq.so and the torch extension (registers torch.ops.torch_mlu.*)."""
    global _torch_loaded
    lib = kernel_lib()
    if not _torch_loaded:
        if not os.path.exists(TORCH_LIB):
            raise ImportError("catch_amd: %s is missing; %s" % (TORCH_LIB, _BUILD_HINT))
        import torch
        torch.ops.load_library(TORCH_LIB)
        _torch_loaded = True
    return lib


def check(status, what="catchq"):
    if status != 0:
        raise CatchqError("%s: %s" % (what, kernel_lib().catchq_status_string(status).decode()))
