"""ctypes binding of ``libdeepshift_hip.so`` (the C ABI declared in ``include/deepshift_hip.h``).

The library is the only compute path of this package: if it is missing, loading fails loudly --
there is no CPU or eager-PyTorch fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdeepshift_hip.so")

DS_Q_ROUND_TO_FIXED = 0
DS_Q_CAST = 1
DS_SMALL_RELU = 0x100
DS_BITS_ZERO_TOP = 0x100
DS_BITS_TOP_UNUSED = 0x200
DS_Q_BORDER_KEPT = 0x100
DS_CHAIN_ONE_LAUNCH = 0x200
DS_CHAIN_LAUNCH_PER_LAYER = 0x400
DS_CHAIN_CONTROL_BYTES = 12288
DS_CHAIN_STATUS_AT = 1536

_c_int = ctypes.c_int
_c_i64 = ctypes.c_int64
_ptr = ctypes.c_void_p
_size = ctypes.c_size_t

class FusedConv(ctypes.Structure):
    """``ds_fused_conv`` of the header: one convolution of a two-convolution launch."""
    _fields_ = [("tiled", _ptr), ("bias", _ptr), ("out", _ptr), ("q", _ptr), ("scale", _ptr), ("shift", _ptr),
                ("residual", _ptr)] + [(name, _c_int) for name in
                                       ("O", "FH", "FW", "crop_h", "crop_w", "bits", "relu", "I", "F", "ph", "pw",
                                        "q_bytes")]


_fcp = ctypes.POINTER(FusedConv)


class ChainLayer(ctypes.Structure):
    """``ds_chain_layer`` of the header: one layer of a one-launch chain of small linear layers."""
    _fields_ = [("tiled", _ptr), ("bias", _ptr)] + [(name, _c_int) for name in ("K", "N", "bits", "base", "relu")]


_clp = ctypes.POINTER(ChainLayer)

# name -> (restype, argtypes); mirrors include/deepshift_hip.h one to one
SIGNATURES = {
    "ds_version": (_c_int, []),
    "ds_status_string": (ctypes.c_char_p, [_c_int]),
    "ds_pack_i32": (_c_int, [_ptr, _ptr, _ptr, _c_int, _c_int, _c_int, _c_int, _ptr]),
    "ds_tiled_bytes": (_size, [_c_int, _c_int, _c_int]),
    "ds_tile_weights_i32": (_c_int, [_ptr, _ptr] + [_c_int] * 6 + [_ptr]),
    "ds_tile_weights_zero_top_i32": (_c_int, [_ptr, _ptr] + [_c_int] * 5 + [_ptr]),
    "ds_convert_stats_f32": (_c_int, [_ptr, _c_i64, _c_int, _c_int, _ptr, _ptr]),
    "ds_convert_weights_f32": (_c_int, [_ptr, _ptr] + [_c_int] * 6 + [_ptr]),
    "ds_convert_codes_f32": (_c_int, [_ptr, _ptr, _ptr, _c_i64, _c_int, _c_int, _ptr]),
    "ds_scan_words_i32": (_c_int, [_ptr, _c_int, _c_int, _c_int, _ptr, _ptr]),
    "ds_check_words_i32": (_c_int, [_ptr] + [_c_int] * 5 + [_ptr, _ptr]),
    "ds_check_bound_i8": (_c_int, [_ptr, _c_i64, _c_int, _ptr, _ptr]),
    "ds_paired_bytes": (_size, [_c_int, _c_int, _c_int]),
    "ds_tile_weights_paired_i32": (_c_int, [_ptr, _ptr] + [_c_int] * 6 + [_ptr]),
    "ds_conv2d_paired_i8": (_c_int, [_ptr] * 4 + [_c_int] * 11 + [_ptr]),
    "ds_conv2d_paired_fused_workspace_bytes": (_size, [_c_int] * 11),
    "ds_conv2d_paired_fused_i8": (_c_int, [_ptr] * 8 + [_c_int] * 18 + [_ptr, _size, _ptr]),
    "ds_quantize_pad_f32_i8": (_c_int, [_ptr, _ptr] + [_c_int] * 8 + [_ptr]),
    "ds_requantize_affine_pad_i8": (_c_int, [_ptr] * 6 + [_c_int] * 10 + [_ptr]),
    "ds_requantize_affine_maxpool_i8": (_c_int, [_ptr] * 5 + [_c_int] * 13 + [_ptr]),
    "ds_linear_workspace_bytes": (_size, [_c_int] * 4),
    "ds_linear_i32": (_c_int, [_ptr] * 4 + [_c_int] * 5 + [_ptr, _size, _ptr]),
    "ds_linear_tiled_workspace_bytes": (_size, [_c_int] * 4),
    "ds_linear_tiled_i32": (_c_int, [_ptr, _c_int, _ptr, _ptr, _ptr] + [_c_int] * 5 + [_ptr, _size, _ptr]),
    "ds_linear_tiled_noalloc_max_bytes": (_size, []),
    "ds_linear_tiled_noalloc_i32": (_c_int, [_ptr, _c_int, _ptr, _ptr, _ptr] + [_c_int] * 5 + [_ptr]),
    "ds_linear_small_f32": (_c_int, [_ptr, _ptr, _ptr, _ptr] + [_c_int] * 8 + [_ptr]),
    "ds_linear_chain_workspace_bytes": (_size, [_c_int, _clp, _c_int]),
    "ds_linear_chain_f32": (_c_int, [_ptr, _clp, _c_int, _ptr, _c_int, _c_int, _c_int, _c_int, _ptr, _size, _ptr]),
    "ds_conv2d_workspace_bytes": (_size, [_c_int] * 10),
    "ds_conv2d_i32": (_c_int, [_ptr] * 4 + [_c_int] * 11 + [_ptr, _size, _ptr]),
    "ds_conv2d_tiled_workspace_bytes": (_size, [_c_int] * 10),
    "ds_conv2d_tiled_i32": (_c_int, [_ptr] * 4 + [_c_int] * 11 + [_ptr, _size, _ptr]),
    "ds_cpu_linear_i32": (_c_int, [_ptr] * 5 + [_c_int] * 4),
    "ds_cpu_conv2d_i32": (_c_int, [_ptr] * 5 + [_c_int] * 10),
    "ds_conv2d_tiled_fusable": (_c_int, [_c_int] * 11),
    "ds_conv2d_tiled_fused_i32": (_c_int, [_ptr] * 8 + [_c_int] * 18 + [_ptr, _size, _ptr]),
    "ds_conv2d_tiled_fused_pair_workspace_bytes": (_size, [_c_int] * 6 + [_fcp, _fcp]),
    "ds_conv2d_tiled_fused_pair_i32": (_c_int, [_ptr] + [_c_int] * 7 + [_fcp, _fcp, _ptr, _size, _ptr]),
    "ds_quantize_f32_i32": (_c_int, [_ptr, _ptr, _c_i64, _c_int, _c_int, _c_int, _ptr]),
    "ds_quantize_pad_f32_i32": (_c_int, [_ptr, _ptr] + [_c_int] * 9 + [_ptr]),
    "ds_quantize_transpose_f32_i32": (_c_int, [_ptr, _ptr] + [_c_int] * 6 + [_ptr]),
    "ds_pad_i32": (_c_int, [_ptr, _ptr] + [_c_int] * 6 + [_ptr]),
    "ds_transpose_i32": (_c_int, [_ptr, _ptr, _c_int, _c_int, _c_int, _ptr]),
    "ds_dequantize_i32_f32": (_c_int, [_ptr, _ptr, _c_i64, _c_int, _ptr]),
    "ds_dequantize_affine_i32_f32": (_c_int, [_ptr] * 5 + [_c_int] * 5 + [_ptr]),
    "ds_requantize_affine_pad_i32": (_c_int, [_ptr] * 6 + [_c_int] * 11 + [_ptr]),
    "ds_requantize_affine_maxpool_i32": (_c_int, [_ptr] * 5 + [_c_int] * 14 + [_ptr]),
    "ds_mul_tiled_bytes": (_size, [_c_int, _c_int]),
    "ds_mul_tile_weights_f32": (_c_int, [_ptr, _ptr] + [_c_int] * 4 + [_ptr]),
    "ds_mul_conv2d_f32": (_c_int, [_ptr] * 4 + [_c_int] * 9 + [_ptr]),
    "ds_mul_linear_f32": (_c_int, [_ptr, _c_int, _ptr, _ptr, _ptr] + [_c_int] * 3 + [_ptr]),
    "ds_valu_calibrate": (_c_int, [_ptr, _c_int, _c_int, _ptr]),
    "ds_copy_i32": (_c_int, [_ptr, _ptr, _c_i64, _ptr]),
    "ds_test_tune": (_c_int, [ctypes.c_char_p, _c_int]),
    "ds_test_fast_div": (_c_int, [_ptr, _ptr, ctypes.c_long, ctypes.c_uint, _c_int, _ptr]),
}

_LIB = None


class DeepShiftError(RuntimeError):
    """A libdeepshift_hip entry point returned a non-zero status."""

    def __init__(self, fn, status, message):
        super().__init__("%s failed: %s (status %d)" % (fn, message, status))
        self.status = status


def lib():
    """The loaded library; raises if it has not been built (``python -m deepshift_amd.build``)."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m deepshift_amd.build` "
                "(there is no fallback path)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _LIB = handle
    return _LIB


def call(name, *args):
    """Invoke a status-returning entry point and raise :class:`DeepShiftError` on failure."""
    handle = lib()
    status = getattr(handle, name)(*args)
    if status != 0:
        raise DeepShiftError(name, status, handle.ds_status_string(status).decode())


def current_stream(device):
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def ptr(tensor):
    return None if tensor is None else ctypes.c_void_p(tensor.data_ptr())
