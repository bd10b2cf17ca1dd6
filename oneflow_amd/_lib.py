"""Loader for the in-tree HIP library ``csrc/libofq_hip.so`` (the C ABI of ``include/ofq.h``).

There is no CPU fallback: if the library is missing the import fails, and every call checks the
returned status and raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libofq_hip.so")

# mirror of the enums in include/ofq.h
OK = 0
ERR_UNSUPPORTED = 5
F32, F16, BF16, F64, I8, U8 = 0, 1, 2, 3, 4, 5
SCHEME = {"symmetric": 0, "affine": 1}
FORMULA = {"google": 0, "cambricon": 1}
ZP_MODE = {"float": 0, "uint8": 1}
LN_STATS_FP32, LN_STATS_FP64 = 0, 1

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_sz = ctypes.c_size_t

# name -> (restype, argtypes); must match include/ofq.h exactly
SIGNATURES = {
    "ofq_status_string": (ctypes.c_char_p, [_i]),
    "ofq_abi_version": (_i, []),
    "ofq_groupwise_dequantize": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i64, _i64, _i64]),
    "ofq_fused_linear_gq_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i64, _i64, _i64, _i64]),
    "ofq_fused_linear_gq": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i64,
                                 _i64, _i64, _i64, _vp, _sz]),
    "ofq_min_max_observer_workspace_bytes": (_sz, [_i, _i64, _i64]),
    "ofq_min_max_observer": (_i, [_vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _i, _i, _vp, _sz]),
    "ofq_moving_average_min_max_observer_workspace_bytes": (_sz, [_i, _i64]),
    "ofq_moving_average_min_max_observer": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i64, _i,
                                                 _i, _i, ctypes.c_float, _i64, _i, _vp, _sz]),
    "ofq_quantization": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i64, _i64, _i, _i, _i, _i]),
    "ofq_fake_quantization": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _i, _i, _i]),
    "ofq_fused_layer_norm_min_max_observer_workspace_bytes": (_sz, [_i, _i64, _i64]),
    "ofq_fused_layer_norm_min_max_observer": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i64,
                                                   _i64, ctypes.c_double, _i, _vp, _sz]),
    "ofq_fused_layer_norm_min_max_observer_static": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i,
                                                          _i64, _i64, ctypes.c_double, _i]),
    "ofq_fused_skip_layer_norm_min_max_observer": (_i, [_vp, _vp, _vp, _vp, ctypes.c_double, _vp,
                                                        _vp, _vp, _vp, _vp, _i, _i64, _i64,
                                                        ctypes.c_double, _i, _vp, _sz]),
    "ofq_fused_layer_norm_min_max_observer_stats": (_i, [_vp, _vp, _vp, _vp, ctypes.c_double, _i,
                                                         _vp, _vp, _vp, _vp, _vp, _i, _i64, _i64,
                                                         ctypes.c_double, _i, _i, _vp, _sz]),
    "ofq_fused_layer_norm_quantization": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i64, _i64,
                                               ctypes.c_double, _i, _i, _vp, _sz]),
    "ofq_fused_layer_norm_quantization_workspace_bytes": (_sz, [_i, _i64, _i64]),
    "ofq_grouped_linear_gq": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i,
                                   _i, _i, _i64]),
    "ofq_fused_glu_gq": (_i, [_vp] * 13 + [_i, _i, _i, _i, _i, _i, _i64, _i64, _i64, _i64]),
    "ofq_groupwise_quantize": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i64, _i64, _i64]),
    "ofq_matmul_quant": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i64]),
    "ofq_matmul_quant_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "ofq_matmul_quant_ws": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i64, _vp, _sz]),
    "ofq_groupwise_repack_bytes": (_sz, [_i, _i64, _i64]),
    "ofq_groupwise_repack": (_i, [_vp, _vp, _vp, _i, _i64, _i64]),
    "ofq_fused_linear_gq_tiled": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i64,
                                       _i64, _i64, _i64]),
}


class OfqError(RuntimeError):
    """A C-ABI call returned a non-zero ofq_status."""

    def __init__(self, fn, status, text):
        super().__init__(f"{fn} failed with status {status}: {text}")
        self.status = status


_lib = None


def lib():
    """The loaded library with prototypes set.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.dirname(LIB_PATH)}` "
                "(or __graft_entry__.build()); there is no CPU fallback")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(fn_name, status):
    if status != OK:
        raise OfqError(fn_name, status, lib().ofq_status_string(status).decode())
