"""ctypes front-end of the CPU oracle (``libofq_oracle.so``, built from ``ofq_oracle.c``).

TEST INFRASTRUCTURE ONLY.  Imported by ``tests/``, by ``__graft_entry__.smoke`` and by the
CPU-baseline leg of ``bench.py``; never by the ``oneflow_amd`` package.

All functions take and return numpy arrays.  fp16 tensors are ``np.float16``; bf16 tensors are
``np.uint16`` bit patterns (numpy has no bf16), see :func:`f32_to_bf16_bits`.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libofq_oracle.so")

F32, F16, BF16 = 0, 1, 2
SYMMETRIC, AFFINE = 0, 1
GOOGLE, CAMBRICON = 0, 1
_SCHEME = {"symmetric": SYMMETRIC, "affine": AFFINE}
_FORMULA = {"google": GOOGLE, "cambricon": CAMBRICON}


def build(force=False):
    """Compile the oracle with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "ofq_oracle.c"))
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libofq_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.ofq_ref_half_to_float.restype = ctypes.c_float
        _lib.ofq_ref_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.ofq_ref_float_to_half.restype = ctypes.c_uint16
        _lib.ofq_ref_float_to_half.argtypes = [ctypes.c_float]
        _lib.ofq_ref_float_to_bf16.restype = ctypes.c_uint16
        _lib.ofq_ref_float_to_bf16.argtypes = [ctypes.c_float]
        _lib.ofq_ref_bf16_to_float.restype = ctypes.c_float
        _lib.ofq_ref_bf16_to_float.argtypes = [ctypes.c_uint16]
    return _lib


def _p(a):
    return None if a is None else ctypes.c_void_p(a.ctypes.data)


def _i64(v):
    return ctypes.c_int64(int(v))


def _c(a, dtype=None):
    if a is None:
        return None
    return np.ascontiguousarray(a, dtype=dtype)


def t_code(arr_or_name):
    """Map a numpy array / name to the oracle's T code.  uint16 means bf16 bits."""
    if isinstance(arr_or_name, str):
        return {"f32": F32, "f16": F16, "bf16": BF16}[arr_or_name]
    dt = arr_or_name.dtype
    if dt == np.float32:
        return F32
    if dt == np.float16:
        return F16
    if dt == np.uint16:
        return BF16
    raise TypeError(f"unsupported T dtype {dt}")


def f32_to_bf16_bits(a):
    """Round fp32 to bf16 (nearest even, NaN -> 0x7FC0); returns uint16 bit patterns."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32)
    bias = ((u >> 16) & 1) + np.uint32(0x7FFF)
    out = ((u + bias) >> 16).astype(np.uint16)
    out[np.isnan(a)] = 0x7FC0
    return out


def bf16_bits_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def to_f32(a):
    """Widen an fp16 / bf16-bits / fp32 array to fp32."""
    if a.dtype == np.uint16:
        return bf16_bits_to_f32(a)
    return a.astype(np.float32)


def min_max_observer(x, quantization_formula="google", quantization_bit=8,
                     quantization_scheme="symmetric", per_layer_quantization=True):
    x = _c(x)
    assert x.dtype in (np.float32, np.float64)
    outer = 1 if per_layer_quantization else x.shape[0]
    scale = np.empty(outer, dtype=x.dtype)
    zp = np.empty(outer, dtype=x.dtype)
    fn = lib().ofq_ref_min_max_observer_f32 if x.dtype == np.float32 else lib().ofq_ref_min_max_observer_f64
    rc = fn(_p(x), _i64(x.size), _i64(outer), int(quantization_bit), _SCHEME[quantization_scheme],
            _FORMULA[quantization_formula], _p(scale), _p(zp))
    if rc != 0:
        raise ValueError("oracle min_max_observer rejected the arguments")
    return scale, zp


def moving_average_min_max_observer(x, current_train_step, moving_max, moving_min, training,
                                    stop_update_after_iters, quantization_formula="google",
                                    quantization_bit=8, quantization_scheme="symmetric",
                                    momentum=0.95):
    """moving_max / moving_min: arrays of one element, updated IN PLACE.  Returns (scale, zp)."""
    x = _c(x)
    assert x.dtype in (np.float32, np.float64)
    assert moving_max.dtype == x.dtype and moving_min.dtype == x.dtype
    scale = np.empty(1, dtype=x.dtype)
    zp = np.empty(1, dtype=x.dtype)
    fn = (lib().ofq_ref_moving_average_min_max_observer_f32 if x.dtype == np.float32
          else lib().ofq_ref_moving_average_min_max_observer_f64)
    rc = fn(_p(x), _i64(x.size), _i64(int(current_train_step)), _i64(int(stop_update_after_iters)),
            int(bool(training)), int(quantization_bit), _SCHEME[quantization_scheme],
            _FORMULA[quantization_formula], ctypes.c_float(momentum), _p(moving_max),
            _p(moving_min), _p(scale), _p(zp))
    if rc != 0:
        raise ValueError("oracle moving_average_min_max_observer rejected the arguments")
    return scale, zp


def _quant(x, scale, zero_point, formula, bit, scheme, zp_mode, fake):
    x = _c(x)
    assert x.dtype in (np.float32, np.float64)
    scale = _c(scale, x.dtype)
    zero_point = _c(zero_point, x.dtype)
    out = np.empty_like(x)
    fn = lib().ofq_ref_quantization_f32 if x.dtype == np.float32 else lib().ofq_ref_quantization_f64
    rc = fn(_p(x), _p(scale), _p(zero_point), _p(out), _i64(x.size), _i64(scale.size),
            _i64(x.shape[0] if x.ndim else 1), int(bit), _SCHEME[scheme], _FORMULA[formula],
            {"cpu": 0, "cuda": 1}[zp_mode], int(fake))
    if rc != 0:
        raise ValueError("oracle quantization rejected the arguments")
    return out


def quantization(x, scale, zero_point, quantization_formula="google", quantization_bit=8,
                 quantization_scheme="symmetric", zp_mode="cpu"):
    return _quant(x, scale, zero_point, quantization_formula, quantization_bit,
                  quantization_scheme, zp_mode, 0)


def fake_quantization(x, scale, zero_point, quantization_formula="google", quantization_bit=8,
                      quantization_scheme="symmetric", zp_mode="cpu"):
    return _quant(x, scale, zero_point, quantization_formula, quantization_bit,
                  quantization_scheme, zp_mode, 1)


def groupwise_quantize(x, num_bits=8, symmetric=True, group_dim=1, group_size=-1, signed=True):
    """x: 2-D fp32 / fp16 / bf16-bits array.  Returns (codes, scale, zero-or-None)."""
    x = _c(x)
    n, k = x.shape
    dim = x.shape[group_dim]
    if group_size < 0:
        group_size = dim
    q = np.zeros((n, k * num_bits // 8), dtype=np.int8 if signed else np.uint8)
    sshape = (n // group_size, k) if group_dim == 0 else (n, k // group_size)
    scale = np.empty(sshape, dtype=x.dtype)
    zero = None if symmetric else np.empty(sshape, dtype=x.dtype)
    rc = lib().ofq_ref_groupwise_quantize(
        _p(x), _p(q), _p(scale), _p(zero), t_code(x), int(bool(signed)), int(num_bits),
        int(bool(symmetric)), int(group_dim), _i64(group_size), _i64(n), _i64(k))
    if rc != 0:
        raise ValueError("oracle groupwise_quantize rejected the arguments")
    return q, scale, zero


def groupwise_dequantize(q, scale, zero=None, num_bits=8, symmetric=True, group_dim=-1,
                         group_size=-1):
    """q: int8/uint8 of any rank, codes packed along the last axis.  Returns an array with the
    dtype of ``scale`` (np.float32 / np.float16 / np.uint16 holding bf16 bits)."""
    q = _c(q)
    scale = _c(scale)
    zero = _c(zero)
    nd = q.ndim
    if group_dim < 0:
        group_dim += nd
    out_shape = list(q.shape)
    out_shape[-1] *= 8 // num_bits
    if group_size < 0:
        group_size = out_shape[group_dim]
    num_groups = out_shape[group_dim] // group_size
    outer = int(np.prod(out_shape[:group_dim], dtype=np.int64)) * num_groups
    inner = int(np.prod(out_shape[group_dim + 1:], dtype=np.int64))
    out = np.empty(out_shape, dtype=scale.dtype)
    rc = lib().ofq_ref_groupwise_dequantize(
        _p(q), _p(scale), _p(zero), _p(out), int(q.dtype == np.int8), t_code(scale), int(num_bits),
        int(bool(symmetric)), _i64(outer), _i64(group_size), _i64(inner))
    if rc != 0:
        raise ValueError("oracle groupwise_dequantize rejected the arguments")
    return out


def fused_linear(x, w, w_scale, w_zero=None, b=None, num_bits=8, symmetric=True, group_dim=-1,
                 group_size=-1, acc="f32"):
    x = _c(x)
    w = _c(w)
    w_scale = _c(w_scale)
    w_zero = _c(w_zero)
    b = _c(b)
    k = x.shape[-1]
    m = x.size // k
    n = w.shape[0]
    if group_dim < 0:
        group_dim += 2
    if group_size < 0:
        group_size = n if group_dim == 0 else k
    out = np.empty(x.shape[:-1] + (n,), dtype=x.dtype)
    rc = lib().ofq_ref_fused_linear(
        _p(x), _p(w), _p(w_scale), _p(w_zero), _p(b), _p(out), int(w.dtype == np.int8), t_code(x),
        int(num_bits), int(bool(symmetric)), int(group_dim), _i64(group_size), _i64(m), _i64(n),
        _i64(k), {"f32": 0, "f64": 1}[acc])
    if rc != 0:
        raise ValueError("oracle fused_linear rejected the arguments")
    return out


def layer_norm_min_max_observer(x, gamma, beta, eps=1e-5, quantization_bit=8):
    x = _c(x)
    gamma = _c(gamma)
    beta = _c(beta)
    cols = x.shape[-1]
    rows = x.size // cols
    y = np.empty_like(x)
    scale = np.empty(1, dtype=np.float32)
    zp = np.empty(1, dtype=np.float32)
    rc = lib().ofq_ref_layer_norm_min_max_observer(
        _p(x), _p(gamma), _p(beta), _p(y), _p(scale), _p(zp), _i64(rows), _i64(cols),
        ctypes.c_double(eps), t_code(x), int(quantization_bit))
    assert rc == 0
    return y, scale, zp


def skip_layer_norm_min_max_observer(x, gamma, beta, bias=None, skip=None, eps=1e-5, alpha=1e1,
                                     quantization_bit=8):
    """skip_layer_norm (skip_layer_norm_kernel.cu:36-67) followed by the per-tensor observer."""
    x = _c(x)
    gamma = _c(gamma)
    beta = _c(beta)
    bias = _c(bias)
    skip = _c(skip)
    cols = x.shape[-1]
    rows = x.size // cols
    y = np.empty_like(x)
    scale = np.empty(1, dtype=np.float32)
    zp = np.empty(1, dtype=np.float32)
    rc = lib().ofq_ref_skip_layer_norm_min_max_observer(
        _p(x), _p(bias), _p(skip), ctypes.c_double(alpha), _p(gamma), _p(beta), _p(y), _p(scale),
        _p(zp), _i64(rows), _i64(cols), ctypes.c_double(eps), t_code(x), int(quantization_bit))
    assert rc == 0
    return y, scale, zp


ACTIVATIONS = {"none": 0, "sigmoid": 1, "relu": 2, "gelu": 3, "fast_gelu": 4, "silu": 5}


def glu_gate(hidden, gate, activation="none"):
    """y = hidden * act(gate) in T (fused_glu_kernel.cu:303-347); 2-D arrays of equal shape."""
    hidden = _c(hidden)
    gate = _c(gate)
    m, n = hidden.shape
    y = np.empty_like(hidden)
    rc = lib().ofq_ref_glu_gate(_p(hidden), _p(gate), _p(y), _i64(m), _i64(n), _i64(n),
                                t_code(hidden), ACTIVATIONS[activation])
    assert rc == 0
    return y


def fused_glu(x, w, w_scale, w_zero=None, b=None, v=None, v_scale=None, v_zero=None, c=None,
              activation="none", num_bits=8, symmetric=True, group_dim=-1, group_size=-1):
    """fused_glu over groupwise-quantised weights: the op's two linears (rounded to T, as the
    reference stores matmul_wx / matmul_vx) and the gating.  Returns (y, matmul_wx, matmul_vx)."""
    wx = fused_linear(x, w, w_scale, w_zero, b, num_bits, symmetric, group_dim, group_size)
    wx2 = wx.reshape(-1, wx.shape[-1])
    if v is not None:
        vx = fused_linear(x, v, v_scale, v_zero, c, num_bits, symmetric, group_dim, group_size)
        y = glu_gate(wx2, vx.reshape(wx2.shape), activation)
        return y.reshape(wx.shape), wx, vx
    n = wx2.shape[1] // 2
    y = glu_gate(np.ascontiguousarray(wx2[:, :n]), np.ascontiguousarray(wx2[:, n:]), activation)
    return y.reshape(wx.shape[:-1] + (n,)), wx, None


def quantize_to_int8(x, scale, quantization_bit=8):
    x = _c(x)
    scale = _c(scale, np.float32)
    out = np.empty(x.shape, dtype=np.int8)
    rc = lib().ofq_ref_quantize_to_int8(_p(x), _p(scale), _p(out), _i64(x.size), _i64(scale.size),
                                        _i64(x.shape[0]), t_code(x), int(quantization_bit))
    assert rc == 0
    return out


def matmul_quant(a, b, a_scale, b_scale, bias=None, out_dtype=np.float16):
    """a[m,k] int8, b[n,k] int8, a_scale fp32[1], b_scale fp32[n]; ``out_dtype`` np.float16,
    np.float32 or np.uint16 (bf16 bits)."""
    a = _c(a, np.int8)
    b = _c(b, np.int8)
    a_scale = _c(a_scale, np.float32).reshape(-1)
    b_scale = _c(b_scale, np.float32)
    bias = _c(bias)
    m, k = a.shape
    n = b.shape[0]
    out = np.empty((m, n), dtype=out_dtype)
    rc = lib().ofq_ref_matmul_quant(_p(a), _p(b), _p(a_scale), _p(b_scale), _p(bias), _p(out),
                                    t_code(out), _i64(m), _i64(n), _i64(k))
    assert rc == 0
    return out
