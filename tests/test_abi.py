"""The C-ABI library: it loads without a GPU, exports every function include/ofq.h declares, the
Python prototypes cover them, and invalid arguments come back as status codes before anything is
launched (so these calls are safe on a machine without a GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ofq.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ofq_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from oneflow_amd import _lib
    return _lib.lib()


def test_header_symbols_are_exported_and_prototyped(lib):
    from oneflow_amd import _lib
    names = _declared_functions()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} declared in ofq.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes prototype"
    assert set(_lib.SIGNATURES) == set(names)
    assert lib.ofq_abi_version() == 1
    assert lib.ofq_status_string(0) == b"ok"
    assert b"unknown" in lib.ofq_status_string(99)


def test_stream_layer_symbols_are_exported(lib):
    """include/ofq_hip_shim.h: the device / stream / event calls behind ep::CudaStream."""
    text = open(os.path.join(ROOT, "include", "ofq_hip_shim.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(ofq_hip_[a-z0-9_]+)\s*\(", text)))
    assert len(names) == 16
    raw = ctypes.CDLL(lib._name)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in ofq_hip_shim.h but not exported"
    raw.ofq_hip_error_string.restype = ctypes.c_char_p
    assert raw.ofq_hip_error_string(0) == b"no error"


# a fake, suitably aligned, never dereferenced device address
P = ctypes.c_void_p(0x10000)
U = ctypes.c_void_p(0x10008)  # not 16-byte aligned
F32, F16, BF16, F64, I8, U8 = 0, 1, 2, 3, 4, 5
OK, NULLP, BAD_DTYPE, BAD_SHAPE, BAD_ATTR, UNSUPPORTED, WORKSPACE, MISALIGNED = 0, 1, 2, 3, 4, 5, 6, 7


def test_dequantize_argument_errors(lib):
    f = lib.ofq_groupwise_dequantize
    assert f(None, P, P, None, P, U8, F16, 3, 1, 4, 128, 1) == BAD_ATTR      # num_bits
    assert f(None, P, P, None, P, F16, F16, 8, 1, 4, 128, 1) == BAD_DTYPE    # codes dtype
    assert f(None, P, P, P, P, I8, F16, 8, 0, 4, 128, 1) == BAD_DTYPE        # asymmetric needs uint8
    assert f(None, P, P, None, P, U8, F64, 8, 1, 4, 128, 1) == BAD_DTYPE     # T
    assert f(None, P, P, None, P, U8, F16, 8, 1, 4, 0, 1) == BAD_SHAPE
    assert f(None, P, P, None, P, U8, F16, 4, 1, 4, 127, 1) == BAD_SHAPE     # odd last axis, 4-bit
    assert f(None, None, P, None, P, U8, F16, 8, 1, 4, 128, 1) == NULLP
    assert f(None, P, P, P, P, U8, F16, 8, 1, 4, 128, 1) == NULLP            # zero with symmetric
    assert f(None, P, P, None, P, U8, F16, 8, 0, 4, 128, 1) == NULLP         # no zero, asymmetric
    assert f(None, U, P, None, P, U8, F16, 8, 1, 4, 128, 1) == MISALIGNED
    assert f(None, None, None, None, None, U8, F16, 8, 1, 0, 128, 1) == OK   # empty tensor


def test_fused_linear_argument_errors(lib):
    f = lib.ofq_fused_linear_gq

    def call(x=P, w=P, s=P, z=None, b=None, o=P, wd=I8, td=F16, bits=4, sym=1, gd=1, gs=128, m=1,
             n=256, k=256):
        return f(None, x, w, s, z, b, o, wd, td, bits, sym, gd, gs, m, n, k, None, 0)
    assert call(bits=5) == BAD_ATTR
    assert call(gd=2) == BAD_ATTR
    assert call(wd=F16) == BAD_DTYPE
    assert call(sym=0, z=P, wd=I8) == BAD_DTYPE
    assert call(td=F64) == BAD_DTYPE
    assert call(k=0) == BAD_SHAPE
    assert call(bits=4, k=255) == BAD_SHAPE
    assert call(gs=0) == BAD_ATTR
    assert call(gs=96) == BAD_SHAPE               # not a divisor of k
    assert call(gs=512) == BAD_SHAPE              # larger than k
    assert call(m=1 << 20, k=1 << 12, n=16, gs=128) == UNSUPPORTED   # m*k beyond int32
    assert call(x=None) == NULLP
    assert call(z=P) == NULLP
    assert call(sym=0, wd=U8) == NULLP
    assert call(w=U) == MISALIGNED
    assert call(m=0) == OK
    assert lib.ofq_fused_linear_gq_workspace_bytes(I8, F16, 4, 1, 1, 128, 1, 4096, 4096) == 0
    # groups along N: no workspace up to 64 rows of x, the dequantised weight beyond
    assert lib.ofq_fused_linear_gq_workspace_bytes(I8, F16, 4, 1, 0, 128, 64, 4096, 4096) == 0
    # (32 tiles of 256 x 128 for m = 65: 8 K slices of fp32 partial sums behind the weight)
    assert lib.ofq_fused_linear_gq_workspace_bytes(I8, F16, 4, 1, 0, 128, 65, 4096, 4096) \
        == 4096 * 4096 * 2 + 8 * 65 * 4096 * 4
    assert lib.ofq_fused_linear_gq_workspace_bytes(I8, F16, 4, 1, 0, 128, 2048, 11008, 4096) == 11008 * 4096 * 2


def test_observer_and_quantization_argument_errors(lib):
    obs = lib.ofq_min_max_observer
    need = lib.ofq_min_max_observer_workspace_bytes(F32, 4096 * 4096, 4096)
    assert need == 4096 * 2 * 4
    assert lib.ofq_min_max_observer_workspace_bytes(F64, 1 << 20, 1) == (1 << 20) // 4096 * 2 * 8
    assert obs(None, P, P, P, F32, 1024, 4, 9, 0, 0, P, 1 << 20) == BAD_ATTR
    assert obs(None, P, P, P, F32, 1024, 4, 1, 0, 0, P, 1 << 20) == BAD_ATTR
    assert obs(None, P, P, P, F32, 1024, 4, 8, 2, 0, P, 1 << 20) == BAD_ATTR
    assert obs(None, P, P, P, F16, 1024, 4, 8, 0, 0, P, 1 << 20) == BAD_DTYPE
    assert obs(None, P, P, P, F32, 1023, 4, 8, 0, 0, P, 1 << 20) == BAD_SHAPE
    assert obs(None, P, P, P, F32, 1024, 4, 8, 0, 1, P, 1 << 20) == UNSUPPORTED  # cambricon per-channel
    assert obs(None, P, P, P, F32, 1024, 4, 8, 0, 0, None, 0) == WORKSPACE
    assert obs(None, P, P, P, F32, 1024, 4, 8, 0, 0, P, 8) == WORKSPACE
    q = lib.ofq_quantization
    assert q(None, P, P, P, P, F32, F32, 1024, 1, 8, 0, 0, 5) == BAD_ATTR        # zp_mode
    assert q(None, P, P, P, P, F32, F16, 1024, 1, 8, 0, 0, 0) == BAD_DTYPE       # out dtype
    assert q(None, P, P, P, P, F32, U8, 1024, 1, 8, 0, 0, 0) == BAD_DTYPE        # symmetric -> int8
    assert q(None, P, P, P, P, F32, I8, 1024, 1, 8, 1, 0, 0) == BAD_DTYPE        # affine -> uint8
    assert q(None, P, P, None, P, F32, F32, 1024, 1, 8, 1, 0, 0) == NULLP        # affine needs zp
    assert q(None, P, P, P, P, F32, F32, 1023, 4, 8, 0, 0, 0) == BAD_SHAPE
    assert q(None, P, P, P, P, F32, F32, 0, 1, 8, 0, 0, 0) == OK
    fq = lib.ofq_fake_quantization
    assert fq(None, P, P, P, P, I8, 1024, 1, 8, 0, 0, 0) == BAD_DTYPE


def test_layer_norm_and_matmul_quant_argument_errors(lib):
    ln = lib.ofq_fused_layer_norm_min_max_observer
    assert lib.ofq_fused_layer_norm_min_max_observer_workspace_bytes(F16, 2048, 4096) == 2048 * 4
    assert ln(None, P, P, P, P, P, P, F16, 8, 64, 1e-5, 1, P, 64) == BAD_ATTR
    assert ln(None, P, P, P, P, P, P, I8, 8, 64, 1e-5, 8, P, 64) == BAD_DTYPE
    assert ln(None, P, P, P, P, P, P, F16, 0, 64, 1e-5, 8, P, 64) == BAD_SHAPE
    assert ln(None, None, P, P, P, P, P, F16, 8, 64, 1e-5, 8, P, 64) == NULLP
    assert ln(None, P, P, P, P, P, P, F16, 8, 64, 1e-5, 8, P, 16) == WORKSPACE
    sl = lib.ofq_fused_skip_layer_norm_min_max_observer
    assert sl(None, P, P, P, 1.0, P, P, P, P, P, F16, 8, 64, 1e-5, 9, P, 64) == BAD_ATTR
    assert sl(None, P, None, None, 1.0, P, P, P, P, P, U8, 8, 64, 1e-5, 8, P, 64) == BAD_DTYPE
    assert sl(None, P, P, P, 1.0, P, P, None, P, P, F16, 8, 64, 1e-5, 8, P, 64) == NULLP
    assert sl(None, P, P, P, 1.0, P, P, P, P, P, F16, 8, 64, 1e-5, 8, None, 0) == WORKSPACE
    mq = lib.ofq_matmul_quant
    assert mq(None, P, P, P, P, None, P, I8, 16, 16, 128) == BAD_DTYPE
    assert mq(None, P, P, P, P, None, P, F16, 16, 16, 0) == BAD_SHAPE
    assert mq(None, P, P, P, P, None, P, F16, 16, 16, 100) == UNSUPPORTED
    assert mq(None, None, P, P, P, None, P, F16, 16, 16, 128) == NULLP
    assert mq(None, U, P, P, P, None, P, F16, 16, 16, 128) == MISALIGNED
    assert mq(None, P, P, P, P, None, P, F16, 0, 16, 128) == OK


def test_grouped_and_glu_argument_errors(lib):
    vp, i64 = ctypes.c_void_p, ctypes.c_int64
    one = (vp * 1)(P.value)
    n1 = (i64 * 1)(16)
    g = lib.ofq_grouped_linear_gq
    assert g(None, 0, None, None, None, None, None, None, None, None, None, I8, F16, 4, 1, 1, 128) == OK
    assert g(None, 65, one, one, one, None, None, one, n1, n1, n1, I8, F16, 4, 1, 1, 128) == BAD_SHAPE
    assert g(None, 1, None, one, one, None, None, one, n1, n1, n1, I8, F16, 4, 1, 1, 128) == NULLP
    assert g(None, 1, one, one, one, None, None, one, n1, n1, n1, F16, F16, 4, 1, 1, 128) == BAD_DTYPE
    assert g(None, 1, one, one, one, None, None, one, n1, n1, n1, U8, F16, 4, 0, 1, 128) == NULLP  # no zeros
    # one problem goes through the single op's checks: num_bits 3 is rejected there
    k128 = (i64 * 1)(128)
    assert g(None, 1, one, one, one, None, None, one, n1, n1, k128, I8, F16, 3, 1, 1, 128) == BAD_ATTR
    f = lib.ofq_fused_glu_gq
    N = None
    assert f(None, P, P, P, N, N, P, P, N, N, P, P, P, 6, I8, F16, 4, 1, 1, 128, 1, 16, 128) == BAD_ATTR
    assert f(None, P, P, P, N, N, P, P, N, N, P, P, P, 5, F16, F16, 4, 1, 1, 128, 1, 16, 128) == BAD_DTYPE
    assert f(None, P, P, P, N, N, P, P, N, N, P, P, P, 5, I8, F16, 4, 1, 1, 128, 0, 16, 128) == OK
    assert f(None, P, P, P, N, N, P, P, N, N, N, P, P, 5, I8, F16, 4, 1, 1, 128, 1, 16, 128) == NULLP  # y
    assert f(None, P, P, P, N, N, P, P, N, P, P, P, P, 5, I8, F16, 4, 1, 1, 128, 1, 16, 128) == NULLP  # c without b
    assert f(None, P, P, P, N, P, P, P, N, N, P, P, P, 5, I8, F16, 4, 1, 1, 128, 1, 16, 128) == NULLP  # b without c
    assert f(None, P, P, P, N, N, P, P, N, N, P, P, N, 5, I8, F16, 4, 1, 1, 128, 1, 16, 128) == NULLP  # matmul_vx
