"""groupwise_dequantize on the GPU against the CPU oracle: bit-exact (both sides perform the same
two roundings in T).  Shape list = the reference's own cases
(python/oneflow/test/modules/test_groupwise_quantization.py:184-206) plus the benchmark shape."""
import numpy as np
import pytest

import helpers as H
from oracle import ofq_oracle as O

pytestmark = pytest.mark.gpu

REFERENCE_CASES = [
    (8, (128, 256), 0, 128), (8, (64, 128, 256), 0, 64), (8, (64, 128, 256), 1, 128),
    (8, (64, 128, 256), 2, 256), (8, (63, 127, 255), 0, 63), (8, (63, 127, 255), 1, 127),
    (8, (63, 127, 255), 2, 255), (8, (128, 256), 1, 64), (8, (128, 256), 0, 32),
    (8, (64, 128, 256), 0, 16), (8, (64, 128, 256), 1, 32), (8, (64, 128, 256), 2, 64),
    (4, (128, 256), 1, 256), (4, (128, 256), 0, 128), (4, (64, 128, 256), 0, 64),
    (4, (64, 128, 256), 1, 128), (4, (64, 128, 256), 2, 256), (4, (128, 256), 1, 64),
    (4, (128, 256), 0, 32), (4, (64, 128, 256), 0, 16), (4, (64, 128, 256), 1, 32),
    (4, (64, 128, 256), 2, 64),
]
VARIANTS = [(True, np.int8), (True, np.uint8), (False, np.uint8)]


def _same_bits(got, ref):
    if got.dtype == np.float32:
        g, r = got.view(np.uint32), ref.view(np.uint32)
    else:
        g, r = got.view(np.uint16), ref.view(np.uint16)
    return np.array_equal(g, r)


@pytest.mark.parametrize("num_bits,shape,group_dim,group_size", REFERENCE_CASES)
@pytest.mark.parametrize("t", ["f16", "f32", "bf16"])
def test_dequantize_matches_oracle_bitwise(num_bits, shape, group_dim, group_size, t):
    import oneflow_amd as flow
    rng = np.random.Generator(np.random.PCG64(hash((num_bits, shape, group_dim, group_size)) % 2**32))
    x = rng.standard_normal(shape).astype(np.float32)
    for symmetric, qdt in VARIANTS:
        q, scale, zero = H.quantize_groupwise(x, num_bits, symmetric, group_dim, group_size, qdt, t)
        ref = O.groupwise_dequantize(q, scale, zero, num_bits, symmetric, group_dim, group_size)
        got = flow._C.groupwise_dequantize(H.to_torch(q), H.to_torch(scale), zero=H.to_torch(zero),
                                           num_bits=num_bits, symmetric=symmetric,
                                           group_dim=group_dim, group_size=group_size)
        got = H.to_numpy(got)
        assert got.shape == ref.shape
        assert _same_bits(got, ref), (symmetric, qdt, np.abs(O.to_f32(got) - O.to_f32(ref)).max())
        # and the reference test's own tolerance against the real-valued input
        if symmetric or True:
            assert np.allclose(O.to_f32(got), O.to_f32(ref), atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("t", ["f16", "bf16"])
def test_dequantize_benchmark_shape(t):
    """uint8 asymmetric [11008,4096], g=128 along K, scale ~U(1e-3,1e-2), zero ~U(100,156)."""
    import oneflow_amd as flow
    n, k, g = 11008, 4096, 128
    q = H.rng_for(2, 0).integers(0, 256, size=(n, k), dtype=np.uint8)
    scale = H.as_T(H.rng_for(2, 1).uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float32), t)
    zero = H.as_T(H.rng_for(2, 2).uniform(100, 156, size=(n, k // g)).astype(np.float32), t)
    ref = O.groupwise_dequantize(q, scale, zero, 8, False, 1, g)
    got = H.to_numpy(flow._C.groupwise_dequantize(H.to_torch(q), H.to_torch(scale),
                                                  zero=H.to_torch(zero), num_bits=8,
                                                  symmetric=False, group_dim=-1, group_size=g))
    assert _same_bits(got, ref)


def test_dequantize_identity_scale():
    """s = 1, z = 0 returns the codes themselves (closed form, no oracle involved)."""
    import oneflow_amd as flow
    import torch
    codes = np.arange(-128, 128, dtype=np.int8).reshape(2, 128)
    scale = np.ones((2, 1), dtype=np.float16)
    got = flow._C.groupwise_dequantize(H.to_torch(codes), H.to_torch(scale), num_bits=8,
                                       symmetric=True, group_dim=1, group_size=128)
    assert torch.equal(got.cpu().float(), torch.from_numpy(codes.astype(np.float32)))
    # int4: nibble order, both containers
    vals = np.tile(np.arange(-8, 8, dtype=np.int8), 4).reshape(1, 64)
    packed = H.pack_int4(vals)
    got = flow._C.groupwise_dequantize(H.to_torch(packed), H.to_torch(np.ones((1, 1), np.float16)),
                                       num_bits=4, symmetric=True, group_dim=1, group_size=64)
    assert torch.equal(got.cpu().float(), torch.from_numpy(vals.astype(np.float32)))
    uvals = np.tile(np.arange(0, 16, dtype=np.uint8), 4).reshape(1, 64)
    got = flow._C.groupwise_dequantize(H.to_torch(H.pack_int4(uvals)),
                                       H.to_torch(np.ones((1, 1), np.float16)),
                                       zero=H.to_torch(np.zeros((1, 1), np.float16)),
                                       num_bits=4, symmetric=False, group_dim=1, group_size=64)
    assert torch.equal(got.cpu().float(), torch.from_numpy(uvals.astype(np.float32)))
