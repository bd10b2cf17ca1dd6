"""groupwise_quantize (weight quantiser + int4 packer) on the GPU against the oracle: codes,
scales and zeros bit-exact; then the whole weight pipeline quantize -> dequantize / fused linear."""
import numpy as np
import pytest

import helpers as H
from oracle import ofq_oracle as O

pytestmark = pytest.mark.gpu


def _run(x, bits, symmetric, group_dim, group_size, signed):
    import torch
    import oneflow_amd as flow
    q, s, z = flow.quantize.groupwise_quantize(
        H.to_torch(x), num_bits=bits, symmetric=symmetric, group_dim=group_dim,
        group_size=group_size, quant_type=torch.int8 if signed else torch.uint8)
    return H.to_numpy(q), H.to_numpy(s), None if z is None else H.to_numpy(z)


VARIANTS = [(True, True), (True, False), (False, False)]


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("symmetric,signed", VARIANTS)
@pytest.mark.parametrize("t", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("n,k,group_dim,group_size", [
    (64, 256, 1, 128), (37, 512, 1, 64), (8, 64, 1, 8), (5, 1024, 1, 512),   # lane-group kernel
    (48, 96, 1, 48), (7, 126, 1, 6), (64, 128, 0, 16), (30, 50, 0, 10),      # strided kernel
    (128, 64, 0, 128), (3, 40, 1, 40),
    (33, 4096, 1, 4096), (20, 11008, 1, 11008), (9, 2048, 1, 1024), (70, 960, 1, 96),  # block per group
])
def test_bit_exact_against_the_oracle(bits, symmetric, signed, t, n, k, group_dim, group_size):
    rng = np.random.Generator(np.random.PCG64(n * 7 + k + bits + group_size))
    x = H.as_T((rng.standard_normal((n, k)) * rng.uniform(0.01, 3.0, size=(n, 1))).astype(np.float32), t)
    qr, sr, zr = O.groupwise_quantize(x, bits, symmetric, group_dim, group_size, signed)
    q, s, z = _run(x, bits, symmetric, group_dim, group_size, signed)
    assert np.array_equal(q.view(np.uint8), qr.view(np.uint8))
    assert np.array_equal(s.view(np.uint8), sr.view(np.uint8))
    if symmetric:
        assert z is None
    else:
        assert np.array_equal(O.to_f32(z), O.to_f32(zr))  # by value: the sign of a zero minimum is free


@pytest.mark.parametrize("bits,signed", [(4, True), (4, False), (8, True), (8, False)])
def test_symmetric_fp16_groups_of_arbitrary_bit_patterns(bits, signed):
    """Symmetric quantisation of fp16 weights divides by the group scale through a corrected
    multiplication with its reciprocal.  Groups of random fp16 bit patterns (every exponent,
    subnormals, both zeros, the largest values; infinities in a few groups, which keep the
    division) against the oracle's `x / scale`, bit for bit."""
    rng = np.random.default_rng(bits * 2 + signed)
    bits16 = rng.integers(0, 65536, size=(6000, 128)).astype(np.uint16)
    x = bits16.view(np.float16)
    x[np.isnan(x)] = np.float16(0.0)
    keep_inf = np.zeros(x.shape[0], bool)
    keep_inf[:5] = True
    x[np.isinf(x) & ~keep_inf[:, None]] = np.float16(65504.0)
    # narrow the spread inside most groups so that the codes are not all 0 or the extremes
    for r in range(100, x.shape[0]):
        e = int(rng.integers(1, 28))
        x[r] = (x[r].view(np.uint16) & np.uint16(0x83FF) | np.uint16(e << 10)).view(np.float16)
    x[5] = np.float16(0.0)
    x[6, :4] = np.array([6e-8, -6e-8, 1.2e-7, 0.0], np.float16)
    qr, sr, _ = O.groupwise_quantize(x, bits, True, 1, 128, signed)
    q, s, _ = _run(x, bits, True, 1, 128, signed)
    rows = ~keep_inf  # (a group with an infinite element has scale inf and codes from 0 * nan)
    assert np.array_equal(q.view(np.uint8)[rows], qr.view(np.uint8)[rows])
    assert np.array_equal(s.view(np.uint16)[rows], sr.view(np.uint16)[rows])


def test_constant_and_zero_groups_and_ties():
    """scale 0 groups get the code of value 0; exact .5 quotients round to even."""
    x = np.zeros((4, 64), np.float32)
    x[1] = 3.5          # constant row: symmetric scale 3.5/7, every code 7
    x[2, :8] = np.array([7, 3.5, 2.5, 1.5, 0.5, -0.5, -1.5, -2.5], np.float32)  # scale 1
    for signed in (True, False):
        q, s, _ = _run(x, 4, True, 1, 64, signed)
        qr, sr, _ = O.groupwise_quantize(x, 4, True, 1, 64, signed)
        assert np.array_equal(q.view(np.uint8), qr.view(np.uint8)) and np.array_equal(s, sr)
        c = H.unpack_int4(q).astype(np.int64) - (0 if signed else 7)
        assert np.all(c[0] == 0) and np.all(c[1] == 7)
        # the offset is added BEFORE rounding (test_groupwise_quantization.py:58-62), so ties
        # fall differently in the two containers
        expect = [7, 4, 2, 2, 0, 0, -2, -2] if signed else [7, 3, 3, 1, 1, -1, -1, -3]
        assert list(c[2, :8]) == expect
    q, s, z = _run(x, 8, False, 1, 64, False)
    assert np.all(q[0] == 0) and np.all(s[0] == 0) and np.all(q[1] == 0) and np.all(z[1] == 3.5)


@pytest.mark.parametrize("bits,symmetric,signed", [(4, True, True), (4, False, False), (8, True, False)])
def test_weight_pipeline_llama_shape(bits, symmetric, signed):
    """fp16 weight [4096,4096] -> quantize (GPU) -> dequantize (GPU) is within half a step of the
    weight, equals the oracle's dequantisation of the oracle's codes bit for bit, and the fused
    linear on the GPU-made codes meets the linear contract against the oracle composition."""
    import torch
    import oneflow_amd as flow
    rng = np.random.Generator(np.random.PCG64(bits))
    n, k, g = 4096, 4096, 128
    wf = H.as_T((rng.standard_normal((n, k)) * 0.02).astype(np.float32), "f16")
    qt, st, zt = flow.quantize.groupwise_quantize(
        H.to_torch(wf), num_bits=bits, symmetric=symmetric, group_dim=1, group_size=g,
        quant_type=torch.int8 if signed else torch.uint8)
    deq = flow._C.groupwise_dequantize(qt, st, zero=zt, num_bits=bits, symmetric=symmetric,
                                       group_dim=1, group_size=g)
    q, s = H.to_numpy(qt), H.to_numpy(st)
    z = None if zt is None else H.to_numpy(zt)
    rows = np.arange(0, n, 97)
    qr, sr, zr = O.groupwise_quantize(wf[rows], bits, symmetric, 1, g, signed)
    assert np.array_equal(q[rows].view(np.uint8), qr.view(np.uint8)) and np.array_equal(s[rows], sr)
    ref_deq = O.groupwise_dequantize(qr, sr, zr, bits, symmetric, 1, g)
    assert np.array_equal(H.to_numpy(deq)[rows].view(np.uint16), ref_deq.view(np.uint16))
    step = np.repeat(s.astype(np.float32), g, axis=1)
    err = np.abs(H.to_numpy(deq).astype(np.float32) - wf.astype(np.float32))
    # half a step plus the fp16 roundings of scale, zero, product and sum (values are < 0.15,
    # where one fp16 ulp is at most 1.2e-4)
    assert np.all(err <= 0.5 * step + 4e-4)
    x = H.as_T(rng.standard_normal((2, k)).astype(np.float32), "f16")
    out = flow._C.fused_linear_with_groupwise_quantized_weight(
        H.to_torch(x), qt, st, w_zero=zt, num_bits=bits, symmetric=symmetric, group_dim=1,
        group_size=g)
    cols = np.arange(0, n, 53)
    ref = O.fused_linear(x, q[cols], s[cols], None if z is None else z[cols], None, bits,
                         symmetric, 1, g)
    H.assert_linear_parity(H.to_numpy(out)[:, cols], ref, "f16", "pipeline")


@pytest.mark.parametrize("num_bits,symmetric", [(4, True), (8, False)])
@pytest.mark.parametrize("dtype_name", ["float16", "bfloat16"])
def test_quantized_linear_module(num_bits, symmetric, dtype_name):
    """QuantizedLinear.from_float against the float layer (within the quantisation error of the
    weights), 3-D inputs, decode and prefill batch sizes, and a state_dict round trip."""
    import torch
    import oneflow_amd as flow
    dtype = getattr(torch, dtype_name)
    torch.manual_seed(3)
    lin = torch.nn.Linear(1024, 768, bias=True, device="cuda", dtype=dtype)
    qt = torch.int8 if symmetric else torch.uint8
    ql = flow.nn.QuantizedLinear.from_float(lin, num_bits=num_bits, symmetric=symmetric,
                                            group_size=128, quant_type=qt)
    wd = flow._C.groupwise_dequantize(ql.weight, ql.weight_scale, zero=ql.weight_zero,
                                      num_bits=num_bits, symmetric=symmetric, group_dim=1,
                                      group_size=128)
    for shape in ((1, 1024), (2, 3, 1024), (150, 1024)):
        x = torch.randn(shape, device="cuda", dtype=dtype)
        y = ql(x)
        assert y.shape == shape[:-1] + (768,) and y.dtype == dtype
        ref = torch.nn.functional.linear(x.float(), wd.float(), lin.bias.float())
        err = (y.float() - ref).norm() / ref.norm()
        assert err < (3e-3 if dtype == torch.float16 else 1e-2), float(err)
        full = torch.nn.functional.linear(x.float(), lin.weight.float(), lin.bias.float())
        assert (y.float() - full).norm() / full.norm() < (0.2 if num_bits == 4 else 0.02)
    clone = flow.nn.QuantizedLinear(1024, 768, True, num_bits, symmetric, 128, qt, dtype, "cuda")
    clone.load_state_dict(ql.state_dict())
    x = torch.randn((4, 1024), device="cuda", dtype=dtype)
    assert torch.equal(clone(x), ql(x))
