"""fused_linear_with_groupwise_quantized_weight on the GPU against the oracle composition
(dequantize in T -> matmul with fp32 accumulation -> + bias -> round to T).
Tolerance (stated contract): rel-L2 <= 1e-3 and max-abs <= 2e-2 (see helpers.assert_linear_parity
for how the absolute bound is read when one ulp of T is larger than 2e-2)."""
import numpy as np
import pytest

import helpers as H
from oracle import ofq_oracle as O

pytestmark = pytest.mark.gpu

# (num_bits, m, k, n, group_dim, group_size): test_groupwise_quantization.py:209-220
REFERENCE_CASES = [
    (8, 1, 64, 128, 0, 128), (8, 1, 64, 128, 1, 64), (8, 16, 64, 128, 0, 128),
    (8, 16, 64, 128, 1, 64), (8, 1, 63, 127, 0, 127), (8, 1, 63, 127, 1, 63),
    (8, 1, 256, 512, 0, 64), (8, 1, 256, 512, 1, 64), (4, 1, 256, 512, 0, 512),
    (4, 1, 256, 512, 1, 256), (4, 1, 256, 512, 0, 64), (4, 1, 256, 512, 1, 64),
]
VARIANTS = [(True, np.int8), (True, np.uint8), (False, np.uint8)]


def _run(x, w, scale, zero, b, num_bits, symmetric, group_dim, group_size):
    import oneflow_amd as flow
    out = flow._C.fused_linear_with_groupwise_quantized_weight(
        H.to_torch(x), H.to_torch(w), H.to_torch(scale), w_zero=H.to_torch(zero), b=H.to_torch(b),
        num_bits=num_bits, symmetric=symmetric, group_dim=group_dim, group_size=group_size)
    return H.to_numpy(out)


@pytest.mark.parametrize("num_bits,m,k,n,group_dim,group_size", REFERENCE_CASES)
@pytest.mark.parametrize("t", ["f16", "f32", "bf16"])
def test_reference_cases(num_bits, m, k, n, group_dim, group_size, t):
    rng = np.random.Generator(np.random.PCG64(hash((num_bits, m, k, n, group_dim, group_size)) % 2**32))
    x = H.as_T(rng.standard_normal((m, k)).astype(np.float32) / 10, t)
    wf = rng.standard_normal((n, k)).astype(np.float32) / 10
    b = H.as_T(rng.standard_normal(n).astype(np.float32) / 10, t)
    for symmetric, qdt in VARIANTS:
        w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, group_dim, group_size, qdt, t)
        ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, group_dim, group_size)
        got = _run(x, w, scale, zero, b, num_bits, symmetric, group_dim, group_size)
        H.assert_linear_parity(got, ref, t, f"{symmetric} {qdt}")
        # the reference test's own criterion
        assert np.allclose(O.to_f32(got), O.to_f32(ref), atol=1e-2, rtol=1e-2)


def _decode_inputs(m, n, k, container):
    x = H.as_T(H.rng_for(3, 0).standard_normal((m, k)).astype(np.float32), "f16")
    if container == np.int8:
        codes = H.rng_for(3, 1).integers(-7, 8, size=(n, k)).astype(np.int8)
    else:
        codes = H.rng_for(3, 1).integers(0, 15, size=(n, k)).astype(np.uint8)
    w = H.pack_int4(codes)
    scale = H.as_T(H.rng_for(3, 2).uniform(1e-3, 1e-2, size=(n, k // 128)).astype(np.float32), "f16")
    b = H.as_T((H.rng_for(3, 3).standard_normal(n) * 0.01).astype(np.float32), "f16")
    return x, w, scale, b


@pytest.mark.parametrize("n,k", [(4096, 4096), (11008, 4096), (4096, 11008)])
@pytest.mark.parametrize("m", [1, 4, 8])
@pytest.mark.parametrize("container", [np.int8, np.uint8])
def test_decode_w4a16_llama_shapes(m, n, k, container):
    """Symmetric int4, g=128 along K, fp16, Llama-7B q/o, gate/up and down shapes."""
    x, w, scale, b = _decode_inputs(m, n, k, container)
    ref = O.fused_linear(x, w, scale, None, b, 4, True, 1, 128)
    got = _run(x, w, scale, None, b, 4, True, 1, 128)
    r, e = H.assert_linear_parity(got, ref, "f16", f"m={m} n={n} k={k}")
    # int8 container: w~ = q*s is not rounded to fp16 inside the kernel (~3e-4 from the oracle);
    # uint8 container: w~ = T(T(u*s) + T(-7s)) carries three roundings of magnitude ~7s around a
    # small value, so it is formed exactly as the oracle does and only the sum order differs
    assert r < (5e-4 if container == np.int8 else 1e-4)


@pytest.mark.parametrize("n,k,g,with_bias", [
    (4096, 256, 128, True), (37, 512, 128, False), (4099, 2048, 256, True), (1000, 3072, 128, True),
    (513, 4096, 512, True), (300, 5120, 128, False), (2048, 8192, 1024, True), (129, 9216, 128, True),
    (64, 11008, 128, True), (77, 13824, 128, True), (50, 14336, 256, False), (33, 16384, 128, True),
    (128256, 256, 128, True),
])
def test_decode_m1_row_per_wave_shapes(n, k, g, with_bias):
    """m = 1, fp16, symmetric int4 in an int8 container: the kernel in which a wave owns whole
    rows.  Every row length class (1 .. 8 KB of codes per row, with a partial last KB), group
    sizes above 128, row counts off the block size, no bias."""
    rng = np.random.default_rng(n * 31 + k)
    x = H.as_T(rng.standard_normal((1, k)).astype(np.float32), "f16")
    codes = rng.integers(-8, 8, size=(n, k)).astype(np.int8)
    w = H.pack_int4(codes)
    scale = H.as_T(rng.uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float32), "f16")
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), "f16") if with_bias else None
    ref = O.fused_linear(x, w, scale, None, b, 4, True, 1, g)
    got = _run(x, w, scale, None, b, 4, True, 1, g)
    r, e = H.assert_linear_parity(got, ref, "f16", f"n={n} k={k} g={g}")
    assert r < 5e-4


@pytest.mark.parametrize("m,n,k,g,with_bias", [
    (2, 4096, 4096, 128, True), (3, 4099, 2048, 256, True), (4, 1000, 3072, 128, False),
    (5, 300, 5120, 128, True), (6, 2048, 8192, 1024, True), (7, 64, 11008, 128, True),
    (8, 4096, 4096, 128, True), (8, 129, 7936, 128, False), (4, 77, 13824, 128, True),
    (3, 33, 16384, 128, True), (2, 50, 14336, 256, False), (8, 20000, 256, 128, True),
    (8, 64, 11008, 128, True), (5, 64, 16384, 128, True), (4, 11008, 4096, 128, True),
    (2, 33000, 512, 128, False), (3, 20000, 1280, 256, True), (8, 11008, 4096, 128, True),
    (6, 1001, 3840, 128, True), (7, 4096, 2304, 256, False), (5, 6, 256, 128, True),
])
def test_decode_few_rows_of_x_long_and_ragged_rows(m, n, k, g, with_bias):
    """2 .. 8 rows of x, fp16, symmetric int4 in an int8 container: every row length up to 16384
    (with lengths that are not a multiple of 2048), group sizes above 128, row counts off the
    block sizes, and the shapes whose x does not fit LDS."""
    rng = np.random.default_rng(n * 31 + k + m)
    x = H.as_T(rng.standard_normal((m, k)).astype(np.float32), "f16")
    codes = rng.integers(-8, 8, size=(n, k)).astype(np.int8)
    w = H.pack_int4(codes)
    scale = H.as_T(rng.uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float32), "f16")
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), "f16") if with_bias else None
    ref = O.fused_linear(x, w, scale, None, b, 4, True, 1, g)
    got = _run(x, w, scale, None, b, 4, True, 1, g)
    r, e = H.assert_linear_parity(got, ref, "f16", f"m={m} n={n} k={k} g={g}")
    assert r < 5e-4


@pytest.mark.parametrize("x_std,s_lo,s_hi", [
    (1e-2, 1e-3, 1e-2), (1e-3, 1e-3, 1e-2), (1e-2, 1e-4, 1e-3), (1.0, 1e-4, 1e-3),
    (3e-3, 1e-4, 1e-3), (100.0, 1e-4, 2e-4), (30.0, 1e-4, 1e-3),
])
@pytest.mark.parametrize("m,group_dim,n,k,g", [
    (1, 1, 4096, 4096, 128), (1, 1, 1024, 11008, 128), (1, 1, 11008, 2048, 256),
    (1, 0, 4096, 4096, 128), (1, 0, 1024, 11008, 64), (1, 0, 512, 512, 16),
    (4, 1, 4096, 4096, 128), (8, 1, 1024, 11008, 128), (2, 1, 11008, 1024, 128),
    (16, 1, 300, 4096, 128), (4, 0, 1024, 4096, 128),
])
def test_decode_does_not_depend_on_the_magnitude_of_x_or_of_the_scales(x_std, s_lo, s_hi, m,
                                                                       group_dim, n, k, g):
    """The contract holds for any magnitude of x and of the scales the output type can carry
    (the reference's arithmetic does not depend on it): activations of 1e-3, scales of 1e-4,
    activations of hundreds (with scales that keep the outputs near 10, where the absolute bound
    of 2e-2 still is the tighter of the two).  fp16, symmetric int4 in an int8 container, both group directions;
    no bias, so that the bound is on the product itself.  A tenth of every row of x is another
    hundred times smaller, so that large and small values meet inside one group."""
    rng = np.random.default_rng(int(x_std * 1e6) + int(s_lo * 1e7) + m * 7 + group_dim + n + k)
    xf = rng.standard_normal((m, k)).astype(np.float32) * x_std
    xf[:, rng.random(k) < 0.1] *= 0.01
    x = H.as_T(xf, "f16")
    codes = rng.integers(-8, 8, size=(n, k)).astype(np.int8)
    w = H.pack_int4(codes)
    sshape = (n, k // g) if group_dim == 1 else (n // g, k)
    scale = H.as_T(rng.uniform(s_lo, s_hi, size=sshape).astype(np.float32), "f16")
    ref = O.fused_linear(x, w, scale, None, None, 4, True, group_dim, g)
    assert np.abs(O.to_f32(ref)).mean() > 6.2e-5, "outputs must be normal halves for the bound to mean something"
    got = _run(x, w, scale, None, None, 4, True, group_dim, g)
    r, e = H.assert_linear_parity(got, ref, "f16", f"x~{x_std} s~{s_lo} m={m} dim={group_dim} {n}x{k}")
    assert r < 5e-4


@pytest.mark.parametrize("m", [1, 8])
def test_same_weights_in_both_containers_differ_by_rounding_of_w_only(m):
    """The same symmetric 4-bit weights stored as int8 codes q and as uint8 codes q + 7: the int8
    fast path scales the exact group sum (q*scale never rounded to fp16), the uint8 path forms
    w~ = T(T(u*s) + T(-7s)) as groupwise_dequantize does.  Both are within the contract of the
    composition; between them the difference is the rounding of w~ alone, bounded here."""
    n, k = 4096, 4096
    x, w_i8, scale, b = _decode_inputs(m, n, k, np.int8)
    codes = H.unpack_int4(w_i8.view(np.uint8)).astype(np.int16)
    codes = np.where(codes > 7, codes - 16, codes)  # sign-extend the nibbles
    w_u8 = H.pack_int4((codes + 7).astype(np.uint8))
    got_i8 = _run(x, w_i8, scale, None, b, 4, True, 1, 128)
    got_u8 = _run(x, w_u8, scale, None, b, 4, True, 1, 128)
    ref_i8 = O.fused_linear(x, w_i8, scale, None, b, 4, True, 1, 128)
    ref_u8 = O.fused_linear(x, w_u8, scale, None, b, 4, True, 1, 128)
    H.assert_linear_parity(got_i8, ref_i8, "f16", "int8 container")
    H.assert_linear_parity(got_u8, ref_u8, "f16", "uint8 container")
    d = H.rel_l2(got_i8.astype(np.float32), got_u8.astype(np.float32))
    assert 0 < d < 1e-3, d


@pytest.mark.parametrize("m,n,k", [(1, 5000, 256), (3, 4099, 384), (16, 6000, 128), (2, 40000, 256),
                                   (5, 33000, 128), (8, 4112, 1024), (16, 688, 256), (12, 100, 128),
                                   (9, 2048, 128)])
@pytest.mark.parametrize("container", [np.int8, np.uint8])
def test_decode_w4a16_row_balanced_shapes(m, n, k, container):
    """n large enough that a block owns more than one 16-row tile, with row counts per block
    that are not multiples of 16, partial last blocks and more blocks than fit the chip at once."""
    rng = np.random.Generator(np.random.PCG64(n + m))
    x = H.as_T(rng.standard_normal((m, k)).astype(np.float32), "f16")
    if container == np.int8:
        codes = rng.integers(-8, 8, size=(n, k)).astype(np.int8)
        values = codes.astype(np.int64)
    else:  # offset codes: value = code - 7, all 16 code points used
        codes = rng.integers(0, 16, size=(n, k)).astype(np.uint8)
        values = codes.astype(np.int64) - 7
    w = H.pack_int4(codes)
    scale = H.as_T(rng.uniform(1e-3, 1e-2, size=(n, k // 128)).astype(np.float32), "f16")
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), "f16")
    ref = O.fused_linear(x, w, scale, None, b, 4, True, 1, 128)
    got = _run(x, w, scale, None, b, 4, True, 1, 128)
    r, e = H.assert_linear_parity(got, ref, "f16", f"m={m} n={n} k={k}")
    assert r < (5e-4 if container == np.int8 else 1e-4)
    # exact integer case through the same path: scales 1, small integer x
    xi = rng.integers(-2, 3, size=(m, k)).astype(np.float16)
    ones = np.ones((n, k // 128), dtype=np.float16)
    got = _run(xi, w, ones, None, None, 4, True, 1, 128)
    exact = xi.astype(np.int64) @ values.T
    assert np.abs(exact).max() < 2048
    assert np.array_equal(got.astype(np.int64), exact)


@pytest.mark.parametrize("m,n,k", [(16, 80, 8192), (8, 48, 11008), (13, 4096, 4096),
                                   (8, 100, 11136), (5, 300, 16512), (6, 4096, 11008),
                                   (16, 5000, 8192), (8, 11008, 11008), (7, 33, 22016),
                                   (16, 4096, 11008), (12, 300, 11136), (16, 11008, 11008),
                                   (16, 64, 16384), (9, 1000, 19200)])
@pytest.mark.parametrize("symmetric,qdt", VARIANTS)
def test_decode_w4a16_large_x(m, n, k, symmetric, qdt):
    """m * k too large for x to be staged in LDS at once, for all three code variants: x staged
    in two, three or four parts of a row's chunk pairs (an odd number of chunks, parts of unequal
    size, one and several tiles per block, two blocks per CU) or read from L2 per chunk."""
    rng = np.random.Generator(np.random.PCG64(m * 131 + n))
    x = H.as_T(rng.standard_normal((m, k)).astype(np.float32), "f16")
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    w, scale, zero = H.quantize_groupwise(wf, 4, symmetric, 1, 128, qdt, "f16")
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), "f16")
    ref = O.fused_linear(x, w, scale, zero, b, 4, symmetric, 1, 128)
    got = _run(x, w, scale, zero, b, 4, symmetric, 1, 128)
    r, e = H.assert_linear_parity(got, ref, "f16", f"m={m} n={n} k={k}")
    assert r < (5e-4 if (symmetric and qdt == np.int8) else 1e-4)
    if symmetric and qdt == np.int8:
        # exact integer case through the same path (closed form, no oracle): scales 1, sparse
        # small-integer x, every sum an integer below 2048
        nn = min(n, 700)
        xi = rng.integers(-2, 3, size=(m, k)).astype(np.float16)
        xi[rng.random((m, k)) < 0.9] = 0
        codes = rng.integers(-8, 8, size=(nn, k)).astype(np.int8)
        ones = np.ones((nn, k // 128), dtype=np.float16)
        exact = xi.astype(np.int64) @ codes.astype(np.int64).T
        assert np.abs(exact).max() < 2048
        got = _run(xi, H.pack_int4(codes), ones, None, None, 4, True, 1, 128)
        assert np.array_equal(got.astype(np.int64), exact)


@pytest.mark.parametrize("m,n,k,group_size", [
    (1, 4096, 4096, 128), (4, 11008, 4096, 64), (16, 5000, 512, 32), (3, 4099, 384, 64),
    (2, 40000, 256, 128), (16, 16400, 1024, 128), (5, 4096, 11008, 128), (7, 100, 128, 16)])
@pytest.mark.parametrize("num_bits", [4, 8])
@pytest.mark.parametrize("t", ["bf16", "f16"])
def test_decode_natural_order_kernel(m, n, k, group_size, num_bits, t):
    """Decode (m <= 16) for bf16 and for 8-bit codes, fp16 with groups shorter than 128, all three
    code variants: row counts per block that are not multiples of 16, partial last blocks, two
    blocks per CU, more outputs per block than threads, groups as short as one lane's load."""
    if num_bits == 4 and group_size % 32 != 0:
        group_size = 32
    rng = np.random.Generator(np.random.PCG64(m * 977 + n + num_bits))
    x = H.as_T(rng.standard_normal((m, k)).astype(np.float32), t)
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), t)
    for symmetric, qdt in VARIANTS:
        w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 1, group_size, qdt, t)
        ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 1, group_size)
        got = _run(x, w, scale, zero, b, num_bits, symmetric, 1, group_size)
        r, e = H.assert_linear_parity(got, ref, t, f"{t} b{num_bits} m={m} n={n} k={k} {symmetric} {qdt}")
        # w~ is formed with the oracle's roundings, only the order of the sum differs: the
        # outputs agree to a rounding of T on a few elements
        # (fp16, int8 container, 4 bits, groups of 128 take the kernel that leaves w~ = q*s
        # unrounded: ~3e-4)
        shortcut = t == "f16" and num_bits == 4 and qdt == np.int8 and group_size % 128 == 0
        assert r < (3e-3 if t == "bf16" else 5e-4 if shortcut else 1e-4), (r, symmetric, qdt)
        # and no element is off by more than one rounding of T (2e-4 absolute where cancellation
        # leaves an output far smaller than its terms)
        gf, rf = O.to_f32(got).astype(np.float64), O.to_f32(ref).astype(np.float64)
        assert (np.abs(gf - rf) <= np.maximum(H.ulp_of(rf, t), 2e-4) * (1 + 1e-9)).all() or shortcut


@pytest.mark.parametrize("n,k,group_size", [
    (4096, 4096, 128), (11008, 4096, 128), (4096, 11008, 128), (5000, 256, 32), (4099, 1536, 64),
    (40000, 2048, 256), (300, 8192, 1024), (130, 5120, 64), (17, 14336, 128), (9000, 416, 32),
    (1, 64, 32)])
@pytest.mark.parametrize("num_bits", [4, 8])
@pytest.mark.parametrize("t", ["bf16", "f16"])
def test_decode_single_row_of_x_every_variant(n, k, group_size, num_bits, t):
    """m = 1 for both 16-bit types, both code widths and all three code variants: rows of 1 to
    8 KB of codes (and beyond, where another kernel takes over), rows that end inside a KB, one
    row per wave and many rows per wave, n not a multiple of the block's waves, groups from one
    lane's share of a row up to 1024."""
    rng = np.random.Generator(np.random.PCG64(n * 31 + k + num_bits))
    x = H.as_T(rng.standard_normal((1, k)).astype(np.float32), t)
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), t)
    for symmetric, qdt in VARIANTS:
        w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 1, group_size, qdt, t)
        ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 1, group_size)
        got = _run(x, w, scale, zero, b, num_bits, symmetric, 1, group_size)
        what = f"{t} b{num_bits} n={n} k={k} g={group_size} {symmetric} {qdt}"
        r, e = H.assert_linear_parity(got, ref, t, what)
        shortcut = t == "f16" and num_bits == 4 and qdt == np.int8 and group_size % 128 == 0
        # w~ formed with the oracle's roundings: what is left is the order of the fp32 sum, which
        # moves a few per cent of the outputs by one rounding of T (5e-4 relative in fp16)
        assert r < (3e-3 if t == "bf16" else 5e-4 if shortcut else 2e-4), (r, what)
        gf, rf = O.to_f32(got).astype(np.float64), O.to_f32(ref).astype(np.float64)
        assert (np.abs(gf - rf) <= np.maximum(H.ulp_of(rf, t), 2e-4) * (1 + 1e-9)).all() or shortcut
    # exact integer case through the same path (closed form, no oracle): scales 1, integer zero
    # points, x in {-1, 0, 1} with so few non-zeros that every sum is an integer T represents
    kk, nn = min(k, 2048), min(n, 600)
    gsz = min(group_size, kk)
    ones = H.as_T(np.ones((nn, kk // gsz), dtype=np.float32), t)
    for symmetric, qdt in VARIANTS:
        offset_127 = num_bits == 8 and symmetric and qdt == np.uint8  # w~ = code - 127
        nnz = {"f16": 16 if offset_127 else 128, "bf16": 2 if offset_127 else 16}[t]
        xi = np.zeros((1, kk), dtype=np.float32)
        pos = rng.choice(kk, size=min(nnz, kk), replace=False)
        xi[0, pos] = rng.choice([-1.0, 1.0], size=pos.size)
        zero, zp = None, 0
        if qdt == np.int8:
            codes = rng.integers(-8, 8, size=(nn, kk)).astype(np.int8)
            values = codes.astype(np.int64)
        else:
            codes = rng.integers(0, 16, size=(nn, kk)).astype(np.uint8)
            values = codes.astype(np.int64)
            if symmetric:
                values = values - ((1 << (num_bits - 1)) - 1)
            else:
                zp = rng.integers(-8, 1, size=(nn, kk // gsz))
                values = values + np.repeat(zp, gsz, axis=1)
                zero = H.as_T(zp.astype(np.float32), t)
        w = H.pack_int4(codes) if num_bits == 4 else codes
        exact = xi.astype(np.int64) @ values.T
        assert np.abs(exact).max() < (256 if t == "bf16" else 2048)
        got = _run(H.as_T(xi, t), w, ones, zero, None, num_bits, symmetric, 1, gsz)
        assert np.array_equal(O.to_f32(got).astype(np.int64), exact), (t, num_bits, symmetric, qdt)


def test_decode_m_invariance_and_integer_case():
    """Row i of an m=8 call agrees with the m=1 call on that row (the two batch sizes take
    different code paths: x staged in LDS or not, so agreement is to fp32-accumulation noise, at
    most one fp16 ulp of the larger neighbour), and with all scales 1 the op is an exact integer
    dot product (closed form, no oracle)."""
    x8, w, scale, b = _decode_inputs(8, 4096, 4096, np.int8)
    out8 = _run(x8, w, scale, None, b, 4, True, 1, 128)
    for i in (0, 5):
        out1 = _run(x8[i:i + 1], w, scale, None, b, 4, True, 1, 128)
        d = np.abs(out1[0].astype(np.float64) - out8[i].astype(np.float64))
        bound = np.maximum(H.ulp_of(out8[i].astype(np.float64), "f16") * 2.0001, 2.5e-4)
        assert (d <= bound).all(), float((d / bound).max())
        assert (d > 0).mean() < 0.3
    # integer case: x small integers, scale 1, |sum| < 2048 is exact in fp16
    rng = np.random.Generator(np.random.PCG64(7))
    k, n = 256, 64
    xi = rng.integers(-2, 3, size=(3, k)).astype(np.float16)
    codes = rng.integers(-7, 8, size=(n, k)).astype(np.int8)
    ones = np.ones((n, k // 128), dtype=np.float16)
    got = _run(xi, H.pack_int4(codes), ones, None, None, 4, True, 1, 128)
    exact = xi.astype(np.int64) @ codes.astype(np.int64).T
    assert np.array_equal(got.astype(np.int64), exact)


@pytest.mark.parametrize("t", ["bf16", "f16"])
def test_prefill_w8a16_sampled(t):
    """x [2048,4096], W uint8 asymmetric [11008,4096], g=64; the GPU computes the full output, the
    oracle a sample of rows and columns (the scalar composition on the full shape takes minutes)."""
    m, n, k, g = 2048, 11008, 4096, 64
    x = H.as_T(H.rng_for(4, 0).standard_normal((m, k)).astype(np.float32), t)
    w = H.rng_for(4, 1).integers(0, 256, size=(n, k), dtype=np.uint8)
    scale = H.as_T(H.rng_for(4, 2).uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float32), t)
    zero = H.as_T(H.rng_for(4, 3).uniform(120, 136, size=(n, k // g)).astype(np.float32), t)
    got = _run(x, w, scale, zero, None, 8, False, 1, g)
    assert got.shape == (m, n)
    rows = np.array([0, 1, 127, 128, 255, 256, 1000, 1023, 1024, 2047])
    cols = np.concatenate([np.arange(0, 40), np.arange(5000, 5040), np.arange(n - 40, n)])
    ref = O.fused_linear(x[rows], w[cols], scale[cols], zero[cols], None, 8, False, 1, g)
    H.assert_linear_parity(got[np.ix_(rows, cols)], ref, t, f"prefill {t}")
    # linearity in x: doubling x doubles every output exactly (power-of-two scaling is exact)
    x2 = H.as_T(O.to_f32(x) * 2.0, t)
    got2 = _run(x2, w, scale, zero, None, 8, False, 1, g)
    assert np.array_equal(O.to_f32(got2), O.to_f32(got) * 2.0)


def _composition_on_all_cores(x, w, scale, zero, g, t):
    """The dequantize -> matmul composition at full size as torch CPU tensor operations on every
    host core: w~ = T(T(q) * s) + z with one rounding per operation (a bf16 / fp16 tensor product
    or sum rounds once, from the exact fp32 value), then an fp32 matmul, rounded to T."""
    import torch
    td = {"bf16": torch.bfloat16, "f16": torch.float16}[t]
    n, k = w.shape
    q = torch.from_numpy(w.astype(np.float32)).to(td).view(n, k // g, g)
    s = H.to_torch(scale, "cpu").view(n, k // g, 1)
    z = H.to_torch(zero, "cpu").view(n, k // g, 1)
    wt = ((q * s) + z).view(n, k).float()
    out = H.to_torch(x, "cpu").float() @ wt.t()
    return H.to_numpy(out.to(td))


@pytest.mark.parametrize("t", ["bf16", "f16"])
def test_prefill_w8a16_full_shape_every_output_both_paths(t):
    """Config 4 at full size (x [2048,4096], W uint8 asymmetric [11008,4096], g = 64) through the
    C ABI twice: with the op's tmp_buffer (weight dequantised once, copy-fed GEMM) and with
    workspace = NULL (weight tiles dequantised inside the GEMM).  EVERY output of both is held to
    the contract against the composition computed on all host cores, which is itself checked
    against the scalar oracle on sampled rows and columns; the two paths differ from each other
    by fp32 summation order only."""
    import torch
    from oneflow_amd import _lib
    L = _lib.lib()
    tcode = {"bf16": _lib.BF16, "f16": _lib.F16}[t]
    m, n, k, g = 2048, 11008, 4096, 64
    x = H.as_T(H.rng_for(4, 0).standard_normal((m, k)).astype(np.float32), t)
    w = H.rng_for(4, 1).integers(0, 256, size=(n, k), dtype=np.uint8)
    scale = H.as_T(H.rng_for(4, 2).uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float32), t)
    zero = H.as_T(H.rng_for(4, 3).uniform(120, 136, size=(n, k // g)).astype(np.float32), t)
    xt, wt, st, zt = map(H.to_torch, (x, w, scale, zero))
    need = L.ofq_fused_linear_gq_workspace_bytes(_lib.U8, tcode, 8, 0, 1, g, m, n, k)
    assert need == n * k * 2
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    outs = []
    for wptr, wbytes in ((ws.data_ptr(), need), (None, 0)):
        out = torch.empty((m, n), dtype=xt.dtype, device="cuda")
        rc = L.ofq_fused_linear_gq(torch.cuda.current_stream().cuda_stream, xt.data_ptr(),
                                   wt.data_ptr(), st.data_ptr(), zt.data_ptr(), None,
                                   out.data_ptr(), _lib.U8, tcode, 8, 0, 1, g, m, n, k, wptr, wbytes)
        assert rc == 0
        torch.cuda.synchronize()
        outs.append(H.to_numpy(out))
    full = _composition_on_all_cores(x, w, scale, zero, g, t)
    rows = np.array([0, 1, 127, 128, 255, 256, 1000, 1023, 1024, 2047])
    cols = np.concatenate([np.arange(0, 40), np.arange(5000, 5040), np.arange(n - 40, n)])
    ref = O.fused_linear(x[rows], w[cols], scale[cols], zero[cols], None, 8, False, 1, g)
    # the all-cores composition against the oracle: same w~, same fp32 products, only the order
    # of the fp32 sum differs (one ulp of T where the sum falls next to a rounding boundary)
    assert H.rel_l2(O.to_f32(full[np.ix_(rows, cols)]), O.to_f32(ref)) < 2e-4
    for name, got in (("tmp_buffer", outs[0]), ("workspace NULL", outs[1])):
        H.assert_linear_parity(got[np.ix_(rows, cols)], ref, t, f"prefill {t} {name} vs oracle")
        H.assert_linear_parity(got, full, t, f"prefill {t} {name}, all 22.5 M outputs")
    assert H.rel_l2(O.to_f32(outs[1]), O.to_f32(outs[0])) < 1e-3


@pytest.mark.parametrize("m", [17, 100, 130])
@pytest.mark.parametrize("num_bits,symmetric,qdt", [(4, True, np.int8), (4, False, np.uint8),
                                                    (8, True, np.uint8)])
def test_prefill_ragged_m_and_n(m, num_bits, symmetric, qdt):
    """m and n that are not multiples of the tile sizes."""
    rng = np.random.Generator(np.random.PCG64(m * 31 + num_bits))
    n, k, g = 200, 256, 64
    for t in ("f16", "bf16"):
        x = H.as_T(rng.standard_normal((m, k)).astype(np.float32) / 10, t)
        wf = rng.standard_normal((n, k)).astype(np.float32) / 10
        b = H.as_T(rng.standard_normal(n).astype(np.float32) / 10, t)
        w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 1, g, qdt, t)
        ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        got = _run(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        H.assert_linear_parity(got, ref, t, f"m={m} {t}")


def test_prefill_with_and_without_workspace():
    """Large m: with the workspace the weight is dequantised once and a copy-fed GEMM runs on it,
    without it the weight tiles are dequantised inside the GEMM.  Both must meet the contract, and
    they differ from each other only by fp32 summation order."""
    import torch
    from oneflow_amd import _lib
    L = _lib.lib()
    m, n, k, g = 1100, 1500, 512, 64
    rng = np.random.Generator(np.random.PCG64(77))
    for t, tcode in (("bf16", _lib.BF16), ("f16", _lib.F16)):
        x = H.as_T(rng.standard_normal((m, k)).astype(np.float32) / 4, t)
        w = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
        scale = H.as_T(rng.uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float32), t)
        zero = H.as_T(rng.uniform(-1.4, -1.1, size=(n, k // g)).astype(np.float32), t)
        b = H.as_T(rng.standard_normal(n).astype(np.float32) / 10, t)
        xt, wt, st, zt, bt = map(H.to_torch, (x, w, scale, zero, b))
        need = L.ofq_fused_linear_gq_workspace_bytes(_lib.U8, tcode, 8, 0, 1, g, m, n, k)
        assert need == n * k * 2
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        outs = []
        for wptr, wbytes in ((ws.data_ptr(), need), (None, 0), (ws.data_ptr(), need - 16)):
            out = torch.empty((m, n), dtype=xt.dtype, device="cuda")
            rc = L.ofq_fused_linear_gq(torch.cuda.current_stream().cuda_stream, xt.data_ptr(),
                                       wt.data_ptr(), st.data_ptr(), zt.data_ptr(), bt.data_ptr(),
                                       out.data_ptr(), _lib.U8, tcode, 8, 0, 1, g, m, n, k, wptr, wbytes)
            assert rc == 0
            outs.append(H.to_numpy(out))
        rows = np.array([0, 255, 256, 700, 1023, 1024, 1099])
        ref = O.fused_linear(x[rows], w, scale, zero, b, 8, False, 1, g)
        for got in outs:
            H.assert_linear_parity(got[rows], ref, t, f"workspace paths {t}")
        # a too-small workspace falls back to the in-tile path: identical to passing none
        assert np.array_equal(outs[1], outs[2])
        assert H.rel_l2(O.to_f32(outs[0]), O.to_f32(outs[1])) < 1e-3


@pytest.mark.parametrize("m,n,k,g", [(17, 300, 1024, 64), (32, 203, 1536, 128), (33, 4100, 512, 32),
                                     (64, 1000, 4096, 128), (48, 129, 256, 64), (50, 2049, 384, 64),
                                     (63, 700, 2048, 256)])
@pytest.mark.parametrize("num_bits", [4, 8])
@pytest.mark.parametrize("t", ["f16", "bf16"])
def test_small_batch_multi_tile_kernel(m, n, k, g, num_bits, t):
    """16 < m <= 64: the decode kernel's row split with 2 or 4 tiles of x per weight tile; needs
    no workspace.  Ragged m, n, partial last blocks and tiles."""
    from oneflow_amd import _lib
    L = _lib.lib()
    rng = np.random.Generator(np.random.PCG64(m * 13 + n + num_bits))
    x = H.as_T((rng.standard_normal((m, k)) / 4).astype(np.float32), t)
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), t)
    tcode = _lib.F16 if t == "f16" else _lib.BF16
    for symmetric, qdt in VARIANTS:
        wcode = _lib.I8 if qdt == np.int8 else _lib.U8
        assert L.ofq_fused_linear_gq_workspace_bytes(wcode, tcode, num_bits, int(symmetric), 1, g,
                                                     m, n, k) == 0
        w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 1, g, qdt, t)
        ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        got = _run(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        r, e = H.assert_linear_parity(got, ref, t, f"{t} b{num_bits} m={m} n={n} k={k} {symmetric} {qdt}")
        assert r < (3e-3 if t == "bf16" else 1e-4)


@pytest.mark.parametrize("m,n,k,g,symmetric,qdt", [
    (33, 11008, 4096, 128, True, np.int8), (64, 4096, 11008, 128, False, np.uint8),
    (17, 16400, 11008, 32, False, np.uint8)])
def test_small_batch_multi_tile_kernel_model_shapes(m, n, k, g, symmetric, qdt):
    """16 < m <= 64 on the shapes of a model: many chunks per wave (the x of a chunk goes through
    the wave's buffer in LDS while the next chunk's is in flight), three and four weight tiles
    per block; the last case leaves no room for the buffers beside the block's scales and zeros
    (64 rows x 344 groups) and takes x straight from L2."""
    rng = np.random.Generator(np.random.PCG64(m * 7 + n))
    x = H.as_T((rng.standard_normal((m, k)) / 4).astype(np.float32), "f16")
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), "f16")
    w, scale, zero = H.quantize_groupwise(wf, 4, symmetric, 1, g, qdt, "f16")
    ref = O.fused_linear(x, w, scale, zero, b, 4, symmetric, 1, g)
    got = _run(x, w, scale, zero, b, 4, symmetric, 1, g)
    r, e = H.assert_linear_parity(got, ref, "f16", f"m={m} n={n} k={k}")
    assert r < 1e-4


@pytest.mark.parametrize("m,n,k", [(65, 300, 1024), (128, 1000, 4096), (130, 520, 2048),
                                   (300, 384, 1024), (257, 203, 1536)])
@pytest.mark.parametrize("num_bits", [4, 8])
def test_midsize_m_split_k(m, n, k, num_bits):
    """64 < m < 1024 with few output tiles: given the workspace the op cuts K into slices that run
    as separate blocks and folds their fp32 partial sums; without it one block walks all of K.
    Both meet the contract and agree with each other up to summation order.  n not a multiple of
    4 takes the scalar fold."""
    import torch
    from oneflow_amd import _lib
    L = _lib.lib()
    g = 64
    rng = np.random.Generator(np.random.PCG64(m * 7 + n + num_bits))
    for t, tcode in (("bf16", _lib.BF16), ("f16", _lib.F16)):
        x = H.as_T(rng.standard_normal((m, k)).astype(np.float32) / 4, t)
        wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
        b = H.as_T(rng.standard_normal(n).astype(np.float32) / 10, t)
        for symmetric, qdt in VARIANTS:
            w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 1, g, qdt, t)
            wcode = _lib.I8 if qdt == np.int8 else _lib.U8
            need = L.ofq_fused_linear_gq_workspace_bytes(wcode, tcode, num_bits, int(symmetric), 1,
                                                         g, m, n, k)
            assert need > 0 and need % (m * n * 4) == 0 and need // (m * n * 4) >= 2, need
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            xt, wt, st, bt = map(H.to_torch, (x, w, scale, b))
            zt = H.to_torch(zero)
            outs = []
            for wptr, wbytes in ((ws.data_ptr(), need), (None, 0)):
                out = torch.empty((m, n), dtype=xt.dtype, device="cuda")
                rc = L.ofq_fused_linear_gq(torch.cuda.current_stream().cuda_stream, xt.data_ptr(),
                                           wt.data_ptr(), st.data_ptr(),
                                           zt.data_ptr() if zt is not None else None, bt.data_ptr(),
                                           out.data_ptr(), wcode, tcode, num_bits, int(symmetric), 1,
                                           g, m, n, k, wptr, wbytes)
                assert rc == 0
                outs.append(H.to_numpy(out))
            ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 1, g)
            for got in outs:
                H.assert_linear_parity(got, ref, t, f"m={m} n={n} k={k} {t} {symmetric} {qdt}")
            assert H.rel_l2(O.to_f32(outs[0]), O.to_f32(outs[1])) < 1e-3


def test_decode_random_shape_sweep():
    """Seeded sweep over the decode dispatch: m 1..16, ragged n, k from one chunk to many, group
    sizes from one lane's load to the whole row, both code widths, all containers, fp16 and bf16:
    every kernel variant and wave count the launchers can pick, each against the oracle."""
    rng = np.random.Generator(np.random.PCG64(20240229))
    n_cases = 0
    for _ in range(90):
        t = ("f16", "bf16")[int(rng.integers(0, 2))]
        num_bits = (4, 8)[int(rng.integers(0, 2))]
        m = int(rng.integers(1, 17))
        ck = 128 if num_bits == 4 else 64
        k = ck * int(rng.choice([1, 2, 3, 4, 8, 16, 32]))
        n = int(rng.choice([1, 15, 16, 17, 100, 688, 1000, 2049, 4100]))
        divisors = [g for g in (16, 32, 64, 128, 256, 512, k) if k % g == 0 and g % (ck // 4) == 0]
        g = int(rng.choice(divisors))
        symmetric, qdt = VARIANTS[int(rng.integers(0, 3))]
        x = H.as_T(rng.standard_normal((m, k)).astype(np.float32), t)
        wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
        b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), t) if rng.integers(0, 2) else None
        w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 1, g, qdt, t)
        ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        got = _run(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        H.assert_linear_parity(got, ref, t, f"{t} b{num_bits} m={m} n={n} k={k} g={g} {symmetric} {qdt}")
        n_cases += 1
    assert n_cases == 90


def test_prefill_random_shape_sweep():
    """The same for m > 16 (tile shapes, K slices with a workspace, ragged edges)."""
    rng = np.random.Generator(np.random.PCG64(777))
    for _ in range(40):
        t = ("f16", "bf16")[int(rng.integers(0, 2))]
        num_bits = (4, 8)[int(rng.integers(0, 2))]
        m = int(rng.choice([17, 31, 64, 129, 200, 257, 300]))
        k = 64 * int(rng.choice([1, 2, 3, 8, 16, 24, 40]))
        n = int(rng.choice([1, 31, 33, 127, 130, 353, 500]))
        lane_k = 32 if num_bits == 4 else 16
        divisors = [g for g in (16, 32, 64, 128, k) if k % g == 0 and g % lane_k == 0]
        g = int(rng.choice(divisors))
        symmetric, qdt = VARIANTS[int(rng.integers(0, 3))]
        x = H.as_T((rng.standard_normal((m, k)) / 4).astype(np.float32), t)
        wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
        b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), t) if rng.integers(0, 2) else None
        w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 1, g, qdt, t)
        ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        got = _run(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        H.assert_linear_parity(got, ref, t, f"{t} b{num_bits} m={m} n={n} k={k} g={g} {symmetric} {qdt}")


@pytest.mark.parametrize("m,n,k,g", [(1, 4096, 4096, 128), (7, 1000, 512, 64), (16, 4100, 256, 32),
                                     (17, 300, 1024, 16), (40, 129, 128, 128), (3, 20000, 128, 64)])
@pytest.mark.parametrize("num_bits", [4, 8])
def test_fp32_activations(m, n, k, g, num_bits):
    """T = float (registered by the reference next to half): the fp32 MFMA kernel, 16 rows of x
    per pass over the weights; fp32 products and sums, so only the summation order differs from
    the oracle."""
    if num_bits == 4 and g % 32 != 0:
        g = 32
    rng = np.random.Generator(np.random.PCG64(m * 3 + n + num_bits))
    x = rng.standard_normal((m, k)).astype(np.float32)
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    b = (rng.standard_normal(n) * 0.01).astype(np.float32)
    for symmetric, qdt in VARIANTS:
        w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 1, g, qdt, "f32")
        ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        got = _run(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        assert H.rel_l2(got, ref) < 2e-6, (symmetric, qdt)
        assert np.allclose(got, ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("t", ["bf16", "f16"])
@pytest.mark.parametrize("m,n", [(700, 11012), (1030, 8300), (1100, 4100), (4000, 4096)])
def test_prefill_192_wide_tiles(t, m, n):
    """m and n for which three or four 256-row tiles of x times the 128-wide weight tiles spill
    into a second, nearly empty round of blocks: the 192-wide tiles, in-tile (m < 1024) and
    copy-fed behind the dequantised weight (m >= 1024, with the workspace); and five row tiles on
    n = 4100, which the copy-fed path covers with 128 x 128 tiles on 8 waves, and 16 on n = 4096,
    which it covers with one round of 256-wide tiles; sampled rows."""
    import torch
    from oneflow_amd import _lib
    L = _lib.lib()
    k, g = 256, 64
    tcode = _lib.F16 if t == "f16" else _lib.BF16
    rng = np.random.Generator(np.random.PCG64(m + n))
    x = H.as_T((rng.standard_normal((m, k)) / 4).astype(np.float32), t)
    w = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
    scale = H.as_T(rng.uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float32), t)
    zero = H.as_T(rng.uniform(-1.4, -1.1, size=(n, k // g)).astype(np.float32), t)
    b = H.as_T(rng.standard_normal(n).astype(np.float32) / 10, t)
    xt, wt, st, zt, bt = map(H.to_torch, (x, w, scale, zero, b))
    need = L.ofq_fused_linear_gq_workspace_bytes(_lib.U8, tcode, 8, 0, 1, g, m, n, k)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    rows = np.unique(np.concatenate([np.arange(0, 3), np.arange(254, 258), np.arange(m - 3, m)]))
    ref = O.fused_linear(x[rows], w, scale, zero, b, 8, False, 1, g)
    for wptr, wbytes in ((ws.data_ptr(), need), (None, 0)):
        out = torch.empty((m, n), dtype=xt.dtype, device="cuda")
        rc = L.ofq_fused_linear_gq(torch.cuda.current_stream().cuda_stream, xt.data_ptr(),
                                   wt.data_ptr(), st.data_ptr(), zt.data_ptr(), bt.data_ptr(),
                                   out.data_ptr(), _lib.U8, tcode, 8, 0, 1, g, m, n, k, wptr, wbytes)
        assert rc == 0
        H.assert_linear_parity(H.to_numpy(out)[rows], ref, t, f"m={m} n={n} {t} ws={wbytes}")


@pytest.mark.parametrize("t", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("m", [1, 9, 20, 70])
@pytest.mark.parametrize("num_bits,k,g", [(4, 384, 96), (4, 768, 192), (8, 192, 48), (8, 576, 96)])
def test_group_sizes_that_are_not_powers_of_two(t, m, num_bits, k, g):
    """Group sizes that are multiples of a lane's load but not powers of two (the kernels' group
    index is then a division, not a shift), through every m regime."""
    n = 200
    rng = np.random.Generator(np.random.PCG64(m + k + g))
    x = H.as_T((rng.standard_normal((m, k)) / 2).astype(np.float32), t)
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), t)
    for symmetric, qdt in VARIANTS:
        w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 1, g, qdt, t)
        ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        got = _run(x, w, scale, zero, b, num_bits, symmetric, 1, g)
        if t == "f32":
            assert np.allclose(got, ref, rtol=1e-4, atol=1e-4)
        else:
            H.assert_linear_parity(got, ref, t, f"{t} b{num_bits} m={m} k={k} g={g} {symmetric} {qdt}")


@pytest.mark.parametrize("t", ["f16", "bf16"])
@pytest.mark.parametrize("m", [2, 16])
def test_decode_vocabulary_sized_n(t, m):
    """An output layer: n = 128256 rows (more 64-row blocks than the chip holds at once)."""
    n, k, g = 128256, 512, 128
    rng = np.random.Generator(np.random.PCG64(5))
    x = H.as_T(rng.standard_normal((m, k)).astype(np.float32), t)
    codes = rng.integers(-8, 8, size=(n, k)).astype(np.int8)
    w = H.pack_int4(codes)
    scale = H.as_T(rng.uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float32), t)
    ref = O.fused_linear(x, w, scale, None, None, 4, True, 1, g)
    got = _run(x, w, scale, None, None, 4, True, 1, g)
    H.assert_linear_parity(got, ref, t, f"{t} lm head")


@pytest.mark.parametrize("t", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("num_bits", [4, 8])
@pytest.mark.parametrize("m,n,k,g", [(1, 512, 256, 512), (1, 4096, 1024, 128), (8, 1000, 512, 200),
                                     (16, 688, 256, 16), (17, 96, 128, 48), (40, 2048, 384, 64),
                                     (64, 320, 256, 32), (3, 11008, 128, 128), (1, 11008, 4096, 128),
                                     (1, 1040, 11008, 16), (1, 4112, 5120, 2056), (40, 256, 11008, 128),
                                     (24, 4096, 1024, 128)])
def test_groups_along_n_streaming(t, num_bits, m, n, k, g):
    """group_dim = 0 (scale / zero [n / g, k], one value per k): the streaming kernel that applies
    a scale per element, through every container, 1, 2 and 4 tiles of x (x through the waves'
    LDS buffers beyond 16 rows; 40 rows of 11008 in two passes), groups from one 16-row
    tile to the whole weight, and n with a ragged last block; one row of x on fp16 / 4-bit /
    int8-container weights takes the kernel in which a wave owns whole rows and the scale meets x
    (rows of 128 bytes to 5.4 KB, groups of one block's rows and of many)."""
    if n % g != 0:
        pytest.skip("group_size has to divide n")
    rng = np.random.Generator(np.random.PCG64(m * 11 + n + k + num_bits))
    x = H.as_T((rng.standard_normal((m, k)) / 2).astype(np.float32), t)
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), t)
    for symmetric, qdt in VARIANTS:
        w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 0, g, qdt, t)
        assert scale.shape == (n // g, k)
        ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 0, g)
        got = _run(x, w, scale, zero, b, num_bits, symmetric, 0, g)
        if t == "f32":
            # (fp32 sums of 11008 terms in another order than the oracle's: 2e-6 at k = 11008)
            assert H.rel_l2(got, ref) < (2e-6 if k <= 4096 else 5e-6), (symmetric, qdt)
            assert np.allclose(got, ref, rtol=1e-4, atol=1e-4)
            continue
        r, _ = H.assert_linear_parity(got, ref, t, f"{t} b{num_bits} m={m} n={n} k={k} g={g} {symmetric} {qdt}")
        # one row of x, fp16, int4 in an int8 container: x * s is rounded once per k instead of
        # q * s per element (~3e-4 from the oracle, as for groups along K)
        shortcut = (t == "f16" and num_bits == 4 and m == 1 and qdt == np.int8 and k % 256 == 0
                    and g % 16 == 0)
        assert r < (3e-3 if t == "bf16" else 5e-4 if shortcut else 1e-4), r


def test_groups_along_n_single_row_exact_case():
    """Closed form for the kernel that applies the scale to x (one row of x, groups along N):
    power-of-two scales that differ per k and per group, small integer x and codes, so that every
    product and sum is exact in fp16 / fp32 and any slip in the pairing of x, scale and code
    positions changes the result."""
    rng = np.random.Generator(np.random.PCG64(99))
    n, k, g = 96, 2304, 32
    x = rng.integers(-2, 3, size=(1, k)).astype(np.float16)
    x[:, rng.random(k) < 0.5] = 0
    codes = rng.integers(-8, 8, size=(n, k)).astype(np.int8)
    scale = rng.choice([0.5, 1.0, 2.0], size=(n // g, k)).astype(np.float16)
    wt = codes.astype(np.float64) * np.repeat(scale.astype(np.float64), g, axis=0)
    exact = x.astype(np.float64) @ wt.T
    assert np.abs(exact).max() < 1024 and np.all(exact * 2 == np.round(exact * 2))
    got = _run(x, H.pack_int4(codes), scale, None, None, 4, True, 0, g)
    assert np.array_equal(got.astype(np.float64), exact)


@pytest.mark.parametrize("m,n,k,g", [(65, 256, 512, 64), (130, 1024, 256, 128), (200, 352, 1024, 16),
                                     (300, 4096, 512, 128)])
@pytest.mark.parametrize("num_bits", [4, 8])
def test_groups_along_n_large_m(m, n, k, g, num_bits):
    """group_dim = 0 beyond 64 rows of x: with the workspace the op asks for (n*k*sizeof(T)) the
    weight is dequantised once and the copy-fed GEMM runs on it; without it the streaming kernel
    takes x 64 rows at a time.  Both meet the contract and agree up to summation order."""
    import torch
    from oneflow_amd import _lib
    L = _lib.lib()
    rng = np.random.Generator(np.random.PCG64(m + n + k + num_bits))
    for t, tcode in (("bf16", _lib.BF16), ("f16", _lib.F16)):
        x = H.as_T(rng.standard_normal((m, k)).astype(np.float32) / 4, t)
        wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
        b = H.as_T(rng.standard_normal(n).astype(np.float32) / 10, t)
        for symmetric, qdt in VARIANTS:
            w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 0, g, qdt, t)
            wcode = _lib.I8 if qdt == np.int8 else _lib.U8
            need = L.ofq_fused_linear_gq_workspace_bytes(wcode, tcode, num_bits, int(symmetric), 0,
                                                         g, m, n, k)
            assert need >= n * k * 2, need   # + fp32 partial sums when K is cut into slices
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            xt, wt, st, bt = map(H.to_torch, (x, w, scale, b))
            zt = H.to_torch(zero)
            outs = []
            for wptr, wbytes in ((ws.data_ptr(), need), (None, 0)):
                out = torch.empty((m, n), dtype=xt.dtype, device="cuda")
                rc = L.ofq_fused_linear_gq(torch.cuda.current_stream().cuda_stream, xt.data_ptr(),
                                           wt.data_ptr(), st.data_ptr(),
                                           zt.data_ptr() if zt is not None else None, bt.data_ptr(),
                                           out.data_ptr(), wcode, tcode, num_bits, int(symmetric), 0,
                                           g, m, n, k, wptr, wbytes)
                assert rc == 0
                outs.append(H.to_numpy(out))
            ref = O.fused_linear(x, w, scale, zero, b, num_bits, symmetric, 0, g)
            for got in outs:
                H.assert_linear_parity(got, ref, t, f"m={m} n={n} k={k} {t} {symmetric} {qdt}")
            assert H.rel_l2(O.to_f32(outs[0]), O.to_f32(outs[1])) < 1e-3


def test_views_off_the_16_byte_grid():
    """Inputs that are views starting off a 16-byte boundary (the kernels use 128-bit accesses):
    the Python layer copies them; results equal those of the aligned tensors."""
    import torch
    import oneflow_amd as flow
    rng = np.random.Generator(np.random.PCG64(31))
    m, n, k, g = 3, 64, 256, 64
    x = H.as_T(rng.standard_normal((m, k)).astype(np.float32), "f16")
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    w, scale, _ = H.quantize_groupwise(wf, 8, True, 1, g, np.int8, "f16")
    b = H.as_T(rng.standard_normal(n).astype(np.float32), "f16")

    def shifted(a):
        t = H.to_torch(a)
        buf = torch.empty(t.numel() + 1, dtype=t.dtype, device="cuda")
        v = buf[1:].view(t.shape)
        v.copy_(t)
        assert v.data_ptr() % 16 != 0
        return v
    ref = _run(x, w, scale, None, b, 8, True, 1, g)
    got = flow._C.fused_linear_with_groupwise_quantized_weight(
        shifted(x), shifted(w), shifted(scale), b=shifted(b), num_bits=8, symmetric=True,
        group_dim=1, group_size=g)
    assert np.array_equal(H.to_numpy(got), ref)
    deq = flow._C.groupwise_dequantize(shifted(w), shifted(scale), num_bits=8, symmetric=True,
                                       group_dim=1, group_size=g)
    assert np.array_equal(H.to_numpy(deq), O.groupwise_dequantize(w, scale, None, 8, True, 1, g))
