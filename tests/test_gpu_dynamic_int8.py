"""Dynamic int8 activation path: fused_layer_norm_min_max_observer -> quantization (int8 codes)
-> matmul_quant.  These two ops are absent from the reference tree; the oracle composes them
from reference rules, so parity with the reference itself is unpinned (see oracle/ofq_oracle.c).
Bars used here: with `exact_statistics` (row statistics in fp64, rounded once, as the oracle takes
them) y bit-exact, scale identical and the int8 codes bit-exact against the oracle; with the
default fp32 statistics (the reference's precision, whose last bit depends on the order of
summation) y within 2 ulp of T of the oracle and codes bit-exact GIVEN the same y and scale;
int32 accumulation exact, scaled output bit-exact."""
import numpy as np
import pytest

import helpers as H
from oracle import ofq_oracle as O

pytestmark = pytest.mark.gpu


def _cfg5_inputs(rows=2048, cols=4096, t="f16"):
    x = H.as_T(H.rng_for(5, 0).standard_normal((rows, cols)).astype(np.float32), t)
    gamma = H.as_T((1 + 0.1 * H.rng_for(5, 1).standard_normal(cols)).astype(np.float32), t)
    beta = H.as_T((0.1 * H.rng_for(5, 2).standard_normal(cols)).astype(np.float32), t)
    return x, gamma, beta


@pytest.mark.parametrize("t,rows,cols", [("f16", 2048, 4096), ("bf16", 64, 4096), ("f32", 33, 1000),
                                         ("f16", 7, 8200), ("f16", 5, 24), ("f16", 12, 11008),
                                         ("f32", 6, 16384), ("bf16", 3, 16392)])
def test_layer_norm_observer(t, rows, cols):
    import oneflow_amd as flow
    x, gamma, beta = _cfg5_inputs(rows, cols, t)
    y_ref, s_ref, z_ref = O.layer_norm_min_max_observer(x, gamma, beta, 1e-5, 8)
    y, s, z = flow._C.fused_layer_norm_min_max_observer(H.to_torch(x), H.to_torch(gamma),
                                                        H.to_torch(beta), 1e-5, 8)
    y_np = H.to_numpy(y)
    yf, yr = O.to_f32(y_np).astype(np.float64), O.to_f32(y_ref).astype(np.float64)
    # A last-bit difference of mean/inv (fp32 vs fp64 statistics) can move the normalised value by
    # one ulp of T; the two roundings of the affine carry it on, and after a cancelling `+ beta`
    # it is measured against a smaller |y|.  Bound: 2 ulp of T at |y_ref| + |beta|; and almost
    # all elements are identical.
    if t == "f32":
        # nothing is rounded to a narrower T, so the fp32 statistics show directly
        assert np.allclose(yf, yr, rtol=4e-6, atol=4e-6)
    else:
        mag = np.abs(yr) + np.abs(O.to_f32(beta).astype(np.float64))[None, :]
        assert (np.abs(yf - yr) <= 2.0001 * H.ulp_of(mag, t)).all()
        assert (yf != yr).mean() < 0.02
    # scale is exactly absmax(y_gpu)/127 in fp32, zero_point 0
    expect = np.float32(np.abs(O.to_f32(y_np)).max()) / np.float32(127.0)
    assert H.to_numpy(s)[0] == expect and H.to_numpy(z)[0] == 0.0
    assert abs(float(H.to_numpy(s)[0]) - float(s_ref[0])) <= 2e-3 * float(s_ref[0])


@pytest.mark.parametrize("t,rows,cols", [("f16", 2048, 4096), ("bf16", 300, 4096), ("f32", 33, 1000),
                                         ("f16", 7, 8200), ("bf16", 5, 24), ("f32", 40, 2048),
                                         ("bf16", 9, 16384), ("f16", 4, 11008)])
@pytest.mark.parametrize("use_bias,use_skip", [(True, True), (False, True), (True, False)])
def test_skip_layer_norm_observer(t, rows, cols, use_bias, use_skip):
    """The residual input of skip_layer_norm in front of the same LayerNorm + observer: every
    kernel variant (one wave per row, one block per row, scalar any-length rows)."""
    import oneflow_amd as flow
    x, gamma, beta = _cfg5_inputs(rows, cols, t)
    bias = H.as_T((0.5 * H.rng_for(6, 0).standard_normal(cols)).astype(np.float32), t) if use_bias else None
    skip = H.as_T(H.rng_for(6, 1).standard_normal((rows, cols)).astype(np.float32), t) if use_skip else None
    alpha = 0.37
    y_ref, s_ref, z_ref = O.skip_layer_norm_min_max_observer(x, gamma, beta, bias, skip, 1e-5, alpha, 8)
    y, s, z = flow._C.fused_skip_layer_norm_min_max_observer(
        H.to_torch(x), H.to_torch(gamma), H.to_torch(beta), H.to_torch(bias), H.to_torch(skip),
        1e-5, alpha, 8)
    y_np = H.to_numpy(y)
    yf, yr = O.to_f32(y_np).astype(np.float64), O.to_f32(y_ref).astype(np.float64)
    if t == "f32":
        assert np.allclose(yf, yr, rtol=4e-6, atol=4e-6)
    else:
        mag = np.abs(yr) + np.abs(O.to_f32(beta).astype(np.float64))[None, :]
        assert (np.abs(yf - yr) <= 2.0001 * H.ulp_of(mag, t)).all()
        assert (yf != yr).mean() < 0.02
    expect = np.float32(np.abs(O.to_f32(y_np)).max()) / np.float32(127.0)
    assert H.to_numpy(s)[0] == expect and H.to_numpy(z)[0] == 0.0
    assert abs(float(H.to_numpy(s)[0]) - float(s_ref[0])) <= 2e-3 * float(s_ref[0])


EXACT_SHAPES = [("f16", 2048, 4096), ("bf16", 2048, 4096), ("f16", 5000, 512), ("bf16", 300, 1024),
                ("f16", 64, 2048), ("f32", 33, 1000), ("f16", 7, 8200), ("f16", 5, 24),
                ("f16", 12, 11008), ("f32", 6, 16384), ("bf16", 3, 16392), ("f32", 40, 2048),
                ("bf16", 4, 20000), ("f16", 3, 4104), ("f16", 4, 20000), ("f16", 9, 16384)]


@pytest.mark.parametrize("t,rows,cols", EXACT_SHAPES)
def test_layer_norm_observer_exact_statistics_matches_the_oracle_bit_for_bit(t, rows, cols):
    """Config 5 at full size and every kernel variant (one wave per row with and without the
    row in registers, rows walked by a wave, one block per row, any-length rows): y bit-exact,
    scale identical (the contract asks for 1 ulp) and the int8 codes quantised from them
    bit-exact against the oracle.  A quarter of the rows carry an offset of 40 standard
    deviations, where a variance from fp32 sums would be off by many ulps."""
    import oneflow_amd as flow
    import torch
    x, gamma, beta = _cfg5_inputs(rows, cols, t)
    xf = O.to_f32(x).copy()
    xf[::4] += 40.0
    x = H.as_T(xf, t)
    y_ref, s_ref, z_ref = O.layer_norm_min_max_observer(x, gamma, beta, 1e-5, 8)
    y, s, z = flow._C.fused_layer_norm_min_max_observer(
        H.to_torch(x), H.to_torch(gamma), H.to_torch(beta), 1e-5, 8, exact_statistics=True)
    y_np = H.to_numpy(y)
    view = np.uint32 if t == "f32" else np.uint16
    assert np.array_equal(y_np.view(view), y_ref.view(view))
    assert H.to_numpy(s)[0] == s_ref[0] and H.to_numpy(z)[0] == 0.0
    if t == "f16":
        a = flow._C.quantization(y, s, z, "google", 8, "symmetric", out_dtype=torch.int8)
        assert np.array_equal(H.to_numpy(a), O.quantize_to_int8(y_ref, s_ref, 8))


@pytest.mark.parametrize("rows,cols", [(2048, 4096), (3, 512), (130, 1024), (257, 2048), (4099, 512),
                                       (5000, 1024)])
@pytest.mark.parametrize("exact", [False, True])
def test_layer_norm_quantization_equals_the_two_ops(rows, cols, exact):
    """LayerNorm -> observer -> int8 codes as one entry point (the normalised tensor is never
    written) against fused_layer_norm_min_max_observer followed by quantization: identical
    codes, scale and zero point, with fp32 and with fp64 row statistics, one row per wave and
    rows walked by a wave (more than 4096 rows); with fp64 statistics also against the oracle.
    A quarter of the rows carry an offset and a few values are large, so that the scale is set
    by a single row."""
    import oneflow_amd as flow
    import torch
    x, gamma, beta = _cfg5_inputs(rows, cols, "f16")
    xf = O.to_f32(x).copy()
    xf[::4] += 40.0
    xf[rows // 2, 7] = 300.0
    x = H.as_T(xf, "f16")
    xt, gt, bt = H.to_torch(x), H.to_torch(gamma), H.to_torch(beta)
    y, s, z = flow._C.fused_layer_norm_min_max_observer(xt, gt, bt, 1e-5, 8, exact_statistics=exact)
    want = flow._C.quantization(y, s, z, "google", 8, "symmetric", out_dtype=torch.int8)
    codes, s2, z2 = flow._C.fused_layer_norm_quantization(xt, gt, bt, 1e-5, 8, exact_statistics=exact)
    assert codes.dtype == torch.int8 and codes.shape == xt.shape
    assert torch.equal(s.view(torch.int32), s2.view(torch.int32)) and z2.item() == 0.0
    assert torch.equal(codes, want)
    if exact:
        y_ref, s_ref, z_ref = O.layer_norm_min_max_observer(x, gamma, beta, 1e-5, 8)
        assert H.to_numpy(s2)[0] == s_ref[0]
        assert np.array_equal(H.to_numpy(codes), O.quantize_to_int8(y_ref, s_ref, 8))


@pytest.mark.parametrize("bits", [2, 5, 8])
def test_layer_norm_quantization_bit_widths_and_a_zero_row_tensor(bits):
    import oneflow_amd as flow
    import torch
    x, gamma, beta = _cfg5_inputs(40, 1024, "f16")
    xt, gt, bt = H.to_torch(x), H.to_torch(gamma), H.to_torch(beta)
    y, s, z = flow._C.fused_layer_norm_min_max_observer(xt, gt, bt, 1e-5, bits)
    want = flow._C.quantization(y, s, z, "google", bits, "symmetric", out_dtype=torch.int8)
    codes, s2, z2 = flow._C.fused_layer_norm_quantization(xt, gt, bt, 1e-5, bits)
    assert torch.equal(codes, want) and torch.equal(s.view(torch.int32), s2.view(torch.int32))
    assert int(codes.max()) <= 2 ** (bits - 1) - 1 and int(codes.min()) >= -(2 ** (bits - 1))
    # y = 0 everywhere (gamma = beta = 0): scale 0, and the codes of 0 / 0 as the two ops give them
    zeros = torch.zeros_like(gt)
    y, s, z = flow._C.fused_layer_norm_min_max_observer(xt, zeros, zeros, 1e-5, bits)
    want = flow._C.quantization(y, s, z, "google", bits, "symmetric", out_dtype=torch.int8)
    codes, s2, z2 = flow._C.fused_layer_norm_quantization(xt, zeros, zeros, 1e-5, bits)
    assert s2.item() == 0.0 and torch.equal(codes, want)


@pytest.mark.parametrize("t,rows,cols,with_params", [("f16", 9, 1000, True), ("bf16", 33, 1024, True),
                                                     ("f32", 5, 512, True), ("f16", 12, 8192, True),
                                                     ("f16", 16, 2048, False)])
def test_layer_norm_quantization_other_shapes_run_the_two_ops(t, rows, cols, with_params):
    """Shapes and dtypes outside the fused kernels: the C entry point reports
    OFQ_ERR_UNSUPPORTED without launching anything, the functional runs the two ops."""
    import oneflow_amd as flow
    import torch
    from oneflow_amd import _lib
    x, gamma, beta = _cfg5_inputs(rows, cols, t)
    xt = H.to_torch(x)
    gt, bt = (H.to_torch(gamma), H.to_torch(beta)) if with_params else (None, None)
    L = _lib.lib()
    dt = {"f16": _lib.F16, "bf16": _lib.BF16, "f32": _lib.F32}[t]
    nbytes = L.ofq_fused_layer_norm_quantization_workspace_bytes(dt, rows, cols)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    codes = torch.full((rows, cols), 77, dtype=torch.int8, device="cuda")
    s = torch.full((1,), -1.0, device="cuda")
    z = torch.full((1,), -1.0, device="cuda")
    st = L.ofq_fused_layer_norm_quantization(
        torch.cuda.current_stream().cuda_stream, xt.data_ptr(),
        gt.data_ptr() if with_params else None, bt.data_ptr() if with_params else None,
        codes.data_ptr(), s.data_ptr(), z.data_ptr(), dt, rows, cols, 1e-5, 8, _lib.LN_STATS_FP32,
        ws.data_ptr(), nbytes)
    torch.cuda.synchronize()
    assert st == _lib.ERR_UNSUPPORTED and s.item() == -1.0 and int(codes.min()) == 77
    y, s1, z1 = flow._C.fused_layer_norm_min_max_observer(xt, gt, bt, 1e-5, 8)
    got, s2, z2 = flow._C.fused_layer_norm_quantization(xt, gt, bt, 1e-5, 8)
    assert torch.equal(s1.view(torch.int32), s2.view(torch.int32))
    if t == "f16":
        want = flow._C.quantization(y, s1, z1, "google", 8, "symmetric", out_dtype=torch.int8)
        assert torch.equal(got, want)


def test_layer_norm_quantization_argument_errors():
    import torch
    from oneflow_amd import _lib
    L = _lib.lib()
    rows, cols = 8, 1024
    x = torch.zeros(rows, cols, dtype=torch.float16, device="cuda")
    g = torch.ones(cols, dtype=torch.float16, device="cuda")
    codes = torch.zeros(rows, cols, dtype=torch.int8, device="cuda")
    s = torch.zeros(1, device="cuda")
    nbytes = L.ofq_fused_layer_norm_quantization_workspace_bytes(_lib.F16, rows, cols)
    assert nbytes == 32 + rows * 8
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream

    def call(bits=8, stats=_lib.LN_STATS_FP32, wsp=ws.data_ptr(), wsb=nbytes, xp=x.data_ptr()):
        return L.ofq_fused_layer_norm_quantization(stream, xp, g.data_ptr(), g.data_ptr(),
                                                   codes.data_ptr(), s.data_ptr(), s.data_ptr(),
                                                   _lib.F16, rows, cols, 1e-5, bits, stats, wsp, wsb)
    assert call() == 0
    assert call(bits=9) == 4 and call(bits=1) == 4 and call(stats=7) == 4
    assert call(wsp=None) == 6 and call(wsb=nbytes - 1) == 6
    assert call(xp=None) == 1
    torch.cuda.synchronize()


@pytest.mark.parametrize("t,rows,cols", [("f16", 2048, 4096), ("bf16", 300, 4096), ("f32", 33, 1000),
                                         ("f16", 7, 8200), ("bf16", 5, 24), ("bf16", 9, 16384),
                                         ("f16", 4, 20000)])
@pytest.mark.parametrize("use_bias,use_skip", [(True, True), (False, True)])
def test_skip_layer_norm_observer_exact_statistics(t, rows, cols, use_bias, use_skip):
    import oneflow_amd as flow
    x, gamma, beta = _cfg5_inputs(rows, cols, t)
    bias = H.as_T((0.5 * H.rng_for(6, 0).standard_normal(cols)).astype(np.float32), t) if use_bias else None
    skip = H.as_T(H.rng_for(6, 1).standard_normal((rows, cols)).astype(np.float32), t) if use_skip else None
    y_ref, s_ref, z_ref = O.skip_layer_norm_min_max_observer(x, gamma, beta, bias, skip, 1e-5, 0.37, 8)
    y, s, z = flow._C.fused_skip_layer_norm_min_max_observer(
        H.to_torch(x), H.to_torch(gamma), H.to_torch(beta), H.to_torch(bias), H.to_torch(skip),
        1e-5, 0.37, 8, exact_statistics=True)
    view = np.uint32 if t == "f32" else np.uint16
    assert np.array_equal(H.to_numpy(y).view(view), y_ref.view(view))
    assert H.to_numpy(s)[0] == s_ref[0] and H.to_numpy(z)[0] == 0.0


def test_skip_layer_norm_without_residual_is_the_plain_op():
    """bias = skip = None adds zeros: the same bits as fused_layer_norm_min_max_observer."""
    import oneflow_amd as flow
    x, gamma, beta = _cfg5_inputs(64, 4096, "f16")
    a = flow._C.fused_layer_norm_min_max_observer(H.to_torch(x), H.to_torch(gamma), H.to_torch(beta), 1e-5, 8)
    b = flow._C.fused_skip_layer_norm_min_max_observer(H.to_torch(x), H.to_torch(gamma), H.to_torch(beta),
                                                       None, None, 1e-5, 1e1, 8)
    for u, v in zip(a, b):
        assert np.array_equal(H.to_numpy(u), H.to_numpy(v))


def test_layer_norm_closed_form():
    """Rows of +-c have mean 0 and variance c^2: y = +-c/sqrt(c^2+eps) * gamma + beta."""
    import oneflow_amd as flow
    cols = 512
    x = np.tile(np.array([1.5, -1.5], np.float32), cols // 2)[None, :].repeat(3, 0)
    y, s, z = flow._C.fused_layer_norm_min_max_observer(H.to_torch(x), None, None, 1e-5, 8)
    expect = np.float32(1.5) * (np.float32(1.0) / np.sqrt(np.float32(2.25) + np.float32(1e-5)))
    y = H.to_numpy(y)
    assert np.allclose(np.abs(y), expect, rtol=2e-7, atol=0) and np.array_equal(np.sign(y), np.sign(x))
    assert np.isclose(H.to_numpy(s)[0], expect / 127.0, rtol=3e-7)


@pytest.mark.parametrize("t", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("cols", [256, 4096, 8192, 20000])
def test_layer_norm_exact_statistics_rows_bit_exact(t, cols):
    """Rows of +-4 (any order) have mean 0, variance 16 and, with eps = 0, inv = 1/4 exactly in
    every summation order, so only the roundings of the affine are left: the bits must equal the
    oracle's, for gamma and beta together, gamma alone (the reference then adds its default beta
    0, which turns a -0 product into +0) and beta alone.  The column counts reach the one-wave,
    one-block and any-length kernels."""
    import oneflow_amd as flow
    rng = np.random.default_rng(cols)
    base = np.concatenate([np.full(cols // 2, 4.0, np.float32), np.full(cols // 2, -4.0, np.float32)])
    x = H.as_T(np.stack([rng.permutation(base) for _ in range(5)]), t)
    gamma_f = (1 + 0.37 * rng.standard_normal(cols)).astype(np.float32)
    gamma_f[::7] = 0.0
    gamma = H.as_T(gamma_f, t)
    beta = H.as_T((0.21 * rng.standard_normal(cols)).astype(np.float32), t)
    for g, b in ((gamma, beta), (gamma, None), (None, beta), (None, None)):
        y_ref, s_ref, _ = O.layer_norm_min_max_observer(x, g, b, 0.0, 8)
        y, s, z = flow._C.fused_layer_norm_min_max_observer(
            H.to_torch(x), None if g is None else H.to_torch(g), None if b is None else H.to_torch(b), 0.0, 8)
        y = H.to_numpy(y)
        view = np.uint32 if t == "f32" else np.uint16
        assert np.array_equal(y.view(view), y_ref.view(view)), (t, cols, g is None, b is None)
        assert H.to_numpy(s)[0] == s_ref[0]


def _scale_with_mantissa(exp, mant):
    return np.array([(np.uint32(exp + 127) << np.uint32(23)) | np.uint32(mant)], dtype=np.uint32).view(np.float32)


@pytest.mark.parametrize("scheme", ["symmetric", "affine"])
def test_quantization_of_every_fp16_value_bit_exact(scheme):
    """fp16 input with one scale per tensor replaces the division by a multiplication with the
    reciprocal and two exact-remainder corrections.  Every finite fp16 value and the infinities
    (both zeros, subnormals included) against scales whose mantissas are the hard cases of a
    division (all ones, just above a power of two, random), scales of either sign, and scales
    outside the range the corrected multiplication is used for: int8 codes, codes stored as fp16
    and fake quantization, all bit for bit what `x / scale` gives in the oracle."""
    import oneflow_amd as flow
    import torch
    bits16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = bits16.view(np.float16)
    x = x[~np.isnan(x)]
    x = np.tile(x, 2)[: (2 * x.size) // 16 * 16].reshape(-1, 16)  # whole 16-element packs
    rng = np.random.default_rng(11)
    scales = [_scale_with_mantissa(e, m) for e, m in
              [(-7, 0x7FFFFF), (-7, 0x7FFFFE), (-3, 0), (-3, 1), (2, 0x7FFFFD), (-12, 0x555555),
               (9, 0x2AAAAA), (-59, 0x7FFFFF), (59, 3), (-70, 0x123456), (70, 0x654321)]]
    scales += [np.array([v], dtype=np.float32) for v in rng.uniform(1e-4, 50.0, size=6)]
    scales += [-scales[0], -scales[5]]
    xf = x.astype(np.float32)
    for sc in scales:
        zp = np.array([0.0 if scheme == "symmetric" else 3.0], dtype=np.float32)
        ref = O.quantization(xf, sc, zp, "google", 8, scheme, zp_mode="cuda")
        ref_fake = O.fake_quantization(xf, sc, zp, "google", 8, scheme, zp_mode="cuda")
        xt, st, zt = H.to_torch(x), H.to_torch(sc), H.to_torch(zp)
        got_f16 = H.to_numpy(flow._C.quantization(xt, st, zt, "google", 8, scheme))
        assert np.array_equal(got_f16.view(np.uint16), ref.astype(np.float16).view(np.uint16)), sc
        got_fake = H.to_numpy(flow._C.fake_quantization(xt, st, zt, "google", 8, scheme))
        assert np.array_equal(got_fake.view(np.uint16),
                              ref_fake.astype(np.float16).view(np.uint16)), sc
        # byte codes: whole 1024-element tiles (the kernel with two 1 KB requests per wave) and a
        # size that is not a multiple of 1024 (the generic kernel)
        code_dt, code_np = (torch.int8, np.int8) if scheme == "symmetric" else (torch.uint8, np.uint8)
        for rows in (x.shape[0], x.shape[0] - 1):
            got_b = H.to_numpy(flow._C.quantization(H.to_torch(x[:rows]), st, zt, "google", 8,
                                                    scheme, out_dtype=code_dt))
            assert np.array_equal(got_b, ref[:rows].astype(code_np)), (sc, rows)


def test_dynamic_quantize_and_matmul_quant():
    import oneflow_amd as flow
    import torch
    m, n, k = 2048, 11008, 4096
    x, gamma, beta = _cfg5_inputs(m, k, "f16")
    y, s, z = flow._C.fused_layer_norm_min_max_observer(H.to_torch(x), H.to_torch(gamma),
                                                        H.to_torch(beta), 1e-5, 8)
    a = flow._C.quantization(y, s, z, "google", 8, "symmetric", out_dtype=torch.int8)
    a_np = H.to_numpy(a)
    # codes: bit-exact against the oracle GIVEN the same y and scale
    a_ref = O.quantize_to_int8(H.to_numpy(y), H.to_numpy(s), 8)
    assert np.array_equal(a_np, a_ref)
    assert np.abs(a_np.astype(np.int32)).max() == 127
    w = H.rng_for(5, 3).integers(-127, 128, size=(n, k)).astype(np.int8)
    w_scale = H.rng_for(5, 4).uniform(1e-3, 1e-2, size=n).astype(np.float32)
    out = H.to_numpy(flow._C.matmul_quant(a, H.to_torch(w), s, H.to_torch(w_scale), None,
                                          torch.float16))
    rows = np.array([0, 31, 32, 127, 128, 1000, 2047])
    cols = np.concatenate([np.arange(0, 64), np.arange(6000, 6064), np.arange(n - 64, n)])
    # exact integer accumulation (int64 brute force) then the fp32 epilogue, rounded once
    acc = a_np[rows].astype(np.int64) @ w[cols].astype(np.int64).T
    sc = (H.to_numpy(s)[0] * w_scale[cols]).astype(np.float32)
    expect = (acc.astype(np.float32) * sc[None, :]).astype(np.float16)
    got = out[np.ix_(rows, cols)]
    assert np.array_equal(got.view(np.uint16), expect.view(np.uint16))
    ref = O.matmul_quant(a_np[rows], w[cols], H.to_numpy(s), w_scale[cols], None, np.float16)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))
    # every one of the 22.5 M outputs: the integer sums are exact in an fp64 matmul on all host
    # cores (|acc| < 2^27), the epilogue is one int -> fp32 conversion, one fp32 product and one
    # rounding to fp16; this composition is pinned by the oracle on the sample above
    acc_all = (torch.from_numpy(a_np).double() @ torch.from_numpy(w).double().t())
    sc_all = torch.from_numpy((H.to_numpy(s)[0] * w_scale).astype(np.float32))
    expect_all = (acc_all.to(torch.int32).to(torch.float32) * sc_all[None, :]).to(torch.float16).numpy()
    assert np.array_equal(expect_all[np.ix_(rows, cols)].view(np.uint16), ref.view(np.uint16))
    assert np.array_equal(out.view(np.uint16), expect_all.view(np.uint16))


@pytest.mark.parametrize("m,n,k,t", [(1, 16, 128, "f32"), (100, 200, 256, "f16"), (130, 33, 384, "bf16")])
def test_matmul_quant_small_exact(m, n, k, t):
    import oneflow_amd as flow
    import torch
    rng = np.random.Generator(np.random.PCG64(m * 1000 + n))
    a = rng.integers(-128, 128, size=(m, k)).astype(np.int8)
    b = rng.integers(-128, 128, size=(n, k)).astype(np.int8)
    a_scale = np.array([0.0123], np.float32)
    b_scale = rng.uniform(1e-3, 1e-2, size=n).astype(np.float32)
    bias = H.as_T(rng.standard_normal(n).astype(np.float32), t)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[t]
    got = H.to_numpy(flow._C.matmul_quant(H.to_torch(a), H.to_torch(b), H.to_torch(a_scale),
                                          H.to_torch(b_scale), H.to_torch(bias), tdt))
    ref = O.matmul_quant(a, b, a_scale, b_scale, bias, {"f32": np.float32, "f16": np.float16,
                                                        "bf16": np.uint16}[t])
    assert np.array_equal(got.view(np.uint16 if t != "f32" else np.uint32),
                          ref.view(np.uint16 if t != "f32" else np.uint32))


@pytest.mark.parametrize("t", ["f32", "bf16"])
@pytest.mark.parametrize("m,n", [(2053, 8196), (700, 11012)])
def test_matmul_quant_wide_tiles_full_output(t, m, n):
    """Shapes that are dispatched to the 256x352 and to the 256x192 tiles, with ragged last tiles
    in both m and n; every output is checked.  The int32 accumulators come from a float64 matmul,
    which is exact here (|sum| <= 128*128*256 < 2^53)."""
    import oneflow_amd as flow
    import torch
    k = 256
    rng = np.random.Generator(np.random.PCG64(99))
    a = rng.integers(-128, 128, size=(m, k)).astype(np.int8)
    b = rng.integers(-128, 128, size=(n, k)).astype(np.int8)
    a_scale = np.array([0.0071], np.float32)
    b_scale = rng.uniform(1e-3, 1e-2, size=n).astype(np.float32)
    bias = H.as_T(rng.standard_normal(n).astype(np.float32), t)
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16}[t]
    got = H.to_numpy(flow._C.matmul_quant(H.to_torch(a), H.to_torch(b), H.to_torch(a_scale),
                                          H.to_torch(b_scale), H.to_torch(bias), tdt))
    acc = (a.astype(np.float64) @ b.astype(np.float64).T)
    assert np.abs(acc).max() < 2**31
    sc = (a_scale[0] * b_scale).astype(np.float32)
    val = (acc.astype(np.float32) * sc[None, :]).astype(np.float32) + O.to_f32(bias)[None, :]
    if t == "f32":
        assert np.array_equal(got, val.astype(np.float32))
    else:
        assert np.array_equal(got, O.f32_to_bf16_bits(val))
    # the oracle itself on a corner that includes the ragged edges
    rows, cols = np.arange(m - 40, m), np.arange(n - 70, n)
    ref = O.matmul_quant(a[rows], b[cols], a_scale, b_scale[cols], bias[cols],
                         {"f32": np.float32, "bf16": np.uint16}[t])
    view = np.uint32 if t == "f32" else np.uint16
    assert np.array_equal(got[np.ix_(rows, cols)].view(view), ref.view(view))


@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (5, 1000, 192), (16, 37, 64), (17, 688, 1024),
                                   (33, 2049, 448), (64, 300, 11008), (200, 130, 192),
                                   (2, 11008, 4096), (3, 1000, 192), (4, 37, 8192), (1, 30000, 64),
                                   (4, 4099, 1088), (2, 70000, 128), (1, 13, 7168), (4, 33, 11008),
                                   (2, 9000, 8192), (4, 9000, 5120), (3, 600, 7232)])
def test_matmul_quant_few_rows_streaming(m, n, k, t):
    """m <= 64 (and any m when k is a multiple of 64 but not of 128) runs the streaming int8
    kernels: up to 2 rows of a with k <= 8192, up to 4 with k <= 4096, the one in which a wave owns
    whole rows of b (every
    row length class incl. partial KBs, one and two blocks per CU, many rows per wave, fewer rows
    than waves), beyond that the MFMA kernel with 1, 2 and 4 tiles of a, ragged n, k from one
    chunk to many, several passes for m = 200.  Bit-exact: int32 sums are order-free and the
    epilogue is the GEMM path's."""
    import oneflow_amd as flow
    import torch
    rng = np.random.Generator(np.random.PCG64(m * 1000 + n + k))
    a = rng.integers(-128, 128, size=(m, k)).astype(np.int8)
    b = rng.integers(-128, 128, size=(n, k)).astype(np.int8)
    a_scale = np.array([0.0317], np.float32)
    b_scale = rng.uniform(1e-3, 1e-2, size=n).astype(np.float32)
    bias = H.as_T(rng.standard_normal(n).astype(np.float32), t) if (m + n) % 2 else None
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[t]
    got = H.to_numpy(flow._C.matmul_quant(H.to_torch(a), H.to_torch(b), H.to_torch(a_scale),
                                          H.to_torch(b_scale), H.to_torch(bias), tdt))
    acc = (a.astype(np.float64) @ b.astype(np.float64).T)
    assert np.abs(acc).max() < 2**31
    sc = (a_scale[0] * b_scale).astype(np.float32)
    val = (acc.astype(np.float32) * sc[None, :]).astype(np.float32)
    if bias is not None:
        val = val + O.to_f32(bias)[None, :]
    if t == "f32":
        assert np.array_equal(got, val.astype(np.float32))
    elif t == "bf16":
        assert np.array_equal(got, O.f32_to_bf16_bits(val))
    else:
        assert np.array_equal(got, val.astype(np.float16))
    # and the oracle on a corner
    rows, cols = np.arange(max(0, m - 3), m), np.arange(max(0, n - 20), n)
    ref = O.matmul_quant(a[rows], b[cols], a_scale, b_scale[cols],
                         None if bias is None else bias[cols],
                         {"f32": np.float32, "f16": np.float16, "bf16": np.uint16}[t])
    view = np.uint32 if t == "f32" else np.uint16
    assert np.array_equal(got[np.ix_(rows, cols)].view(view), ref.view(view))


@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("m,n,k", [(65, 8192, 256), (80, 4100, 1024), (256, 4096, 4096), (200, 3001, 640),
                                   (512, 1100, 6144), (130, 2789, 1152), (768, 4096, 384),
                                   (1024, 4096, 256), (600, 5000, 640), (2200, 4096, 256),
                                   (3000, 4100, 128)])
def test_matmul_quant_one_launch_tile_choices(m, n, k, t):
    """Shapes for which one launch without K slices and without a workspace is the path: 64 x 64
    tiles (128 to 768 of them, m <= 768), 128 x 128 tiles where 256-row tiles would leave CUs
    idle, 256 x 256 tiles where they make one round of two; ragged last tiles in both
    directions; bit-identical to the oracle's int64 sums and fp32 epilogue."""
    import torch
    from oneflow_amd import _lib
    L = _lib.lib()
    rng = np.random.Generator(np.random.PCG64(m * 3 + n + k))
    a = rng.integers(-128, 128, size=(m, k)).astype(np.int8)
    b = rng.integers(-128, 128, size=(n, k)).astype(np.int8)
    a_scale = np.array([0.0173], np.float32)
    b_scale = rng.uniform(1e-3, 1e-2, size=n).astype(np.float32)
    bias = H.as_T(rng.standard_normal(n).astype(np.float32), t)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[t]
    tcode = {"f32": _lib.F32, "f16": _lib.F16, "bf16": _lib.BF16}[t]
    assert L.ofq_matmul_quant_workspace_bytes(m, n, k) == 0
    at, bt, ast, bst, biast = map(H.to_torch, (a, b, a_scale, b_scale, bias))
    out = torch.full((m, n), float("nan"), dtype=tdt, device="cuda")
    rc = L.ofq_matmul_quant(torch.cuda.current_stream().cuda_stream, at.data_ptr(), bt.data_ptr(),
                            ast.data_ptr(), bst.data_ptr(), biast.data_ptr(), out.data_ptr(), tcode,
                            m, n, k)
    assert rc == 0
    view = np.uint32 if t == "f32" else np.uint16
    ref = O.matmul_quant(a, b, a_scale, b_scale, bias,
                         {"f32": np.float32, "f16": np.float16, "bf16": np.uint16}[t])
    assert np.array_equal(H.to_numpy(out).view(view), ref.view(view))


@pytest.mark.parametrize("t", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("m,n,k", [(65, 256, 2048), (128, 1000, 4096), (200, 130, 1024), (512, 384, 1024),
                                   (300, 203, 1536), (40, 256, 8192)])
def test_matmul_quant_k_slices(m, n, k, t):
    """64 < m with few output tiles: with the workspace the op asks for, K is cut into slices whose
    int32 partial sums are added by a second kernel.  Integer sums do not depend on the order, so
    the result equals the one-kernel path bit for bit, and both equal the oracle."""
    import torch
    from oneflow_amd import _lib
    L = _lib.lib()
    rng = np.random.Generator(np.random.PCG64(m + n + k))
    a = rng.integers(-128, 128, size=(m, k)).astype(np.int8)
    b = rng.integers(-128, 128, size=(n, k)).astype(np.int8)
    a_scale = np.array([0.0211], np.float32)
    b_scale = rng.uniform(1e-3, 1e-2, size=n).astype(np.float32)
    bias = H.as_T(rng.standard_normal(n).astype(np.float32), t)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[t]
    tcode = {"f32": _lib.F32, "f16": _lib.F16, "bf16": _lib.BF16}[t]
    need = L.ofq_matmul_quant_workspace_bytes(m, n, k)
    assert need > 0 and need % (m * n * 4) == 0 and need // (m * n * 4) >= 2, need
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    at, bt, ast, bst, biast = map(H.to_torch, (a, b, a_scale, b_scale, bias))
    outs = []
    for wptr, wbytes in ((ws.data_ptr(), need), (None, 0)):
        out = torch.empty((m, n), dtype=tdt, device="cuda")
        rc = L.ofq_matmul_quant_ws(torch.cuda.current_stream().cuda_stream, at.data_ptr(),
                                   bt.data_ptr(), ast.data_ptr(), bst.data_ptr(), biast.data_ptr(),
                                   out.data_ptr(), tcode, m, n, k, wptr, wbytes)
        assert rc == 0
        outs.append(H.to_numpy(out))
    view = np.uint32 if t == "f32" else np.uint16
    assert np.array_equal(outs[0].view(view), outs[1].view(view))
    ref = O.matmul_quant(a, b, a_scale, b_scale, bias,
                         {"f32": np.float32, "f16": np.float16, "bf16": np.uint16}[t])
    assert np.array_equal(outs[0].view(view), ref.view(view))
