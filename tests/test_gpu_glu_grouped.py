"""The linears' neighbours over groupwise-quantised weights: several problems in one call
(grouped_matmul_bias's counterpart) and the gated linear unit (fused_glu's counterpart), on the GPU
against the oracle.  Linear outputs: the op's contract (rel-L2 <= 1e-3, max-abs <= 2e-2); the
gating: bit-exact for 'none' / 'relu', one rounding of T for the smooth activations (expf, erff
and tanhf of the device library and of the host libm may differ in the last fp32 bit)."""
import numpy as np
import pytest

import helpers as H
from oracle import ofq_oracle as O

pytestmark = pytest.mark.gpu

VARIANTS = [(True, np.int8), (True, np.uint8), (False, np.uint8)]


def _problem(rng, m, n, k, num_bits, symmetric, qdt, g, t, bias=True):
    x = H.as_T(rng.standard_normal((m, k)).astype(np.float32), t)
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    w, scale, zero = H.quantize_groupwise(wf, num_bits, symmetric, 1, g, qdt, t)
    b = H.as_T((rng.standard_normal(n) * 0.1).astype(np.float32), t) if bias else None
    return x, w, scale, zero, b


@pytest.mark.parametrize("t", ["f16", "bf16"])
@pytest.mark.parametrize("num_bits", [4, 8])
@pytest.mark.parametrize("m,k,ns", [(1, 1024, (512, 128, 128)), (8, 512, (300, 300)),
                                    (16, 256, (40, 4099, 17)), (3, 128, (20000, 20000)),
                                    (1, 4096, (4096, 4096, 4096)), (1, 2048, (5000, 300, 6000)),
                                    (1, 256, (9000, 37))])
@pytest.mark.parametrize("g", [64, 128])
def test_grouped_decode_one_launch(t, num_bits, m, k, ns, g):
    """Problems of equal (m, k): q/k/v-like row counts, ragged ones, and enough rows for two
    blocks per CU; shared x (the decode case) for the first problems, an own x for the last."""
    import oneflow_amd as flow
    rng = np.random.Generator(np.random.PCG64(m * 100 + k + num_bits))
    for symmetric, qdt in VARIANTS:
        probs = [_problem(rng, m, n, k, num_bits, symmetric, qdt, g, t, bias=(i != 1))
                 for i, n in enumerate(ns)]
        xs = [probs[0][0]] * (len(ns) - 1) + [probs[-1][0]]
        tt = H.to_torch
        outs = flow._C.grouped_linear_with_groupwise_quantized_weight(
            [tt(x) for x in xs], [tt(p[1]) for p in probs], [tt(p[2]) for p in probs],
            w_zeros=None if symmetric else [tt(p[3]) for p in probs], bs=[tt(p[4]) for p in probs],
            num_bits=num_bits, symmetric=symmetric, group_dim=1, group_size=g)
        assert len(outs) == len(ns)
        # fp16, int8 container, 4 bits, groups of 128: the kernel that leaves q*s unrounded
        shortcut = t == "f16" and num_bits == 4 and qdt == np.int8 and g == 128
        for x, p, out in zip(xs, probs, outs):
            ref = O.fused_linear(x, p[1], p[2], p[3], p[4], num_bits, symmetric, 1, g)
            r, e = H.assert_linear_parity(H.to_numpy(out), ref, t, f"{t} b{num_bits} {symmetric} {qdt}")
            assert r < (3e-3 if t == "bf16" else 5e-4 if shortcut else 1e-4)


def test_grouped_mixed_shapes_and_many_problems():
    """Problems of different (m, k) are grouped by shape as in the reference kernel; m > 16 and
    fp32 run one by one; more than 8 problems of a shape take several launches."""
    import oneflow_amd as flow
    rng = np.random.Generator(np.random.PCG64(5))
    shapes = [(2, 64, 256)] * 10 + [(20, 48, 256), (2, 32, 128), (20, 16, 256), (1, 33, 128)]
    for t in ("f16", "f32"):
        probs = [_problem(rng, m, n, k, 8, True, np.int8, 64, t) for m, n, k in shapes]
        tt = H.to_torch
        outs = flow._C.grouped_linear_with_groupwise_quantized_weight(
            [tt(p[0]) for p in probs], [tt(p[1]) for p in probs], [tt(p[2]) for p in probs],
            bs=[tt(p[4]) for p in probs], num_bits=8, symmetric=True, group_dim=1, group_size=64)
        for p, out in zip(probs, outs):
            ref = O.fused_linear(p[0], p[1], p[2], None, p[4], 8, True, 1, 64)
            if t == "f32":
                assert np.allclose(H.to_numpy(out), ref, rtol=1e-4, atol=1e-4)
            else:
                H.assert_linear_parity(H.to_numpy(out), ref, t, "mixed")


def _glu_call(L, _lib, torch, x, w, ws, wz, b, v, vs, vz, c, act, wcode, tcode, bits, sym, g, m, n, k):
    tt = H.to_torch
    xt, wt, wst, wzt, bt, vt, vst, vzt, ct = map(tt, (x, w, ws, wz, b, v, vs, vz, c))
    split = v is not None
    y = torch.empty((m, n), dtype=xt.dtype, device="cuda")
    wx = torch.empty((m, n if split else 2 * n), dtype=xt.dtype, device="cuda")
    vx = torch.empty((m, n), dtype=xt.dtype, device="cuda") if split else None
    ptr = lambda a: a.data_ptr() if a is not None else None
    rc = L.ofq_fused_glu_gq(torch.cuda.current_stream().cuda_stream, ptr(xt), ptr(wt), ptr(wst),
                            ptr(wzt), ptr(bt), ptr(vt), ptr(vst), ptr(vzt), ptr(ct), ptr(y), ptr(wx),
                            ptr(vx), O.ACTIVATIONS[act], wcode, tcode, bits, int(sym), 1, g, m, n, k)
    assert rc == 0, rc
    return H.to_numpy(y), H.to_numpy(wx), (H.to_numpy(vx) if split else None)


@pytest.mark.parametrize("t", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("m,n,k", [(1, 1024, 512), (16, 344, 256), (40, 136, 256), (5, 37, 128),
                                   (2, 9000, 256)])
@pytest.mark.parametrize("split", [True, False])
@pytest.mark.parametrize("g", [64, 128])
def test_glu_all_activations(t, m, n, k, split, g):
    import torch
    from oneflow_amd import _lib
    L = _lib.lib()
    tcode = {"f16": _lib.F16, "bf16": _lib.BF16, "f32": _lib.F32}[t]
    rng = np.random.Generator(np.random.PCG64(m + n + k))
    bits = 4
    for symmetric, qdt in ((True, np.int8), (True, np.uint8), (False, np.uint8)):
        wcode = _lib.I8 if qdt == np.int8 else _lib.U8
        rows = n if split else 2 * n
        x, w, ws, wz, b = _problem(rng, m, rows, k, bits, symmetric, qdt, g, t)
        v = vs = vz = c = None
        if split:
            _, v, vs, vz, c = _problem(rng, m, n, k, bits, symmetric, qdt, g, t)
        for act in O.ACTIVATIONS:
            y, wx, vx = _glu_call(L, _lib, torch, x, w, ws, wz, b, v, vs, vz, c, act, wcode, tcode,
                                  bits, symmetric, g, m, n, k)
            # the two linears: the op's contract against the oracle
            wx_ref = O.fused_linear(x, w, ws, wz, b, bits, symmetric, 1, g)
            if t == "f32":
                assert np.allclose(wx, wx_ref, rtol=1e-4, atol=1e-4)
            else:
                H.assert_linear_parity(wx, wx_ref, t, f"wx {act}")
            if split:
                vx_ref = O.fused_linear(x, v, vs, vz, c, bits, symmetric, 1, g)
                if t == "f32":
                    assert np.allclose(vx, vx_ref, rtol=1e-4, atol=1e-4)
                else:
                    H.assert_linear_parity(vx, vx_ref, t, f"vx {act}")
                hidden, gate = wx, vx
            else:
                hidden, gate = np.ascontiguousarray(wx[:, :n]), np.ascontiguousarray(wx[:, n:])
            # the gating: against the oracle ON THE GPU's own linear outputs
            y_ref = O.glu_gate(hidden, gate, act)
            if act in ("none", "relu"):
                assert np.array_equal(y, y_ref), act
            else:
                yf, yr = O.to_f32(y).astype(np.float64), O.to_f32(y_ref).astype(np.float64)
                if t == "f32":
                    # (1 + erf) and (1 + tanh) cancel for negative gates: a last-bit difference
                    # of erff / tanhf is an absolute error of 2^-23 on that sum
                    slack = np.abs(O.to_f32(hidden).astype(np.float64) * O.to_f32(gate)) * 4e-7
                    assert (np.abs(yf - yr) <= 2e-6 * np.abs(yr) + slack + 1e-7).all(), act
                else:
                    # a last-bit difference of the activation moves act(gate) by one rounding of
                    # T and the product by about two
                    assert (np.abs(yf - yr) <= 2.0001 * H.ulp_of(yr, t) + 1e-7).all(), act
                    assert (yf != yr).mean() < 0.02, act


@pytest.mark.parametrize("m,n,k", [(1, 1000, 4096), (1, 11008, 4096), (1, 4100, 2048), (1, 5003, 1024),
                                   (1, 12000, 256), (1, 4097, 3840),
                                   (2, 344, 2048), (3, 136, 5120), (4, 2000, 4096),
                                   (5, 37, 3072), (8, 1100, 4096), (8, 33, 11008), (4, 65, 11008),
                                   (8, 11008, 4096), (16, 2000, 4096), (6, 1200, 8192)])
def test_glu_and_grouped_few_rows_of_x_symmetric_int4_fp16(m, n, k):
    """fp16, symmetric int4 in an int8 container, groups of 128, 1 .. 16 rows of x at real row
    lengths (the decode case of both ops; one row of x takes the kernels in which a wave owns
    whole weight rows -- one row or row pair per wave up to 4096 rows, beyond that a wave walks
    its rows, with rows of 1 and 2 KB of codes, row counts off the block sizes and a row that
    ends inside a KB; the last three shapes need two stagings of x in the GLU kernel, with one
    and with two blocks per CU).  Split GLU + a grouped call with three row counts on a shared
    x."""
    import torch
    import oneflow_amd as flow
    from oneflow_amd import _lib
    L = _lib.lib()
    rng = np.random.Generator(np.random.PCG64(m * 7 + n + k))
    x, w, ws, _, b = _problem(rng, m, n, k, 4, True, np.int8, 128, "f16")
    _, v, vs, _, c = _problem(rng, m, n, k, 4, True, np.int8, 128, "f16")
    for act in ("fast_gelu", "silu", "none"):
        y, wx, vx = _glu_call(L, _lib, torch, x, w, ws, None, b, v, vs, None, c, act, _lib.I8,
                              _lib.F16, 4, True, 128, m, n, k)
        r, _ = H.assert_linear_parity(wx, O.fused_linear(x, w, ws, None, b, 4, True, 1, 128), "f16", "wx")
        assert r < 5e-4
        r, _ = H.assert_linear_parity(vx, O.fused_linear(x, v, vs, None, c, 4, True, 1, 128), "f16", "vx")
        assert r < 5e-4
        y_ref = O.glu_gate(wx, vx, act)
        yf, yr = O.to_f32(y).astype(np.float64), O.to_f32(y_ref).astype(np.float64)
        assert (np.abs(yf - yr) <= 2.0001 * H.ulp_of(yr, "f16") + 1e-7).all(), act
    ns = (n, max(1, n // 4), n + 13)
    probs = [_problem(rng, m, nn, k, 4, True, np.int8, 128, "f16", bias=(i != 1))
             for i, nn in enumerate(ns)]
    tt = H.to_torch
    outs = flow._C.grouped_linear_with_groupwise_quantized_weight(
        [tt(x)] * 3, [tt(p[1]) for p in probs], [tt(p[2]) for p in probs], w_zeros=None,
        bs=[tt(p[4]) for p in probs], num_bits=4, symmetric=True, group_dim=1, group_size=128)
    for p, out in zip(probs, outs):
        ref = O.fused_linear(x, p[1], p[2], None, p[4], 4, True, 1, 128)
        r, _ = H.assert_linear_parity(H.to_numpy(out), ref, "f16", f"grouped n={p[1].shape[0]}")
        assert r < 5e-4


def test_glu_functional_matches_reference_style_composition():
    """flow._C.fused_glu_with_groupwise_quantized_weight against dequantize -> matmul -> gate in
    float64 (how the reference test builds its expectation, test_fused_glu.py:31-83), Llama
    gate/up width at m = 1, SiLU."""
    import oneflow_amd as flow
    rng = np.random.Generator(np.random.PCG64(9))
    m, n, k, g = 1, 11008, 512, 128
    x, w, ws, _, _ = _problem(rng, m, n, k, 4, True, np.int8, g, "f16", bias=False)
    _, v, vs, _, _ = _problem(rng, m, n, k, 4, True, np.int8, g, "f16", bias=False)
    tt = H.to_torch
    y = flow._C.fused_glu_with_groupwise_quantized_weight(
        tt(x), tt(w), tt(ws), v=tt(v), v_scale=tt(vs), activation="silu", num_bits=4,
        symmetric=True, group_dim=1, group_size=g)
    wd = O.groupwise_dequantize(w, ws, None, 4, True, 1, g).astype(np.float64)
    vd = O.groupwise_dequantize(v, vs, None, 4, True, 1, g).astype(np.float64)
    hx = x.astype(np.float64) @ wd.T
    gx = x.astype(np.float64) @ vd.T
    want = hx * (gx / (1 + np.exp(-gx)))
    got = H.to_numpy(y).astype(np.float64)
    assert H.rel_l2(got, want) < 2e-3
    with pytest.raises(flow.CheckFailedError):
        flow._C.fused_glu_with_groupwise_quantized_weight(tt(x), tt(w), tt(ws), c=tt(x[0]))


def test_module_wrappers():
    """nn.QuantizedGLU and nn.GroupedQuantizedLinear give what their QuantizedLinear parts give
    one by one (the linears agree up to summation order, the gating is then applied to them)."""
    import torch
    import oneflow_amd as flow
    torch.manual_seed(3)
    k, n = 512, 384
    lin = [torch.nn.Linear(k, nn_, bias=True).half().cuda() for nn_ in (n, n, 128)]
    x = torch.randn(3, k, dtype=torch.float16, device="cuda")
    q = [flow.nn.QuantizedLinear.from_float(l, num_bits=4, symmetric=False, group_size=128,
                                            quant_type=torch.uint8) for l in lin]
    outs = flow.nn.GroupedQuantizedLinear(q)(x)
    for o, m in zip(outs, q):
        assert H.rel_l2(H.to_numpy(o), H.to_numpy(m(x))) < 1e-3
    glu = flow.nn.QuantizedGLU(q[0], q[1], activation="silu")
    y = glu(x)
    ref = O.glu_gate(H.to_numpy(q[0](x)), H.to_numpy(q[1](x)), "silu")
    assert H.rel_l2(H.to_numpy(y), ref) < 2e-3
    with pytest.raises(ValueError):
        flow.nn.QuantizedGLU(q[0], q[2])
