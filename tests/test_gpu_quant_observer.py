"""min_max_observer / quantization / fake_quantization on the GPU against the oracle.
Bars: codes bit-exact; scale and zero_point within 1 ulp (they are in fact identical: max/min are
exact and the division is correctly rounded on both sides)."""
import numpy as np
import pytest

import helpers as H
from oracle import ofq_oracle as O

pytestmark = pytest.mark.gpu


def _bits(a):
    return a.view(np.uint32) if a.dtype == np.float32 else a.view(np.uint64)


def _ulp_diff(a, b):
    ia = _bits(a).astype(np.int64)
    ib = _bits(b).astype(np.int64)
    return int(np.abs(ia - ib).max())


def _same_values_and_nan(a, b):
    """bit-exact including the sign of zero; NaNs must coincide."""
    na, nb = np.isnan(a), np.isnan(b)
    return np.array_equal(na, nb) and np.array_equal(_bits(a)[~na], _bits(b)[~nb])


# shapes/attribute grid of the reference tests (test_min_max_observer.py:137-148)
@pytest.mark.parametrize("shape", [(9, 40, 20, 10), (4096, 64), (3, 5), (300001,), (2, 700000), (70000, 3)])
@pytest.mark.parametrize("bits", [8, 4, 2])
@pytest.mark.parametrize("scheme", ["symmetric", "affine"])
@pytest.mark.parametrize("per_layer", [True, False])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_observer_quantize_fake(shape, bits, scheme, per_layer, dtype):
    import oneflow_amd as flow
    if len(shape) == 1 and not per_layer and scheme == "affine":
        pytest.skip("one-element channels: the affine scale is (max - min) / .. = 0, and what "
                    "follows is 0/0 in the reference too")
    rng = np.random.Generator(np.random.PCG64(hash((shape, bits, scheme, per_layer)) % 2**32))
    x = (rng.random(shape) - 0.5).astype(dtype)
    s_ref, z_ref = O.min_max_observer(x, "google", bits, scheme, per_layer)
    xt = H.to_torch(x)
    s, z = flow._C.min_max_observer(xt, "google", bits, scheme, per_layer)
    s_np, z_np = H.to_numpy(s), H.to_numpy(z)
    assert s_np.shape == s_ref.shape
    assert _ulp_diff(s_np, s_ref) <= 1 and _ulp_diff(z_np, z_ref) <= 1
    assert np.array_equal(_bits(s_np), _bits(s_ref)) and np.array_equal(z_np, z_ref)
    for zp_mode_gpu, zp_mode_ref in (("uint8", "cpu"), ("float", "cuda")):
        q_ref = O.quantization(x, s_ref, z_ref, "google", bits, scheme, zp_mode=zp_mode_ref)
        q = H.to_numpy(flow._C.quantization(xt, s, z, "google", bits, scheme, zp_mode=zp_mode_gpu))
        assert _same_values_and_nan(q, q_ref)
        f_ref = O.fake_quantization(x, s_ref, z_ref, "google", bits, scheme, zp_mode=zp_mode_ref)
        f = H.to_numpy(flow._C.fake_quantization(xt, s, z, "google", bits, scheme,
                                                 zp_mode=zp_mode_gpu))
        assert _same_values_and_nan(f, f_ref)


def test_config1_weight_4096():
    """fp32 weight [4096,4096] ~N(0,0.02): per-channel symmetric 8-bit observer, quantization and
    the fake-quantization round trip; codes bit-exact, scales identical."""
    import oneflow_amd as flow
    w = (H.rng_for(1, 0).standard_normal((4096, 4096)) * 0.02).astype(np.float32)
    s_ref, z_ref = O.min_max_observer(w, "google", 8, "symmetric", False)
    wt = H.to_torch(w)
    s, z = flow._C.min_max_observer(wt, "google", 8, "symmetric", False)
    assert np.array_equal(H.to_numpy(s).view(np.uint32), s_ref.view(np.uint32))
    assert np.array_equal(H.to_numpy(z), z_ref)
    q = H.to_numpy(flow._C.quantization(wt, s, z, "google", 8, "symmetric"))
    q_ref = O.quantization(w, s_ref, z_ref, "google", 8, "symmetric")
    assert np.array_equal(q.view(np.uint32), q_ref.view(np.uint32))
    f = H.to_numpy(flow._C.fake_quantization(wt, s, z, "google", 8, "symmetric"))
    f_ref = O.fake_quantization(w, s_ref, z_ref, "google", 8, "symmetric")
    assert np.array_equal(f.view(np.uint32), f_ref.view(np.uint32))
    # size-independent properties: codes integral, in range, each row's absmax maps to +-127,
    # |w/s - code| <= 0.5, and the int8 output option narrows the same codes
    assert np.array_equal(q, np.rint(q)) and q.min() >= -128 and q.max() <= 127
    assert np.array_equal(np.abs(q).max(axis=1), np.full(4096, 127.0, np.float32))
    # (the fp32 quotient carries up to 127 * 2^-24 of rounding error)
    assert np.abs(w.astype(np.float64) / s_ref[:, None].astype(np.float64) - q).max() <= 0.5 + 127 * 2.0 ** -23
    import torch
    q8 = flow._C.quantization(wt, s, z, "google", 8, "symmetric", out_dtype=torch.int8)
    assert np.array_equal(H.to_numpy(q8).astype(np.float32), q)


def test_round_half_even_and_known_answers():
    """Tie vectors and the known-answer row of the reference's CPU kernels."""
    import oneflow_amd as flow
    x = np.array([0.5, 1.5, 2.5, -2.5, -0.5, 3.5, -1.5, 126.5, 127.5, 200.0, -128.5, -300.0],
                 dtype=np.float32)
    one = H.to_torch(np.ones(1, np.float32))
    zero = H.to_torch(np.zeros(1, np.float32))
    q = H.to_numpy(flow._C.quantization(H.to_torch(x), one, zero, "google", 8, "symmetric"))
    expect = np.array([0, 2, 2, -2, -0.0, 4, -2, 126, 127, 127, -128, -128], dtype=np.float32)
    assert np.array_equal(q.view(np.uint32), expect.view(np.uint32))
    inp = np.array([[0.5, -1.0, 0.25, 0.3], [2.5, 1.5, -0.5, 0.1]], dtype=np.float32)
    s, z = flow._C.min_max_observer(H.to_torch(inp), "google", 8, "symmetric", False)
    assert [float(v).hex() for v in H.to_numpy(s)] == ["0x1.0204080000000p-7", "0x1.42850a0000000p-6"]
    q = H.to_numpy(flow._C.quantization(H.to_torch(inp), s, z, "google", 8, "symmetric"))
    assert q.ravel().tolist() == [64, -127, 32, 38, 127, 76, -25, 5]


def test_cambricon_and_all_zero_channel():
    import oneflow_amd as flow
    x = np.array([[0.3, -6.0, 2.0, 1.0]], dtype=np.float32)
    s_ref, z_ref = O.min_max_observer(x, "cambricon", 8, "symmetric", True)
    s, z = flow._C.min_max_observer(H.to_torch(x), "cambricon", 8, "symmetric", True)
    assert np.array_equal(H.to_numpy(s), s_ref) and s_ref[0] == np.floor(np.log2(6.0)) - 6
    q_ref = O.quantization(x, s_ref, z_ref, "cambricon", 8, "symmetric")
    q = H.to_numpy(flow._C.quantization(H.to_torch(x), s, z, "cambricon", 8, "symmetric"))
    assert np.array_equal(q, q_ref)
    # an all-zero channel has scale 0 and NaN codes, as in the reference (0/0)
    xz = np.zeros((2, 8), np.float32)
    xz[1] = 1.0
    s, z = flow._C.min_max_observer(H.to_torch(xz), "google", 8, "symmetric", False)
    q = H.to_numpy(flow._C.quantization(H.to_torch(xz), s, z, "google", 8, "symmetric"))
    assert np.isnan(q[0]).all() and np.array_equal(q[1], np.full(8, 127.0, np.float32))


@pytest.mark.parametrize("scheme", ["symmetric", "affine"])
@pytest.mark.parametrize("formula", ["google", "cambricon"])
@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_moving_average_observer_sequence(scheme, formula, dt):
    """A training sequence that crosses stop_update_after_iters, then eval mode: moving values,
    scale and zero point must equal the oracle's after every call (same values bit for bit: the
    extremes are exact and the scalar arithmetic is the oracle's)."""
    import torch
    import oneflow_amd as flow
    if formula == "cambricon" and scheme == "affine":
        pytest.skip("cambricon ignores the scheme")
    rng = np.random.Generator(np.random.PCG64(17))
    obs = flow.nn.MovingAverageMinMaxObserver(stop_update_after_iters=3, quantization_formula=formula,
                                              quantization_bit=8, quantization_scheme=scheme,
                                              momentum=0.9).cuda()
    rmax, rmin = np.zeros(1, dt), np.zeros(1, dt)
    for step in range(6):
        if step == 5:
            obs.eval()
        x = (rng.standard_normal((37, 1031)) * (1 + step)).astype(dt)
        st = torch.tensor([step], dtype=torch.int64, device="cuda")
        s, z = obs(H.to_torch(x), st)
        rs, rz = O.moving_average_min_max_observer(x, step, rmax, rmin, step < 5, 3, formula, 8,
                                                   scheme, 0.9)
        assert np.array_equal(H.to_numpy(obs.moving_max), rmax), step
        assert np.array_equal(H.to_numpy(obs.moving_min), rmin), step
        assert np.array_equal(H.to_numpy(s), rs) and np.array_equal(H.to_numpy(z), rz), step
    # the values froze after step 3
    assert np.array_equal(rmax, H.to_numpy(obs.moving_max))
    obs.reset_running_stats()
    assert float(obs.moving_max[0]) == 0.0


def test_moving_average_observer_large_and_checks():
    import torch
    import oneflow_amd as flow
    x = H.rng_for(9, 0).standard_normal((4096, 4096)).astype(np.float32)
    mmax = torch.zeros(1, device="cuda")
    mmin = torch.zeros(1, device="cuda")
    st = torch.zeros(1, dtype=torch.int64, device="cuda")
    s, z = flow._C.moving_average_min_max_observer(H.to_torch(x), st, mmax, mmin, True, 1, "google",
                                                   8, "affine", 0.95)
    assert float(mmax[0]) == float(x.max()) and float(mmin[0]) == float(x.min())
    assert np.float32(s.item()) == (x.max() - x.min()) / np.float32(255.0)
    with pytest.raises(flow.CheckFailedError):
        flow._C.moving_average_min_max_observer(H.to_torch(x), st, mmax, mmin, True, 0, "google", 8,
                                                "affine", 0.95)
    with pytest.raises(flow.CheckFailedError):
        flow._C.moving_average_min_max_observer(H.to_torch(x), st.to(torch.int32), mmax, mmin, True, 1,
                                                "google", 8, "affine", 0.95)


def test_fake_quantization_straight_through_gradient():
    """in_grad = out_grad, no gradient for scale / zero_point
    (core/autograd/gradient_funcs/fake_quantization.cpp:36-42)."""
    import torch
    import oneflow_amd as flow
    x = torch.randn((64, 256), device="cuda", requires_grad=True)
    s, z = flow._C.min_max_observer(x.detach(), "google", 8, "symmetric", False)
    y = flow._C.fake_quantization(x, s, z, "google", 8, "symmetric")
    assert y.requires_grad
    g = torch.randn_like(y)
    y.backward(g)
    assert torch.equal(x.grad, g)
    with torch.no_grad():
        y2 = flow._C.fake_quantization(x, s, z, "google", 8, "symmetric")
    assert not y2.requires_grad and torch.equal(y2, y.detach())


@pytest.mark.parametrize("per_layer", [True, False])
@pytest.mark.parametrize("scheme", ["symmetric", "affine"])
def test_qat_conv_is_the_convolution_of_the_fake_quantized_operands(per_layer, scheme):
    """python/oneflow/nn/qat/conv.py: QatConv2d = conv(fake_quant(x; moving-average observer),
    fake_quant(w; min/max observer)).  The fake-quantized operands are checked bit for bit against
    the oracle's observers and fake quantization, the output against the host framework's
    convolution on those operands, and the gradient passes straight through to x and w."""
    import torch
    import oneflow_amd as flow
    rng = np.random.default_rng(3)
    conv = flow.qat.QatConv2d(4, 6, 3, padding=1, quantization_scheme=scheme,
                              weight_quant_per_layer=per_layer).cuda()
    x = torch.from_numpy(rng.standard_normal((2, 4, 8, 8)).astype(np.float32)).cuda().requires_grad_()
    conv.train()
    y = conv(x)
    xn, wn = x.detach().cpu().numpy(), conv.weight.detach().cpu().numpy()
    # input: first training step of the moving-average observer = the tensor's own extremes
    s_in, z_in = O.moving_average_min_max_observer(
        xn, 0, np.zeros(1, np.float32), np.zeros(1, np.float32), True, 1, "google", 8, scheme, 0.95)
    x_fq = O.fake_quantization(xn, s_in, z_in, "google", 8, scheme, zp_mode="cuda")
    s_w, z_w = O.min_max_observer(wn, "google", 8, scheme, per_layer)
    w_fq = O.fake_quantization(wn, s_w, z_w, "google", 8, scheme, zp_mode="cuda")
    want = torch.nn.functional.conv2d(torch.from_numpy(x_fq).cuda(), torch.from_numpy(w_fq).cuda(),
                                      conv.bias.detach(), padding=1)
    assert torch.allclose(y.detach(), want, rtol=1e-5, atol=1e-5)
    y.sum().backward()
    assert x.grad is not None and conv.weight.grad is not None
    # straight-through: d y / d x = conv_transpose of ones with the fake-quantized weight
    xx = x.detach().clone().requires_grad_()
    torch.nn.functional.conv2d(xx, torch.from_numpy(w_fq).cuda(), None, padding=1).sum().backward()
    assert torch.allclose(x.grad, xx.grad, rtol=1e-5, atol=1e-5)
