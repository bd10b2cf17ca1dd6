"""Every op of the path inside a captured HIP graph (the runtime captures user kernels that derive
CudaGraphSupport, oneflow/core/kernel/user_kernel.cpp:714-734): the graph is replayed several
times with new input contents, with eager work and synchronisations between the replays, and
every replay must equal the eager result on the same inputs bit for bit."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu


def _capture_and_check(make_inputs, run, n_replays=3):
    """make_inputs(seed) -> list of torch tensors (same shapes every time); run(*inputs) ->
    tensor or tuple of tensors."""
    import torch
    static = [t.clone() for t in make_inputs(0)]
    run(*static)  # warm-up outside capture (first-launch attribute calls, allocator growth)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = run(*static)
    outs = out if isinstance(out, (tuple, list)) else (out,)
    for seed in range(1, n_replays + 1):
        fresh = make_inputs(seed)
        for s, f in zip(static, fresh):
            s.copy_(f)
        g.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs if o is not None]
        eager = run(*fresh)  # eager work between replays, on the same inputs
        eager = eager if isinstance(eager, (tuple, list)) else (eager,)
        eager = [e for e in eager if e is not None]
        torch.cuda.synchronize()
        assert len(got) == len(eager)
        for a, b in zip(got, eager):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), seed


def _t(a):
    return H.to_torch(a)


def test_dequantize_and_weight_quantize_in_a_graph():
    import oneflow_amd as flow

    def inputs(seed):
        rng = H.rng_for(20, seed)
        return [_t((rng.standard_normal((256, 512)) * 0.05).astype(np.float16))]

    def run(w):
        q, s, z = flow.quantize.groupwise_quantize(w, num_bits=4, symmetric=False, group_dim=1,
                                                   group_size=64, quant_type=__import__("torch").uint8)
        d = flow._C.groupwise_dequantize(q, s, zero=z, num_bits=4, symmetric=False, group_dim=1,
                                         group_size=64)
        return q, s, z, d
    _capture_and_check(inputs, run)


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (8, 11008, 4096), (1, 11008, 4096), (200, 512, 512),
                                   (1100, 704, 512)])
def test_fused_linear_in_a_graph(m, n, k):
    import oneflow_amd as flow
    rng = H.rng_for(21, 0)
    codes = rng.integers(-8, 8, size=(n, k)).astype(np.int8)
    w = _t(H.pack_int4(codes))
    scale = _t(rng.uniform(1e-3, 1e-2, size=(n, k // 128)).astype(np.float16))
    b = _t((rng.standard_normal(n) * 0.01).astype(np.float16))

    def inputs(seed):
        return [_t(H.rng_for(22, seed).standard_normal((m, k)).astype(np.float16))]

    def run(x):
        return flow._C.fused_linear_with_groupwise_quantized_weight(
            x, w, scale, b=b, num_bits=4, symmetric=True, group_dim=1, group_size=128)
    _capture_and_check(inputs, run)


@pytest.mark.parametrize("m", [1, 40, 100])
def test_fused_linear_groups_along_n_in_a_graph(m):
    """group_dim = 0: the streaming kernel (m <= 64) and, beyond, dequantise + copy-fed GEMM in the
    workspace the Python layer allocates before capture."""
    import oneflow_amd as flow
    rng = H.rng_for(27, 0)
    n, k, g = 512, 512, 64
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    w, scale, zero = H.quantize_groupwise(wf, 4, False, 0, g, np.uint8, "f16")
    w, scale, zero = _t(w), _t(scale), _t(zero)

    def inputs(seed):
        return [_t(H.rng_for(28, seed).standard_normal((m, k)).astype(np.float16))]

    def run(x):
        return flow._C.fused_linear_with_groupwise_quantized_weight(
            x, w, scale, w_zero=zero, num_bits=4, symmetric=False, group_dim=0, group_size=g)
    _capture_and_check(inputs, run)


@pytest.mark.parametrize("rows", [300, 4])
def test_dynamic_int8_chain_in_a_graph(rows):
    """LayerNorm+observer -> quantization to int8 -> matmul_quant, captured as one graph."""
    import torch
    import oneflow_amd as flow
    cols, n = 1024, 704   # 4 rows: the streaming int8 kernel; 300: the tiled GEMM
    rng = H.rng_for(23, 0)
    gamma = _t((1 + 0.1 * rng.standard_normal(cols)).astype(np.float16))
    beta = _t((0.1 * rng.standard_normal(cols)).astype(np.float16))
    wq = _t(rng.integers(-127, 128, size=(n, cols)).astype(np.int8))
    wscale = _t(rng.uniform(1e-3, 1e-2, size=n).astype(np.float32))

    def inputs(seed):
        return [_t(H.rng_for(24, seed).standard_normal((rows, cols)).astype(np.float16))]

    def run(x):
        y, s, z = flow._C.fused_layer_norm_min_max_observer(x, gamma, beta, 1e-5, 8)
        a = flow._C.quantization(y, s, z, "google", 8, "symmetric", out_dtype=torch.int8)
        o = flow._C.matmul_quant(a, wq, s, wscale, None, torch.float16)
        return y, s, a, o
    _capture_and_check(inputs, run)


def test_observers_and_fake_quant_in_a_graph():
    import oneflow_amd as flow

    def inputs(seed):
        return [_t((H.rng_for(25, seed).standard_normal((64, 4100)) * (seed + 1)).astype(np.float32))]

    def run(x):
        s, z = flow._C.min_max_observer(x, "google", 8, "affine", False)
        q = flow._C.quantization(x, s, z, "google", 8, "affine")
        f = flow._C.fake_quantization(x, s, z, "google", 8, "affine")
        return s, z, q, f
    _capture_and_check(inputs, run)


def test_moving_average_observer_in_a_graph():
    """The step counter lives on the device, so a captured observer follows it from replay to
    replay: the moving values after each replay equal an eager module fed the same sequence."""
    import torch
    import oneflow_amd as flow
    cap = flow.nn.MovingAverageMinMaxObserver(stop_update_after_iters=2, momentum=0.8).cuda()
    ref = flow.nn.MovingAverageMinMaxObserver(stop_update_after_iters=2, momentum=0.8).cuda()
    x = torch.zeros((128, 256), device="cuda")
    step = torch.zeros(1, dtype=torch.int64, device="cuda")
    x.copy_(_t(H.rng_for(26, 100).standard_normal((128, 256)).astype(np.float32)))
    cap(x, step)                      # warm-up, then start both modules from scratch
    cap.reset_running_stats()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        s, z = cap(x, step)
    cap.reset_running_stats()
    for i in range(5):
        xi = _t((H.rng_for(26, i).standard_normal((128, 256)) * (i + 1)).astype(np.float32))
        x.copy_(xi)
        step.fill_(i)
        g.replay()
        torch.cuda.synchronize()
        rs, rz = ref(xi, torch.tensor([i], dtype=torch.int64, device="cuda"))
        torch.cuda.synchronize()
        assert torch.equal(cap.moving_max, ref.moving_max) and torch.equal(cap.moving_min, ref.moving_min), i
        assert torch.equal(s, rs) and torch.equal(z, rz), i


def test_grouped_glu_and_skip_layer_norm_in_a_graph():
    """The decoder-block neighbours: q/k/v as one grouped call, the gated unit, and the residual
    LayerNorm + observer, captured together."""
    import oneflow_amd as flow
    import torch
    k, g = 512, 128
    rng = H.rng_for(21, 0)
    ws = []
    for n in (512, 128, 128, 1376, 1376):
        codes = rng.integers(0, 256, size=(n, k // 2)).astype(np.uint8)
        sc = rng.uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float16)
        ze = rng.uniform(-0.08, -0.04, size=(n, k // g)).astype(np.float16)
        ws.append((_t(codes), _t(sc), _t(ze)))
    gamma = _t((1 + 0.1 * rng.standard_normal(k)).astype(np.float16))

    def inputs(seed):
        r = H.rng_for(22, seed)
        return [_t(r.standard_normal((2, k)).astype(np.float16)),
                _t(r.standard_normal((2, k)).astype(np.float16))]

    def run(x, skip):
        h, s, z = flow._C.fused_skip_layer_norm_min_max_observer(x, gamma, None, None, skip, 1e-5,
                                                                 1.0, 8)
        q, kk, v = flow._C.grouped_linear_with_groupwise_quantized_weight(
            [h, h, h], [w[0] for w in ws[:3]], [w[1] for w in ws[:3]],
            w_zeros=[w[2] for w in ws[:3]], num_bits=4, symmetric=False, group_dim=1, group_size=g)
        y = flow._C.fused_glu_with_groupwise_quantized_weight(
            h, ws[3][0], ws[3][1], w_zero=ws[3][2], v=ws[4][0], v_scale=ws[4][1], v_zero=ws[4][2],
            activation="silu", num_bits=4, symmetric=False, group_dim=1, group_size=g)
        return h, s, q, kk, v, y
    _capture_and_check(inputs, run)
