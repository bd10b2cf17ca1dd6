"""The C++ OneFlow adapter (oneflow_amd/plugin): registrations carry the reference's op names,
device/dtype predicates and tmp_buffer sizing; on the GPU, a kernel looked up from the registry and
run through a KernelComputeContext gives the same bits as the direct C-ABI call."""
import ctypes
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PLUGIN = os.path.join(ROOT, "oneflow_amd", "plugin", "libofq_oneflow_plugin.so")
# DataType / DeviceType values of oneflow/core/common/data_type.proto and device_type.proto
K_FLOAT, K_DOUBLE, K_INT8, K_UINT8, K_FLOAT16, K_BFLOAT16 = 2, 3, 4, 7, 9, 11
K_CPU, K_CUDA = 1, 2


@pytest.fixture(scope="module")
def plugin():
    if not os.path.exists(PLUGIN):
        pytest.fail(f"{PLUGIN} missing: run __graft_entry__.build()")
    return ctypes.CDLL(PLUGIN)


def test_registrations(plugin):
    n = plugin.ofq_plugin_registration_count()
    seen = {}
    for i in range(n):
        name = ctypes.create_string_buffer(128)
        prio, tmp = ctypes.c_int(), ctypes.c_int()
        assert plugin.ofq_plugin_registration_info(i, name, 128, ctypes.byref(prio), ctypes.byref(tmp)) == 0
        seen.setdefault(name.value.decode(), []).append((prio.value, tmp.value))
    assert set(seen) == {"groupwise_dequantize", "fused_linear_with_groupwise_quantized_weight",
                         "min_max_observer", "moving_average_min_max_observer", "quantization",
                         "fake_quantization", "fused_layer_norm_min_max_observer",
                         "fused_layer_norm_quantization", "matmul_quant",
                         "fused_glu_with_groupwise_quantized_weight",
                         "grouped_linear_with_groupwise_quantized_weight"}
    for name in ("fused_layer_norm_min_max_observer", "matmul_quant",
                 "fused_glu_with_groupwise_quantized_weight",
                 "grouped_linear_with_groupwise_quantized_weight"):
        assert len(seen[name]) == 3  # half, bfloat16, float
    assert all(t == 1 for _, t in seen["fused_layer_norm_min_max_observer"])
    assert all(t == 1 for _, t in seen["matmul_quant"])   # K slices at 64 < m
    assert len(seen["groupwise_dequantize"]) == 3 and len(seen["min_max_observer"]) == 2
    assert len(seen["moving_average_min_max_observer"]) == 2
    # every kernel outranks a stock registration (priority 0); the observers and the fused linear
    # (dequantised weight at large m) declare a tmp_buffer
    assert all(p == 10 for v in seen.values() for p, _ in v)
    assert all(t == 1 for _, t in seen["min_max_observer"] + seen["moving_average_min_max_observer"])
    assert all(t == 1 for _, t in seen["fused_linear_with_groupwise_quantized_weight"])
    assert all(t == 0 for _, t in seen["quantization"] + seen["groupwise_dequantize"])
    has = plugin.ofq_plugin_has_kernel
    assert has(b"groupwise_dequantize", K_CUDA, b"scale", K_FLOAT16) == 1
    assert has(b"groupwise_dequantize", K_CUDA, b"scale", K_BFLOAT16) == 1
    assert has(b"groupwise_dequantize", K_CPU, b"scale", K_FLOAT16) == 0
    assert has(b"groupwise_dequantize", K_CUDA, b"scale", K_DOUBLE) == 0
    assert has(b"fused_linear_with_groupwise_quantized_weight", K_CUDA, b"out", K_FLOAT16) == 1
    assert has(b"quantization", K_CUDA, b"in", K_DOUBLE) == 1
    assert has(b"quantization", K_CUDA, b"in", K_FLOAT16) == 0
    assert has(b"matmul", K_CUDA, b"out", K_FLOAT16) == 0
    assert has(b"matmul_quant", K_CUDA, b"out", K_FLOAT16) == 1
    assert has(b"matmul_quant", K_CUDA, b"out", K_DOUBLE) == 0
    assert has(b"fused_layer_norm_min_max_observer", K_CUDA, b"y", K_BFLOAT16) == 1
    assert has(b"grouped_linear_with_groupwise_quantized_weight", K_CPU, b"ys", K_FLOAT16) == 0
    plugin.ofq_plugin_observer_tmp_bytes.restype = ctypes.c_longlong
    shape = (ctypes.c_longlong * 2)(4096, 4096)
    assert plugin.ofq_plugin_observer_tmp_bytes(K_FLOAT, shape, 2, 0) == 4096 * 2 * 4
    assert plugin.ofq_plugin_observer_tmp_bytes(K_FLOAT, shape, 2, 1) == (4096 * 4096 // 4096) * 2 * 4  # one (min, max) pair per 4096-element slice
    # fused linear: a tmp_buffer for the dequantised weight at large m, for fp32 partial sums of
    # K slices at mid-size m with few output tiles, none for decode
    ll = ctypes.c_longlong
    plugin.ofq_plugin_fused_linear_tmp_bytes.restype = ll
    plugin.ofq_plugin_fused_linear_tmp_bytes.argtypes = [ctypes.c_int] * 2 + [ll] * 3 + [ctypes.c_int] * 2 + [ll] * 2
    tmp = plugin.ofq_plugin_fused_linear_tmp_bytes
    assert tmp(K_BFLOAT16, K_UINT8, 2048, 11008, 4096, 8, 0, 1, 64) == 11008 * 4096 * 2
    assert tmp(K_FLOAT16, K_INT8, 1, 4096, 4096, 4, 1, 1, 128) == 0
    assert tmp(K_FLOAT16, K_INT8, 128, 4096, 4096, 4, 1, 1, 128) == 8 * 128 * 4096 * 4
    assert tmp(K_FLOAT16, K_INT8, 64, 4096, 4096, 4, 1, 1, 128) == 0
    assert tmp(K_FLOAT16, K_INT8, 16, 4096, 4096, 4, 1, 1, 128) == 0
    assert tmp(K_FLOAT, K_UINT8, 2048, 4096, 4096, 8, 0, 1, 64) == 0


@pytest.mark.gpu
def test_fused_linear_through_the_adapter(plugin):
    import torch
    import helpers as H
    import oneflow_amd as flow
    rng = np.random.default_rng(11)
    m, n, k, g = 4, 512, 1024, 128
    x = rng.standard_normal((m, k)).astype(np.float16)
    w = H.pack_int4(rng.integers(-7, 8, size=(n, k)).astype(np.int8))
    scale = rng.uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float16)
    b = (rng.standard_normal(n) * 0.01).astype(np.float16)
    xt, wt, st, bt = map(H.to_torch, (x, w, scale, b))
    direct = flow._C.fused_linear_with_groupwise_quantized_weight(
        xt, wt, st, b=bt, num_bits=4, symmetric=True, group_dim=1, group_size=g)
    out = torch.empty_like(direct)
    vp, ll = ctypes.c_void_p, ctypes.c_longlong
    plugin.ofq_plugin_run_fused_linear.argtypes = [vp] * 7 + [ctypes.c_int] * 2 + [ll] * 3 + [ctypes.c_int] * 2 + [ll] * 2
    rc = plugin.ofq_plugin_run_fused_linear(
        torch.cuda.current_stream().cuda_stream, xt.data_ptr(), wt.data_ptr(), st.data_ptr(), None,
        bt.data_ptr(), out.data_ptr(), K_FLOAT16, K_INT8, m, n, k, 4, 1, 1, g)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(out, direct)


@pytest.mark.gpu
def test_dynamic_int8_ops_through_the_adapter(plugin):
    """fused_layer_norm_min_max_observer (plain and with the skip_layer_norm inputs) and
    matmul_quant looked up from the registry and run through a KernelComputeContext: the same bits
    as the direct calls."""
    import torch
    import helpers as H
    import oneflow_amd as flow
    rng = np.random.default_rng(12)
    rows, cols = 64, 1024
    x = H.to_torch(rng.standard_normal((rows, cols)).astype(np.float16))
    skip = H.to_torch(rng.standard_normal((rows, cols)).astype(np.float16))
    gamma = H.to_torch((1 + 0.1 * rng.standard_normal(cols)).astype(np.float16))
    beta = H.to_torch((0.1 * rng.standard_normal(cols)).astype(np.float16))
    vp, ll, dbl, ci = ctypes.c_void_p, ctypes.c_longlong, ctypes.c_double, ctypes.c_int
    run = plugin.ofq_plugin_run_layer_norm_observer
    run.argtypes = [vp] * 6 + [dbl] + [vp] * 4 + [ll, ci, ll, ll, dbl, ci]
    stream = torch.cuda.current_stream().cuda_stream
    for sk in (None, skip):
        if sk is None:
            want = flow._C.fused_layer_norm_min_max_observer(x, gamma, beta, 1e-5, 8)
        else:
            want = flow._C.fused_skip_layer_norm_min_max_observer(x, gamma, beta, None, sk, 1e-5, 0.5, 8)
        y = torch.empty_like(x)
        s = torch.empty(1, dtype=torch.float32, device="cuda")
        z = torch.empty(1, dtype=torch.float32, device="cuda")
        tmp = torch.empty(rows * 4, dtype=torch.uint8, device="cuda")
        rc = run(stream, x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), None,
                 sk.data_ptr() if sk is not None else None, 0.5, y.data_ptr(), s.data_ptr(),
                 z.data_ptr(), tmp.data_ptr(), rows * 4, K_FLOAT16, rows, cols, 1e-5, 8)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(y, want[0]) and torch.equal(s, want[1]) and torch.equal(z, want[2])
    # LayerNorm -> int8 codes as one op: the shapes the library serves with its two kernels, and
    # one it does not (the kernel class then runs the two ops inside the op's tmp_buffer)
    lnq = plugin.ofq_plugin_run_layer_norm_quantization
    lnq.argtypes = [vp] * 8 + [ll, ci, ll, ll, dbl, ci]
    tmpb = plugin.ofq_plugin_ln_quantization_tmp_bytes
    tmpb.argtypes = [ci, ll, ll]
    tmpb.restype = ll
    for r2, c2 in ((64, 1024), (9, 1000)):
        x2 = H.to_torch(rng.standard_normal((r2, c2)).astype(np.float16))
        g2 = H.to_torch((1 + 0.1 * rng.standard_normal(c2)).astype(np.float16))
        b2 = H.to_torch((0.1 * rng.standard_normal(c2)).astype(np.float16))
        y2, s2, z2 = flow._C.fused_layer_norm_min_max_observer(x2, g2, b2, 1e-5, 8)
        want = flow._C.quantization(y2, s2, z2, "google", 8, "symmetric", out_dtype=torch.int8)
        nbytes = tmpb(K_FLOAT16, r2, c2)
        assert nbytes >= r2 * c2 * 2
        tmp = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        codes = torch.full((r2, c2), 99, dtype=torch.int8, device="cuda")
        s = torch.empty(1, dtype=torch.float32, device="cuda")
        z = torch.empty(1, dtype=torch.float32, device="cuda")
        rc = lnq(stream, x2.data_ptr(), g2.data_ptr(), b2.data_ptr(), codes.data_ptr(), s.data_ptr(),
                 z.data_ptr(), tmp.data_ptr(), nbytes, K_FLOAT16, r2, c2, 1e-5, 8)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(codes, want) and torch.equal(s, s2) and z.item() == 0.0
    m, n, k = 48, 200, 256
    a = H.to_torch(rng.integers(-128, 128, size=(m, k)).astype(np.int8))
    b = H.to_torch(rng.integers(-127, 128, size=(n, k)).astype(np.int8))
    a_s = H.to_torch(np.array([0.02], np.float32))
    b_s = H.to_torch(rng.uniform(1e-3, 1e-2, size=n).astype(np.float32))
    want = flow._C.matmul_quant(a, b, a_s, b_s, None, torch.float16)
    out = torch.empty_like(want)
    mq = plugin.ofq_plugin_run_matmul_quant
    mq.argtypes = [vp] * 7 + [ci, ll, ll, ll]
    assert mq(stream, a.data_ptr(), b.data_ptr(), a_s.data_ptr(), b_s.data_ptr(), None,
              out.data_ptr(), K_FLOAT16, m, n, k) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, want)


@pytest.mark.gpu
def test_grouped_linear_through_the_adapter(plugin):
    import torch
    import helpers as H
    import oneflow_amd as flow
    rng = np.random.default_rng(13)
    m, k, g, ns = 2, 512, 128, (256, 64, 64)
    x = H.to_torch(rng.standard_normal((m, k)).astype(np.float16))
    ws = [H.to_torch(rng.integers(-128, 128, size=(n, k // 2)).astype(np.int8)) for n in ns]
    scs = [H.to_torch(rng.uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float16)) for n in ns]
    want = flow._C.grouped_linear_with_groupwise_quantized_weight(
        [x] * 3, ws, scs, num_bits=4, symmetric=True, group_dim=1, group_size=g)
    outs = [torch.empty_like(w) for w in want]
    vp, ll, ci = ctypes.c_void_p, ctypes.c_longlong, ctypes.c_int
    arr = lambda ts: (vp * 3)(*[t.data_ptr() for t in ts])
    run = plugin.ofq_plugin_run_grouped_linear
    run.argtypes = [vp, ci, vp, vp, vp, vp, vp, ci, ci, ll, ll, ci, ll]
    rc = run(torch.cuda.current_stream().cuda_stream, 3, x.data_ptr(), arr(ws), arr(scs), arr(outs),
             (ll * 3)(*ns), K_FLOAT16, K_INT8, m, k, 4, g)
    assert rc == 0
    torch.cuda.synchronize()
    for o, w in zip(outs, want):
        assert torch.equal(o, w)


def _bind_stream_hooks(plugin):
    vp, ci, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    protos = {
        "ofq_plugin_stream_new": (vp, [ci]), "ofq_plugin_stream_view": (vp, [ci, vp]),
        "ofq_plugin_stream_delete": (None, [vp]), "ofq_plugin_stream_raw": (vp, [vp]),
        "ofq_plugin_stream_device_type": (ci, [vp]),
        "ofq_plugin_stream_sync": (ci, [vp, ctypes.c_char_p, ci]),
        "ofq_plugin_stream_get_async_error": (ci, [vp, ctypes.c_char_p, ci]),
        "ofq_plugin_stream_on_execution_context_setup": (ci, [vp]),
        "ofq_plugin_stream_cu_count": (ci, [vp]),
        "ofq_plugin_stream_grid_with_waves": (ctypes.c_uint, [vp, sz, sz, sz]),
        "ofq_plugin_event_new": (vp, []), "ofq_plugin_event_delete": (None, [vp]),
        "ofq_plugin_stream_record_event": (None, [vp, vp]),
        "ofq_plugin_stream_wait_event": (None, [vp, vp]),
        "ofq_plugin_event_query_done": (ci, [vp]), "ofq_plugin_event_sync": (ci, [vp]),
        "ofq_plugin_last_async_error": (ci, [ctypes.c_char_p, ci]),
    }
    for name, (res, args) in protos.items():
        f = getattr(plugin, name)
        f.restype, f.argtypes = res, args


def test_stream_hooks_are_exported(plugin):
    _bind_stream_hooks(plugin)


@pytest.mark.gpu
def test_hip_stream_behind_ep_cuda_stream(plugin):
    """ep::CudaStream / ep::CudaEvent over HIP (oneflow_amd/plugin/ep_hip): a stream of its own,
    a registered kernel run on it through a KernelComputeContext, RecordEvent / QueryDone / Sync,
    WaitEvent from a second stream, the CU count and the launch-size helper built on it, and
    OnExecutionContextSetup."""
    import torch
    import helpers as H
    import oneflow_amd as flow
    _bind_stream_hooks(plugin)
    dev = torch.cuda.current_device()
    rng = np.random.default_rng(21)
    m, n, k, g = 1, 2048, 4096, 128
    x = rng.standard_normal((m, k)).astype(np.float16)
    w = H.pack_int4(rng.integers(-7, 8, size=(n, k)).astype(np.int8))
    scale = rng.uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float16)
    xt, wt, st = map(H.to_torch, (x, w, scale))
    direct = flow._C.fused_linear_with_groupwise_quantized_weight(
        xt, wt, st, num_bits=4, symmetric=True, group_dim=1, group_size=g)
    torch.cuda.synchronize()
    s1 = plugin.ofq_plugin_stream_new(dev)
    s2 = plugin.ofq_plugin_stream_new(dev)
    ev = plugin.ofq_plugin_event_new()
    try:
        assert plugin.ofq_plugin_stream_device_type(s1) == K_CUDA
        assert plugin.ofq_plugin_stream_on_execution_context_setup(s1) == 0
        raw1 = plugin.ofq_plugin_stream_raw(s1)
        assert raw1 and raw1 != plugin.ofq_plugin_stream_raw(s2)
        cus = plugin.ofq_plugin_stream_cu_count(s1)
        assert cus == torch.cuda.get_device_properties(dev).multi_processor_count == 256
        # InitLaunchConfigWithWaves (cuda_stream.h:116-124): min(waves * CUs * threads/CU / block,
        # blocks needed)
        tpc = torch.cuda.get_device_properties(dev).max_threads_per_multi_processor
        assert plugin.ofq_plugin_stream_grid_with_waves(s1, 1 << 30, 256, 32) == 32 * cus * (tpc // 256)
        assert plugin.ofq_plugin_stream_grid_with_waves(s1, 1000, 256, 32) == 4
        out = torch.empty_like(direct)
        vp, ll = ctypes.c_void_p, ctypes.c_longlong
        run = plugin.ofq_plugin_run_fused_linear
        run.argtypes = [vp] * 7 + [ctypes.c_int] * 2 + [ll] * 3 + [ctypes.c_int] * 2 + [ll] * 2
        assert run(raw1, xt.data_ptr(), wt.data_ptr(), st.data_ptr(), None, None, out.data_ptr(),
                   K_FLOAT16, K_INT8, m, n, k, 4, 1, 1, g) == 0
        plugin.ofq_plugin_stream_record_event(s1, ev)
        # the second stream waits for the event, then runs the same kernel into a second buffer
        plugin.ofq_plugin_stream_wait_event(s2, ev)
        out2 = torch.empty_like(direct)
        assert run(plugin.ofq_plugin_stream_raw(s2), xt.data_ptr(), wt.data_ptr(), st.data_ptr(),
                   None, None, out2.data_ptr(), K_FLOAT16, K_INT8, m, n, k, 4, 1, 1, g) == 0
        assert plugin.ofq_plugin_event_sync(ev) == 0
        assert plugin.ofq_plugin_event_query_done(ev) == 1
        assert torch.equal(out, direct)   # the event has completed, so the first kernel has
        buf = ctypes.create_string_buffer(256)
        assert plugin.ofq_plugin_stream_sync(s2, buf, 256) == 0
        assert torch.equal(out2, direct)
        assert plugin.ofq_plugin_stream_get_async_error(s1, buf, 256) == 0
    finally:
        plugin.ofq_plugin_event_delete(ev)
        plugin.ofq_plugin_stream_delete(s1)   # synchronises and destroys its stream
        plugin.ofq_plugin_stream_delete(s2)


@pytest.mark.gpu
def test_errors_of_the_device_runtime_surface_through_get_async_error(plugin):
    """CudaStream::GetAsyncError is the device runtime's last error, cleared by the query
    (cuda_stream.cpp:240-247).  The error is made on the host (a device ordinal that does not
    exist): nothing faulty reaches the GPU.  Two routes: the stream is asked directly; and a
    kernel of the library runs in between -- its launch check reads the runtime's record, the
    C ABI reports OFQ_ERR_LAUNCH, and the runtime's query after Compute
    (stateful_opkernel.cpp:1007) still gets the error."""
    import torch
    import helpers as H
    from oneflow_amd import _lib
    _bind_stream_hooks(plugin)
    L = ctypes.CDLL(_lib.lib()._name)
    dev = torch.cuda.current_device()
    view = plugin.ofq_plugin_stream_view(dev, torch.cuda.current_stream().cuda_stream)
    buf = ctypes.create_string_buffer(256)
    try:
        assert plugin.ofq_plugin_stream_get_async_error(view, buf, 256) == 0
        assert L.ofq_hip_set_device(9999) != 0
        assert plugin.ofq_plugin_stream_get_async_error(view, buf, 256) == -1
        assert b"invalid device" in buf.value.lower()
        assert plugin.ofq_plugin_stream_get_async_error(view, buf, 256) == 0   # cleared by the query

        rng = np.random.default_rng(22)
        m, n, k, g = 1, 256, 512, 128
        xt = H.to_torch(rng.standard_normal((m, k)).astype(np.float16))
        wt = H.to_torch(H.pack_int4(rng.integers(-7, 8, size=(n, k)).astype(np.int8)))
        st = H.to_torch(rng.uniform(1e-3, 1e-2, size=(n, k // g)).astype(np.float16))
        out = torch.empty((m, n), dtype=torch.float16, device="cuda")
        vp, ll = ctypes.c_void_p, ctypes.c_longlong
        run = plugin.ofq_plugin_run_fused_linear
        run.argtypes = [vp] * 7 + [ctypes.c_int] * 2 + [ll] * 3 + [ctypes.c_int] * 2 + [ll] * 2
        args = (torch.cuda.current_stream().cuda_stream, xt.data_ptr(), wt.data_ptr(), st.data_ptr(),
                None, None, out.data_ptr(), K_FLOAT16, K_INT8, m, n, k, 4, 1, 1, g)
        assert L.ofq_hip_set_device(9999) != 0
        assert run(*args) == -2                       # Compute, then GetAsyncError: the error
        assert plugin.ofq_plugin_last_async_error(buf, 256) > 0
        assert b"invalid device" in buf.value.lower()
        assert run(*args) == 0                        # nothing is left behind
        torch.cuda.synchronize()
        assert L.ofq_hip_get_async_error() == 0
    finally:
        plugin.ofq_plugin_stream_delete(view)


class _Infer:
    """One op-definition call described through the plugin's hooks."""

    def __init__(self, plugin, op):
        vp, ci, ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong
        p = plugin
        p.ofq_plugin_infer_new.restype = vp
        p.ofq_plugin_infer_delete.argtypes = [vp]
        p.ofq_plugin_infer_add_input.argtypes = [vp, ctypes.c_char_p, ci, ctypes.POINTER(ll), ci, ci]
        p.ofq_plugin_infer_attr_int.argtypes = [vp, ctypes.c_char_p, ll]
        p.ofq_plugin_infer_attr_bool.argtypes = [vp, ctypes.c_char_p, ci]
        p.ofq_plugin_infer_attr_double.argtypes = [vp, ctypes.c_char_p, ctypes.c_double]
        p.ofq_plugin_infer_attr_string.argtypes = [vp, ctypes.c_char_p, ctypes.c_char_p]
        p.ofq_plugin_infer_run.argtypes = [vp, ctypes.c_char_p]
        p.ofq_plugin_infer_output.argtypes = [vp, ctypes.c_char_p, ci, ctypes.POINTER(ll), ci, ctypes.POINTER(ci)]
        self.p, self.op, self.c = p, op.encode(), p.ofq_plugin_infer_new()

    def inp(self, name, shape, dtype, index=0):
        arr = (ctypes.c_longlong * len(shape))(*shape)
        self.p.ofq_plugin_infer_add_input(self.c, name.encode(), index, arr, len(shape), dtype)
        return self

    def attrs(self, **kw):
        for k, v in kw.items():
            if isinstance(v, bool):
                self.p.ofq_plugin_infer_attr_bool(self.c, k.encode(), int(v))
            elif isinstance(v, int):
                self.p.ofq_plugin_infer_attr_int(self.c, k.encode(), v)
            elif isinstance(v, float):
                self.p.ofq_plugin_infer_attr_double(self.c, k.encode(), v)
            else:
                self.p.ofq_plugin_infer_attr_string(self.c, k.encode(), v.encode())
        return self

    def run(self):
        rc = self.p.ofq_plugin_infer_run(self.c, self.op)
        if rc != 0:
            buf = ctypes.create_string_buffer(512)
            self.p.ofq_plugin_infer_error(buf, 512)
            return buf.value.decode()
        return None

    def out(self, name, index=0):
        shape = (ctypes.c_longlong * 8)()
        dt = ctypes.c_int()
        rank = self.p.ofq_plugin_infer_output(self.c, name.encode(), index, shape, 8, ctypes.byref(dt))
        return (None, None) if rank < 0 else (tuple(shape[:rank]), dt.value)

    def __del__(self):
        self.p.ofq_plugin_infer_delete(self.c)


def test_op_definitions_of_the_added_ops(plugin):
    """Shape and dtype inference of the four ops without a definition in the reference tree
    (oneflow_amd/plugin/ofq_oneflow_ops.cpp), in the style of
    fused_linear_with_groupwise_quantized_weight_op.cpp:27-94: outputs inferred, the same shape
    rules as the functional layer, violations reported as errors and not as aborts."""
    quant = dict(num_bits=4, symmetric=True, group_dim=1, group_size=128)
    # LayerNorm + observer, with the skip_layer_norm inputs
    c = (_Infer(plugin, "fused_layer_norm_min_max_observer").inp("x", (2, 7, 4096), K_FLOAT16)
         .inp("gamma", (4096,), K_FLOAT16).inp("beta", (4096,), K_FLOAT16)
         .inp("skip", (2, 7, 4096), K_FLOAT16).attrs(epsilon=1e-5, alpha=0.5, quantization_bit=8))
    assert c.run() is None
    assert c.out("y") == ((2, 7, 4096), K_FLOAT16)
    assert c.out("scale") == ((1,), K_FLOAT) and c.out("zero_point") == ((1,), K_FLOAT)
    bad = (_Infer(plugin, "fused_layer_norm_min_max_observer").inp("x", (4, 4096), K_FLOAT16)
           .inp("gamma", (4095,), K_FLOAT16).attrs(epsilon=1e-5, alpha=0.5, quantization_bit=8))
    assert "Check failed" in bad.run()
    bad = (_Infer(plugin, "fused_layer_norm_min_max_observer").inp("x", (4, 4096), K_FLOAT16)
           .attrs(epsilon=1e-5, alpha=0.5, quantization_bit=9))
    assert "quantization_bit" in bad.run()
    bad = (_Infer(plugin, "fused_layer_norm_min_max_observer").inp("x", (4, 4096), K_FLOAT16)
           .inp("beta", (4096,), K_FLOAT).attrs(epsilon=1e-5, alpha=0.5, quantization_bit=8))
    assert "Check failed" in bad.run()
    # LayerNorm -> int8 codes
    c = (_Infer(plugin, "fused_layer_norm_quantization").inp("x", (2, 7, 4096), K_FLOAT16)
         .inp("gamma", (4096,), K_FLOAT16).inp("beta", (4096,), K_FLOAT16)
         .attrs(epsilon=1e-5, quantization_bit=8))
    assert c.run() is None
    assert c.out("out") == ((2, 7, 4096), K_INT8)
    assert c.out("scale") == ((1,), K_FLOAT) and c.out("zero_point") == ((1,), K_FLOAT)
    bad = (_Infer(plugin, "fused_layer_norm_quantization").inp("x", (4096,), K_FLOAT16)
           .attrs(epsilon=1e-5, quantization_bit=8))
    assert "Check failed" in bad.run()
    bad = (_Infer(plugin, "fused_layer_norm_quantization").inp("x", (4, 4096), K_FLOAT16)
           .inp("gamma", (4096,), K_BFLOAT16).attrs(epsilon=1e-5, quantization_bit=8))
    assert "Check failed" in bad.run()
    # matmul_quant
    c = (_Infer(plugin, "matmul_quant").inp("a", (3, 2048, 4096), K_INT8).inp("b", (11008, 4096), K_INT8)
         .inp("a_scale", (1,), K_FLOAT).inp("b_scale", (11008,), K_FLOAT)
         .inp("bias", (11008,), K_FLOAT16).attrs(out_dtype=K_FLOAT16))
    assert c.run() is None and c.out("out") == ((3, 2048, 11008), K_FLOAT16)
    bad = (_Infer(plugin, "matmul_quant").inp("a", (8, 4096), K_INT8).inp("b", (64, 4000), K_INT8)
           .inp("a_scale", (1,), K_FLOAT).inp("b_scale", (64,), K_FLOAT).attrs(out_dtype=K_FLOAT16))
    assert "Check failed" in bad.run()
    bad = (_Infer(plugin, "matmul_quant").inp("a", (8, 4096), K_UINT8).inp("b", (64, 4096), K_INT8)
           .inp("a_scale", (1,), K_FLOAT).inp("b_scale", (64,), K_FLOAT).attrs(out_dtype=K_FLOAT16))
    assert "Check failed" in bad.run()
    # GLU over two weights, and over one weight of 2n rows
    c = (_Infer(plugin, "fused_glu_with_groupwise_quantized_weight").inp("x", (5, 4096), K_FLOAT16)
         .inp("w", (11008, 2048), K_INT8).inp("w_scale", (11008, 32), K_FLOAT16)
         .inp("v", (11008, 2048), K_INT8).inp("v_scale", (11008, 32), K_FLOAT16)
         .attrs(activation="silu", **quant))
    assert c.run() is None
    assert c.out("y") == ((5, 11008), K_FLOAT16) and c.out("matmul_vx") == ((5, 11008), K_FLOAT16)
    c = (_Infer(plugin, "fused_glu_with_groupwise_quantized_weight").inp("x", (5, 4096), K_FLOAT16)
         .inp("w", (22016, 2048), K_INT8).inp("w_scale", (22016, 32), K_FLOAT16)
         .inp("b", (22016,), K_FLOAT16).attrs(activation="fast_gelu", **quant))
    assert c.run() is None
    assert c.out("y") == ((5, 11008), K_FLOAT16) and c.out("matmul_wx") == ((5, 22016), K_FLOAT16)
    assert c.out("matmul_vx") == (None, None)
    bad = (_Infer(plugin, "fused_glu_with_groupwise_quantized_weight").inp("x", (5, 4096), K_FLOAT16)
           .inp("w", (64, 2048), K_INT8).inp("w_scale", (64, 31), K_FLOAT16)
           .attrs(activation="silu", **quant))
    assert "Check failed" in bad.run()
    bad = (_Infer(plugin, "fused_glu_with_groupwise_quantized_weight").inp("x", (5, 4096), K_FLOAT16)
           .inp("w", (64, 2048), K_INT8).inp("w_scale", (64, 32), K_FLOAT16)
           .attrs(activation="swish", **quant))
    assert "Check failed" in bad.run()
    # asymmetric codes need uint8 and a zero point
    asym = dict(quant, symmetric=False)
    bad = (_Infer(plugin, "fused_glu_with_groupwise_quantized_weight").inp("x", (5, 4096), K_FLOAT16)
           .inp("w", (64, 2048), K_INT8).inp("w_scale", (64, 32), K_FLOAT16)
           .inp("w_zero", (64, 32), K_FLOAT16).attrs(activation="silu", **asym))
    assert "Check failed" in bad.run()
    # grouped linear: q / k / v
    c = _Infer(plugin, "grouped_linear_with_groupwise_quantized_weight").attrs(**quant)
    for i, n in enumerate((4096, 1024, 1024)):
        c.inp("xs", (1, 4096), K_FLOAT16, i).inp("ws", (n, 2048), K_INT8, i)
        c.inp("w_scales", (n, 32), K_FLOAT16, i).inp("bs", (n,), K_FLOAT16, i)
    assert c.run() is None
    assert [c.out("ys", i) for i in range(3)] == [((1, n), K_FLOAT16) for n in (4096, 1024, 1024)]
    bad = _Infer(plugin, "grouped_linear_with_groupwise_quantized_weight").attrs(**quant)
    bad.inp("xs", (1, 4096), K_FLOAT16, 0).inp("ws", (64, 2048), K_INT8, 0).inp("w_scales", (64, 32), K_FLOAT16, 0)
    bad.inp("xs", (1, 4096), K_FLOAT16, 1).inp("ws", (64, 2048), K_INT8, 1)
    assert "Check failed" in bad.run()
