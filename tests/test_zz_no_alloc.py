"""The entry point that allocates nothing (ofq_fused_layer_norm_min_max_observer_static) against
the workspace-taking entry point it is a variant of, through the C ABI: identical bits, on two
calls in a row, the second with a smaller input (the static scratch keeps the first call's
contents), and the capacity limit."""
import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu


def _call(static, x, gamma, beta, eps, bits):
    from oneflow_amd import _lib
    L = _lib.lib()
    rows, cols = x.shape
    y = torch.empty_like(x)
    scale = torch.full((1,), -1.0, dtype=torch.float32, device=x.device)
    zp = torch.full((1,), -1.0, dtype=torch.float32, device=x.device)
    dt = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}[x.dtype]
    stream = torch.cuda.current_stream().cuda_stream
    if static:
        st = L.ofq_fused_layer_norm_min_max_observer_static(
            stream, x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), y.data_ptr(), scale.data_ptr(),
            zp.data_ptr(), dt, rows, cols, eps, bits)
    else:
        nbytes = L.ofq_fused_layer_norm_min_max_observer_workspace_bytes(dt, rows, cols)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        st = L.ofq_fused_layer_norm_min_max_observer(
            stream, x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), y.data_ptr(), scale.data_ptr(),
            zp.data_ptr(), dt, rows, cols, eps, bits, ws.data_ptr(), nbytes)
    torch.cuda.synchronize()
    return st, y, scale, zp


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_static_scratch_entry_matches_workspace_entry(dtype):
    gen = torch.Generator(device="cpu").manual_seed(7)
    # a large call first, whose partial maxima stay in the scratch, then a smaller one with
    # smaller values: stale partials would raise its scale
    for rows, cols, amp in ((2048, 4096, 3.0), (96, 1024, 0.25), (5, 20000, 1.0)):
        x = (torch.randn(rows, cols, generator=gen) * amp).to(dtype).cuda()
        gamma = (1 + 0.1 * torch.randn(cols, generator=gen)).to(dtype).cuda()
        beta = (0.1 * torch.randn(cols, generator=gen)).to(dtype).cuda()
        st_a, y_a, s_a, z_a = _call(False, x, gamma, beta, 1e-5, 8)
        st_b, y_b, s_b, z_b = _call(True, x, gamma, beta, 1e-5, 8)
        assert st_a == 0 and st_b == 0
        assert torch.equal(y_a.view(torch.uint8), y_b.view(torch.uint8))
        assert torch.equal(s_a.view(torch.int32), s_b.view(torch.int32)) and s_b.item() > 0
        assert z_b.item() == 0.0


def test_static_scratch_entry_rejects_more_rows_than_its_capacity():
    from oneflow_amd import _lib
    rows, cols = 65537, 8
    x = torch.zeros(rows, cols, dtype=torch.float16, device="cuda")
    g = torch.ones(cols, dtype=torch.float16, device="cuda")
    st, y, s, z = _call(True, x, g, g, 1e-5, 8)
    assert st == 9 and _lib.lib().ofq_status_string(st).decode().startswith("input exceeds")
    assert s.item() == -1.0  # nothing was launched
    st, y, s, z = _call(True, x[:65536], g, g, 1e-5, 8)
    assert st == 0 and s.item() == np.float32(1.0) / np.float32(127.0)  # y = beta = 1
