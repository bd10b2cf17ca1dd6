"""The entry point that allocates nothing (ofq_fused_layer_norm_min_max_observer_static) against
the workspace-taking entry point it is a variant of, through the C ABI: identical bits, on two
calls in a row, the second with a smaller input (the static scratch keeps the first call's
contents), and the capacity limit."""
import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu


def _call(static, x, gamma, beta, eps, bits, sync=True):
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
    if sync:
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


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("cols", [512, 1024, 2048, 4096])
def test_static_scratch_entry_when_a_wave_walks_several_rows(dtype, cols):
    """More than 4096 rows of 512 * {1, 2, 4, 8} elements: 2048 waves walk the rows with the next
    row requested ahead and leave one partial maximum each; then a small call whose values are
    smaller (its scale must not see the 2048 partials the large call left)."""
    gen = torch.Generator(device="cpu").manual_seed(cols)
    for rows, amp in ((4097 + cols // 8, 2.0), (40, 0.125)):
        x = (torch.randn(rows, cols, generator=gen) * amp).to(dtype).cuda()
        gamma = (1 + 0.1 * torch.randn(cols, generator=gen)).to(dtype).cuda()
        beta = (0.1 * torch.randn(cols, generator=gen)).to(dtype).cuda()
        st_a, y_a, s_a, z_a = _call(False, x, gamma, beta, 1e-5, 8)
        st_b, y_b, s_b, z_b = _call(True, x, gamma, beta, 1e-5, 8)
        assert st_a == 0 and st_b == 0
        assert torch.equal(y_a.view(torch.uint8), y_b.view(torch.uint8))
        assert torch.equal(s_a.view(torch.int32), s_b.view(torch.int32)) and s_b.item() > 0


def test_static_scratch_entry_back_to_back_on_one_stream_without_a_host_wait():
    """Two calls queued on one stream with nothing between them (the documented use): the second
    call's kernels run behind the first call's finalize, so each sees its own partials.  Large
    amplitudes first, then a smaller input with small ones; both against the workspace entry."""
    gen = torch.Generator(device="cpu").manual_seed(99)
    cases = []
    for rows, cols, amp in ((3000, 2048, 4.0), (64, 2048, 0.1), (6000, 512, 2.0), (7, 8200, 0.5)):
        x = (torch.randn(rows, cols, generator=gen) * amp).to(torch.float16).cuda()
        gamma = (1 + 0.1 * torch.randn(cols, generator=gen)).to(torch.float16).cuda()
        beta = (0.1 * torch.randn(cols, generator=gen)).to(torch.float16).cuda()
        cases.append((x, gamma, beta))
    want = [_call(False, x, g, b, 1e-5, 8) for x, g, b in cases]
    torch.cuda.synchronize()
    got = [_call(True, x, g, b, 1e-5, 8, sync=False) for x, g, b in cases]   # queued, not waited for
    torch.cuda.synchronize()
    for (st_a, y_a, s_a, z_a), (st_b, y_b, s_b, z_b) in zip(want, got):
        assert st_a == 0 and st_b == 0
        assert torch.equal(y_a.view(torch.uint8), y_b.view(torch.uint8))
        assert torch.equal(s_a.view(torch.int32), s_b.view(torch.int32)) and s_b.item() > 0


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
