"""The offline tile-major copy of 4-bit weights (ofq_groupwise_repack) and the fused linear that
reads it (ofq_fused_linear_gq_tiled): the layout is the documented one, and the outputs carry the
same bits as the row-major call, which the other tests hold against the oracle."""
import numpy as np
import pytest

import helpers as H
from oracle import ofq_oracle as O

pytestmark = pytest.mark.gpu


def _row_split(n):
    """rows per block and blocks of the row-balanced decode kernel (include/ofq.h: a function of
    n alone; 256 CUs, at most 64 rows per block)."""
    grid = 256
    if -(-n // grid) > 64:
        grid = 512
    if -(-n // grid) > 64:
        grid = -(-n // 64)
    rpb = max(16, -(-n // grid))
    return rpb, -(-n // rpb)


def _tiled_reference(w, n, k):
    rpb, grid = _row_split(n)
    tpb = -(-rpb // 16)
    nch = k // 128
    wb = w.view(np.uint8).reshape(n, k // 2)
    out = np.zeros((grid, tpb, nch, 4, 16, 16), dtype=np.uint8)  # [b][t][c][kb][r][16 bytes]
    for b in range(grid):
        for t in range(tpb):
            for r in range(16):
                row_l = 16 * t + r
                row = b * rpb + row_l
                if row_l < rpb and row < n:
                    out[b, t, :, :, r, :] = wb[row].reshape(nch, 4, 16)
    return out.reshape(-1)


@pytest.mark.parametrize("n,k", [(4096, 512), (11008, 256), (100, 256), (4099, 384), (33000, 128),
                                 (16, 128), (17, 128)])
def test_tile_major_layout_is_the_documented_one(n, k):
    import oneflow_amd as flow
    rng = np.random.default_rng(n + k)
    w = rng.integers(-128, 128, size=(n, k // 2)).astype(np.int8)
    tiled = H.to_numpy(flow._C.groupwise_repack(H.to_torch(w), 4)).view(np.uint8)
    ref = _tiled_reference(w, n, k)
    assert tiled.shape == ref.shape
    assert np.array_equal(tiled, ref)


VARIANTS = [(True, np.int8), (True, np.uint8), (False, np.uint8)]


@pytest.mark.parametrize("m,n,k,g", [
    (1, 4096, 4096, 128), (2, 4096, 4096, 128), (4, 4096, 4096, 128), (8, 4096, 4096, 128),
    (16, 4096, 2048, 256), (12, 4096, 4096, 128), (3, 11008, 4096, 128), (8, 11008, 4096, 128), (4, 4096, 11008, 128),
    (5, 4096, 11008, 128), (8, 4096, 11008, 128), (7, 11008, 11008, 128), (5, 100, 256, 128), (2, 4099, 384, 128), (7, 33000, 128, 128),
    (16, 17, 1024, 512), (6, 20000, 256, 128),
])
def test_tiled_linear_has_the_bits_of_the_row_major_call(m, n, k, g):
    """Every container / zero mode, one tile per block, 43 rows per block with a partial last
    tile, two blocks per CU, more blocks than CUs, row counts off the tile size, x staged in two
    halves (8 rows of 11008); and against the oracle
    within the op's contract."""
    import oneflow_amd as flow
    rng = np.random.default_rng(m * 131 + n + k)
    x = H.as_T(rng.standard_normal((m, k)).astype(np.float32), "f16")
    b = H.as_T((rng.standard_normal(n) * 0.01).astype(np.float32), "f16")
    for symmetric, qdt in VARIANTS:
        wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
        w, scale, zero = H.quantize_groupwise(wf, 4, symmetric, 1, g, qdt, "f16")
        tt = H.to_torch
        kw = dict(w_zero=None if symmetric else tt(zero), b=tt(b), num_bits=4, symmetric=symmetric,
                  group_dim=1, group_size=g)
        row_major = H.to_numpy(flow._C.fused_linear_with_groupwise_quantized_weight(
            tt(x), tt(w), tt(scale), **kw))
        tiled = flow._C.groupwise_repack(tt(w), 4)
        got = H.to_numpy(flow._C.fused_linear_with_tiled_groupwise_quantized_weight(
            tt(x), tiled, tt(scale), **kw))
        if m == 1:
            # one row of x: the row-major call takes the kernels in which a wave owns whole rows
            # (another summation order); both are within the contract of the oracle
            ref = O.fused_linear(x, w, scale, zero, b, 4, symmetric, 1, g)
            H.assert_linear_parity(got, ref, "f16", "tiled, one row of x")
        else:
            assert np.array_equal(got.view(np.uint16), row_major.view(np.uint16)), (symmetric, qdt)


def test_tiled_entry_point_says_what_it_does_not_serve():
    import torch
    import oneflow_amd as flow
    from oneflow_amd import _lib
    L = _lib.lib()
    assert L.ofq_groupwise_repack_bytes(4, 4096, 4096) == 4096 * 2048
    assert L.ofq_groupwise_repack_bytes(4, 11008, 4096) == 256 * 48 * 2048  # 43 rows -> 3 tiles
    assert L.ofq_groupwise_repack_bytes(4, 4096, 4160) == 0                  # 128 does not divide k
    assert L.ofq_groupwise_repack_bytes(8, 4096, 4096) == 0                  # 4-bit codes only
    w = torch.zeros((64, 2048), dtype=torch.int8, device="cuda")
    tiled = flow._C.groupwise_repack(w, 4)
    scale = torch.ones((64, 32), dtype=torch.float16, device="cuda")
    # 17 rows of x, bf16, and 8 rows of 11008 (x beyond LDS): the row-major call serves those
    for x in (torch.zeros((17, 4096), dtype=torch.float16, device="cuda"),
              torch.zeros((2, 4096), dtype=torch.bfloat16, device="cuda")):
        with pytest.raises(flow.OfqError) as e:
            flow._C.fused_linear_with_tiled_groupwise_quantized_weight(
                x, tiled, scale.to(x.dtype), num_bits=4, symmetric=True, group_dim=1, group_size=128)
        assert e.value.status == 5  # OFQ_ERR_UNSUPPORTED


def test_module_reads_the_decode_copy_for_few_rows():
    import torch
    import oneflow_amd as flow
    lin = torch.nn.Linear(1024, 300, bias=True).half().cuda()
    q = flow.nn.QuantizedLinear.from_float(lin, num_bits=4, symmetric=True, group_size=128)
    xs = [torch.randn((m, 1024), dtype=torch.float16, device="cuda") for m in (1, 4, 16, 40)]
    before = [q(x) for x in xs]
    q.make_decode_copy()
    assert "weight_tiled" not in q.state_dict()
    for x, ref in zip(xs, before):
        assert torch.equal(q(x), ref)
