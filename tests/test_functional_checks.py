"""The host layer rejects what the reference functors reject, with the reference's messages
(oneflow/core/functional/impl/quantization.cpp:155-220, :264-372), and refuses CPU tensors
instead of falling back.  No GPU needed: every check fires before the library is called."""
import pytest
import torch

import oneflow_amd as flow
from oneflow_amd import CheckFailedError


def _w(n=8, k=64, bits=8, dtype=torch.uint8):
    return torch.zeros((n, k * bits // 8), dtype=dtype)


def test_groupwise_dequantize_checks():
    s = torch.ones((8, 1), dtype=torch.float16)
    with pytest.raises(CheckFailedError, match="num_bits should be 4 or 8."):
        flow._C.groupwise_dequantize(_w(), s, num_bits=3)
    with pytest.raises(CheckFailedError, match=r"group_dim should be in range \[-2,2\)."):
        flow._C.groupwise_dequantize(_w(), s, group_dim=2)
    with pytest.raises(CheckFailedError, match=r"group_size should be in range \(0,64\]."):
        flow._C.groupwise_dequantize(_w(), s, group_size=65)
    with pytest.raises(CheckFailedError, match="group_size should be a divisor of 64."):
        flow._C.groupwise_dequantize(_w(), s, group_size=24)
    with pytest.raises(CheckFailedError, match="The dtype of tensor in should be uint8."):
        flow._C.groupwise_dequantize(_w(dtype=torch.int8), s, zero=s, symmetric=False)
    with pytest.raises(CheckFailedError, match="The dtype of tensor in should be int8 or uint8."):
        flow._C.groupwise_dequantize(_w(dtype=torch.int32), s)
    with pytest.raises(CheckFailedError, match="The size of the 1-th dimension of tensor scale should be equal to 1"):
        flow._C.groupwise_dequantize(_w(), torch.ones((8, 2), dtype=torch.float16))
    with pytest.raises(CheckFailedError, match="When symmetric is False, tensor zero should be specified."):
        flow._C.groupwise_dequantize(_w(), s, symmetric=False)
    with pytest.raises(CheckFailedError, match="When symmetric is True, tensor zero should be None."):
        flow._C.groupwise_dequantize(_w(), s, zero=s)
    with pytest.raises(CheckFailedError, match="The shape of zero tensor should be equal to tensor scale."):
        flow._C.groupwise_dequantize(_w(), s, zero=torch.ones((8, 2), dtype=torch.float16), symmetric=False)
    # 4-bit: the packed axis counts double; group_size=-1 means the whole (unpacked) axis
    with pytest.raises(CheckFailedError, match="tensors must live on the GPU"):
        flow._C.groupwise_dequantize(_w(bits=4), s, num_bits=4)


def test_fused_linear_checks():
    x = torch.zeros((2, 64), dtype=torch.float16)
    s = torch.ones((8, 1), dtype=torch.float16)
    f = flow._C.fused_linear_with_groupwise_quantized_weight
    with pytest.raises(CheckFailedError, match="greater than or equal to 2"):
        f(torch.zeros(64, dtype=torch.float16), _w(), s)
    with pytest.raises(CheckFailedError, match="The size of second dimension of tensor w should be equal to 32"):
        f(x, _w(), s, num_bits=4)
    with pytest.raises(CheckFailedError, match=r"group_dim should be in range \[-2,2\)."):
        f(x, _w(), s, group_dim=-3)
    with pytest.raises(CheckFailedError, match="The dtype of the w_scale tensor should be the same as the x tensor."):
        f(x, _w(), s.float())
    with pytest.raises(CheckFailedError, match="The size of the 0-th dimension of tensor w_scale should be equal to tensor w."):
        f(x, _w(), torch.ones((4, 1), dtype=torch.float16))
    with pytest.raises(CheckFailedError, match="The dtype of the b tensor should be the same as the x tensor."):
        f(x, _w(), s, b=torch.zeros(8))
    with pytest.raises(CheckFailedError, match="The number of dimensions for tensor b should be equal to 1."):
        f(x, _w(), s, b=torch.zeros((8, 1), dtype=torch.float16))
    with pytest.raises(CheckFailedError, match="When symmetric is False, tensor w_zero should be specified."):
        f(x, _w(), s, symmetric=False)
    # group_dim=0: scale is [n/g, k]
    with pytest.raises(CheckFailedError, match="The size of the 1-th dimension of tensor w_scale should be equal to 64."):
        f(x, _w(), torch.ones((2, 63), dtype=torch.float16), group_dim=0, group_size=4)
    with pytest.raises(CheckFailedError, match="tensors must live on the GPU"):
        f(x, _w(), s, group_size=64)


def test_observer_and_quantization_checks():
    x = torch.zeros((4, 8))
    with pytest.raises(CheckFailedError, match="quantization_bit"):
        flow._C.min_max_observer(x, "google", 9, "symmetric", True)
    with pytest.raises(CheckFailedError, match="quantization_scheme"):
        flow._C.min_max_observer(x, "google", 8, "asymmetric", True)
    with pytest.raises(CheckFailedError, match="quantization_formula"):
        flow._C.min_max_observer(x, "tflite", 8, "symmetric", True)
    with pytest.raises(CheckFailedError, match="per-channel mode is not supported in cambricon scheme"):
        flow._C.min_max_observer(x, "cambricon", 8, "symmetric", False)
    with pytest.raises(CheckFailedError, match="no min_max_observer kernel for dtype"):
        flow._C.min_max_observer(x.half(), "google", 8, "symmetric", True)
    with pytest.raises(CheckFailedError, match="scale.elem_cnt"):
        flow._C.quantization(x, torch.ones(3), torch.zeros(3), "google", 8, "symmetric")
    with pytest.raises(CheckFailedError, match="tensors must live on the GPU"):
        flow._C.quantization(x, torch.ones(4), torch.zeros(4), "google", 8, "symmetric")
    with pytest.raises(CheckFailedError, match="tensors must live on the GPU"):
        flow.nn.MinMaxObserver()(x)
    with pytest.raises(CheckFailedError, match="a and b should be int8"):
        flow._C.matmul_quant(x, x, torch.ones(1), torch.ones(4))


def test_module_wrappers_keep_reference_signatures():
    import inspect
    sig = inspect.signature(flow.nn.MinMaxObserver.__init__)
    assert list(sig.parameters)[1:] == ["quantization_formula", "quantization_bit",
                                        "quantization_scheme", "per_layer_quantization"]
    assert sig.parameters["per_layer_quantization"].default is True
    sig = inspect.signature(flow._C.fused_linear_with_groupwise_quantized_weight)
    kw = [n for n, p in sig.parameters.items() if p.kind == p.KEYWORD_ONLY]
    assert kw == ["w_zero", "b", "num_bits", "symmetric", "group_dim", "group_size"]
    assert sig.parameters["num_bits"].default == 8 and sig.parameters["group_size"].default == -1
    sig = inspect.signature(flow._C.groupwise_dequantize)
    kw = [n for n, p in sig.parameters.items() if p.kind == p.KEYWORD_ONLY]
    assert kw == ["zero", "num_bits", "symmetric", "group_dim", "group_size"]


def test_glu_grouped_and_skip_layer_norm_checks():
    """The argument rules of FusedGluFunctor (nn_functor.cpp:3724-3800), of the grouped tuples
    (GroupedMatmulBiasFunctor: equal lengths) and of skip_layer_norm's inputs."""
    x = torch.zeros((2, 64), dtype=torch.float16)
    s = torch.ones((8, 1), dtype=torch.float16)
    glu = flow._C.fused_glu_with_groupwise_quantized_weight
    with pytest.raises(CheckFailedError, match="unsupported activation"):
        glu(x, _w(), s, activation="tanh")
    with pytest.raises(CheckFailedError, match="expected existance of b while providing c"):
        glu(x, _w(), s, c=torch.zeros(8, dtype=torch.float16))
    with pytest.raises(CheckFailedError, match="expected existance of c, when provide tensors w, v and b"):
        glu(x, _w(), s, b=torch.zeros(8, dtype=torch.float16), v=_w(), v_scale=s)
    with pytest.raises(CheckFailedError, match="v should have the shape and dtype of w"):
        glu(x, _w(), s, v=_w(n=4), v_scale=torch.ones((4, 1), dtype=torch.float16))
    with pytest.raises(CheckFailedError, match="not divisible by 2"):
        glu(x, _w(n=7), torch.ones((7, 1), dtype=torch.float16))
    with pytest.raises(CheckFailedError, match="tensors must live on the GPU"):
        glu(x, _w(), s, v=_w(), v_scale=s, activation="silu")
    grp = flow._C.grouped_linear_with_groupwise_quantized_weight
    with pytest.raises(CheckFailedError, match="should have the same length"):
        grp([x, x], [_w()], [s])
    with pytest.raises(CheckFailedError, match="bs should have the length of xs"):
        grp([x], [_w()], [s], bs=[None, None])
    with pytest.raises(CheckFailedError, match="The size of second dimension of tensor w"):
        grp([x], [_w(k=32)], [s])
    with pytest.raises(CheckFailedError, match="tensors must live on the GPU"):
        grp([x, x], [_w(), _w(n=4)], [s, torch.ones((4, 1), dtype=torch.float16)])
    sln = flow._C.fused_skip_layer_norm_min_max_observer
    with pytest.raises(CheckFailedError, match="skip should have the shape and dtype of x"):
        sln(x, skip=torch.zeros((2, 32), dtype=torch.float16))
    with pytest.raises(CheckFailedError, match="bias should be 1-D"):
        sln(x, bias=torch.zeros((1, 64), dtype=torch.float16))
    with pytest.raises(CheckFailedError, match=r"quantization_bit should be in range \(1, 8\]."):
        sln(x, quantization_bit=9)


def test_quantized_linear_drops_a_stale_decode_copy():
    """The tile-major copy made by make_decode_copy belongs to one weight tensor and one version
    of its contents: loading a state dict, writing to the weight in place or assigning a new weight
    drops it (otherwise 2..16 rows of x would read the old weights and every other batch size the
    new ones); moving the module keeps it."""
    import torch
    from oneflow_amd.nn import QuantizedLinear
    mod = QuantizedLinear(256, 64, bias=True, num_bits=4, group_size=128, device="cpu")
    assert mod._decode_copy() is None and "weight_tiled" not in mod.state_dict()
    fake = torch.zeros(64 * 128, dtype=torch.int8)
    mod._set_decode_copy(fake)
    assert mod._decode_copy() is fake
    assert "weight_tiled" not in mod.state_dict()
    mod.to(torch.device("cpu"))          # a move: still the same weights
    mod.float()                          # only floating-point buffers are converted
    assert mod._decode_copy() is not None
    sd = {k: v.clone() for k, v in mod.state_dict().items()}
    mod.load_state_dict(sd)
    assert mod._decode_copy() is None
    mod._set_decode_copy(fake)
    mod.weight.add_(1)                   # written in place
    assert mod._decode_copy() is None
    mod._set_decode_copy(fake)
    mod.weight = torch.ones_like(mod.weight)   # reassigned
    assert mod._decode_copy() is None
