"""Host-side mirror of OneFlow's ``flow._C`` entry points for the quantized-inference ops.

Signatures, keyword names, defaults and argument checks follow
``oneflow/core/functional/functional_api.yaml:1061-1093`` and the functors in
``oneflow/core/functional/impl/quantization.cpp`` (same messages), so a test written against
``flow._C.groupwise_dequantize`` / ``flow._C.fused_linear_with_groupwise_quantized_weight`` /
``flow._C.min_max_observer`` / ``flow._C.quantization`` / ``flow._C.fake_quantization`` reads the
same against this module.  Tensors are ``torch`` tensors on the GPU; torch is used only to own
device memory and to name the current stream -- all arithmetic happens in the HIP library behind
the C ABI of ``include/ofq.h``.

One deliberate difference: the reference functor routes ``m > 8`` of the fused linear through
``groupwise_dequantize`` + matmul (quantization.cpp:341-350); here every ``m`` goes to the fused
op, whose kernels cover both regimes.
"""
import ctypes

import torch

from . import _lib
from ._lib import BF16, F16, F32, F64, I8, U8


class CheckFailedError(RuntimeError):
    """Raised where the reference functor's CHECK_OR_RETURN would fail."""


def _check(cond, msg):
    if not cond:
        raise CheckFailedError(msg)


_DT = {
    torch.float32: F32,
    torch.float16: F16,
    torch.bfloat16: BF16,
    torch.float64: F64,
    torch.int8: I8,
    torch.uint8: U8,
}


def _dt(t):
    try:
        return _DT[t.dtype]
    except KeyError:
        raise CheckFailedError(f"unsupported dtype {t.dtype}") from None


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise CheckFailedError("tensors must live on the GPU: this build has no CPU kernels")


def _contig(t):
    # the runtime hands kernels contiguous inputs (op_interpreter_util.cpp:156) in buffers of its
    # own allocator (512-byte aligned); a view that starts off a 16-byte boundary is copied, since
    # the kernels use 128-bit accesses
    if t is None:
        return None
    t = t.contiguous()
    return t.clone() if t.data_ptr() % 16 else t


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)


# --------------------------------------------------------------------------------------------
# groupwise_dequantize: GroupwiseDequantizeFunctor, quantization.cpp:155-220
# --------------------------------------------------------------------------------------------
def groupwise_dequantize(in_, scale, *, zero=None, num_bits=8, symmetric=True, group_dim=-1,
                         group_size=-1):
    _check(num_bits in (4, 8), "num_bits should be 4 or 8.")
    nd = in_.dim()
    _check(nd >= 1, "The number of dimensions for tensor in should be greater than or equal to 1.")
    gd = nd + group_dim if group_dim < 0 else group_dim
    _check(0 <= gd < nd, f"group_dim should be in range [-{nd},{nd}).")
    per = 8 // num_bits
    group_dim_size = in_.shape[gd] * (per if gd == nd - 1 else 1)
    gs = group_dim_size if group_size < 0 else group_size
    _check(0 < gs <= group_dim_size, f"group_size should be in range (0,{group_dim_size}].")
    _check(group_dim_size % gs == 0, f"group_size should be a divisor of {group_dim_size}.")
    num_groups = group_dim_size // gs
    if symmetric:
        _check(in_.dtype in (torch.uint8, torch.int8),
               "The dtype of tensor in should be int8 or uint8.")
    else:
        _check(in_.dtype == torch.uint8, "The dtype of tensor in should be uint8.")
    _check(scale.dim() == nd,
           "The number of dimensions of tensor scale should be equal to tensor in.")
    for i in range(nd):
        if i == gd:
            _check(scale.shape[i] == num_groups,
                   f"The size of the {i}-th dimension of tensor scale should be equal to {num_groups}")
        elif i == nd - 1:
            _check(scale.shape[i] == in_.shape[i] * per,
                   f"The size of the {i}-th dimension of tensor scale should be equal to "
                   f"{in_.shape[i] * per}.")
        else:
            _check(scale.shape[i] == in_.shape[i],
                   f"The size of the {i}-th dimension of tensor scale should be equal to tensor in.")
    if not symmetric:
        _check(zero is not None, "When symmetric is False, tensor zero should be specified.")
        _check(zero.dtype == scale.dtype,
               "The dtype of the zero tensor should be the same as the scale tensor.")
        _check(zero.shape == scale.shape,
               "The shape of zero tensor should be equal to tensor scale.")
    else:
        _check(zero is None, "When symmetric is True, tensor zero should be None.")
    # kernels are registered on the dtype of scale (groupwise_quantization_kernels.cu:456-463);
    # bf16 is added here
    _check(scale.dtype in (torch.float16, torch.float32, torch.bfloat16),
           f"no groupwise_dequantize kernel for scale dtype {scale.dtype}")
    _require_gpu(in_, scale, zero)
    in_, scale, zero = _contig(in_), _contig(scale), _contig(zero)
    out_shape = list(in_.shape)
    out_shape[-1] *= per
    out = torch.empty(out_shape, dtype=scale.dtype, device=in_.device)
    outer = 1
    for d in out_shape[:gd]:
        outer *= d
    outer *= num_groups
    inner = 1
    for d in out_shape[gd + 1:]:
        inner *= d
    st = _lib.lib().ofq_groupwise_dequantize(
        _stream(in_), _ptr(in_), _ptr(scale), _ptr(zero), _ptr(out), _dt(in_), _dt(scale),
        num_bits, int(symmetric), outer, gs, inner)
    _lib.check("ofq_groupwise_dequantize", st)
    return out


# --------------------------------------------------------------------------------------------
# fused_linear_with_groupwise_quantized_weight:
# FusedLinearWithGroupwiseQuantizedWeightFunctor, quantization.cpp:264-372
# --------------------------------------------------------------------------------------------
def _check_fused_linear_args(x, w, w_scale, w_zero, b, num_bits, symmetric, group_dim,
                             group_size):
    """The argument checks of FusedLinearWithGroupwiseQuantizedWeightFunctor
    (oneflow/core/functional/impl/quantization.cpp:264-340); returns (m, n, k, group_dim,
    group_size) with the negative defaults resolved."""
    _check(x.dim() >= 2,
           "The number of dimensions for tensor x should be greater than or equal to 2.")
    k = x.shape[-1]
    m = x.numel() // k if k else 0
    _check(num_bits in (4, 8), "num_bits should be 4 or 8.")
    _check(w.dim() == 2, "The number of dimensions for tensor w should be equal to 2.")
    per = 8 // num_bits
    _check(k % per == 0,
           "The size of the last dimension of x should be a multiple of (8/num_bits).")
    _check(w.shape[1] == k // per,
           f"The size of second dimension of tensor w should be equal to {k // per}")
    n = w.shape[0]
    gd = 2 + group_dim if group_dim < 0 else group_dim
    _check(gd in (0, 1), "group_dim should be in range [-2,2).")
    group_dim_size = n if gd == 0 else k
    gs = group_dim_size if group_size < 0 else group_size
    _check(0 < gs <= group_dim_size, f"group_size should be in range (0,{group_dim_size}].")
    _check(group_dim_size % gs == 0, f"group_size should be a divisor of {group_dim_size}.")
    num_groups = group_dim_size // gs
    if symmetric:
        _check(w.dtype in (torch.uint8, torch.int8),
               "The dtype of tensor w should be int8 or uint8.")
    else:
        _check(w.dtype == torch.uint8, "The dtype of tensor w should be uint8.")
    _check(w_scale.dim() == 2,
           "The number of dimensions of tensor w_scale should be equal to 2.")
    for i in range(2):
        if i == gd:
            _check(w_scale.shape[i] == num_groups,
                   f"The size of the {i}-th dimension of tensor w_scale should be equal to "
                   f"{num_groups}")
        elif i == 1:
            _check(w_scale.shape[i] == k,
                   f"The size of the {i}-th dimension of tensor w_scale should be equal to {k}.")
        else:
            _check(w_scale.shape[i] == w.shape[i],
                   f"The size of the {i}-th dimension of tensor w_scale should be equal to tensor w.")
    _check(w_scale.dtype == x.dtype,
           "The dtype of the w_scale tensor should be the same as the x tensor.")
    if not symmetric:
        _check(w_zero is not None, "When symmetric is False, tensor w_zero should be specified.")
        _check(w_zero.dtype == w_scale.dtype,
               "The dtype of the w_zero tensor should be the same as the w_scale tensor.")
        _check(w_zero.shape == w_scale.shape,
               "The shape of w_zero tensor should be equal to tensor w_scale.")
    else:
        _check(w_zero is None, "When symmetric is True, tensor w_zero should be None.")
    if b is not None:
        _check(b.dtype == x.dtype, "The dtype of the b tensor should be the same as the x tensor.")
        _check(b.dim() == 1, "The number of dimensions for tensor b should be equal to 1.")
        _check(b.shape[0] == n,
               "The size of first dimension of tensor b should be equal to the size of first "
               "dimension of tensor w")
    _check(x.dtype in (torch.float16, torch.float32, torch.bfloat16),
           f"no fused_linear_with_groupwise_quantized_weight kernel for dtype {x.dtype}")
    return m, n, k, gd, gs


def fused_linear_with_groupwise_quantized_weight(x, w, w_scale, *, w_zero=None, b=None,
                                                 num_bits=8, symmetric=True, group_dim=-1,
                                                 group_size=-1):
    m, n, k, gd, gs = _check_fused_linear_args(x, w, w_scale, w_zero, b, num_bits, symmetric,
                                               group_dim, group_size)
    _require_gpu(x, w, w_scale, w_zero, b)
    x, w, w_scale, w_zero, b = map(_contig, (x, w, w_scale, w_zero, b))
    out = torch.empty(tuple(x.shape[:-1]) + (n,), dtype=x.dtype, device=x.device)
    L = _lib.lib()
    ws_bytes = L.ofq_fused_linear_gq_workspace_bytes(_dt(w), _dt(x), num_bits, int(symmetric), gd,
                                                     gs, m, n, k)
    ws = _workspace(ws_bytes, x.device) if ws_bytes else None
    st = L.ofq_fused_linear_gq(_stream(x), _ptr(x), _ptr(w), _ptr(w_scale), _ptr(w_zero), _ptr(b),
                               _ptr(out), _dt(w), _dt(x), num_bits, int(symmetric), gd, gs, m, n,
                               k, _ptr(ws), ws_bytes)
    _lib.check("ofq_fused_linear_gq", st)
    return out


def groupwise_repack(w, num_bits=4):
    """Extension (no counterpart in the reference): the tile-major copy of row-major 4-bit codes
    ``w`` [n, k/2] that ``fused_linear_with_tiled_groupwise_quantized_weight`` reads, as a flat
    uint8 / int8 tensor of ``ofq_groupwise_repack_bytes`` elements.  Done once, offline."""
    _check(w.dim() == 2 and w.dtype in (torch.int8, torch.uint8), "w should be 2-D int8 / uint8 codes")
    _check(num_bits == 4, "only 4-bit codes have a tile-major form")
    _require_gpu(w)
    w = _contig(w)
    n, k = w.shape[0], w.shape[1] * 2
    L = _lib.lib()
    nbytes = L.ofq_groupwise_repack_bytes(num_bits, n, k)
    _check(nbytes > 0, f"no tile-major form for n={n}, k={k} (k should be a multiple of 128)")
    tiled = torch.empty(nbytes, dtype=w.dtype, device=w.device)
    st = L.ofq_groupwise_repack(_stream(w), _ptr(w), _ptr(tiled), num_bits, n, k)
    _lib.check("ofq_groupwise_repack", st)
    return tiled


def fused_linear_with_tiled_groupwise_quantized_weight(x, w_tiled, w_scale, *, w_zero=None, b=None,
                                                       num_bits=4, symmetric=True, group_dim=-1,
                                                       group_size=-1):
    """``fused_linear_with_groupwise_quantized_weight`` on the copy ``groupwise_repack`` made of
    ``w`` (n and k are taken from ``w_scale`` and ``x``); the same bits as the row-major call.
    For up to 16 rows of ``x`` in fp16 with groups of a multiple of 128 along K; raises
    ``OfqError`` (unsupported) otherwise -- keep the row-major weight for those calls."""
    _check(x.dim() >= 2 or x.dim() == 1, "x should have at least one dimension")
    k = x.shape[-1]
    m = x.numel() // k
    n = w_scale.shape[0]
    gd = group_dim if group_dim >= 0 else group_dim + 2
    _check(gd == 1, "the tile-major copy serves groups along K only")
    gs = group_size if group_size >= 0 else k
    _check(w_tiled.dim() == 1 and w_tiled.dtype in (torch.int8, torch.uint8),
           "w_tiled should be the flat tensor groupwise_repack returns")
    _check((w_zero is None) == bool(symmetric), "w_zero is given exactly when symmetric is False")
    _require_gpu(x, w_tiled, w_scale, w_zero, b)
    L = _lib.lib()
    _check(w_tiled.numel() == L.ofq_groupwise_repack_bytes(num_bits, n, k),
           "w_tiled does not have the size of the tile-major copy of an [n, k] weight")
    x, w_scale, w_zero, b = map(_contig, (x, w_scale, w_zero, b))
    out = torch.empty(tuple(x.shape[:-1]) + (n,), dtype=x.dtype, device=x.device)
    st = L.ofq_fused_linear_gq_tiled(_stream(x), _ptr(x), _ptr(w_tiled), _ptr(w_scale),
                                     _ptr(w_zero), _ptr(b), _ptr(out), _dt(w_tiled), _dt(x),
                                     num_bits, int(symmetric), gd, gs, m, n, k)
    _lib.check("ofq_fused_linear_gq_tiled", st)
    return out


def grouped_linear_with_groupwise_quantized_weight(xs, ws, w_scales, *, w_zeros=None, bs=None,
                                                   num_bits=8, symmetric=True, group_dim=-1,
                                                   group_size=-1):
    """``fused_linear_with_groupwise_quantized_weight`` over tuples of problems, the quantised
    counterpart of ``grouped_matmul_bias(xs, weights, biases)`` (functional_api.yaml:2759-2760;
    checks of GroupedMatmulBiasFunctor: equal tuple lengths).  Problems of equal (m, k) with
    m <= 16 run as one launch.  Returns the list of outputs."""
    count = len(xs)
    _check(count > 0, "xs should not be empty")
    _check(count <= 64, "at most 64 problems per call")
    _check(len(ws) == count and len(w_scales) == count, "xs, ws and w_scales should have the same length")
    _check(w_zeros is None or len(w_zeros) == count, "w_zeros should have the length of xs")
    _check(bs is None or len(bs) == count, "bs should have the length of xs")
    w_zeros = list(w_zeros) if w_zeros is not None else [None] * count
    bs = list(bs) if bs is not None else [None] * count
    dims = [_check_fused_linear_args(xs[i], ws[i], w_scales[i], w_zeros[i], bs[i], num_bits,
                                     symmetric, group_dim, group_size) for i in range(count)]
    _check(all(x.dtype == xs[0].dtype for x in xs) and all(w.dtype == ws[0].dtype for w in ws),
           "all problems should share the dtypes of x and w")
    _check(all(d[3] == dims[0][3] and d[4] == dims[0][4] for d in dims),
           "all problems should share group_dim and group_size")
    _require_gpu(*xs, *ws, *w_scales, *w_zeros, *bs)
    xs, ws, w_scales = [list(map(_contig, t)) for t in (xs, ws, w_scales)]
    w_zeros, bs = list(map(_contig, w_zeros)), list(map(_contig, bs))
    outs = [torch.empty(tuple(x.shape[:-1]) + (d[1],), dtype=x.dtype, device=x.device)
            for x, d in zip(xs, dims)]
    arr = lambda ts: (ctypes.c_void_p * count)(*[_ptr(t) for t in ts])
    i64 = lambda v: (ctypes.c_int64 * count)(*v)
    L = _lib.lib()
    st = L.ofq_grouped_linear_gq(
        _stream(xs[0]), count, arr(xs), arr(ws), arr(w_scales), None if symmetric else arr(w_zeros),
        arr(bs), arr(outs), i64([d[0] for d in dims]), i64([d[1] for d in dims]),
        i64([d[2] for d in dims]), _dt(ws[0]), _dt(xs[0]), num_bits, int(symmetric), dims[0][3],
        dims[0][4])
    _lib.check("ofq_grouped_linear_gq", st)
    return outs


_ACTIVATIONS = {"none": 0, "sigmoid": 1, "relu": 2, "gelu": 3, "fast_gelu": 4, "silu": 5}


def fused_glu_with_groupwise_quantized_weight(x, w, w_scale, *, w_zero=None, b=None, v=None,
                                              v_scale=None, v_zero=None, c=None,
                                              activation="none", num_bits=8, symmetric=True,
                                              group_dim=-1, group_size=-1):
    """``fused_glu(x, w, b, v, c, activation)`` (functional_api.yaml:774-775, checks of
    FusedGluFunctor, nn_functor.cpp:3724-3800) with groupwise-quantised ``w`` / ``v``:
    ``y = (x w~^T + b) * act(x v~^T + c)``; without ``v`` the 2n rows of ``w`` hold the
    hidden-state rows first and the gate rows second."""
    _check(activation in _ACTIVATIONS, f"unsupported activation {activation!r}")
    split = v is not None
    if b is not None:
        if split:
            _check(c is not None, "expected existance of c, when provide tensors w, v and b")
    else:
        _check(c is None, "expected existance of b while providing c")
    m, n_w, k, gd, gs = _check_fused_linear_args(x, w, w_scale, w_zero, b, num_bits, symmetric,
                                                 group_dim, group_size)
    if split:
        _check(v_scale is not None, "v_scale should be specified with v")
        _check(tuple(v.shape) == tuple(w.shape) and v.dtype == w.dtype,
               "v should have the shape and dtype of w")
        _check_fused_linear_args(x, v, v_scale, v_zero, c, num_bits, symmetric, group_dim,
                                 group_size)
        n = n_w
    else:
        _check(v_scale is None and v_zero is None and c is None,
               "v_scale, v_zero and c belong to v")
        _check(n_w % 2 == 0, "dimension 0 of 'w' is not divisible by 2")
        n = n_w // 2
    _require_gpu(x, w, w_scale, w_zero, b, v, v_scale, v_zero, c)
    x, w, w_scale, w_zero, b, v, v_scale, v_zero, c = map(
        _contig, (x, w, w_scale, w_zero, b, v, v_scale, v_zero, c))
    lead = tuple(x.shape[:-1])
    y = torch.empty(lead + (n,), dtype=x.dtype, device=x.device)
    matmul_wx = torch.empty(lead + (n_w,), dtype=x.dtype, device=x.device)
    matmul_vx = torch.empty(lead + (n,), dtype=x.dtype, device=x.device) if split else None
    st = _lib.lib().ofq_fused_glu_gq(
        _stream(x), _ptr(x), _ptr(w), _ptr(w_scale), _ptr(w_zero), _ptr(b), _ptr(v), _ptr(v_scale),
        _ptr(v_zero), _ptr(c), _ptr(y), _ptr(matmul_wx), _ptr(matmul_vx), _ACTIVATIONS[activation],
        _dt(w), _dt(x), num_bits, int(symmetric), gd, gs, m, n, k)
    _lib.check("ofq_fused_glu_gq", st)
    return y


# --------------------------------------------------------------------------------------------
# min_max_observer / quantization / fake_quantization
# functors quantization.cpp:34-153; attribute checks oneflow/user/ops/min_max_observer_op.cpp:58-70,
# quantization_op.cpp:92-104
# --------------------------------------------------------------------------------------------
def _check_quant_attrs(quantization_formula, quantization_bit, quantization_scheme):
    _check(1 < quantization_bit <= 8, "quantization_bit should be in range (1, 8].")
    _check(quantization_scheme in ("symmetric", "affine"),
           "quantization_scheme should be symmetric or affine.")
    _check(quantization_formula in ("google", "cambricon"),
           "quantization_formula should be google or cambricon.")


def min_max_observer(in_, quantization_formula="google", quantization_bit=8,
                     quantization_scheme="symmetric", per_layer_quantization=True):
    """Returns ``(scale, zero_point)``; shape ``[1]`` per layer or ``[in.shape[0]]`` per channel
    (min_max_observer_op.cpp:21-38)."""
    _check_quant_attrs(quantization_formula, quantization_bit, quantization_scheme)
    _check(in_.dtype in (torch.float32, torch.float64),
           f"no min_max_observer kernel for dtype {in_.dtype}")
    if quantization_formula == "cambricon":
        _check(per_layer_quantization, " per-channel mode is not supported in cambricon scheme")
    _require_gpu(in_)
    in_ = _contig(in_)
    channels = 1 if per_layer_quantization else in_.shape[0]
    scale = torch.empty(channels, dtype=in_.dtype, device=in_.device)
    zero_point = torch.empty(channels, dtype=in_.dtype, device=in_.device)
    L = _lib.lib()
    ws_bytes = L.ofq_min_max_observer_workspace_bytes(_dt(in_), in_.numel(), channels)
    ws = _workspace(ws_bytes, in_.device)
    st = L.ofq_min_max_observer(_stream(in_), _ptr(in_), _ptr(scale), _ptr(zero_point), _dt(in_),
                                in_.numel(), channels, quantization_bit,
                                _lib.SCHEME[quantization_scheme],
                                _lib.FORMULA[quantization_formula], _ptr(ws), ws_bytes)
    _lib.check("ofq_min_max_observer", st)
    return scale, zero_point


def moving_average_min_max_observer(in_, current_train_step, moving_max, moving_min, training,
                                    stop_update_after_iters, quantization_formula="google",
                                    quantization_bit=8, quantization_scheme="symmetric",
                                    momentum=0.95):
    """MovingAverageMinMaxObserverFunctor (quantization.cpp:59-91, functional_api.yaml:1079-1084).
    ``moving_max`` / ``moving_min`` (shape ``[1]``, dtype of ``in``) are updated in place while
    training and ``current_train_step <= stop_update_after_iters``; ``current_train_step`` is a
    device tensor of one int64 and is read on the device.  Returns ``(scale, zero_point)``."""
    _check_quant_attrs(quantization_formula, quantization_bit, quantization_scheme)
    _check(stop_update_after_iters > 0, "stop_update_after_iters should be greater than 0")
    _check(in_.dtype in (torch.float32, torch.float64),
           f"no moving_average_min_max_observer kernel for dtype {in_.dtype}")
    # shape rules of moving_average_min_max_observer_op.cpp:29-32
    for name, t in (("moving_max", moving_max), ("moving_min", moving_min),
                    ("current_train_step", current_train_step)):
        _check(t.dim() == 1 and t.shape[0] == 1, f"{name} should have shape [1]")
    _check(moving_max.dtype == in_.dtype and moving_min.dtype == in_.dtype,
           "moving_max and moving_min should have the dtype of in")
    _check(current_train_step.dtype == torch.int64, "current_train_step should be int64")
    _require_gpu(in_, current_train_step, moving_max, moving_min)
    _check(moving_max.is_contiguous() and moving_min.is_contiguous(),
           "moving_max and moving_min are updated in place and must be contiguous")
    in_ = _contig(in_)
    scale = torch.empty(1, dtype=in_.dtype, device=in_.device)
    zero_point = torch.empty(1, dtype=in_.dtype, device=in_.device)
    L = _lib.lib()
    ws_bytes = L.ofq_moving_average_min_max_observer_workspace_bytes(_dt(in_), in_.numel())
    ws = _workspace(ws_bytes, in_.device)
    st = L.ofq_moving_average_min_max_observer(
        _stream(in_), _ptr(in_), _ptr(current_train_step), _ptr(moving_max), _ptr(moving_min),
        _ptr(scale), _ptr(zero_point), _dt(in_), in_.numel(), quantization_bit,
        _lib.SCHEME[quantization_scheme], _lib.FORMULA[quantization_formula], float(momentum),
        int(stop_update_after_iters), int(bool(training)), _ptr(ws), ws_bytes)
    _lib.check("ofq_moving_average_min_max_observer", st)
    return scale, zero_point


def _quant_common(fn_name, in_, scale, zero_point, quantization_formula, quantization_bit,
                  quantization_scheme, out_dtype, zp_mode):
    _check_quant_attrs(quantization_formula, quantization_bit, quantization_scheme)
    _check(in_.dtype in (torch.float32, torch.float64, torch.float16, torch.bfloat16),
           f"no {fn_name} kernel for dtype {in_.dtype}")
    param_dtype = in_.dtype if in_.dtype in (torch.float32, torch.float64) else torch.float32
    _check(scale.dtype == param_dtype, f"scale should have dtype {param_dtype}")
    _check(zero_point is None or zero_point.dtype == param_dtype,
           f"zero_point should have dtype {param_dtype}")
    # per-channel iff scale has more than one element (quantization_op.cpp:66-69)
    if scale.numel() > 1:
        _check(scale.numel() == in_.shape[0], "scale.elem_cnt() should equal in.shape[0]")
        _check(zero_point is None or zero_point.numel() == in_.shape[0],
               "zero_point.elem_cnt() should equal in.shape[0]")
    _require_gpu(in_, scale, zero_point)
    return _contig(in_), _contig(scale), _contig(zero_point)


def quantization(in_, scale, zero_point, quantization_formula="google", quantization_bit=8,
                 quantization_scheme="symmetric", *, out_dtype=None, zp_mode="float"):
    """``out_dtype`` (extension): ``torch.int8`` / ``torch.uint8`` to get integer codes instead
    of codes stored in the input dtype.  ``zp_mode`` selects how an affine zero point is read:
    ``"float"`` (the CUDA kernel's rule) or ``"uint8"`` (the CPU kernel's rule)."""
    in_, scale, zero_point = _quant_common("quantization", in_, scale, zero_point,
                                           quantization_formula, quantization_bit,
                                           quantization_scheme, out_dtype, zp_mode)
    out = torch.empty(in_.shape, dtype=out_dtype or in_.dtype, device=in_.device)
    st = _lib.lib().ofq_quantization(
        _stream(in_), _ptr(in_), _ptr(scale), _ptr(zero_point), _ptr(out), _dt(in_), _dt(out),
        in_.numel(), scale.numel(), quantization_bit, _lib.SCHEME[quantization_scheme],
        _lib.FORMULA[quantization_formula], _lib.ZP_MODE[zp_mode])
    _lib.check("ofq_quantization", st)
    return out


class _FakeQuantizationSTE(torch.autograd.Function):
    """The reference's gradient of fake_quantization: the output gradient passes to ``in``
    unchanged, scale and zero_point get none
    (oneflow/core/autograd/gradient_funcs/fake_quantization.cpp:36-42)."""

    @staticmethod
    def forward(ctx, in_, scale, zero_point, formula, bit, scheme, zp_mode):
        return _fake_quantization_forward(in_.detach(), scale, zero_point, formula, bit, scheme,
                                          zp_mode)

    @staticmethod
    def backward(ctx, grad):
        return grad, None, None, None, None, None, None


def fake_quantization(in_, scale, zero_point, quantization_formula="google", quantization_bit=8,
                      quantization_scheme="symmetric", *, zp_mode="float"):
    if torch.is_grad_enabled() and in_.requires_grad:
        return _FakeQuantizationSTE.apply(in_, scale, zero_point, quantization_formula,
                                          quantization_bit, quantization_scheme, zp_mode)
    return _fake_quantization_forward(in_, scale, zero_point, quantization_formula,
                                      quantization_bit, quantization_scheme, zp_mode)


def _fake_quantization_forward(in_, scale, zero_point, quantization_formula, quantization_bit,
                               quantization_scheme, zp_mode):
    in_, scale, zero_point = _quant_common("fake_quantization", in_, scale, zero_point,
                                           quantization_formula, quantization_bit,
                                           quantization_scheme, None, zp_mode)
    out = torch.empty_like(in_)
    st = _lib.lib().ofq_fake_quantization(
        _stream(in_), _ptr(in_), _ptr(scale), _ptr(zero_point), _ptr(out), _dt(in_), in_.numel(),
        scale.numel(), quantization_bit, _lib.SCHEME[quantization_scheme],
        _lib.FORMULA[quantization_formula], _lib.ZP_MODE[zp_mode])
    _lib.check("ofq_fake_quantization", st)
    return out


# --------------------------------------------------------------------------------------------
# Ops named by the task but absent from the reference tree
# --------------------------------------------------------------------------------------------
def fused_layer_norm_min_max_observer(x, gamma=None, beta=None, epsilon=1e-5, quantization_bit=8,
                                      *, exact_statistics=False):
    """LayerNorm over the last axis + per-tensor symmetric observer of the result.
    Returns ``(y, scale, zero_point)`` with fp32 ``scale`` / ``zero_point`` of shape ``[1]``.
    ``exact_statistics``: mean and variance of a row accumulated in fp64 and rounded once (the
    correctly rounded fp32 statistics, independent of the order of summation) instead of
    accumulated in fp32."""
    _check(1 < quantization_bit <= 8, "quantization_bit should be in range (1, 8].")
    _check(x.dtype in (torch.float16, torch.bfloat16, torch.float32),
           f"no fused_layer_norm_min_max_observer kernel for dtype {x.dtype}")
    cols = x.shape[-1]
    for name, p in (("gamma", gamma), ("beta", beta)):
        if p is not None:
            _check(p.dtype == x.dtype and p.numel() == cols,
                   f"{name} should have the dtype of x and x.shape[-1] elements")
    _require_gpu(x, gamma, beta)
    x, gamma, beta = _contig(x), _contig(gamma), _contig(beta)
    rows = x.numel() // cols
    y = torch.empty_like(x)
    scale = torch.empty(1, dtype=torch.float32, device=x.device)
    zero_point = torch.empty(1, dtype=torch.float32, device=x.device)
    L = _lib.lib()
    ws_bytes = L.ofq_fused_layer_norm_min_max_observer_workspace_bytes(_dt(x), rows, cols)
    ws = _workspace(ws_bytes, x.device)
    if exact_statistics:
        st = L.ofq_fused_layer_norm_min_max_observer_stats(
            _stream(x), _ptr(x), None, None, 0.0, 0, _ptr(gamma), _ptr(beta), _ptr(y),
            _ptr(scale), _ptr(zero_point), _dt(x), rows, cols, float(epsilon), quantization_bit,
            _lib.LN_STATS_FP64, _ptr(ws), ws_bytes)
    else:
        st = L.ofq_fused_layer_norm_min_max_observer(
            _stream(x), _ptr(x), _ptr(gamma), _ptr(beta), _ptr(y), _ptr(scale), _ptr(zero_point),
            _dt(x), rows, cols, float(epsilon), quantization_bit, _ptr(ws), ws_bytes)
    _lib.check("ofq_fused_layer_norm_min_max_observer", st)
    return y, scale, zero_point


def fused_layer_norm_quantization(x, gamma=None, beta=None, epsilon=1e-5, quantization_bit=8,
                                  *, exact_statistics=False):
    """``fused_layer_norm_min_max_observer`` followed by ``quantization`` (symmetric, per layer,
    int8 codes) of its output -- the dynamic activation quantisation in front of
    ``matmul_quant``.  Returns ``(codes, scale, zero_point)``; the normalised tensor is not
    returned.  For fp16 rows of 512, 1024, 2048 or 4096 elements with gamma and beta the library
    runs it as two kernels that never write the normalised tensor; every other case is the two
    ops in a row.  The codes and the scale carry the same bits either way."""
    _check(1 < quantization_bit <= 8, "quantization_bit should be in range (1, 8].")
    _check(x.dtype in (torch.float16, torch.bfloat16, torch.float32),
           f"no fused_layer_norm_quantization kernel for dtype {x.dtype}")
    cols = x.shape[-1]
    for name, p in (("gamma", gamma), ("beta", beta)):
        if p is not None:
            _check(p.dtype == x.dtype and p.numel() == cols,
                   f"{name} should have the dtype of x and x.shape[-1] elements")
    _require_gpu(x, gamma, beta)
    x, gamma, beta = _contig(x), _contig(gamma), _contig(beta)
    rows = x.numel() // cols
    L = _lib.lib()
    codes = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    scale = torch.empty(1, dtype=torch.float32, device=x.device)
    zero_point = torch.empty(1, dtype=torch.float32, device=x.device)
    ws_bytes = L.ofq_fused_layer_norm_quantization_workspace_bytes(_dt(x), rows, cols)
    ws = _workspace(ws_bytes, x.device)
    st = L.ofq_fused_layer_norm_quantization(
        _stream(x), _ptr(x), _ptr(gamma), _ptr(beta), _ptr(codes), _ptr(scale), _ptr(zero_point),
        _dt(x), rows, cols, float(epsilon), quantization_bit,
        _lib.LN_STATS_FP64 if exact_statistics else _lib.LN_STATS_FP32, _ptr(ws), ws_bytes)
    if st == _lib.ERR_UNSUPPORTED:
        y, scale, zero_point = fused_layer_norm_min_max_observer(
            x, gamma, beta, epsilon, quantization_bit, exact_statistics=exact_statistics)
        codes = quantization(y, scale, zero_point, "google", quantization_bit, "symmetric",
                             out_dtype=torch.int8)
        return codes, scale, zero_point
    _lib.check("ofq_fused_layer_norm_quantization", st)
    return codes, scale, zero_point


def fused_skip_layer_norm_min_max_observer(x, gamma=None, beta=None, bias=None, skip=None,
                                           epsilon=1e-5, alpha=1e1, quantization_bit=8,
                                           *, exact_statistics=False):
    """``skip_layer_norm`` (same arguments and defaults as the reference functional,
    functional_api.yaml:1545-1546: the row normalised is ``(x + bias) + skip * alpha`` in the
    dtype of x) + per-tensor symmetric observer of the result.  Returns
    ``(y, scale, zero_point)``."""
    _check(1 < quantization_bit <= 8, "quantization_bit should be in range (1, 8].")
    _check(x.dtype in (torch.float16, torch.bfloat16, torch.float32),
           f"no fused_skip_layer_norm_min_max_observer kernel for dtype {x.dtype}")
    _check(x.dim() >= 2, "number of axes of x should be greater than or equal to 2")
    cols = x.shape[-1]
    for name, p in (("gamma", gamma), ("beta", beta), ("bias", bias)):
        if p is not None:
            _check(p.dtype == x.dtype and p.dim() == 1 and p.numel() == cols,
                   f"{name} should be 1-D with the dtype of x and x.shape[-1] elements")
    if skip is not None:
        _check(skip.dtype == x.dtype and tuple(skip.shape) == tuple(x.shape),
               "skip should have the shape and dtype of x")
    _require_gpu(x, gamma, beta, bias, skip)
    x, gamma, beta, bias, skip = map(_contig, (x, gamma, beta, bias, skip))
    rows = x.numel() // cols
    y = torch.empty_like(x)
    scale = torch.empty(1, dtype=torch.float32, device=x.device)
    zero_point = torch.empty(1, dtype=torch.float32, device=x.device)
    L = _lib.lib()
    ws_bytes = L.ofq_fused_layer_norm_min_max_observer_workspace_bytes(_dt(x), rows, cols)
    ws = _workspace(ws_bytes, x.device)
    if exact_statistics:
        st = L.ofq_fused_layer_norm_min_max_observer_stats(
            _stream(x), _ptr(x), _ptr(bias), _ptr(skip), float(alpha), 1, _ptr(gamma),
            _ptr(beta), _ptr(y), _ptr(scale), _ptr(zero_point), _dt(x), rows, cols,
            float(epsilon), quantization_bit, _lib.LN_STATS_FP64, _ptr(ws), ws_bytes)
    else:
        st = L.ofq_fused_skip_layer_norm_min_max_observer(
            _stream(x), _ptr(x), _ptr(bias), _ptr(skip), float(alpha), _ptr(gamma), _ptr(beta),
            _ptr(y), _ptr(scale), _ptr(zero_point), _dt(x), rows, cols, float(epsilon),
            quantization_bit, _ptr(ws), ws_bytes)
    _lib.check("ofq_fused_skip_layer_norm_min_max_observer", st)
    return y, scale, zero_point


def matmul_quant(a, b, a_scale, b_scale, bias=None, out_dtype=torch.float16):
    """int8 ``a[m,k]`` x int8 ``b[n,k]`` -> ``out_dtype[m,n]``; exact int32 accumulation, then
    ``acc * (a_scale * b_scale[n]) + bias[n]``."""
    _check(a.dtype == torch.int8 and b.dtype == torch.int8, "a and b should be int8")
    _check(a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[1],
           "a should be [m,k] and b [n,k]")
    _check(a_scale.dtype == torch.float32 and a_scale.numel() == 1,
           "a_scale should be one float32")
    _check(b_scale.dtype == torch.float32 and b_scale.numel() == b.shape[0],
           "b_scale should be float32 with b.shape[0] elements")
    if bias is not None:
        _check(bias.dtype == out_dtype and bias.numel() == b.shape[0],
               "bias should have the output dtype and b.shape[0] elements")
    _require_gpu(a, b, a_scale, b_scale, bias)
    a, b, a_scale, b_scale, bias = map(_contig, (a, b, a_scale, b_scale, bias))
    m, k = a.shape
    n = b.shape[0]
    out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    L = _lib.lib()
    ws_bytes = L.ofq_matmul_quant_workspace_bytes(m, n, k)
    ws = _workspace(ws_bytes, a.device) if ws_bytes else None
    st = L.ofq_matmul_quant_ws(_stream(a), _ptr(a), _ptr(b), _ptr(a_scale), _ptr(b_scale),
                               _ptr(bias), _ptr(out), _dt(out), m, n, k, _ptr(ws), ws_bytes)
    _lib.check("ofq_matmul_quant_ws", st)
    return out
