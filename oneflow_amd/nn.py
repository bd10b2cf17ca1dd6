"""``nn.Module`` wrappers with the constructor arguments and call signatures of the reference
modules (python/oneflow/nn/modules/min_max_observer.py:94-114, quantization.py:88-109,
fake_quantization.py, moving_average_min_max_observer.py:119-153); each forwards to the matching
``_C`` function."""
import torch

from . import functional as _C
from ._lib import OfqError


class MinMaxObserver(torch.nn.Module):
    def __init__(self, quantization_formula="google", quantization_bit=8,
                 quantization_scheme="symmetric", per_layer_quantization=True):
        super().__init__()
        self.quantization_formula = quantization_formula
        self.quantization_bit = quantization_bit
        self.quantization_scheme = quantization_scheme
        self.per_layer_quantization = per_layer_quantization

    def forward(self, input):
        return _C.min_max_observer(input, self.quantization_formula, self.quantization_bit,
                                   self.quantization_scheme, self.per_layer_quantization)


class Quantization(torch.nn.Module):
    def __init__(self, quantization_formula="google", quantization_bit=8,
                 quantization_scheme="symmetric"):
        super().__init__()
        self.quantization_formula = quantization_formula
        self.quantization_bit = quantization_bit
        self.quantization_scheme = quantization_scheme

    def forward(self, input, scale, zero_point):
        return _C.quantization(input, scale, zero_point, self.quantization_formula,
                               self.quantization_bit, self.quantization_scheme)


class FakeQuantization(torch.nn.Module):
    def __init__(self, quantization_formula="google", quantization_bit=8,
                 quantization_scheme="symmetric"):
        super().__init__()
        self.quantization_formula = quantization_formula
        self.quantization_bit = quantization_bit
        self.quantization_scheme = quantization_scheme

    def forward(self, input, scale, zero_point):
        return _C.fake_quantization(input, scale, zero_point, self.quantization_formula,
                                    self.quantization_bit, self.quantization_scheme)


class MovingAverageMinMaxObserver(torch.nn.Module):
    """Per-tensor observer with exponential moving extremes kept in the buffers ``moving_max`` /
    ``moving_min`` (move the module to the GPU before use; the buffers take the dtype of the
    first input if it differs)."""

    def __init__(self, stop_update_after_iters=1, quantization_formula="google",
                 quantization_bit=8, quantization_scheme="symmetric", momentum=0.95):
        super().__init__()
        self.quantization_formula = quantization_formula
        self.stop_update_after_iters = stop_update_after_iters
        self.quantization_bit = quantization_bit
        self.quantization_scheme = quantization_scheme
        self.momentum = momentum
        self.register_buffer("moving_max", torch.zeros(1))
        self.register_buffer("moving_min", torch.zeros(1))

    def reset_running_stats(self):
        self.moving_max.fill_(0)
        self.moving_min.fill_(0)

    def forward(self, input, current_train_step):
        if self.moving_max.dtype != input.dtype:
            self.moving_max = self.moving_max.to(input.dtype)
            self.moving_min = self.moving_min.to(input.dtype)
        return _C.moving_average_min_max_observer(
            input, current_train_step, self.moving_max, self.moving_min, self.training,
            self.stop_update_after_iters, self.quantization_formula, self.quantization_bit,
            self.quantization_scheme, self.momentum)


class QuantizedLinear(torch.nn.Module):
    """``y = x @ dequantize(weight).T + bias`` on groupwise int4/int8 weights through
    ``_C.fused_linear_with_groupwise_quantized_weight`` -- the module the reference leaves to its
    users (its test builds the packed tensors by hand,
    python/oneflow/test/modules/test_groupwise_quantization.py:124-182).  Buffers: ``weight``
    ``[out_features, in_features * num_bits / 8]`` (int8 or uint8), ``weight_scale`` and, when
    asymmetric, ``weight_zero`` ``[out_features, in_features / group_size]``, optional ``bias``;
    they are plain buffers, so ``state_dict`` round-trips the packed format."""

    def __init__(self, in_features, out_features, bias=True, num_bits=4, symmetric=True,
                 group_size=128, quant_type=torch.int8, dtype=torch.float16, device=None):
        super().__init__()
        if num_bits not in (4, 8):
            raise ValueError("num_bits should be 4 or 8.")
        if in_features % group_size != 0:
            raise ValueError("group_size should be a divisor of in_features.")
        if not symmetric and quant_type != torch.uint8:
            raise ValueError("asymmetric codes are uint8.")
        self.in_features, self.out_features = in_features, out_features
        self.num_bits, self.symmetric, self.group_size = num_bits, symmetric, group_size
        groups = in_features // group_size
        self.register_buffer("weight", torch.zeros((out_features, in_features * num_bits // 8),
                                                   dtype=quant_type, device=device))
        self.register_buffer("weight_scale", torch.ones((out_features, groups), dtype=dtype,
                                                        device=device))
        self.register_buffer("weight_zero", None if symmetric else torch.zeros(
            (out_features, groups), dtype=dtype, device=device))
        self.register_buffer("bias", torch.zeros(out_features, dtype=dtype, device=device)
                             if bias else None)
        # the optional tile-major copy of `weight` (make_decode_copy): a buffer, so that it moves
        # with the module, but not part of state_dict; `_tiled_from` names the weight tensor and
        # the version of its contents the copy was made from
        self.register_buffer("weight_tiled", None, persistent=False)
        self._tiled_from = None

    @classmethod
    def from_float(cls, linear, num_bits=4, symmetric=True, group_size=128,
                   quant_type=torch.int8):
        """Quantises the weight of a ``torch.nn.Linear`` that lives on the GPU (fp16, bf16 or
        fp32) with ``quantize.groupwise_quantize``."""
        from . import quantize
        w = linear.weight.detach()
        mod = cls(linear.in_features, linear.out_features, linear.bias is not None, num_bits,
                  symmetric, group_size, quant_type, w.dtype, w.device)
        q, scale, zero = quantize.groupwise_quantize(w, num_bits=num_bits, symmetric=symmetric,
                                                     group_dim=1, group_size=group_size,
                                                     quant_type=quant_type)
        mod.weight, mod.weight_scale = q, scale
        if not symmetric:
            mod.weight_zero = zero
        if linear.bias is not None:
            mod.bias = linear.bias.detach().clone()
        return mod

    def make_decode_copy(self):
        """Extension: keeps a tile-major copy of the 4-bit weight beside the row-major one
        (``_C.groupwise_repack``; not part of ``state_dict``).  ``forward`` then reads it for 2 to
        16 rows of fp16 ``x`` and the row-major weight for everything else."""
        self._set_decode_copy(_C.groupwise_repack(self.weight, self.num_bits))
        return self

    def _set_decode_copy(self, tiled):
        self.weight_tiled = tiled
        self._tiled_from = (self.weight.data_ptr(), self.weight._version)

    def _decode_copy(self):
        """The tile-major copy if it still belongs to ``weight``; a copy made from a weight that
        has since been reassigned or written to (``load_state_dict``, ``copy_``) is dropped, so
        that every batch size reads the same weights."""
        if self.weight_tiled is None:
            return None
        if self._tiled_from != (self.weight.data_ptr(), self.weight._version):
            self.weight_tiled, self._tiled_from = None, None
        return self.weight_tiled

    def _apply(self, fn, *args, **kwargs):
        # .to() / .cuda() move weight and its copy together: the copy stays valid if it was
        valid = self._decode_copy() is not None
        super()._apply(fn, *args, **kwargs)
        if valid and self.weight_tiled is not None:
            self._tiled_from = (self.weight.data_ptr(), self.weight._version)
        return self

    def _load_from_state_dict(self, *args, **kwargs):
        super()._load_from_state_dict(*args, **kwargs)
        self.weight_tiled, self._tiled_from = None, None

    def forward(self, x):
        tiled = self._decode_copy()
        if tiled is not None and x.dtype == torch.float16 and self.group_size % 128 == 0:
            m = x.numel() // x.shape[-1]
            if 2 <= m <= 16:
                try:
                    return _C.fused_linear_with_tiled_groupwise_quantized_weight(
                        x, tiled, self.weight_scale, w_zero=self.weight_zero, b=self.bias,
                        num_bits=self.num_bits, symmetric=self.symmetric, group_dim=1,
                        group_size=self.group_size)
                except OfqError as e:  # e.g. m * k beyond what the kernel stages in LDS
                    if e.status != 5:  # OFQ_ERR_UNSUPPORTED
                        raise
        return _C.fused_linear_with_groupwise_quantized_weight(
            x, self.weight, self.weight_scale, w_zero=self.weight_zero, b=self.bias,
            num_bits=self.num_bits, symmetric=self.symmetric, group_dim=1,
            group_size=self.group_size)

    def extra_repr(self):
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"num_bits={self.num_bits}, symmetric={self.symmetric}, group_size={self.group_size}")


class QuantizedGLU(torch.nn.Module):
    """``y = (x W^T + b) * act(x V^T + c)`` over two ``QuantizedLinear`` weights of equal shape
    (``hidden`` = W, b and ``gate`` = V, c) through ``_C.fused_glu_with_groupwise_quantized_weight``
    -- a Llama MLP's ``up_proj`` / ``gate_proj`` pair with ``activation="silu"``."""

    def __init__(self, hidden, gate, activation="silu"):
        super().__init__()
        for a in ("in_features", "out_features", "num_bits", "symmetric", "group_size"):
            if getattr(hidden, a) != getattr(gate, a):
                raise ValueError(f"hidden and gate differ in {a}")
        if (hidden.bias is None) != (gate.bias is None):
            raise ValueError("hidden and gate should both have a bias or neither")
        self.hidden, self.gate, self.activation = hidden, gate, activation

    @classmethod
    def from_float(cls, hidden_linear, gate_linear, activation="silu", **quant_args):
        return cls(QuantizedLinear.from_float(hidden_linear, **quant_args),
                   QuantizedLinear.from_float(gate_linear, **quant_args), activation)

    def forward(self, x):
        h, g = self.hidden, self.gate
        return _C.fused_glu_with_groupwise_quantized_weight(
            x, h.weight, h.weight_scale, w_zero=h.weight_zero, b=h.bias, v=g.weight,
            v_scale=g.weight_scale, v_zero=g.weight_zero, c=g.bias, activation=self.activation,
            num_bits=h.num_bits, symmetric=h.symmetric, group_dim=1, group_size=h.group_size)


class GroupedQuantizedLinear(torch.nn.Module):
    """Several ``QuantizedLinear`` modules applied to the same input in one call (the q, k and v
    projections of an attention block) through
    ``_C.grouped_linear_with_groupwise_quantized_weight``; returns the tuple of outputs."""

    def __init__(self, linears):
        super().__init__()
        linears = list(linears)
        for a in ("in_features", "num_bits", "symmetric", "group_size"):
            if any(getattr(m, a) != getattr(linears[0], a) for m in linears):
                raise ValueError(f"the linears differ in {a}")
        self.linears = torch.nn.ModuleList(linears)

    def forward(self, x):
        ls = list(self.linears)
        biases = [m.bias for m in ls]
        if any(b is None for b in biases):
            if not all(b is None for b in biases):
                raise ValueError("either every linear has a bias or none")
            biases = None
        return tuple(_C.grouped_linear_with_groupwise_quantized_weight(
            [x] * len(ls), [m.weight for m in ls], [m.weight_scale for m in ls],
            w_zeros=None if ls[0].symmetric else [m.weight_zero for m in ls], bs=biases,
            num_bits=ls[0].num_bits, symmetric=ls[0].symmetric, group_dim=1,
            group_size=ls[0].group_size))
