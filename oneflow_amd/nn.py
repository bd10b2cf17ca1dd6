"""``nn.Module`` wrappers with the constructor arguments and call signatures of the reference
modules (python/oneflow/nn/modules/min_max_observer.py:94-114, quantization.py:88-109,
fake_quantization.py, moving_average_min_max_observer.py:119-153); each forwards to the matching
``_C`` function."""
import torch

from . import functional as _C


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

    def forward(self, x):
        return _C.fused_linear_with_groupwise_quantized_weight(
            x, self.weight, self.weight_scale, w_zero=self.weight_zero, b=self.bias,
            num_bits=self.num_bits, symmetric=self.symmetric, group_dim=1,
            group_size=self.group_size)

    def extra_repr(self):
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"num_bits={self.num_bits}, symmetric={self.symmetric}, group_size={self.group_size}")
