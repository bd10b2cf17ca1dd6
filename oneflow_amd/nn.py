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
