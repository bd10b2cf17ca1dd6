"""``nn.Module`` wrappers with the constructor arguments and call signatures of the reference
modules (python/oneflow/nn/modules/min_max_observer.py:94-114, quantization.py:88-109,
fake_quantization.py); each forwards to the matching ``_C`` function."""
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
