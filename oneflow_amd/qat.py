"""Quantization-aware-training wrappers of the reference, python/oneflow/nn/qat/conv.py:22-57 and
the three classes below them: a convolution whose input and weight pass through fake quantization,
the input's scale coming from a moving-average observer and the weight's from a min/max observer
(per layer or per output channel).  Same constructor arguments and defaults; the observers and the
fake quantization are this library's kernels (``oneflow_amd.nn``), the convolution itself is the
host framework's.  Gradients flow straight through the fake quantization
(oneflow/core/autograd/gradient_funcs/fake_quantization.cpp:36-42)."""
import torch

from . import nn as _nn


def get_conv_fake_quantized(input, input_observer, current_train_step, weight, weight_observer,
                            fake_quantizer):
    in_scale, in_zero_point = input_observer(input, current_train_step)
    input_fake_quanted = fake_quantizer(input, in_scale, in_zero_point)
    w_scale, w_zero_point = weight_observer(weight)
    weight_fake_quanted = fake_quantizer(weight, w_scale, w_zero_point)
    return input_fake_quanted, weight_fake_quanted


def init_conv_fake_quants(self, quantization_formula="google", quantization_bit=8,
                          quantization_scheme="symmetric", weight_quant_per_layer=True,
                          input_quant_momentum=0.95):
    self.input_min_max_observer = _nn.MovingAverageMinMaxObserver(
        stop_update_after_iters=1, quantization_formula=quantization_formula,
        quantization_bit=quantization_bit, quantization_scheme=quantization_scheme,
        momentum=input_quant_momentum)
    self.register_buffer("current_train_step", torch.zeros(1, dtype=torch.int64))
    self.weight_min_max_observer = _nn.MinMaxObserver(
        quantization_formula=quantization_formula, quantization_bit=quantization_bit,
        quantization_scheme=quantization_scheme, per_layer_quantization=weight_quant_per_layer)
    self.fake_quantizer = _nn.FakeQuantization(
        quantization_formula=quantization_formula, quantization_bit=quantization_bit,
        quantization_scheme=quantization_scheme)


def _qat_conv(base):
    class _QatConv(base):
        def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                     groups=1, bias=True, padding_mode="zeros", quantization_formula="google",
                     quantization_bit=8, quantization_scheme="symmetric",
                     weight_quant_per_layer=True, input_quant_momentum=0.95, **kwargs):
            super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation,
                             groups, bias, padding_mode, **kwargs)
            self.channel_pos = "channels_first"
            init_conv_fake_quants(self, quantization_formula=quantization_formula,
                                  quantization_bit=quantization_bit,
                                  quantization_scheme=quantization_scheme,
                                  weight_quant_per_layer=weight_quant_per_layer,
                                  input_quant_momentum=input_quant_momentum)

        def forward(self, x):
            fake_quan_input, fake_quan_weight = get_conv_fake_quantized(
                x, self.input_min_max_observer, self.current_train_step, self.weight,
                self.weight_min_max_observer, self.fake_quantizer)
            return self._conv_forward(fake_quan_input, fake_quan_weight, self.bias)

    return _QatConv


QatConv1d = _qat_conv(torch.nn.Conv1d)
QatConv1d.__name__ = QatConv1d.__qualname__ = "QatConv1d"
QatConv2d = _qat_conv(torch.nn.Conv2d)
QatConv2d.__name__ = QatConv2d.__qualname__ = "QatConv2d"
QatConv3d = _qat_conv(torch.nn.Conv3d)
QatConv3d.__name__ = QatConv3d.__qualname__ = "QatConv3d"
