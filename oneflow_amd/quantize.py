"""Weight quantiser + packer: fp16/bf16/fp32 weights -> the groupwise int4/int8 format that
``_C.groupwise_dequantize`` and ``_C.fused_linear_with_groupwise_quantized_weight`` consume.

The reference has no op for this; the format is defined by the helpers of its own test
(``python/oneflow/test/modules/test_groupwise_quantization.py:26-81``), whose signature and
arithmetic ``groupwise_quantize`` follows: ``(num_bits, symmetric, x, group_dim, group_size,
quant_type) -> (quantized, scale, zero)``.
"""
import torch

from . import _lib
from .functional import CheckFailedError, _check, _contig, _dt, _ptr, _require_gpu, _stream


def groupwise_quantize(x, *, num_bits=8, symmetric=True, group_dim=-1, group_size=-1,
                       quant_type=torch.int8):
    """x: 2-D weight [n, k] on the GPU.  Returns ``(quantized, scale, zero)``; ``zero`` is None
    when ``symmetric``.  4-bit codes are packed two per byte along k, element 2i in the high
    nibble; scale/zero have the dtype of x."""
    _check(num_bits in (4, 8), "num_bits should be 4 or 8.")
    _check(x.dim() == 2, "x should be a 2-D weight [n, k].")
    gd = group_dim + 2 if group_dim < 0 else group_dim
    _check(gd in (0, 1), "group_dim should be in range [-2,2).")
    n, k = x.shape
    dim = x.shape[gd]
    gs = dim if group_size < 0 else group_size
    _check(0 < gs <= dim, f"group_size should be in range (0,{dim}].")
    _check(dim % gs == 0, f"group_size should be a divisor of {dim}.")
    _check(quant_type in (torch.int8, torch.uint8), "quant_type should be int8 or uint8.")
    if not symmetric:
        _check(quant_type == torch.uint8, "asymmetric codes are uint8.")
    _check(x.dtype in (torch.float16, torch.bfloat16, torch.float32),
           "x should be float16, bfloat16 or float32.")
    if num_bits == 4:
        _check(k % 2 == 0 and (gd == 0 or gs % 2 == 0), "4-bit codes are packed in pairs along k.")
    _require_gpu(x)
    x = _contig(x)
    q = torch.empty((n, k * num_bits // 8), dtype=quant_type, device=x.device)
    sshape = (n // gs, k) if gd == 0 else (n, k // gs)
    scale = torch.empty(sshape, dtype=x.dtype, device=x.device)
    zero = None if symmetric else torch.empty(sshape, dtype=x.dtype, device=x.device)
    L = _lib.lib()
    _lib.check("ofq_groupwise_quantize",
               L.ofq_groupwise_quantize(_stream(x), _ptr(x), _ptr(q), _ptr(scale), _ptr(zero),
                                        _dt(x), _dt(q), num_bits, int(symmetric), gd, gs, n, k))
    return q, scale, zero


__all__ = ["groupwise_quantize", "CheckFailedError"]
