"""MI355X-native kernels for OneFlow's quantized-inference op family.

``oneflow_amd._C`` mirrors the ``flow._C.*`` functions of the reference for this path;
``oneflow_amd.nn`` mirrors its thin ``nn.Module`` wrappers, ``oneflow_amd.qat`` its
quantization-aware-training convolutions; ``oneflow_amd.quantize`` produces the
packed weight format the ops consume.  The HIP library is loaded lazily on
first call and there is no CPU fallback.
"""
from . import functional as _C  # noqa: F401  (same spelling as the reference's flow._C)
from . import nn  # noqa: F401
from . import qat  # noqa: F401
from . import quantize  # noqa: F401
from ._lib import LIB_PATH, OfqError  # noqa: F401
from .functional import CheckFailedError  # noqa: F401

__all__ = ["_C", "nn", "qat", "quantize", "LIB_PATH", "OfqError", "CheckFailedError"]
