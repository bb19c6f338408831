from . import backend, low_precision, utils  # noqa: F401
from .quantized_tensor import QuantizedTensor, QuantizedTensorPair  # noqa: F401

__all__ = ["QuantizedTensor", "QuantizedTensorPair"]
