from .quantized_linear import QuantizedLinear
