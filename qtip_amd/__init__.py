"""MI355X-native implementation of QTIP's quantized-linear inference path.

Layout mirrors the part of the reference package it replaces:
  qtip_amd.codebook            op registry (lib/codebook/__init__.py)
  qtip_amd.codebook.bitshift   BitshiftLinear & co. (lib/codebook/bitshift.py)
  qtip_amd.utils.matmul_had    RHT helpers (lib/utils/matmul_had.py)
  qtip_amd.utils.kernel_decompress / kernel_check
  qtip_amd.linear.quantized_linear  QuantizedLinear (lib/linear/quantized_linear.py)
  qtip_amd.ops                 thin tensor-level wrappers over the C ABI
"""
__version__ = "0.1.0"
