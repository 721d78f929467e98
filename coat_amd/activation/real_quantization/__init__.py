"""FP8 op library (reference: coat/activation/real_quantization/__init__.py:3-25)."""
from ._dequantize import fp8_dequantize
from ._division import fp8_division
from ._division_transpose import fp8_division_transpose
from ._quantize import fp8_quantize
from ._quantize_pertensor import fp8_quantize_pertensor
from ._quantize_pertensor_transpose import fp8_quantize_pertensor_transpose
from ._quantize_transpose import fp8_quantize_transpose
from ._transpose import fp8_transpose
