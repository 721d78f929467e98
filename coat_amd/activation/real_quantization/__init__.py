"""FP8 op library (reference: coat/activation/real_quantization/__init__.py:3-25)."""
from ._dequantize import fp8_dequantize
from ._division import fp8_division
from ._division_transpose import fp8_division_transpose
from ._quantize import fp8_quantize
from ._quantize_perblock import fp8_quantize_perblock
from ._quantize_pertensor import fp8_quantize_pertensor
from ._quantize_pertensor_transpose import fp8_quantize_pertensor_transpose
from ._quantize_transpose import fp8_quantize_transpose
from ._transpose import fp8_transpose
from .add_bwd import fp8_add_Ifp_Ifp_Ofp_Opt
from .add_fwd import fp8_add_Ifp_Ifp_Ofp_Og16
from .func_layernorm_noparam import (fp8_layernorm_noparam_backward, fp8_layernorm_noparam_backward_add,
                                     fp8_layernorm_noparam_forward)
from .func_layernorm_param import fp8_layernorm_param_backward, fp8_layernorm_param_forward
from .silu_mul import (fp8_silu_mul_backward, fp8_silu_mul_backward_joined, fp8_silu_mul_forward,
                       fp8_silu_mul_forward_from_bf16)
from .func_rmsnorm import fp8_rmsnorm_backward, fp8_rmsnorm_backward_add, fp8_rmsnorm_forward
from .gelu_bwd import fp8_gelu_backward
from .gelu_fwd import fp8_gelu_forward
from .mul_bwd import fp8_mul_backward
from .mul_fwd import fp8_mul_forward
from .silu_bwd import fp8_silu_backward
from .silu_fwd import fp8_silu_forward
from .linear import (fp8_linear_backward, fp8_linear_backward_grouped, fp8_linear_forward, fp8_linear_forward_add,
                     fp8_linear_forward_grouped, fp8matmul_add, fp8matmul_grouped)
from .func_quantize import Coat_quantize_bgn, Coat_quantize_end
