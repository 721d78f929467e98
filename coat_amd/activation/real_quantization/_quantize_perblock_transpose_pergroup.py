"""Per-block FP8 quantize of x, its transpose, and the 1 x QB per-group quantization of the same x in one pass.
Reference: coat/activation/real_quantization/_quantize_perblock_transpose_pergroup.py:175-246.  With
``only_transposed`` the plain per-block pair is returned uninitialised, as in the reference (:139-141, :193-198)."""
import torch

from ._quantize_perblock import _perblock


def fp8_quantize_perblock_transpose_pergroup(x, QB, fp8type, scale_dtype=torch.bfloat16, only_transposed=False):
    return _perblock(x, QB, fp8type, scale_dtype, not only_transposed, True, True,
                     "fp8_quantize_perblock_transpose_pergroup")
