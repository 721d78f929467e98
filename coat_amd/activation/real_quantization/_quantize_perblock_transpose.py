"""Per-block FP8 quantize of x together with the transposed codes and scales.
Reference: coat/activation/real_quantization/_quantize_perblock_transpose.py:136-190."""
import torch

from ._quantize_perblock import _perblock


def fp8_quantize_perblock_transpose(x, QB, fp8type, scale_dtype=torch.bfloat16, only_transposed=False):
    (y, s_y), (y_t, s_y_t), _ = _perblock(x, QB, fp8type, scale_dtype, not only_transposed, True, False,
                                          "fp8_quantize_perblock_transpose")
    if not only_transposed:
        return (y, s_y), (y_t, s_y_t)
    return y_t, s_y_t
