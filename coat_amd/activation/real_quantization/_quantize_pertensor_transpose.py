"""Per-tensor FP8 quantize through Group Scaling, with the transposed copy the backward GEMMs need.
Reference: coat/activation/real_quantization/_quantize_pertensor_transpose.py:106-150."""
import torch

from ... import _hip
from ._division import _division
from ._quantize_pertensor import group_scales_and_max
from .common import convert_str_to_fp8, flatten_2d, known_scale_max, restore


def fp8_quantize_pertensor_transpose(x, QB, fp8type, transpose_output_2d=False, stochastic=False,
                                     scale_dtype=torch.bfloat16):
    """Returns (qy, s_y_max 0-dim, qy_t); qy_t is [N, M] unless the input was 3-D and
    transpose_output_2d is False (then it is reshaped per batch, reference :145-150).
    stochastic goes to the division pass (reference :140-142).  A tensor whose producer kernel already merged the
    maximum of its group scales (``common.tag_scale_max``) skips the scale pass."""
    fp8type = convert_str_to_fp8[fp8type]
    s_y_max = known_scale_max(x, fp8type)
    x, batch = flatten_2d(x)
    x = _hip.dense(x)
    if s_y_max is None:
        _, s_y_max = group_scales_and_max(x, QB, fp8type, scale_dtype, want_pg=False)
    qy, s_y_max, qy_t = _division(x, fp8type, s_y_max, True, True, "fp8_quantize_pertensor_transpose",
                                   stochastic, max_as=scale_dtype)
    if batch is not None and not transpose_output_2d:
        qy_t = qy_t.reshape(batch, -1, qy_t.shape[-1])
    return restore(qy, batch), s_y_max, qy_t
