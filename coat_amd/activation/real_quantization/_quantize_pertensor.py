"""Per-tensor FP8 quantize through Group Scaling: per-group scales, their maximum, one division pass.
Reference: coat/activation/real_quantization/_quantize_pertensor.py:106-147."""
import torch

from ... import _hip
from ._division import _division
from .common import convert_str_to_fp8, flatten_2d, known_scale_max, new_max, restore


def group_scales_and_max(x, QB, fp8type, scale_dtype=torch.bfloat16, want_pg=True):
    """(s_pg [M, N/QB] or None, maximum of the fp32 group scales as a 0-dim fp32 tensor) in one pass over x.

    Rounding to scale_dtype is monotone, so rounding the maximum (which the division pass does) equals the reference's ``s_y.max()`` over the rounded scales (reference :139)."""
    M, N = x.shape
    s_pg = torch.empty((M, N // QB), dtype=scale_dtype, device=x.device) if want_pg else None
    s_max = new_max(x.device)
    _hip.check(_hip.lib().coat_fp8_group_scales(_hip.ptr(x), _hip.dt(x), _hip.ptr(s_pg), _hip.dt(scale_dtype),
                                                _hip.ptr(s_max), M, N, QB, _hip.fp8(fp8type), _hip.stream(x.device)),
               "fp8_group_scales")
    return s_pg, s_max


def fp8_quantize_pertensor(x, QB, fp8type, stochastic=False, scale_dtype=torch.bfloat16, want_pg=True):
    """Returns (y fp8, s_y_max 0-dim, s_y per-group).  stochastic goes to the division pass (reference :140).
    ``want_pg=False``: the per-group scales are not wanted (None is returned for them), and a tensor whose producer
    kernel already merged their maximum (``common.tag_scale_max``) skips the scale pass."""
    fp8type = convert_str_to_fp8[fp8type]  # the reference accepts only the string here (:118)
    s_y_max = None if want_pg else known_scale_max(x, fp8type)
    x, batch = flatten_2d(x)
    x = _hip.dense(x)
    s_y = None
    if s_y_max is None:
        s_y, s_y_max = group_scales_and_max(x, QB, fp8type, scale_dtype, want_pg=want_pg)
    y, s_y_max, _ = _division(x, fp8type, s_y_max, True, False, "fp8_quantize_pertensor", stochastic,
                                max_as=scale_dtype)
    return restore(y, batch), s_y_max, None if s_y is None else restore(s_y, batch)
