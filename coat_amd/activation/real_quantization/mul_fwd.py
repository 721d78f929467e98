"""FP8 multiply forward (gate * up): two per-group FP8 inputs, per-tensor FP8 output and its transpose.
Reference: coat/activation/real_quantization/mul_fwd.py:191-254."""
import torch

from ... import _hip
from ._division import _division
from ._fused import new_max, prep_pg
from .common import restore


def fp8_mul_forward(x1, s_x1, x2, s_x2, QB, transpose_output_2d=False):
    """Returns (qy, s_y_max, qy_t) in x2's fp8 dtype."""
    x1, s_x1, batch = prep_pg(x1, s_x1)
    x2, s_x2, _ = prep_pg(x2, s_x2)
    assert x1.shape == x2.shape
    assert s_x1.shape == s_x2.shape
    if s_x2.dtype != s_x1.dtype:
        s_x2 = s_x2.to(s_x1.dtype)
    M, N = x1.shape
    y = torch.empty_like(x1, dtype=torch.bfloat16)
    s_max = new_max(x1.device)
    _hip.check(_hip.lib().coat_fp8_mul_forward(
        _hip.ptr(x1), _hip.ptr(s_x1), _hip.ptr(x2), _hip.ptr(s_x2), _hip.fp8(x1.dtype), _hip.dt(s_x1), _hip.ptr(y),
        None, _hip.ptr(s_max), M, N, QB, _hip.stream(x1.device)), "fp8_mul_forward")
    qy, s_y_max, qy_t = _division(y, x2.dtype, s_max, True, True, "fp8_mul_forward", max_as=s_x1.dtype)
    if batch is not None and not transpose_output_2d:
        qy_t = qy_t.reshape(batch, -1, qy.shape[-1])
    return restore(qy, batch), s_y_max, qy_t
