"""FP8 GELU forward.  Reference: coat/activation/real_quantization/gelu_fwd.py:152-203."""
import torch

from ... import _hip
from ._division import _division
from ._fused import new_max, prep_pg
from .common import restore


def fp8_gelu_forward(x, s_x, QB, transpose_output_2d=False):
    """Returns (qy, s_y_max, qy_t) in x's fp8 dtype."""
    x, s_x, batch = prep_pg(x, s_x)
    M, N = x.shape
    y = torch.empty_like(x, dtype=torch.bfloat16)
    s_max = new_max(x.device)
    _hip.check(_hip.lib().coat_fp8_gelu_forward(_hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(y),
                                                None, _hip.ptr(s_max), M, N, QB, _hip.stream(x.device)), "fp8_gelu_forward")
    qy, s_y_max, qy_t = _division(y, x.dtype, s_max, True, True, "fp8_gelu_forward", max_as=s_x.dtype)
    if batch is not None and not transpose_output_2d:
        qy_t = qy_t.reshape(batch, -1, qy.shape[-1])
    return restore(qy, batch), s_y_max, qy_t
