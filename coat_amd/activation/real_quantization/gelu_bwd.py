"""FP8 GELU backward.  Reference: coat/activation/real_quantization/gelu_bwd.py:173-230."""
import torch

from ... import _hip
from ._division import _division
from ._fused import new_max, prep_bf16, prep_pg
from .common import as_fp8_dtype, restore


def fp8_gelu_backward(x, s_x, g, QB, fp8type):
    """Returns (qy, s_y_max): per-tensor FP8 of the gradient (no transpose, as in the reference)."""
    x, s_x, batch = prep_pg(x, s_x)
    g = prep_bf16(g)
    M, N = x.shape
    fp8type = as_fp8_dtype(fp8type)
    y = torch.empty_like(g, dtype=torch.bfloat16)
    s_max = new_max(x.device)
    _hip.check(_hip.lib().coat_fp8_gelu_backward(
        _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(g), _hip.ptr(y), None, _hip.ptr(s_max),
        _hip.fp8(fp8type), M, N, QB, _hip.stream(x.device)), "fp8_gelu_backward")
    qy, s_y_max, _ = _division(y, fp8type, s_max, True, False, "fp8_gelu_backward", max_as=torch.bfloat16)
    return restore(qy, batch), s_y_max
