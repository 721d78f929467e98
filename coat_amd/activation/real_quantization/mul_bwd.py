"""FP8 multiply backward.  Reference: coat/activation/real_quantization/mul_bwd.py:221-315."""
import torch

from ... import _hip
from ._division import _division
from ._fused import new_max, prep_bf16, prep_pg
from .common import as_fp8_dtype, restore


def fp8_mul_backward(x1, s_x1, x2, s_x2, g, QB, fp8type, stochastic=False, output_quantized_transpose=False):
    """Returns (y1 bf16, (y2 bf16, s_y2)) or (y1 bf16, (qy2, s_y2_max, qy2_t)):
    y1 = g * x2 is the gradient of x1, y2 = g * x1 the gradient of x2.
    ``stochastic`` is accepted and has no effect, as in the reference (mul_bwd.py:236-239 allocates noise that the
    kernel never reads, and the division at :305 is called without the flag)."""
    x1, s_x1, batch = prep_pg(x1, s_x1)
    x2, s_x2, _ = prep_pg(x2, s_x2)
    g = prep_bf16(g)
    assert x1.shape == x2.shape
    assert s_x1.shape == s_x2.shape
    if s_x2.dtype != s_x1.dtype:
        s_x2 = s_x2.to(s_x1.dtype)
    M, N = x1.shape
    fp8type = as_fp8_dtype(fp8type)
    y1 = torch.empty_like(g, dtype=torch.bfloat16)
    y2 = torch.empty_like(g, dtype=torch.bfloat16)
    want_pg = not output_quantized_transpose
    s_y2 = torch.empty_like(s_x1, dtype=torch.bfloat16) if want_pg else None
    s_max = None if want_pg else new_max(x1.device)
    _hip.check(_hip.lib().coat_fp8_mul_backward(
        _hip.ptr(x1), _hip.ptr(s_x1), _hip.ptr(x2), _hip.ptr(s_x2), _hip.fp8(x1.dtype), _hip.dt(s_x1), _hip.ptr(g),
        _hip.ptr(y1), _hip.ptr(y2), _hip.ptr(s_y2), _hip.ptr(s_max), _hip.fp8(fp8type), M, N, QB,
        _hip.stream(x1.device)), "fp8_mul_backward")
    if want_pg:
        return restore(y1, batch), (restore(y2, batch), restore(s_y2, batch))
    qy2, s_y2_max, qy2_t = _division(y2, fp8type, s_max, True, True, "fp8_mul_backward", max_as=torch.bfloat16)
    return restore(y1, batch), (restore(qy2, batch), s_y2_max, qy2_t)
