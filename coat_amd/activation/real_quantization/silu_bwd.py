"""FP8 SiLU backward.  Reference: coat/activation/real_quantization/silu_bwd.py:170-238."""
import torch

from ... import _hip
from ._division import _division
from ._fused import new_max, prep_bf16, prep_pg
from .common import as_fp8_dtype, restore


def fp8_silu_backward(x, s_x, g, QB, fp8type, stochastic=False, output_quantized_transpose=False):
    """Returns (y bf16, s_y per-group) or, with output_quantized_transpose, (qy, s_y_max, qy_t [N, M]).
    ``stochastic`` is accepted and has no effect, as in the reference (silu_bwd.py:170-242 never reads it)."""
    x, s_x, batch = prep_pg(x, s_x)
    g = prep_bf16(g)
    M, N = x.shape
    fp8type = as_fp8_dtype(fp8type)
    y = torch.empty_like(g, dtype=torch.bfloat16)
    want_pg = not output_quantized_transpose
    s_y = torch.empty_like(s_x, dtype=torch.bfloat16) if want_pg else None
    s_max = None if want_pg else new_max(x.device)
    _hip.check(_hip.lib().coat_fp8_silu_backward(
        _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(g), _hip.ptr(y), _hip.ptr(s_y),
        _hip.ptr(s_max), _hip.fp8(fp8type), M, N, QB, _hip.stream(x.device)), "fp8_silu_backward")
    if want_pg:
        return restore(y, batch), restore(s_y, batch)
    qy, s_y_max, qy_t = _division(y, fp8type, s_max, True, True, "fp8_silu_backward", max_as=torch.bfloat16)
    return restore(qy, batch), s_y_max, qy_t
