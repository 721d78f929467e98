"""FP8 SiLU forward: per-group FP8 in, per-group FP8 out.
Reference: coat/activation/real_quantization/silu_fwd.py:152-198."""
import torch

from ... import _hip
from ._fused import prep_pg
from .common import restore


def fp8_silu_forward(x, s_x, QB):
    x, s_x, batch = prep_pg(x, s_x)
    M, N = x.shape
    y = torch.empty_like(x)
    s_y = torch.empty_like(s_x)  # in the dtype of the input scales, as the reference allocates it (:166-167)
    _hip.check(_hip.lib().coat_fp8_silu_forward(_hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(y),
                                                _hip.ptr(s_y), M, N, QB, _hip.stream(x.device)), "fp8_silu_forward")
    return restore(y, batch), restore(s_y, batch)
