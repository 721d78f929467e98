"""Per-group FP8 dequantize to bf16.  Reference: coat/activation/real_quantization/_dequantize.py:119-156."""
import torch

from ... import _hip
from .common import flatten_2d, restore


def fp8_dequantize(x, s_x, QB):
    x, batch = flatten_2d(x)
    s_x, _ = flatten_2d(s_x)
    x, s_x = _hip.dense(x), _hip.dense(s_x)
    M, N = x.shape
    y = torch.empty_like(x, dtype=torch.bfloat16)
    _hip.check(_hip.lib().coat_fp8_dequantize(_hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(y),
                                              M, N, QB, _hip.stream(x.device)), "fp8_dequantize")
    return restore(y, batch)
