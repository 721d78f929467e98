"""Per-group (1 x QB) FP8 quantize.  Reference: coat/activation/real_quantization/_quantize.py:120-163."""
import torch

from ... import _hip
from .common import as_fp8_dtype, flatten_2d, restore


def fp8_quantize(x, QB, fp8type, scale_dtype=torch.bfloat16):
    """x [.., N] -> (y fp8 same shape, s_y [.., N/QB]); s = (amax + 1e-10) / fp8max, y = fp8(x / s)."""
    x, batch = flatten_2d(x)
    x = _hip.dense(x)
    M, N = x.shape
    fp8type = as_fp8_dtype(fp8type)
    y = torch.empty_like(x, dtype=fp8type)
    s_y = torch.empty((M, N // QB), dtype=scale_dtype, device=x.device)
    _hip.check(_hip.lib().coat_fp8_quantize(_hip.ptr(x), _hip.dt(x), _hip.ptr(y), _hip.ptr(s_y), _hip.dt(s_y), M, N, QB,
                                            _hip.fp8(fp8type), _hip.stream(x.device)), "fp8_quantize")
    return restore(y, batch), restore(s_y, batch)
