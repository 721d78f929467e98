"""Per-group FP8 quantize of x and of x^T in one pass.
Reference: coat/activation/real_quantization/_quantize_transpose.py:175-226 (outputs are always 2-D)."""
import torch

from ... import _hip
from .common import as_fp8_dtype, flatten_2d


def fp8_quantize_transpose(x, QB, fp8type, scale_dtype=torch.bfloat16):
    x, _ = flatten_2d(x)
    x = _hip.dense(x)
    M, N = x.shape
    fp8type = as_fp8_dtype(fp8type)
    y = torch.empty_like(x, dtype=fp8type)
    y_t = torch.empty((N, M), dtype=fp8type, device=x.device)
    s_y = torch.empty((M, N // QB), dtype=scale_dtype, device=x.device)
    s_y_t = torch.empty((N, M // QB), dtype=scale_dtype, device=x.device)
    _hip.check(_hip.lib().coat_fp8_quantize_transpose(
        _hip.ptr(x), _hip.dt(x), _hip.ptr(y), _hip.ptr(s_y), _hip.ptr(y_t), _hip.ptr(s_y_t), _hip.dt(s_y), M, N, QB,
        _hip.fp8(fp8type), _hip.stream(x.device)), "fp8_quantize_transpose")
    return (y, s_y), (y_t, s_y_t)
