"""FP8 byte transpose.  Reference: coat/activation/real_quantization/_transpose.py:85-115."""
import torch

from ... import _hip
from .common import flatten_2d


def fp8_transpose(x, transpose_output_2d=False):
    x, batch = flatten_2d(x)
    x = _hip.dense(x)
    M, N = x.shape
    y = torch.empty((N, M), dtype=x.dtype, device=x.device)
    _hip.check(_hip.lib().coat_fp8_transpose(_hip.ptr(x), _hip.ptr(y), M, N, _hip.stream(x.device)), "fp8_transpose")
    if batch is not None and not transpose_output_2d:
        y = y.reshape(batch, -1, y.shape[-1])
    return y
