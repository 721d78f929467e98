"""Per-block FP8 quantize: one scale per QB x QB block of the (flattened) 2-D input.
Reference: coat/activation/real_quantization/_quantize_perblock.py:107-150 (outputs are always 2-D)."""
import torch

from ... import _hip
from .common import as_fp8_dtype, flatten_2d


def _perblock(x, QB, fp8type, scale_dtype, plain, transposed, pergroup, name):
    """The one kernel behind the three per-block entry points; absent outputs are returned as the uninitialised tensors the
    reference returns for them."""
    x, _ = flatten_2d(x)
    x = _hip.dense(x)
    M, N = x.shape
    assert M % QB == 0 and N % QB == 0, f"{name}: both dimensions of {tuple(x.shape)} must be multiples of QB = {QB}"
    fp8type = as_fp8_dtype(fp8type)
    dev = x.device

    def pair(shape, s_shape):
        return torch.empty(shape, dtype=fp8type, device=dev), torch.empty(s_shape, dtype=scale_dtype, device=dev)

    y, s_y = pair((M, N), (M // QB, N // QB))
    y_t, s_y_t = pair((N, M), (N // QB, M // QB)) if transposed is not None else (None, None)
    y_pg, s_y_pg = pair((M, N), (M, N // QB)) if pergroup else (None, None)
    p = _hip.ptr
    _hip.check(_hip.lib().coat_fp8_quantize_perblock(
        p(x), _hip.dt(x), p(y) if plain else None, p(s_y) if plain else None, p(y_t) if transposed else None,
        p(s_y_t) if transposed else None, p(y_pg), p(s_y_pg), _hip.dt(s_y), M, N, QB, _hip.fp8(fp8type),
        _hip.stream(dev)), name)
    return (y, s_y), (y_t, s_y_t), (y_pg, s_y_pg)


def fp8_quantize_perblock(x, QB, fp8type, scale_dtype=torch.bfloat16):
    (y, s_y), _, _ = _perblock(x, QB, fp8type, scale_dtype, True, None, False, "fp8_quantize_perblock")
    return y, s_y
