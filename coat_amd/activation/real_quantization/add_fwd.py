"""Residual add, forward: bf16 + bf16 -> bf16 sum and its per-group FP8.
Reference: coat/activation/real_quantization/add_fwd.py:162-213."""
import torch

from ... import _hip
from ._fused import prep_bf16
from .common import as_fp8_dtype, flatten_2d, restore


def fp8_add_Ifp_Ifp_Ofp_Og16(x1, x2, fp8type, QB):
    """Returns (y bf16, (q fp8, s per-group)); the FP8 copy quantizes the fp32 sum, not the rounded bf16."""
    _, batch = flatten_2d(x1)
    for t in (x1, x2):
        if t.dtype != torch.bfloat16:
            raise ValueError(f"fp8_add_Ifp_Ifp_Ofp_Og16 takes bf16 inputs, got {t.dtype}")
    x1, x2 = prep_bf16(x1), prep_bf16(x2)
    assert x1.shape == x2.shape
    M, N = x1.shape
    fp8type = as_fp8_dtype(fp8type)
    y1 = torch.empty_like(x1, dtype=torch.bfloat16)
    y2 = torch.empty_like(x2, dtype=fp8type)
    s_y2 = torch.empty((M, N // QB), dtype=torch.bfloat16, device=x2.device)
    _hip.check(_hip.lib().coat_fp8_add_fwd(_hip.ptr(x1), _hip.ptr(x2), _hip.ptr(y1), _hip.ptr(y2), _hip.ptr(s_y2),
                                           _hip.fp8(fp8type), M, N, QB, _hip.stream(x1.device)), "fp8_add_Ifp_Ifp_Ofp_Og16")
    return restore(y1, batch), (restore(y2, batch), restore(s_y2, batch))
