"""Residual add, backward: bf16 + bf16 -> bf16 sum, its per-tensor FP8 and the per-group scales.
Reference: coat/activation/real_quantization/add_bwd.py:147-200."""
import torch

from ... import _hip
from ._division import _division
from ._fused import new_max, prep_bf16
from .common import as_fp8_dtype, flatten_2d, restore


def fp8_add_Ifp_Ifp_Ofp_Opt(x1, x2, QB, fp8type, stochastic=False):
    """Returns (y bf16, (q fp8 per-tensor, s_max 0-dim, s per-group)); the division quantizes the bf16 sum
    (stochastic applies to that division, reference :192)."""
    _, batch = flatten_2d(x1)
    for t in (x1, x2):
        if t.dtype != torch.bfloat16:
            raise ValueError(f"fp8_add_Ifp_Ifp_Ofp_Opt takes bf16 inputs, got {t.dtype}")
    x1, x2 = prep_bf16(x1), prep_bf16(x2)
    assert x1.shape == x2.shape
    M, N = x1.shape
    fp8type = as_fp8_dtype(fp8type)
    y1 = torch.empty_like(x1, dtype=torch.bfloat16)
    s_y2 = torch.empty((M, N // QB), dtype=torch.bfloat16, device=x2.device)
    s_max = new_max(x1.device)
    _hip.check(_hip.lib().coat_fp8_add_bwd(_hip.ptr(x1), _hip.ptr(x2), _hip.ptr(y1), _hip.ptr(s_y2), _hip.ptr(s_max),
                                           _hip.fp8(fp8type), M, N, QB, _hip.stream(x1.device)), "fp8_add_Ifp_Ifp_Ofp_Opt")
    qy2, s_y2_max, _ = _division(y1, fp8type, s_max, True, False, "fp8_add_Ifp_Ifp_Ofp_Opt", stochastic,
                                 max_as=torch.bfloat16)
    return restore(y1, batch), (restore(qy2, batch), s_y2_max, restore(s_y2, batch))
