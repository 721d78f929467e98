"""Per-tensor FP8 quantize by a given scale, also (or only) written transposed.
Reference: coat/activation/real_quantization/_division_transpose.py:147-210."""
from ... import _hip
from ._division import _division
from .common import as_fp8_dtype, flatten_2d, restore


def fp8_division_transpose(x, QB, fp8type, s_y=None, stochastic=False, only_transposed=False):
    """Returns (y, s_y, y_t [N, M]) or, with only_transposed, (y_t, s_y).
    stochastic: reference :103-119, noise indexed by the element's position in x."""
    x, batch = flatten_2d(x)
    x = _hip.dense(x)
    y, s_y, y_t = _division(x, as_fp8_dtype(fp8type), s_y, not only_transposed, True, "fp8_division_transpose",
                             stochastic)
    if only_transposed:
        return y_t, s_y
    return restore(y, batch), s_y, y_t
