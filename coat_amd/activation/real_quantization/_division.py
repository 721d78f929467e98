"""Per-tensor FP8 quantize by a given scalar scale.
Reference: coat/activation/real_quantization/_division.py:153-207."""
import torch

from ... import _hip
from .common import FP8_MAX_VALUE, SCALE_MIN_THRES, as_fp8_dtype, flatten_2d, new_max, read_max, restore

# the seed the reference's kernels pass to tl.rand (reference :110; _division_transpose.py:117)
STOCHASTIC_SEED = 0


def absmax_scale(x, fp8type):
    """(x.abs().max() + 1e-10) / fp8max in x's dtype (reference :178-179), one pass over x."""
    amax = new_max(x.device)
    _hip.check(_hip.lib().coat_absmax(_hip.ptr(x), _hip.dt(x), _hip.ptr(amax), x.numel(), _hip.stream(x.device)), "absmax")
    return (read_max(amax).to(x.dtype) + SCALE_MIN_THRES) / FP8_MAX_VALUE[fp8type]


def _division(x, fp8type, s_y, want_q, want_qt, what, stochastic=False, max_as=None):
    """q and / or q^T of x divided by a per-tensor scale.  ``max_as`` (a torch dtype): ``s_y`` is the fp32 buffer
    (``new_max``) into which a producer kernel merged the maximum of its group scales; the division kernel rounds the
    maximum to that dtype itself and writes the rounded scale, which is returned (no separate conversion launch)."""
    M, N = x.shape
    if s_y is None:
        s_y = absmax_scale(x, fp8type)
    if max_as is not None and (stochastic or M * N == 0):
        s_y = read_max(s_y).to(max_as)  # the kernel that reads the slots itself is not used on this path
        max_as = None
    if max_as is None and s_y.numel() != 1:
        raise ValueError(f"{what}: the scale must be a single element, got shape {tuple(s_y.shape)}")
    s_dev = s_y if s_y.is_cuda else s_y.to(x.device)
    y = torch.empty_like(x, dtype=fp8type) if want_q else None
    y_t = torch.empty((N, M), dtype=fp8type, device=x.device) if want_qt else None
    if max_as is not None:
        if s_dev.dtype != torch.float32 or s_dev.numel() != _hip.MAX_WORDS:
            raise ValueError(f"{what}: the running maximum must be fp32")
        s_out = torch.empty((), dtype=max_as, device=x.device)
        _hip.check(_hip.lib().coat_fp8_division_from_max(
            _hip.ptr(x), _hip.dt(x), _hip.ptr(s_dev), _hip.ptr(s_out), _hip.dt(s_out), _hip.ptr(y), _hip.ptr(y_t), M, N,
            _hip.fp8(fp8type), _hip.stream(x.device)), what)
        return y, s_out, y_t
    if stochastic:
        _hip.check(_hip.lib().coat_fp8_division_stochastic(
            _hip.ptr(x), _hip.dt(x), _hip.ptr(s_dev), _hip.dt(s_dev), _hip.ptr(y), _hip.ptr(y_t), M, N,
            _hip.fp8(fp8type), STOCHASTIC_SEED, _hip.stream(x.device)), what)
    else:
        _hip.check(_hip.lib().coat_fp8_division(_hip.ptr(x), _hip.dt(x), _hip.ptr(s_dev), _hip.dt(s_dev), _hip.ptr(y),
                                                _hip.ptr(y_t), M, N, _hip.fp8(fp8type), _hip.stream(x.device)), what)
    return y, s_y, y_t


def _outputs_for(x, fp8type):
    M, N = x.shape
    return (torch.empty((M, N), dtype=fp8type, device=x.device), torch.empty((N, M), dtype=fp8type, device=x.device),
            torch.empty((), dtype=torch.bfloat16, device=x.device))


def _rmsnorm_division(x, s_x, w, rstd, s_max, QB, what):
    """(q, s, q_t) of bf16(x * rstd * w) divided by the bf16-rounded ``s_max``, with the tensor recomputed tile by tile
    from the norm's inputs instead of being stored and read back (same codes as ``_division`` on the stored tensor)."""
    M, N = x.shape
    q, q_t, s_out = _outputs_for(x, x.dtype)
    _hip.check(_hip.lib().coat_fp8_rmsnorm_division(
        _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(w), _hip.dt(w), _hip.ptr(rstd),
        _hip.ptr(s_max), _hip.ptr(s_out), _hip.ptr(q), _hip.ptr(q_t), M, N, QB, _hip.stream(x.device)), what)
    return q, s_out, q_t


def _layernorm_division(x, s_x, w, b, mean, rstd, s_max, QB, what):
    """(q, s, q_t) of the fp32 tensor (x - mean) * rstd (* w + b) divided by the bf16-rounded ``s_max``, recomputed tile
    by tile from the norm's inputs (same codes as ``_division`` on the stored fp32 tensor)."""
    M, N = x.shape
    q, q_t, s_out = _outputs_for(x, x.dtype)
    _hip.check(_hip.lib().coat_fp8_layernorm_division(
        _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(w), _hip.ptr(b),
        -1 if w is None else _hip.dt(w), _hip.ptr(mean), _hip.ptr(rstd), _hip.ptr(s_max), _hip.ptr(s_out), _hip.ptr(q),
        _hip.ptr(q_t), M, N, QB, _hip.stream(x.device)), what)
    return q, s_out, q_t


def _product_division(a, s_a, b, s_b, b_pitch, sb_pitch, s_max, QB, what):
    """(q, s, q_t) of bf16(dequant(a) * dequant(b)) divided by the bf16-rounded ``s_max``, recomputed from the factors.
    ``b`` may be a column slice (row pitches in codes / scales, 0 = dense)."""
    M, N = a.shape
    q, q_t, s_out = _outputs_for(a, a.dtype)
    _hip.check(_hip.lib().coat_fp8_product_division(
        _hip.ptr(a), _hip.ptr(s_a), _hip.dt(s_a), _hip.ptr(b), _hip.ptr(s_b), _hip.dt(s_b), _hip.fp8(a.dtype),
        _hip.ptr(s_max), _hip.ptr(s_out), _hip.ptr(q), _hip.ptr(q_t), M, N, QB, b_pitch, sb_pitch,
        _hip.stream(a.device)), what)
    return q, s_out, q_t


def fp8_division(x, QB, fp8type, s_y=None, stochastic=False):
    """x -> (y fp8, s_y); y = fp8(x / float(s_y)); s_y defaults to (absmax + 1e-10) / fp8max.
    stochastic: the reference's noise-then-round branch (reference :96-112, :130-150), same Philox stream."""
    x, batch = flatten_2d(x)
    x = _hip.dense(x)
    y, s_y, _ = _division(x, as_fp8_dtype(fp8type), s_y, True, False, "fp8_division", stochastic)
    return restore(y, batch), s_y
