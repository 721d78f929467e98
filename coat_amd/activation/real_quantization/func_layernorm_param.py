"""FP8 LayerNorm with weight and bias, forward / backward.
Reference: coat/activation/real_quantization/func_layernorm_param.py:243-367."""
import torch

from ... import _hip
from ._fused import prep_bf16, prep_pg
from .common import restore
from .func_layernorm_noparam import _forward

_PARTIALS = 512  # blocks of the dx kernel; each contributes one fp32 partial row of dw and of db


def fp8_layernorm_param_forward(x, s_x, w, b, QB, eps, transpose_output_2d=False):
    """Returns (qy, s_y_max, qy_t, (w, b, mean, rstd, num_warps)); qy is per-tensor FP8 in x's dtype."""
    w = _hip.dense(w)
    b = _hip.dense(b.to(w.dtype))
    qy, s_y_max, qy_t, mean, rstd = _forward(x, s_x, w, b, QB, eps, transpose_output_2d, "fp8_layernorm_param_forward")
    num_warps = 8  # kept in the tuple for signature compatibility; the HIP kernels do not use it
    return qy, s_y_max, qy_t, (w, b, mean, rstd, num_warps)


def fp8_layernorm_param_backward(x, s_x, g, QB, w, b, m, v, num_warps):
    """Returns (dx bf16, dw, db in w's dtype); ``m`` / ``v`` are the mean / rstd saved by the forward."""
    x, s_x, batch = prep_pg(x, s_x)
    g = prep_bf16(g)
    M, N = g.shape
    w = _hip.dense(w)
    mean, rstd = _hip.dense(m.to(torch.float32)), _hip.dense(v.to(torch.float32))
    dx = torch.empty_like(g, dtype=torch.bfloat16)
    dw = torch.empty((N,), dtype=w.dtype, device=w.device)
    db = torch.empty((N,), dtype=w.dtype, device=w.device)
    nparts = min(_PARTIALS, M)
    pw = torch.empty((nparts, N), dtype=torch.float32, device=w.device)
    pb = torch.empty((nparts, N), dtype=torch.float32, device=w.device)
    _hip.check(_hip.lib().coat_fp8_layernorm_backward(
        _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(g), _hip.ptr(w), _hip.dt(w), _hip.ptr(mean),
        _hip.ptr(rstd), _hip.ptr(dx), _hip.ptr(dw), _hip.ptr(db), _hip.ptr(pw), _hip.ptr(pb), nparts, M, N, QB,
        _hip.stream(x.device)), "fp8_layernorm_param_backward")
    return restore(dx, batch), dw, db
