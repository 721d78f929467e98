"""FP8 LayerNorm without affine parameters, forward / backward.
Reference: coat/activation/real_quantization/func_layernorm_noparam.py:188-297."""
import torch

from ... import _hip
from ._division import _division, _layernorm_division
from ._fused import new_max, prep_bf16, prep_pg
from .common import no_stochastic, restore


def _forward(x, s_x, w, b, QB, eps, transpose_output_2d, who):
    x, s_x, batch = prep_pg(x, s_x)
    M, N = x.shape
    # the reference keeps the normalised tensor in fp32 (:205); here the division recomputes it tile by tile from x, mean
    # and rstd, so it is only stored when the row count does not allow the tiled kernel
    recompute = M % 16 == 0 and M > 0
    y = None if recompute else torch.empty_like(x, dtype=torch.float32)
    s_row = torch.empty((M,), dtype=torch.bfloat16, device=x.device)
    mean = torch.empty((M,), dtype=torch.float32, device=x.device)
    rstd = torch.empty((M,), dtype=torch.float32, device=x.device)
    s_max = new_max(x.device)
    if w is not None:
        w, b = _hip.dense(w), _hip.dense(b)
    _hip.check(_hip.lib().coat_fp8_layernorm_forward(
        _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(w), _hip.ptr(b),
        -1 if w is None else _hip.dt(w), _hip.ptr(y), _hip.ptr(s_row), _hip.ptr(mean), _hip.ptr(rstd), _hip.ptr(s_max),
        M, N, QB, float(eps), _hip.stream(x.device)), who)
    if recompute:
        qy, s_y_max, qy_t = _layernorm_division(x, s_x, w, b, mean, rstd, s_max, QB, who)
    else:
        qy, s_y_max, qy_t = _division(y, x.dtype, s_max, True, True, who, max_as=torch.bfloat16)
    if batch is not None and not transpose_output_2d:
        qy_t = qy_t.reshape(batch, -1, N)
    return restore(qy, batch), s_y_max, qy_t, mean, rstd


def fp8_layernorm_noparam_forward(x, s_x, QB, eps, transpose_output_2d=False):
    """Returns (qy, s_y_max, qy_t, (mean, rstd, num_warps)); qy is per-tensor FP8 in x's dtype."""
    qy, s_y_max, qy_t, mean, rstd = _forward(x, s_x, None, None, QB, eps, transpose_output_2d,
                                             "fp8_layernorm_noparam_forward")
    num_warps = 8  # kept in the tuple for signature compatibility; the HIP kernels do not use it
    return qy, s_y_max, qy_t, (mean, rstd, num_warps)


def fp8_layernorm_noparam_backward_add(x, s_x, g, QB, m, v, num_warps, residual_grad, fp8type, stochastic=False):
    """``fp8_layernorm_noparam_backward`` followed by ``fp8_add_Ifp_Ifp_Ofp_Opt(residual_grad, dx, QB, fp8type)`` with the
    addition inside the backward kernel (the reference runs them one after the other, coat/models/coat_olmo.py:318-339): dx is
    rounded to bf16 as it would be stored and added to the bf16 ``residual_grad`` in fp32.  Returns ``(y, (q, s_max, s_pg))``:
    the bf16 sum, its per-tensor FP8 codes with their scale and the per-group scales of the sum, bit-identical to the two calls."""
    from .add_bwd import fp8_add_Ifp_Ifp_Ofp_Opt
    from .common import as_fp8_dtype
    if residual_grad.dtype != torch.bfloat16:
        dx = fp8_layernorm_noparam_backward(x, s_x, g, QB, m, v, num_warps)
        return fp8_add_Ifp_Ifp_Ofp_Opt(residual_grad, dx, QB, fp8type, stochastic=stochastic)
    fp8type = as_fp8_dtype(fp8type)
    x, s_x, batch = prep_pg(x, s_x)
    g, r = prep_bf16(g), prep_bf16(residual_grad)
    if r.shape != g.shape:
        raise ValueError("the residual gradient must have the gradient's shape")
    M, N = g.shape
    mean, rstd = _hip.dense(m.to(torch.float32)), _hip.dense(v.to(torch.float32))
    y = torch.empty_like(g, dtype=torch.bfloat16)
    s_pg = torch.empty((M, N // QB), dtype=torch.bfloat16, device=x.device)
    s_max = new_max(x.device)
    _hip.check(_hip.lib().coat_fp8_layernorm_backward_add(
        _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(g), None, -1, _hip.ptr(mean), _hip.ptr(rstd),
        _hip.ptr(r), _hip.ptr(y), _hip.ptr(s_pg), _hip.ptr(s_max), _hip.fp8(fp8type), None, None, None, None, 0, M, N, QB,
        _hip.stream(x.device)), "fp8_layernorm_noparam_backward_add")
    q, s_out, _ = _division(y, fp8type, s_max, True, False, "fp8_layernorm_noparam_backward_add", stochastic,
                            max_as=torch.bfloat16)
    return restore(y, batch), (restore(q, batch), s_out, restore(s_pg, batch))


def fp8_layernorm_noparam_backward(x, s_x, g, QB, m, v, num_warps, stochastic=False):
    """Returns dx (bf16); ``m`` / ``v`` are the mean / rstd saved by the forward."""
    no_stochastic(stochastic, "the reference's kernel uses e_bit / m_bit that it never receives "
                  "(func_layernorm_noparam.py:180), so there is no behaviour to match")
    x, s_x, batch = prep_pg(x, s_x)
    g = prep_bf16(g)
    M, N = g.shape
    mean, rstd = _hip.dense(m.to(torch.float32)), _hip.dense(v.to(torch.float32))
    dx = torch.empty_like(g, dtype=torch.bfloat16)
    _hip.check(_hip.lib().coat_fp8_layernorm_backward(
        _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(g), None, -1, _hip.ptr(mean), _hip.ptr(rstd),
        _hip.ptr(dx), None, None, None, None, 0, M, N, QB, _hip.stream(x.device)), "fp8_layernorm_noparam_backward")
    return restore(dx, batch)
