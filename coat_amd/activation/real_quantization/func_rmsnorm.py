"""FP8 RMSNorm forward / backward.
Reference: coat/activation/real_quantization/func_rmsnorm.py:223-335."""
import torch

from ... import _hip
from ._division import _division, _rmsnorm_division
from ._fused import new_max, prep_bf16, prep_pg
from .common import restore

_DW_PARTIALS = 512  # blocks of the dx kernel; each contributes one fp32 partial row of dw


def fp8_rmsnorm_forward(x, s_x, w, QB, eps, transpose_output_2d=False):
    """Returns (qy, s_y_max, qy_t, (w, rstd, num_warps)); qy is per-tensor FP8 in x's dtype."""
    x, s_x, batch = prep_pg(x, s_x)
    M, N = x.shape
    w = _hip.dense(w)
    # the division recomputes y from x, rstd and w tile by tile, so y is not stored (needs whole 16 x 16 blocks,
    # which the transposed output needs anyway)
    recompute = M % 16 == 0 and M > 0
    y = None if recompute else torch.empty_like(x, dtype=torch.bfloat16)
    s_row = torch.empty((M,), dtype=torch.bfloat16, device=x.device)
    rstd = torch.empty((M,), dtype=torch.float32, device=x.device)
    s_max = new_max(x.device)
    _hip.check(_hip.lib().coat_fp8_rmsnorm_forward(
        _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(w), _hip.dt(w), _hip.ptr(y), _hip.ptr(s_row),
        _hip.ptr(rstd), _hip.ptr(s_max), M, N, QB, float(eps), _hip.stream(x.device)), "fp8_rmsnorm_forward")
    if recompute:
        qy, s_y_max, qy_t = _rmsnorm_division(x, s_x, w, rstd, s_max, QB, "fp8_rmsnorm_forward")
    else:
        qy, s_y_max, qy_t = _division(y, x.dtype, s_max, True, True, "fp8_rmsnorm_forward", max_as=torch.bfloat16)
    if batch is not None and not transpose_output_2d:
        qy_t = qy_t.reshape(batch, -1, N)
    num_warps = 8  # kept in the tuple for signature compatibility; the HIP kernels do not use it
    return restore(qy, batch), s_y_max, qy_t, (w, rstd, num_warps)


def fp8_rmsnorm_backward(x, s_x, g, w, v, QB, num_warps):
    """Returns (dx bf16, dw in w's dtype); ``v`` is the rstd saved by the forward.

    ``g`` may also be a tuple of two or three bf16 gradients of the normalised tensor: the kernel then uses
    ``g[0] + g[1] (+ g[2])`` with the roundings of that chain of bf16 additions (what the reference's modules compute
    before the call, coat/models/coat_llama.py:328 and :742), without the separate passes over the tensors."""
    return _rmsnorm_backward(x, s_x, g, w, v, QB, None, None, False)


def fp8_rmsnorm_backward_add(x, s_x, g, w, v, QB, num_warps, residual_grad, fp8type, stochastic=False):
    """``fp8_rmsnorm_backward`` followed by ``fp8_add_Ifp_Ifp_Ofp_Opt(residual_grad, dx, QB, fp8type)`` with the
    addition inside the backward kernel (the reference runs them one after the other, coat/models/coat_llama.py:331-339 and
    :745-754): dx is rounded to bf16 as it would be stored and added to the bf16 ``residual_grad`` in fp32.
    Returns ``(y, (q, s_max, s_pg), dw)``: the bf16 sum, its per-tensor FP8 codes with their scale, the per-group scales
    of the sum, and the weight gradient; all bit-identical to the two calls."""
    from .add_bwd import fp8_add_Ifp_Ifp_Ofp_Opt
    from .common import as_fp8_dtype
    N = x.shape[-1]
    if N > 8192 or residual_grad.dtype != torch.bfloat16:  # rows the wave-per-row kernels do not take: the two kernels
        dx, dw = _rmsnorm_backward(x, s_x, g, w, v, QB, None, None, False)
        y, quant = fp8_add_Ifp_Ifp_Ofp_Opt(residual_grad, dx, QB, fp8type, stochastic=stochastic)
        return y, quant, dw
    return _rmsnorm_backward(x, s_x, g, w, v, QB, residual_grad, as_fp8_dtype(fp8type), stochastic)


def _rmsnorm_backward(x, s_x, g, w, v, QB, residual_grad, fp8type, stochastic):
    x, s_x, batch = prep_pg(x, s_x)
    extra = [None, None]
    if isinstance(g, (tuple, list)):
        if not 1 <= len(g) <= 3:
            raise ValueError("fp8_rmsnorm_backward takes one to three gradients")
        more = [prep_bf16(t) for t in g[1:]]
        g = g[0]
        for i, t in enumerate(more):
            extra[i] = t
    g = prep_bf16(g)
    M, N = g.shape
    for t in extra:
        if t is not None and t.shape != g.shape:
            raise ValueError("the gradients must have the same shape")
    w = _hip.dense(w)
    rstd = _hip.dense(v.to(torch.float32))
    dx = torch.empty_like(g, dtype=torch.bfloat16)
    dw = torch.empty((N,), dtype=w.dtype, device=w.device)
    nparts = min(_DW_PARTIALS, M)
    partial = torch.empty((nparts, N), dtype=torch.float32, device=w.device)
    if residual_grad is None:
        _hip.check(_hip.lib().coat_fp8_rmsnorm_backward(
            _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(g), _hip.ptr(extra[0]), _hip.ptr(extra[1]),
            _hip.ptr(w), _hip.dt(w), _hip.ptr(rstd),
            _hip.ptr(dx), _hip.ptr(dw), _hip.ptr(partial), nparts, M, N, QB, _hip.stream(x.device)), "fp8_rmsnorm_backward")
        return restore(dx, batch), dw
    r = prep_bf16(residual_grad)
    if r.shape != g.shape:
        raise ValueError("the residual gradient must have the gradient's shape")
    s_pg = torch.empty((M, N // QB), dtype=torch.bfloat16, device=x.device)
    s_max = new_max(x.device)
    _hip.check(_hip.lib().coat_fp8_rmsnorm_backward_add(
        _hip.ptr(x), _hip.fp8(x.dtype), _hip.ptr(s_x), _hip.dt(s_x), _hip.ptr(g), _hip.ptr(extra[0]), _hip.ptr(extra[1]),
        _hip.ptr(w), _hip.dt(w), _hip.ptr(rstd), _hip.ptr(r), _hip.ptr(dx), _hip.ptr(s_pg), _hip.ptr(s_max), _hip.fp8(fp8type),
        _hip.ptr(dw), _hip.ptr(partial), nparts, M, N, QB, _hip.stream(x.device)), "fp8_rmsnorm_backward_add")
    q, s_q, _ = _division(dx, fp8type, s_max, True, False, "fp8_rmsnorm_backward_add", stochastic, max_as=torch.bfloat16)
    return restore(dx, batch), (restore(q, batch), s_q, restore(s_pg, batch)), dw
