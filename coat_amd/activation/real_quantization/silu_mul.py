"""SiLU(gate) * up in one kernel per direction.  Not a function of the reference: its MLP calls fp8_silu_forward then
fp8_mul_forward (coat/models/coat_llama.py:664-668) and fp8_mul_backward then fp8_silu_backward (:741-748).  The fused
kernels return bit-identical tensors and save one pass over the FP8 SiLU output and the bf16 round trip of the product's
gradient."""
import torch

from ... import _hip
from ._division import _division
from ._fused import new_max, prep_bf16, prep_pg
from .common import as_fp8_dtype, restore


def fp8_silu_mul_forward(gate_x, gate_s, up_x, up_s, QB, transpose_output_2d=False):
    """Equivalent to ``silu_x, silu_s = fp8_silu_forward(gate_x, gate_s, QB)`` followed by
    ``fp8_mul_forward(silu_x, silu_s, up_x, up_s, QB, transpose_output_2d)``.
    Returns (silu_x, silu_s, mul_x, mul_s, mul_x_t)."""
    gate_x, gate_s, batch = prep_pg(gate_x, gate_s)
    up_x, up_s, _ = prep_pg(up_x, up_s)
    assert gate_x.shape == up_x.shape and gate_s.shape == up_s.shape and gate_x.dtype == up_x.dtype
    if up_s.dtype != gate_s.dtype:
        up_s = up_s.to(gate_s.dtype)
    M, N = gate_x.shape
    silu_x = torch.empty_like(gate_x)
    silu_s = torch.empty_like(gate_s, dtype=torch.bfloat16)
    y = torch.empty_like(gate_x, dtype=torch.bfloat16)
    s_max = new_max(gate_x.device)
    _hip.check(_hip.lib().coat_fp8_silu_mul_forward(
        _hip.ptr(gate_x), _hip.ptr(gate_s), _hip.ptr(up_x), _hip.ptr(up_s), _hip.fp8(gate_x.dtype), _hip.dt(gate_s),
        _hip.ptr(silu_x), _hip.ptr(silu_s), _hip.ptr(y), _hip.ptr(s_max), M, N, QB, _hip.stream(gate_x.device)),
        "fp8_silu_mul_forward")
    mul_x, mul_s, mul_x_t = _division(y, up_x.dtype, s_max.to(torch.bfloat16), True, True, "fp8_silu_mul_forward")
    if batch is not None and not transpose_output_2d:
        mul_x_t = mul_x_t.reshape(batch, -1, N)
    return restore(silu_x, batch), restore(silu_s, batch), restore(mul_x, batch), mul_s, mul_x_t


def fp8_silu_mul_backward(gate_x, gate_s, up_x, up_s, silu_x, silu_s, g, QB, fp8type, stochastic=False):
    """Equivalent to ``mul_g1, up_grad = fp8_mul_backward(silu_x, silu_s, up_x, up_s, g, QB, fp8type,
    output_quantized_transpose=True)`` followed by ``gate_grad = fp8_silu_backward(gate_x, gate_s, mul_g1, QB, fp8type,
    output_quantized_transpose=True)``.  Returns ((gate_q, gate_s, gate_q_t), (up_q, up_s, up_q_t)).
    ``stochastic`` has no effect, as in both of those reference functions."""
    gate_x, gate_s, batch = prep_pg(gate_x, gate_s)
    up_x, up_s, _ = prep_pg(up_x, up_s)
    silu_x, silu_s, _ = prep_pg(silu_x, silu_s)
    g = prep_bf16(g)
    sd = gate_s.dtype
    up_s, silu_s = up_s.to(sd), silu_s.to(sd)
    M, N = gate_x.shape
    fp8type = as_fp8_dtype(fp8type)
    y_gate = torch.empty_like(g)
    y_up = torch.empty_like(g)
    m_gate, m_up = new_max(g.device), new_max(g.device)
    _hip.check(_hip.lib().coat_fp8_silu_mul_backward(
        _hip.ptr(gate_x), _hip.ptr(gate_s), _hip.ptr(up_x), _hip.ptr(up_s), _hip.ptr(silu_x), _hip.ptr(silu_s),
        _hip.fp8(gate_x.dtype), _hip.dt(gate_s), _hip.ptr(g), _hip.ptr(y_gate), _hip.ptr(m_gate), _hip.ptr(y_up),
        _hip.ptr(m_up), _hip.fp8(fp8type), M, N, QB, _hip.stream(g.device)), "fp8_silu_mul_backward")
    gq, gs, gq_t = _division(y_gate, fp8type, m_gate.to(torch.bfloat16), True, True, "fp8_silu_mul_backward")
    uq, us, uq_t = _division(y_up, fp8type, m_up.to(torch.bfloat16), True, True, "fp8_silu_mul_backward")
    return (restore(gq, batch), gs, gq_t), (restore(uq, batch), us, uq_t)
