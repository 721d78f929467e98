"""SiLU(gate) * up in one kernel per direction.  Not a function of the reference: its MLP calls fp8_silu_forward then
fp8_mul_forward (coat/models/coat_llama.py:664-668) and fp8_mul_backward then fp8_silu_backward (:741-748).  The fused
kernels return bit-identical tensors and save one pass over the FP8 SiLU output and the bf16 round trip of the product's
gradient."""
import torch

from ... import _hip
from ._division import _division, _product_division
from ._fused import new_max, prep_bf16, prep_pg
from .common import as_fp8_dtype, restore


def _sliced_pair(gate_x, gate_s, up_x, up_s):
    """gate / up as 2-D row-sliced views when they are column slices of one wider tensor (same row pitch, rows 16-byte
    aligned): returns (gate_x, gate_s, up_x, up_s, batch, in_pitch, s_pitch).  Anything else is made dense."""
    batch = gate_x.shape[0] if gate_x.dim() == 3 else None
    views = []
    for t in (gate_x, gate_s, up_x, up_s):
        if t.dim() == 3:
            t = t.reshape(-1, t.shape[-1])  # a view whenever the leading dimensions merge, which a column slice allows
        views.append(t)
    gx, gs, ux, us = views
    ok = (gx.is_cuda and gx.shape == ux.shape and gs.shape == us.shape and gs.dtype == us.dtype
          and all(t.dim() == 2 and t.stride(1) == 1 for t in views)
          and gx.stride(0) == ux.stride(0) and gs.stride(0) == us.stride(0)
          and gx.stride(0) % 16 == 0 and gx.data_ptr() % 16 == 0 and ux.data_ptr() % 16 == 0)
    if ok and (gx.stride(0) != gx.shape[1] or gs.stride(0) != gs.shape[1]):
        return gx, gs, ux, us, batch, gx.stride(0), gs.stride(0)
    gx, gs, batch = prep_pg(gate_x, gate_s)
    ux, us, _ = prep_pg(up_x, up_s)
    return gx, gs, ux, us, batch, 0, 0


def fp8_silu_mul_forward(gate_x, gate_s, up_x, up_s, QB, transpose_output_2d=False):
    """Equivalent to ``silu_x, silu_s = fp8_silu_forward(gate_x, gate_s, QB)`` followed by
    ``fp8_mul_forward(silu_x, silu_s, up_x, up_s, QB, transpose_output_2d)``.
    Returns (silu_x, silu_s, mul_x, mul_s, mul_x_t)."""
    if up_s.dtype != gate_s.dtype:
        up_s = up_s.to(gate_s.dtype)
    gate_x, gate_s, up_x, up_s, batch, in_pitch, s_pitch = _sliced_pair(gate_x, gate_s, up_x, up_s)
    assert gate_x.shape == up_x.shape and gate_s.shape == up_s.shape and gate_x.dtype == up_x.dtype
    M, N = gate_x.shape
    silu_x = torch.empty((M, N), dtype=gate_x.dtype, device=gate_x.device)
    silu_s = torch.empty(gate_s.shape, dtype=torch.bfloat16, device=gate_x.device)
    # the division recomputes the product from the SiLU codes just written and from up, so the bf16 product is not stored
    recompute = M % 16 == 0 and M > 0 and N > 0
    y = None if recompute else torch.empty((M, N), dtype=torch.bfloat16, device=gate_x.device)
    s_max = new_max(gate_x.device)
    _hip.check(_hip.lib().coat_fp8_silu_mul_forward(
        _hip.ptr(gate_x), _hip.ptr(gate_s), _hip.ptr(up_x), _hip.ptr(up_s), _hip.fp8(gate_x.dtype), _hip.dt(gate_s),
        _hip.ptr(silu_x), _hip.ptr(silu_s), _hip.ptr(y), _hip.ptr(s_max), M, N, QB, in_pitch, s_pitch,
        _hip.stream(gate_x.device)), "fp8_silu_mul_forward")
    if recompute:
        mul_x, mul_s, mul_x_t = _product_division(silu_x, silu_s, up_x, up_s, in_pitch, s_pitch, s_max, QB,
                                                  "fp8_silu_mul_forward")
    else:
        mul_x, mul_s, mul_x_t = _division(y, up_x.dtype, s_max, True, True, "fp8_silu_mul_forward", max_as=torch.bfloat16)
    if batch is not None and not transpose_output_2d:
        mul_x_t = mul_x_t.reshape(batch, -1, N)
    return restore(silu_x, batch), restore(silu_s, batch), restore(mul_x, batch), mul_s, mul_x_t


def fp8_silu_mul_forward_from_bf16(gate, up, QB, fp8type="E4M3", transpose_output_2d=False):
    """``gate_x, gate_s = fp8_quantize(gate, QB, fp8type)``, ``up_x, up_s = fp8_quantize(up, QB, fp8type)`` and
    ``fp8_silu_mul_forward(gate_x, gate_s, up_x, up_s, QB, transpose_output_2d)`` in one pass over the two bf16 tensors.
    Returns (gate_x, gate_s, up_x, up_s, silu_x, silu_s, mul_x, mul_s, mul_x_t), bit-identical to that chain."""
    fp8type = as_fp8_dtype(fp8type)
    assert gate.shape == up.shape
    batch = gate.shape[0] if gate.dim() == 3 else None
    g2, u2 = prep_bf16(gate), prep_bf16(up)
    M, N = g2.shape
    dev = g2.device
    if N % QB != 0:
        raise ValueError(f"fp8_silu_mul_forward_from_bf16: the last dimension {N} is not a multiple of the group size {QB}")
    outs = [torch.empty((M, N), dtype=fp8type, device=dev) for _ in range(3)]
    scales = [torch.empty((M, N // QB), dtype=torch.bfloat16, device=dev) for _ in range(3)]
    (gate_x, up_x, silu_x), (gate_s, up_s, silu_s) = outs, scales
    recompute = M % 16 == 0 and M > 0 and N > 0
    y = None if recompute else torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    s_max = new_max(dev)
    _hip.check(_hip.lib().coat_fp8_silu_mul_forward_bf16(
        _hip.ptr(g2), _hip.ptr(u2), _hip.fp8(fp8type), _hip.ptr(gate_x), _hip.ptr(gate_s), _hip.ptr(up_x), _hip.ptr(up_s),
        _hip.ptr(silu_x), _hip.ptr(silu_s), _hip.ptr(y), _hip.ptr(s_max), M, N, QB, _hip.stream(dev)),
        "fp8_silu_mul_forward_from_bf16")
    if recompute:
        mul_x, mul_s, mul_x_t = _product_division(silu_x, silu_s, up_x, up_s, 0, 0, s_max, QB, "fp8_silu_mul_forward_from_bf16")
    else:
        mul_x, mul_s, mul_x_t = _division(y, fp8type, s_max, True, True, "fp8_silu_mul_forward_from_bf16",
                                          max_as=torch.bfloat16)
    if batch is not None and not transpose_output_2d:
        mul_x_t = mul_x_t.reshape(batch, -1, N)
    r = lambda t: restore(t, batch)  # noqa: E731
    return r(gate_x), r(gate_s), r(up_x), r(up_s), r(silu_x), r(silu_s), r(mul_x), mul_s, mul_x_t


def _silu_mul_backward_values(gate_x, gate_s, up_x, up_s, silu_x, silu_s, g, QB, fp8type, joined):
    """Runs the fused backward kernel.  joined: the two bf16 gradients are written side by side, [up | gate], into one
    [M, 2N] tensor.  Returns (y_gate, y_up, m_gate, m_up, batch, joined tensor or None)."""
    sd = gate_s.dtype
    up_s, silu_s = up_s.to(sd), silu_s.to(sd)
    gate_x, gate_s, up_x, up_s, batch, in_pitch, s_pitch = _sliced_pair(gate_x, gate_s, up_x, up_s)
    silu_x, silu_s, _ = prep_pg(silu_x, silu_s)
    g = prep_bf16(g)
    M, N = gate_x.shape
    both = None
    if joined:
        both = torch.empty((M, 2 * N), dtype=torch.bfloat16, device=g.device)
        y_up, y_gate, y_pitch = both[:, :N], both[:, N:], 2 * N
    else:
        y_gate, y_up, y_pitch = torch.empty_like(g), torch.empty_like(g), 0
    m_gate = new_max(g.device)
    m_up = m_gate if joined else new_max(g.device)  # joined: one maximum over both halves
    _hip.check(_hip.lib().coat_fp8_silu_mul_backward(
        _hip.ptr(gate_x), _hip.ptr(gate_s), _hip.ptr(up_x), _hip.ptr(up_s), _hip.ptr(silu_x), _hip.ptr(silu_s),
        _hip.fp8(gate_x.dtype), _hip.dt(gate_s), _hip.ptr(g), _hip.ptr(y_gate), _hip.ptr(m_gate), _hip.ptr(y_up),
        _hip.ptr(m_up), _hip.fp8(fp8type), M, N, QB, in_pitch, s_pitch, y_pitch, _hip.stream(g.device)),
        "fp8_silu_mul_backward")
    return y_gate, y_up, m_gate, m_up, batch, both


def fp8_silu_mul_backward(gate_x, gate_s, up_x, up_s, silu_x, silu_s, g, QB, fp8type, stochastic=False):
    """Equivalent to ``mul_g1, up_grad = fp8_mul_backward(silu_x, silu_s, up_x, up_s, g, QB, fp8type,
    output_quantized_transpose=True)`` followed by ``gate_grad = fp8_silu_backward(gate_x, gate_s, mul_g1, QB, fp8type,
    output_quantized_transpose=True)``.  Returns ((gate_q, gate_s, gate_q_t), (up_q, up_s, up_q_t)).
    ``stochastic`` has no effect, as in both of those reference functions."""
    fp8type = as_fp8_dtype(fp8type)
    y_gate, y_up, m_gate, m_up, batch, _ = _silu_mul_backward_values(gate_x, gate_s, up_x, up_s, silu_x, silu_s, g, QB,
                                                                     fp8type, False)
    gq, gs, gq_t = _division(y_gate, fp8type, m_gate, True, True, "fp8_silu_mul_backward", max_as=torch.bfloat16)
    uq, us, uq_t = _division(y_up, fp8type, m_up, True, True, "fp8_silu_mul_backward", max_as=torch.bfloat16)
    return (restore(gq, batch), gs, gq_t), (restore(uq, batch), us, uq_t)


def fp8_silu_mul_backward_joined(gate_x, gate_s, up_x, up_s, silu_x, silu_s, g, QB, fp8type):
    """The backward of a fused up/gate projection's activation (coat/models/coat_olmo.py:594-606): equivalent to
    ``mul_g1, (up_g, up_gs) = fp8_mul_backward(silu_x, silu_s, up_x, up_s, g, QB, fp8type)``,
    ``gate_g, gate_gs = fp8_silu_backward(gate_x, gate_s, mul_g1, QB, fp8type)``,
    ``both = torch.cat([up_g, gate_g], dim=-1)``, ``s = torch.max(torch.cat([up_gs, gate_gs]))`` and
    ``fp8_division_transpose(both, QB, fp8type, s)``, without the concatenation copies.
    Returns (q [M, 2N] (3-D if the inputs were), s 0-dim bf16, q_t [2N, M])."""
    fp8type = as_fp8_dtype(fp8type)
    _, _, m_gate, m_up, batch, both = _silu_mul_backward_values(gate_x, gate_s, up_x, up_s, silu_x, silu_s, g, QB,
                                                                fp8type, True)
    # rounding is monotone: the rounded maximum is the maximum of the bf16 group scales
    q, s, q_t = _division(both, fp8type, m_gate, True, True, "fp8_silu_mul_backward_joined", max_as=torch.bfloat16)
    return restore(q, batch), s, q_t
