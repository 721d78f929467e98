"""The COAT Llama decoder layer, forward + backward, as a chain of the CPU oracle's operations.  TEST INFRASTRUCTURE ONLY.

Follows the reference's call order (paths relative to the reference repository):
  coat/models/coat_llama.py:223-283 / :286-347   residual branch point + RMSNorm + q / k / v projections, and backward
  coat/models/coat_llama.py:420-453 / :456-488   output projection + residual add, and backward
  coat/models/coat_llama.py:603-682 / :685-766   RMSNorm + gate / up + SiLU * up + down projection + residual add, and backward
  coat/models/coat_llama.py:981-1074             attention between the projections (bf16 in the reference; torch's fp32
                                                 SDPA with autograd here, rotary embedding left to the caller's q / k)
with the weights in the reference's default memory-efficient mode (re-quantized from the master weight with the
absmax scale, coat/utils/_fp8_weightcache.py:11-28).  Every operation is the one of oracle/activation_ref.py, which is
where each of them is pinned; this file adds no arithmetic of its own.  Used as the CPU baseline of the layer benchmark.
"""
import torch
import torch.nn.functional as F

from . import activation_ref as R

E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2
QB = 16


def _weights(W, names):
    """(codes, transposed codes, scale) of each master weight: rq/_division.py:178-179 scale, then division."""
    out = []
    for n in names:
        q, s = R.fp8_division(W[n], QB, "E4M3")
        out.append((q, R.fp8_transpose(q), s))
    return out


def _pt_e5m2(g):
    """A bf16 gradient -> per-tensor e5m2 in both layouts (rq/_quantize_pertensor_transpose.py:106-150)."""
    q, s, q_t = R.fp8_quantize_pertensor_transpose(g, QB, "E5M2")
    return q, s, q_t


def decoder_layer_step(x, gy, W, heads, batch, eps=1e-5):
    """x, gy bf16 [batch * seq, H]; W: master weights (bf16) named q, k, v, o, gate, up, down, norm1, norm2.
    Returns (output bf16 [T, H], input gradient bf16 [T, H], dict of weight gradients)."""
    T, H = x.shape
    S, hd = T // batch, H // heads
    # ---- forward
    qx, sx = R.fp8_quantize(x, QB, "E4M3")                                   # Coat_quantize_bgn
    ln1, ln1_s, ln1_t, rstd1 = R.fp8_rmsnorm_forward(qx, sx, W["norm1"], QB, eps)
    wq, wk, wv = _weights(W, ("q", "k", "v"))
    proj = [R.fp8_linear_forward(ln1, ln1_s, w[0], w[2], False, QB) for w in (wq, wk, wv)]
    heads_in = [p.float().view(batch, S, heads, hd).transpose(1, 2).requires_grad_(True) for p in proj]
    with torch.enable_grad():
        attn = F.scaled_dot_product_attention(*heads_in, is_causal=True).transpose(1, 2).reshape(T, H)
    flash = attn.detach().bfloat16()
    fq, fs, _ = R.fp8_quantize_pertensor(flash, QB, "E4M3")
    (wo,) = _weights(W, ("o",))
    h1, (q1, s1) = R.fp8_add_Ifp_Ifp_Ofp_Og16(x, R.fp8_linear_forward(fq, fs, wo[0], wo[2], False, QB), E4, QB)
    ln2, ln2_s, ln2_t, rstd2 = R.fp8_rmsnorm_forward(q1, s1, W["norm2"], QB, eps)
    wg, wu, wd = _weights(W, ("gate", "up", "down"))
    gate_x, gate_s = R.fp8_linear_forward(ln2, ln2_s, wg[0], wg[2], True, QB)
    up_x, up_s = R.fp8_linear_forward(ln2, ln2_s, wu[0], wu[2], True, QB)
    silu_x, silu_s = R.fp8_silu_forward(gate_x, gate_s, QB)
    mul_x, mul_s, mul_t = R.fp8_mul_forward(silu_x, silu_s, up_x, up_s, QB)
    h2, (q2, s2) = R.fp8_add_Ifp_Ifp_Ofp_Og16(h1, R.fp8_linear_forward(mul_x, mul_s, wd[0], wd[2], False, QB), E4, QB)
    # ---- backward (Coat_quantize_end: the incoming gradient as bf16 + per-tensor e5m2 with its group scales)
    grads = {}
    fp_g = gy
    g8, g8_s, g8_t = _pt_e5m2(gy)
    # MLP residual
    fc3_g, grads["down"] = R.fp8_linear_backward(mul_t, mul_s, g8, g8_s, g8_t, wd[1], wd[2], QB)
    g1, (g2, g2_s, g2_t) = R.fp8_mul_backward(silu_x, silu_s, up_x, up_s, fc3_g, QB, "E5M2", True)
    sg, sg_s, sg_t = R.fp8_silu_backward(gate_x, gate_s, g1, QB, "E5M2", True)
    fc1_g, grads["gate"] = R.fp8_linear_backward(ln2_t, ln2_s, sg, sg_s, sg_t, wg[1], wg[2], QB)
    fc2_g, grads["up"] = R.fp8_linear_backward(ln2_t, ln2_s, g2, g2_s, g2_t, wu[1], wu[2], QB)
    in_g, grads["norm2"] = R.fp8_rmsnorm_backward(q1, s1, fc1_g + fc2_g, W["norm2"], rstd2, QB, accumulate=torch.float32)
    fp_g, (g8, g8_s, _) = R.fp8_add_Ifp_Ifp_Ofp_Opt(fp_g, in_g, QB, "E5M2")
    # after attention
    flash_t, _ = R.fp8_division_transpose(flash, QB, "E4M3", fs, only_transposed=True)
    fc4_g, grads["o"] = R.fp8_linear_backward(flash_t, fs, g8, g8_s, R.fp8_transpose(g8), wo[1], wo[2], QB)
    # attention
    dq, dk, dv = torch.autograd.grad(attn, heads_in, fc4_g.float())
    # before attention
    dgrads = []
    for name, d, w in (("q", dq, wq), ("k", dk, wk), ("v", dv, wv)):
        dq8, dq8_s, dq8_t = _pt_e5m2(d.transpose(1, 2).reshape(T, H).bfloat16())
        dx, grads[name] = R.fp8_linear_backward(ln1_t, ln1_s, dq8, dq8_s, dq8_t, w[1], w[2], QB)
        dgrads.append(dx)
    in_g, grads["norm1"] = R.fp8_rmsnorm_backward(qx, sx, dgrads[0] + dgrads[1] + dgrads[2], W["norm1"], rstd1, QB,
                                                  accumulate=torch.float32)
    fp_g, _ = R.fp8_add_Ifp_Ifp_Ofp_Opt(fp_g, in_g, QB, "E5M2")
    return h2, fp_g, grads
