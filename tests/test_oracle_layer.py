"""CPU: the decoder-layer chain of the oracle (oracle/layer_ref.py) against the same layer in fp32 torch with autograd.

Every operation of the chain is pinned where it is defined (tests/test_oracle_activation.py); what is checked here is the
wiring of the chain: output, input gradient and every weight gradient agree with the fp32 layer within the noise of the
FP8 flow (e4m3 activations 2^-4, e5m2 gradients 2^-3 per element), which a wrong operand, a missing transpose or a
dropped residual would exceed many times over."""
import torch
import torch.nn.functional as F

from oracle import layer_ref


def test_oracle_layer_chain_follows_the_fp32_layer():
    torch.manual_seed(0)
    H, heads, I, B, S = 512, 8, 1536, 2, 64
    W = {n: (torch.randn(shape) * 0.02).bfloat16() for n, shape in
         (("q", (H, H)), ("k", (H, H)), ("v", (H, H)), ("o", (H, H)), ("gate", (I, H)), ("up", (I, H)), ("down", (H, I)))}
    W["norm1"] = (1 + 0.1 * torch.randn(H)).bfloat16()
    W["norm2"] = (1 + 0.1 * torch.randn(H)).bfloat16()
    x = torch.randn(B * S, H).bfloat16()
    gy = (torch.randn(B * S, H) * 1e-2).bfloat16()
    y, gx, grads = layer_ref.decoder_layer_step(x, gy, W, heads, B)

    P = {k: v.float().requires_grad_(True) for k, v in W.items()}
    xin = x.float().requires_grad_(True)
    h = F.rms_norm(xin, (H,), P["norm1"], 1e-5)
    q, k, v = (F.linear(h, P[n]).view(B, S, heads, H // heads).transpose(1, 2) for n in ("q", "k", "v"))
    a = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(B * S, H)
    x1 = xin + F.linear(a, P["o"])
    h2 = F.rms_norm(x1, (H,), P["norm2"], 1e-5)
    out = x1 + F.linear(F.silu(F.linear(h2, P["gate"])) * F.linear(h2, P["up"]), P["down"])
    out.backward(gy.float())

    def rel(got, want):
        return ((got.float() - want.float()).norm() / want.float().norm()).item()

    assert y.dtype == torch.bfloat16 and rel(y, out) < 0.02          # measured 0.008
    assert rel(gx, xin.grad) < 0.03                                   # measured 0.013
    for n, g in grads.items():
        assert g.shape == P[n].shape and rel(g, P[n].grad) < 0.16, n  # measured 0.075 .. 0.108
    # a dropped MLP branch would move the output by the branch's norm: 0.086 of the output here, four times the bar
    assert rel(x1.detach(), out) > 0.06
