"""GPU: the bf16 causal attention forward kernel against fp32 attention of the same bf16 inputs.

Stated tolerance: the output is bf16 of an fp32 accumulation of products of bf16 probabilities (2^-9 relative each) with
bf16 values, so |out - ref| <= 2^-8 max|v| per element is about twice what is measured (printed); the
log-sum-exp is fp32 and agrees to 1e-4 absolute (the exponentials run through v_exp_f32).  The backward (torch's
memory-efficient attention backward fed with this forward's output and log-sum-exp) is compared with fp32 autograd."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def reference(q, k, v, causal=True):
    B, H, S, D = q.shape
    s = (q.float() @ k.float().transpose(-1, -2)) / math.sqrt(D)
    if causal:
        s = s.masked_fill(torch.triu(torch.ones(S, S, device=q.device, dtype=torch.bool), 1), float("-inf"))
    return torch.softmax(s, -1) @ v.float(), torch.logsumexp(s, -1)


def make(dev, B, S, H, D, seed, Hkv=None, scale=1.0):
    g = torch.Generator(device=dev).manual_seed(seed)
    Hkv = H if Hkv is None else Hkv
    q = (torch.randn(B, S, H, D, generator=g, device=dev) * scale).bfloat16().transpose(1, 2)
    k = (torch.randn(B, S, Hkv, D, generator=g, device=dev) * scale).bfloat16().transpose(1, 2)
    v = torch.randn(B, S, Hkv, D, generator=g, device=dev).bfloat16().transpose(1, 2)
    return q, k, v


@pytest.mark.parametrize("B,S,H,causal", [(1, 128, 1, True), (2, 256, 3, True), (1, 200, 2, True), (2, 1024, 4, True),
                                          (1, 192, 2, False), (1, 72, 1, True), (1, 2048, 2, True)])
def test_attention_forward_matches_fp32_attention(dev, B, S, H, causal):
    from coat_amd.models._attention import attention_forward
    q, k, v = make(dev, B, S, H, 128, 1 + S, scale=1.5)
    out, lse = attention_forward(q, k, v, causal=causal)
    assert out.shape == (B, H, S, 128) and out.stride() == q.stride() and lse.shape == (B, H, S)
    ref, ref_lse = reference(q, k, v, causal)
    err = (out.float() - ref).abs().max().item()
    lerr = (lse - ref_lse).abs().max().item()
    print(f"[measured] attention forward B {B} S {S} H {H} causal {causal}: max |out - ref| {err:.2e} "
          f"(bar {2.0 ** -8 * v.float().abs().max().item():.2e}), max |lse - ref| {lerr:.2e} (bar 1e-4)")
    assert err <= 2.0 ** -8 * v.float().abs().max().item()
    assert lerr <= 1e-4


def test_attention_forward_grouped_query_and_column_slices(dev):
    """Fewer key / value heads than query heads, and q / k / v taken as column slices of one fused projection output."""
    from coat_amd.models._attention import attention_forward
    B, S, H, Hkv, D = 2, 320, 4, 2, 128
    g = torch.Generator(device=dev).manual_seed(5)
    fused = torch.randn(B, S, (H + 2 * Hkv) * D, generator=g, device=dev).bfloat16()
    q = fused[..., : H * D].view(B, S, H, D).transpose(1, 2)
    k = fused[..., H * D: (H + Hkv) * D].view(B, S, Hkv, D).transpose(1, 2)
    v = fused[..., (H + Hkv) * D:].view(B, S, Hkv, D).transpose(1, 2)
    out, lse = attention_forward(q, k, v, causal=True)
    ref, ref_lse = reference(q, k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1))
    assert (out.float() - ref).abs().max().item() <= 2.0 ** -8 * v.float().abs().max().item()
    assert (lse - ref_lse).abs().max().item() <= 1e-4


def test_attention_autograd_matches_fp32_autograd(dev):
    """sdpa() on the layers' case: forward from this library, backward from torch's kernel fed with its output and lse."""
    from coat_amd.models._attention import _CausalAttention, sdpa
    B, S, H, D = 2, 512, 4, 128
    q, k, v = (t.detach().requires_grad_(True) for t in make(dev, B, S, H, D, 9))
    out = sdpa(q, k, v, is_causal=True)
    assert isinstance(out.grad_fn, _CausalAttention._backward_cls)
    go = torch.randn(B, S, H, D, generator=torch.Generator(device=dev).manual_seed(10), device=dev).bfloat16().transpose(1, 2)
    out.backward(go)
    qf, kf, vf = (t.detach().float().requires_grad_(True) for t in (q, k, v))
    s = (qf @ kf.transpose(-1, -2)) / math.sqrt(D)
    s = s.masked_fill(torch.triu(torch.ones(S, S, device=dev, dtype=torch.bool), 1), float("-inf"))
    (torch.softmax(s, -1) @ vf).backward(go.float())
    for name, got, want in (("dq", q.grad, qf.grad), ("dk", k.grad, kf.grad), ("dv", v.grad, vf.grad)):
        rel = ((got.float() - want).norm() / want.norm()).item()
        print(f"[measured] attention backward {name}: relative Frobenius {rel:.2e} (bar 1e-2)")
        assert rel < 1e-2, (name, rel)
