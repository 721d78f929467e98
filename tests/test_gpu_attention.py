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
    """The oracle (oracle/attention_ref.py: fp32 attention of the bf16 inputs), evaluated on the device for speed."""
    from oracle import attention_ref
    return attention_ref.attention(q, k, v, causal=causal)


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


def _scale_pass_max(t, fp8):
    """What the scale pass of fp8_quantize_pertensor would merge for the bf16 tensor t: the maximum fp32 group scale."""
    from coat_amd.activation.real_quantization._quantize_pertensor import group_scales_and_max
    from coat_amd.activation.real_quantization.common import read_max
    t2 = t.reshape(-1, t.shape[-1]).contiguous()
    return read_max(group_scales_and_max(t2, 16, fp8, want_pg=False)[1])


@pytest.mark.parametrize("fp8", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_forward_hands_over_the_scale_maximum_of_its_output(dev, fp8):
    """coat_attention_forward_bf16 with s_max: the buffer holds, bit for bit, the maximum group scale that
    coat_fp8_group_scales finds on the stored output (ragged length: rows beyond the sequence do not count)."""
    from coat_amd.activation.real_quantization.common import new_max, read_max
    from coat_amd.models._attention import attention_forward
    B, H, S, D = 2, 4, 333, 128
    g = torch.Generator().manual_seed(11)
    q, k, v = [(torch.randn(B, S, H, D, generator=g) * 3).bfloat16().to(dev).transpose(1, 2) for _ in range(3)]
    buf = new_max(dev)
    out, _ = attention_forward(q, k, v, causal=True, out_scale_max=buf, out_fp8=fp8)
    ref, _ = attention_forward(q, k, v, causal=True)
    assert torch.equal(out, ref)
    assert read_max(buf).item() == _scale_pass_max(out.transpose(1, 2).reshape(B * S, H * D), fp8).item() > 0


def test_layer_quantizations_fed_by_handed_over_maxima_are_bit_identical(dev, monkeypatch):
    """The attention module tags its output (forward) and the RoPE backward tags the q / k gradients with the scale maximum
    their kernels merged; fp8_quantize_pertensor(_transpose) then skip their scale pass.  Same codes, same scale and the
    scale pass really skipped: compared with the untagged path on the same tensors."""
    import coat_amd.activation.real_quantization._quantize_pertensor as QP
    from coat_amd.activation.real_quantization import fp8_quantize_pertensor, fp8_quantize_pertensor_transpose
    from coat_amd.activation.real_quantization.common import known_scale_max
    from coat_amd.models.coat_llama import CoatLlamaConfig, LlamaSdpaAttentionWithoutLinear
    cfg = CoatLlamaConfig(hidden_size=512, intermediate_size=1024, num_attention_heads=4, num_key_value_heads=4)
    attn = LlamaSdpaAttentionWithoutLinear(cfg, 0).train()
    B, S, Hd = 2, 160, 512
    g = torch.Generator().manual_seed(12)
    qs, ks, vs = [torch.randn(B, S, Hd, generator=g).bfloat16().to(dev).requires_grad_(True) for _ in range(3)]
    out, _, _ = attn(qs, ks, vs)
    assert known_scale_max(out, torch.float8_e4m3fn) is not None and known_scale_max(out, torch.float8_e5m2) is None
    calls = []
    real = QP.group_scales_and_max
    monkeypatch.setattr(QP, "group_scales_and_max", lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    import coat_amd.activation.real_quantization._quantize_pertensor_transpose as QPT
    monkeypatch.setattr(QPT, "group_scales_and_max", QP.group_scales_and_max)
    q1, s1, _ = fp8_quantize_pertensor(out, 16, "E4M3", want_pg=False)
    assert not calls
    q0, s0, _ = fp8_quantize_pertensor(out.detach().clone(), 16, "E4M3", want_pg=False)
    assert len(calls) == 1 and torch.equal(q0.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(s0, s1)
    # an in-place change after the hand-over invalidates the tag
    from coat_amd.activation.real_quantization.common import tag_scale_max
    out2 = tag_scale_max(out.detach().clone(), out._coat_scale_max[0], torch.float8_e4m3fn)
    assert known_scale_max(out2, torch.float8_e4m3fn) is not None
    out2.mul_(2)
    assert known_scale_max(out2, torch.float8_e4m3fn) is None
    # backward: the gradients of the q and k projections arrive tagged for e5m2, the one of v (torch's backward) untagged
    seen = {}
    qs.register_hook(lambda gr: seen.__setitem__("q", gr))
    ks.register_hook(lambda gr: seen.__setitem__("k", gr))
    vs.register_hook(lambda gr: seen.__setitem__("v", gr))
    out.backward(torch.randn(B, S, Hd, generator=g).bfloat16().to(dev) * 1e-2)
    assert known_scale_max(seen["v"], torch.float8_e5m2) is None
    for name in ("q", "k"):
        gr = seen[name]
        assert known_scale_max(gr, torch.float8_e5m2) is not None
        n = len(calls)
        a = fp8_quantize_pertensor_transpose(gr, 16, "E5M2", transpose_output_2d=True)
        assert len(calls) == n
        b = fp8_quantize_pertensor_transpose(gr.detach().clone(), 16, "E5M2", transpose_output_2d=True)
        assert len(calls) == n + 1
        for x, y in zip(a, b):
            assert torch.equal(x.view(torch.uint8) if x.dtype != torch.bfloat16 else x, y.view(torch.uint8) if y.dtype != torch.bfloat16 else y)


def test_fused_qkv_gradient_arrives_with_the_maximum_of_all_three_parts(dev):
    """OLMo's fused projection: the backward of fused_qkv_rotary writes dq and dk (inverse rotations) and dv (copy) into one
    gradient and all three kernels merge into one maximum buffer; quantizing that gradient per tensor with and without the
    hand-over gives the same codes and scale, whichever part holds the largest value."""
    from coat_amd.activation.real_quantization import fp8_quantize_pertensor_transpose
    from coat_amd.activation.real_quantization.common import known_scale_max
    from coat_amd.models.coat_llama import fused_qkv_rotary
    B, S, H, KV, D = 2, 96, 4, 2, 128
    g = torch.Generator().manual_seed(13)
    for big in range(3):  # the largest gradient sits in q, then k, then v
        qkv = torch.randn(B, S, (H + 2 * KV) * D, generator=g).bfloat16().to(dev).requires_grad_(True)
        seen = {}
        qkv.register_hook(lambda gr: seen.__setitem__("g", gr))
        q, k, v = fused_qkv_rotary(qkv, H, KV, D, 10000.0, grad_fp8=torch.float8_e5m2)
        grads = [torch.randn(t.shape, generator=g).bfloat16().to(dev) * (8.0 if i == big else 1.0) for i, t in enumerate((q, k, v))]
        torch.autograd.backward([q, k, v], grads)
        gr = seen["g"]
        assert known_scale_max(gr, torch.float8_e5m2) is not None
        a = fp8_quantize_pertensor_transpose(gr, 16, "E5M2", transpose_output_2d=True)
        b = fp8_quantize_pertensor_transpose(gr.detach().clone(), 16, "E5M2", transpose_output_2d=True)
        assert torch.equal(a[0].view(torch.uint8), b[0].view(torch.uint8)) and torch.equal(a[1], b[1])
        assert torch.equal(a[2].view(torch.uint8), b[2].view(torch.uint8))
        # and the gradient itself equals the one of the untagged path
        qkv2 = qkv.detach().clone().requires_grad_(True)
        q2, k2, v2 = fused_qkv_rotary(qkv2, H, KV, D, 10000.0)
        torch.autograd.backward([q2, k2, v2], grads)
        assert torch.equal(qkv2.grad, gr)
