"""GPU checks at the full sizes of the benchmark configurations, where the CPU oracle would take minutes: each kernel is
held to size-independent properties, evaluated on the GPU with plain torch fp32 arithmetic.

* quantize family: round trip within half a code step of the group maximum, the largest member of every group maps
  to the largest finite code, q^T of the per-tensor path is the byte transpose of q, the transposing kernels agree
  with the non-transposing ones bit for bit;
* GEMM: |C - C_ref| <= 2^-7 |C_ref| + 2^-14 sum|a||b| s_A s_B with C_ref from an fp32 matmul of the decoded operands
  (its own accumulation error, K 2^-24 sum|a||b|, is inside the second term);
* SiLU / mul: dequantized outputs against torch's fp32 formula within one e4m3 step of the tensor maximum;
* AdamW: step 1 from the fresh state against the closed form, Dynamic-Range-Expansion invariants (exponent on the
  1/16 grid, largest code per group = 448), and identical bytes on a second run.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu
E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


def _rq():
    import coat_amd.activation.real_quantization as rq
    return rq


def randn(dev, shape, seed, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator(device=dev).manual_seed(seed)
    return (torch.randn(shape, generator=g, device=dev) * scale).to(dtype)


def test_quantize_family_llama_activation(dev):
    rq = _rq()
    from coat_amd.activation.real_quantization._quantize_transpose import fp8_quantize_transpose
    M, N, QB = 8192, 11008, 16
    x = randn(dev, (M, N), 1)
    x[::97, ::89] *= 64
    q, s = rq.fp8_quantize(x, QB, "E4M3")
    xg = x.float().reshape(M, N // QB, QB)
    amax = xg.abs().amax(dim=2, keepdim=True)
    deq = q.float().reshape(M, N // QB, QB) * s.float().unsqueeze(-1)
    # bf16 storage of the scale (2^-9 relative) + half an e4m3 step (2^-4 relative at worst) of the group maximum
    assert ((deq - xg).abs() <= amax * (2.0 ** -4 + 2.0 ** -8) + 1e-12).all()
    assert ((q.view(torch.uint8).reshape(M, N // QB, QB) & 0x7F).amax(dim=2) == 0x7E).all()
    (q2, s2), (qt, st) = fp8_quantize_transpose(x, QB, "E4M3")
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2, s)
    qx, sx = rq.fp8_quantize(x.t().contiguous(), QB, "E4M3")
    assert torch.equal(qt.view(torch.uint8), qx.view(torch.uint8)) and torch.equal(st, sx)
    for fp8 in ("E4M3", "E5M2"):
        qp, sp, qpt = rq.fp8_quantize_pertensor_transpose(x, QB, fp8)
        assert torch.equal(qpt.view(torch.uint8), qp.view(torch.uint8).t())
        qp1, sp1 = rq.fp8_quantize_pertensor(x, QB, fp8)[:2]
        assert torch.equal(qp1.view(torch.uint8), qp.view(torch.uint8)) and torch.equal(sp1, sp)
        mx = 448.0 if fp8 == "E4M3" else 57344.0
        assert abs(sp.float().item() * mx / x.float().abs().max().item() - 1) <= 2.0 ** -8
        step = 2.0 ** -4 if fp8 == "E4M3" else 2.0 ** -3
        assert ((qp.float() * sp.float() - x.float()).abs() <= x.float().abs() * step + sp.float() * (2.0 ** -10 if fp8 == "E4M3" else 2.0 ** -17)).all()
    back = rq.fp8_dequantize(q, s, QB)
    assert torch.equal(back.float(), deq.reshape(M, N).bfloat16().float())


@pytest.mark.parametrize("M,N,K,fa", [(8192, 11008, 4096, E4), (8192, 4096, 11008, E5), (11008, 4096, 8192, E5)])
def test_gemm_llama_mlp_shapes(dev, M, N, K, fa):
    from coat_amd.activation.real_quantization import linear
    a = randn(dev, (M, K), 2, 1.0, torch.float32).to(fa)
    b = randn(dev, (N, K), 3, 1.0, torch.float32).to(E4)
    sa = torch.tensor(0.02, device=dev).bfloat16()
    sb = torch.tensor(0.013, device=dev).bfloat16()
    c = linear.fp8matmul(a, b.t(), False, sa, sb, 16)
    scale = sa.float() * sb.float()
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        rows = 2048  # bound the fp32 temporaries
        for r0 in range(0, M, rows):
            af = a[r0:r0 + rows].float()
            ref = (af @ b.float().t()) * scale
            bound = (af.abs() @ b.float().abs().t()) * scale * 2.0 ** -14
            err = (c[r0:r0 + rows].float() - ref).abs()
            assert (err <= ref.abs() * 2.0 ** -7 + bound).all(), (r0, (err / (ref.abs() + 1e-6)).max().item())
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev


def test_silu_mul_llama_mlp(dev):
    rq = _rq()
    M, N, QB = 8192, 11008, 16
    gate, up = randn(dev, (M, N), 4), randn(dev, (M, N), 5)
    qg, sg = rq.fp8_quantize(gate, QB, "E4M3")
    qu, su = rq.fp8_quantize(up, QB, "E4M3")
    gd = (qg.float().reshape(M, N // QB, QB) * sg.float().unsqueeze(-1)).reshape(M, N)
    ud = (qu.float().reshape(M, N // QB, QB) * su.float().unsqueeze(-1)).reshape(M, N)
    qs, ss = rq.fp8_silu_forward(qg, sg, QB)
    ref = torch.nn.functional.silu(gd)
    sd = (qs.float().reshape(M, N // QB, QB) * ss.float().unsqueeze(-1)).reshape(M, N)
    gmax = ref.reshape(M, N // QB, QB).abs().amax(dim=2, keepdim=True).expand(M, N // QB, QB).reshape(M, N)
    assert ((sd - ref).abs() <= gmax * (2.0 ** -4 + 2.0 ** -8) + 1e-12).all()
    qm, sm, qmt = rq.fp8_mul_forward(qs, ss, qu, su, QB)
    assert torch.equal(qmt.view(torch.uint8), qm.view(torch.uint8).t())
    prod = (sd * ud).bfloat16().float()
    assert abs(sm.float().item() * 448.0 / prod.abs().max().item() - 1) <= 2.0 ** -7
    assert ((qm.float() * sm.float() - prod).abs() <= prod.abs() * 2.0 ** -4 + sm.float() * 2.0 ** -10).all()


def test_adamw_llama_weight(dev):
    from coat_amd.optimizer import qoptim_cuda as Q
    n = 11008 * 4096
    ng = n // 128
    hp = dict(beta1=0.9, beta2=0.95, lr=1e-3, wd=0.1, eps=1e-8)

    def fresh():
        p = randn(dev, (n,), 6, 0.02, torch.float32)
        z8 = lambda: torch.zeros(n, dtype=E4, device=dev)
        zf = lambda v: torch.full((ng,), v, dtype=torch.float32, device=dev)
        return p, [z8(), zf(0.0), zf(1.0), zf(1.0), z8(), zf(0.0), zf(1.0), zf(1.0)]

    g = randn(dev, (n,), 7, 1e-3, torch.float32) * torch.logspace(-1, 1, 128, device=dev).repeat(ng)
    p, st = fresh()
    p0 = p.clone()
    Q.fp8_adamw_expand_step(p, g, *st, *hp.values(), 1, 128, 16)
    # closed form of step 1 from zero moments: m_hat = g, v_hat = g^2
    ref = p0 * (1 - hp["lr"] * hp["wd"]) - hp["lr"] * g / (g.abs() + hp["eps"])
    assert torch.allclose(p, ref, rtol=3e-6, atol=1e-9)
    m8, sm, km, cm, v8, sv, kv, cv = st
    for codes, s, k, c, target in ((m8, sm, km, cm, (1 - hp["beta1"]) * g), (v8, sv, kv, cv, (1 - hp["beta2"]) * g * g)):
        assert ((k * 16).round() == k * 16).all() and (k > 0).all() and (k <= 16).all()
        assert (s > 0).all() and (c > 0).all()
        cg = codes.view(torch.uint8).reshape(ng, 128) & 0x7F
        assert (cg.amax(dim=1) == 0x7E).all()
        # dequantize: sign * (|code * s|)^(1/k) * c reproduces the moment within an e4m3 step mapped through 1/k
        y = codes.float().reshape(ng, 128) * s.unsqueeze(1)
        deq = y.sign() * y.abs().pow(1.0 / k.unsqueeze(1)) * c.unsqueeze(1)
        t = target.reshape(ng, 128)
        nz = cg > 0x08  # normal codes: relative step 2^-4 of the expanded value
        rel = ((deq - t).abs() / t.abs().clamp_min(1e-30))[nz]
        assert (rel <= (2.0 ** -4 + 1e-3) / k.unsqueeze(1).expand(ng, 128)[nz] * 1.05 + 1e-4).all(), rel.max().item()
    # determinism: a second run from the same inputs writes the same bytes
    p2, st2 = fresh()
    Q.fp8_adamw_expand_step(p2, g, *st2, *hp.values(), 1, 128, 16)
    assert torch.equal(p2, p)
    for a, b in zip(st, st2):
        assert torch.equal(a.view(torch.uint8) if a.dtype == E4 else a, b.view(torch.uint8) if b.dtype == E4 else b)
