"""Pins oracle/activation_ref.py by closed forms, invariants and torch.nn.functional + autograd."""

import pytest
import torch
import torch.nn.functional as F

from oracle import activation_ref as R

E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


def _x(M, N, seed=0, outliers=True, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, N, generator=g)
    if outliers:
        x[torch.rand(M, N, generator=g) < 0.001] *= 100
    return x.to(dtype)


def test_quantize_hand_made_groups():
    x = torch.zeros(2, 32)
    x[0, :16] = torch.arange(16) * 28.0          # amax 420 -> s = (420+1e-10)/448 = 0.9375, x/s = 29.8667 * i
    x[0, 16:] = -448.0                            # s = 1 -> code 0xFE everywhere
    x[1, 0] = 1.0                                 # s = 1/448 -> code of 448 = 0x7E, rest 0
    q, s = R.fp8_quantize(x, 16, "E4M3")
    assert s.dtype == torch.bfloat16 and s.shape == (2, 2)
    assert s[0, 0].item() == 0.9375 and s[0, 1].item() == 1.0 and s[1, 1].float().item() == pytest.approx(1e-10 / 448, rel=1e-2)
    assert (q[0, 16:].view(torch.uint8) == 0xFE).all()
    assert q[1, 0].view(torch.uint8).item() == 0x7E and (q[1, 1:].view(torch.uint8) == 0).all()
    want = (torch.arange(16) * 28.0 / 0.9375).to(E4)
    assert torch.equal(q[0, :16].view(torch.uint8), want.view(torch.uint8))
    assert q[0, 15].float().item() == 448.0


@pytest.mark.parametrize("fp8,QB", [("E4M3", 16), ("E5M2", 16), ("E4M3", 128)])
def test_quantize_scale_and_error_bound(fp8, QB):
    x = _x(64, 256, 1)
    q, s = R.fp8_quantize(x, QB, fp8)
    fmax = R.FP8_MAX_VALUE[R.STR2FP8[fp8]]
    amax = x.double().reshape(64, -1, QB).abs().amax(dim=2)
    s64 = ((amax.float() + torch.tensor(1e-10)).double() / fmax)  # the add is an fp32 add in the kernel
    assert torch.equal(s, s64.float().bfloat16()) or torch.equal(s, ((amax.float() + 1e-10) / fmax).bfloat16())
    deq = q.double().reshape(64, -1, QB) * ((amax.float() + 1e-10) / fmax).double().unsqueeze(2)
    err = (deq - x.double().reshape(64, -1, QB)).abs()
    mant = 3 if fp8 == "E4M3" else 2
    # half a step of the binade of the scaled value, at most 2^-(mant+1) relative to the group max
    assert (err <= amax.unsqueeze(2) * 2.0 ** -(mant + 1) * (1 + 1e-6) + 1e-12).all()
    # the group maximum itself is reproduced exactly up to fp32 rounding of the scale
    assert ((q.float().reshape(64, -1, QB).abs().amax(dim=2) == fmax) | (amax == 0)).all()


def test_reference_tests_definition_is_95_percent_equal():
    x = _x(256, 512, 2, dtype=torch.float32)
    q, s = R.fp8_quantize(x, 16, "E4M3")
    qb, sb = R.quantize_tensor_ref_test(x, 16, "E4M3")
    assert torch.equal(s, sb)  # 1e-10 is far below one bf16 ulp of these scales
    eq = (q.view(torch.uint8) == qb.view(torch.uint8)).float().mean().item()
    assert 0.95 <= eq < 1.0  # tests/test_utils.py:98-119 bar; the two definitions are not identical


def test_quantize_transpose_is_quantize_of_transpose():
    x = _x(64, 96, 3)
    (q, s), (qt, st) = R.fp8_quantize_transpose(x, 16, "E4M3")
    q2, s2 = R.fp8_quantize(x.t().contiguous(), 16, "E4M3")
    assert torch.equal(qt.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(st, s2)
    q1, s1 = R.fp8_quantize(x, 16, "E4M3")
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(s, s1)
    assert qt.shape == (96, 64) and st.shape == (96, 4)


def test_perblock_hand_made_blocks():
    x = torch.zeros(32, 32)
    x[:16, :16] = (torch.arange(256).reshape(16, 16) % 16) * 28.0   # block (0,0): amax 420 -> s = 0.9375
    x[:16, 16:] = -448.0                                            # block (0,1): s = 1, every code 0xFE
    x[20, 3] = 1.0                                                  # block (1,0): s = 1/448, that element codes 448
    q, s = R.fp8_quantize_perblock(x, 16, "E4M3")
    assert s.dtype == torch.bfloat16 and s.shape == (2, 2)
    assert s[0, 0].item() == 0.9375 and s[0, 1].item() == 1.0
    assert s[1, 0].float().item() == pytest.approx(1.0 / 448, rel=4e-3) and s[1, 1].float().item() == pytest.approx(1e-10 / 448, rel=1e-2)
    assert (q[:16, 16:].view(torch.uint8) == 0xFE).all()
    want = ((torch.arange(256).reshape(16, 16) % 16) * 28.0 / 0.9375).to(E4)
    assert torch.equal(q[:16, :16].view(torch.uint8), want.view(torch.uint8))
    assert q[20, 3].view(torch.uint8).item() == 0x7E
    rest = q[16:, :].view(torch.uint8).clone()
    rest[4, 3] = 0
    assert (rest == 0).all()


@pytest.mark.parametrize("fp8,QB,sdt", [("E4M3", 16, torch.bfloat16), ("E5M2", 32, torch.float32), ("E4M3", 128, torch.float32)])
def test_perblock_scales_by_loops_and_error_bound(fp8, QB, sdt):
    M, N = 2 * QB, 3 * QB
    x = _x(M, N, 11)
    q, s = R.fp8_quantize_perblock(x, QB, fp8, scale_dtype=sdt)
    fmax = R.FP8_MAX_VALUE[R.STR2FP8[fp8]]
    mant = 3 if fp8 == "E4M3" else 2
    xl = x.double().tolist()
    for bi in range(M // QB):
        for bj in range(N // QB):
            amax = 0.0
            for r in range(QB):          # plain loops: nothing shared with the oracle's reshape / amax
                for c in range(QB):
                    amax = max(amax, abs(xl[bi * QB + r][bj * QB + c]))
            s32 = (torch.tensor(amax, dtype=torch.float32) + torch.tensor(1e-10)) / fmax
            assert s[bi, bj].item() == s32.to(sdt).item()
            blk = q[bi * QB:(bi + 1) * QB, bj * QB:(bj + 1) * QB].double() * s32.double()
            err = (blk - x[bi * QB:(bi + 1) * QB, bj * QB:(bj + 1) * QB].double()).abs()
            assert (err <= amax * 2.0 ** -(mant + 1) * (1 + 1e-6) + 1e-12).all()
            assert q[bi * QB:(bi + 1) * QB, bj * QB:(bj + 1) * QB].float().abs().max().item() == fmax


def test_perblock_of_one_block_is_division_by_the_fp32_scale():
    x = _x(64, 64, 12, dtype=torch.float32)
    q, s = R.fp8_quantize_perblock(x, 64, "E4M3", scale_dtype=torch.float32)
    s32 = (x.abs().max() + torch.tensor(1e-10)) / 448.0
    qd, _ = R.fp8_division(x, 16, "E4M3", s32)
    assert s.shape == (1, 1) and s.item() == s32.item()
    assert torch.equal(q.view(torch.uint8), qd.view(torch.uint8))


def test_perblock_transpose_and_pergroup_parts():
    x = _x(64, 96, 13)
    (q, s), (qt, st), (qg, sg) = R.fp8_quantize_perblock_transpose_pergroup(x, 32, "E4M3", scale_dtype=torch.float32)
    q0, s0 = R.fp8_quantize_perblock(x, 32, "E4M3", scale_dtype=torch.float32)
    assert torch.equal(q.view(torch.uint8), q0.view(torch.uint8)) and torch.equal(s, s0)
    assert qt.shape == (96, 64) and st.shape == (3, 2)
    assert torch.equal(qt.view(torch.uint8), q0.view(torch.uint8).t()) and torch.equal(st, s0.t())
    qg0, sg0 = R.fp8_quantize(x, 32, "E4M3", scale_dtype=torch.float32)       # the pinned per-group quantizer
    assert torch.equal(qg.view(torch.uint8), qg0.view(torch.uint8)) and torch.equal(sg, sg0)
    qt1, st1 = R.fp8_quantize_perblock_transpose(x, 32, "E4M3", scale_dtype=torch.float32, only_transposed=True)
    assert torch.equal(qt1.view(torch.uint8), qt.view(torch.uint8)) and torch.equal(st1, st)
    # the transposed pair is the per-block quantization of x^T (blocks are square)
    q2, s2 = R.fp8_quantize_perblock(x.t().contiguous(), 32, "E4M3", scale_dtype=torch.float32)
    assert torch.equal(qt.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(st, s2)


def test_perblock_against_the_reference_tests_definition():
    """tests/test_fp8_quantize.py:42-48 with tests/test_utils.py:53-60: fp32 [1024, 2048], QB 16, >= 95 % equal codes."""
    x = _x(1024, 2048, 14, outliers=False, dtype=torch.float32)
    q, s = R.fp8_quantize_perblock(x, 16, "E4M3")
    qb, sb = R.quantize_tensor_ref_test_perblock(x, 16, "E4M3")
    assert torch.equal(s, sb)
    eq = (q.view(torch.uint8) == qb.view(torch.uint8)).float().mean().item()
    assert 0.95 <= eq < 1.0


@pytest.mark.parametrize("fp8", ["E4M3", "E5M2"])
def test_pertensor_paths(fp8):
    x = _x(64, 128, 4)
    q, s, s_pg = R.fp8_quantize_pertensor(x, 16, fp8)
    fmax = R.FP8_MAX_VALUE[R.STR2FP8[fp8]]
    assert s.dtype == torch.bfloat16 and s.numel() == 1
    # rounding is monotone: max of rounded scales == rounded scale of the tensor maximum
    assert s.item() == ((x.float().abs().max() + 1e-10) / fmax).bfloat16().item()
    want = R.cast_fp8(x.float() / s.float(), fp8)
    assert torch.equal(q.view(torch.uint8), want.view(torch.uint8))
    q2, s2, qt = R.fp8_quantize_pertensor_transpose(x, 16, fp8)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and s2.item() == s.item()
    assert torch.equal(qt.view(torch.uint8), q.view(torch.uint8).t())
    assert torch.equal(R.fp8_transpose(q).view(torch.uint8), q.view(torch.uint8).t())
    # s_y=None: scale evaluated in the input dtype (bf16 here)
    q3, s3 = R.fp8_division(x, 16, fp8)
    assert s3.dtype == torch.bfloat16 and s3.item() == ((x.abs().max().float() + 1e-10).bfloat16().float() / fmax).bfloat16().item()
    # saturation instead of NaN when the given scale is too small
    q4, _ = R.fp8_division(x, 16, fp8, (s.float() / 4).bfloat16())
    assert q4.float().isfinite().all() and q4.float().abs().max().item() == fmax


def test_dequantize():
    x = _x(32, 64, 5)
    q, s = R.fp8_quantize(x, 16, "E4M3")
    y = R.fp8_dequantize(q, s, 16)
    want = (q.double().reshape(32, 4, 16) * s.double().unsqueeze(2)).reshape(32, 64)
    assert torch.equal(y, want.float().bfloat16())  # product of an 4-bit and an 8-bit significand is exact in fp32


def test_matmul_against_float64():
    g = torch.Generator().manual_seed(6)
    a = (torch.randn(64, 128, generator=g)).to(E4)
    b = (torch.randn(96, 128, generator=g)).to(E5)
    sa, sb = torch.tensor(0.02).bfloat16(), torch.tensor(0.5).bfloat16()
    bias = torch.randn(96, generator=g).bfloat16()
    c = R.fp8matmul(a, b.t(), False, sa, sb, 16, bias)
    ref = (a.double() @ b.double().t()) * (sa.double() * sb.double()) + bias.double()
    assert c.dtype == torch.bfloat16 and (c.double() - ref).abs().max() <= ref.abs().max() * 2.0 ** -8
    cq, cs = R.fp8matmul(a, b.t(), True, sa, sb, 16)
    assert cq.dtype == E4 and cs.shape == (64, 6)
    deq = R.fp8_dequantize(cq, cs, 16).double()
    ref2 = (a.double() @ b.double().t()) * (sa.double() * sb.double())
    assert ((deq - ref2).abs() <= ref2.reshape(64, 6, 16).abs().amax(dim=2).repeat_interleave(16, dim=1) * 2.0 ** -4 * 1.02 + 1e-9).all()
    # linear backward: dgrad = g @ w, wgrad = g^T @ x through the stored transposes
    xq, wq, gq = a, (torch.randn(96, 128, generator=g)).to(E4), (torch.randn(64, 96, generator=g)).to(E5)
    dx, dw = R.fp8_linear_backward(xq.t().contiguous(), sa, gq, sb, gq.t().contiguous(), wq.t().contiguous(), sa, 16)
    rdx = (gq.double() @ wq.double()) * (sb.double() * sa.double())
    rdw = (gq.double().t() @ xq.double()) * (sb.double() * sa.double())
    assert dx.shape == (64, 128) and dw.shape == (96, 128)
    assert (dx.double() - rdx).abs().max() <= rdx.abs().max() * 2.0 ** -8
    assert (dw.double() - rdw).abs().max() <= rdw.abs().max() * 2.0 ** -8


def _pg(x, fp8="E4M3"):
    return R.fp8_quantize(x, 16, fp8)


def test_silu_gelu_mul_values_against_torch_functional():
    x = _x(32, 64, 7, outliers=False)
    g = _x(32, 64, 8, outliers=False) * 0.01
    q, s = _pg(x)
    xd = R._dequant32(q, s, 16).double().requires_grad_(True)
    # forward values
    qy, sy = R.fp8_silu_forward(q, s, 16)
    ref = F.silu(xd)
    want_q, want_s = R._quantize_pg(ref.detach().float(), 16, E4)
    assert (qy.view(torch.uint8) != want_q.view(torch.uint8)).float().mean() < 2e-3  # fp32 vs fp64 exp, 1 code step
    assert torch.equal(sy, want_s) or (sy.float() - want_s.float()).abs().max() <= want_s.float().abs().max() * 2 ** -7
    # backward values
    ref.backward(g.double())
    v = R.silu_backward_value(q, s, g, 16)
    assert torch.allclose(v.double(), xd.grad, rtol=1e-5, atol=1e-9)
    xd.grad = None
    ref = F.gelu(xd)
    # 1 + erf(x/sqrt 2) cancels for negative x: the fp32 formula is absolutely, not relatively, accurate
    assert torch.allclose(R.gelu_forward_value(q, s, 16).double(), ref.detach(), rtol=1e-5, atol=5e-7)
    ref.backward(g.double())
    assert torch.allclose(R.gelu_backward_value(q, s, g, 16).double(), xd.grad, rtol=1e-5, atol=5e-9)
    # mul
    x2 = _x(32, 64, 9, outliers=False)
    q2, s2 = _pg(x2)
    qm, sm, qmt = R.fp8_mul_forward(q, s, q2, s2, 16)
    prod = (R._dequant32(q, s, 16) * R._dequant32(q2, s2, 16))
    assert sm.numel() == 1 and torch.equal(qmt.view(torch.uint8), qm.view(torch.uint8).t())
    assert torch.equal(qm.view(torch.uint8), R.cast_fp8(prod.bfloat16().float() / sm.float(), E4).view(torch.uint8))
    assert sm.item() == ((prod.abs().max() + 1e-10) / 448).bfloat16().item()
    y1, (qy2, s2m, qy2t) = R.fp8_mul_backward(q, s, q2, s2, g, 16, "E5M2", output_quantized_transpose=True)
    assert torch.equal(y1, (g.float() * R._dequant32(q2, s2, 16)).bfloat16()) and qy2.dtype == E5
    assert torch.equal(qy2t.view(torch.uint8), qy2.view(torch.uint8).t())


def test_add_paths():
    a, b = _x(32, 64, 10), _x(32, 64, 11)
    y, (q, s) = R.fp8_add_Ifp_Ifp_Ofp_Og16(a, b, E4, 16)
    v = a.float() + b.float()
    assert torch.equal(y, v.bfloat16())
    wq, ws = R._quantize_pg(v, 16, E4)
    assert torch.equal(q.view(torch.uint8), wq.view(torch.uint8)) and torch.equal(s, ws)
    y2, (q2, s2, spg) = R.fp8_add_Ifp_Ifp_Ofp_Opt(a, b, 16, "E5M2")
    assert torch.equal(y2, y) and s2.item() == spg.max().item()
    assert torch.equal(q2.view(torch.uint8), R.cast_fp8(y.float() / s2.float(), E5).view(torch.uint8))  # divides the bf16 sum


def test_rmsnorm_against_functional_and_autograd():
    M, N = 48, 256
    x = _x(M, N, 12, outliers=False)
    g = _x(M, N, 13, outliers=False) * 0.01
    w = (1 + 0.1 * _x(1, N, 14, outliers=False).float()).reshape(N).bfloat16()
    q, s = _pg(x)
    xd = R._dequant32(q, s, 16).double().requires_grad_(True)
    wd = w.double().requires_grad_(True)
    ref = F.rms_norm(xd, (N,), wd, 1e-5)
    v, rstd = R.rmsnorm_forward_value(q, s, w, 16, 1e-5)
    assert torch.allclose(v.double(), ref.detach(), rtol=2e-6, atol=1e-8)
    assert torch.allclose(rstd.double(), (xd.detach().pow(2).mean(dim=1) + 1e-5).rsqrt(), rtol=1e-6)
    ref.backward(g.double())
    dx, dw = R.fp8_rmsnorm_backward(q, s, g, w, rstd, 16)
    assert (dx.double() - xd.grad).abs().max() <= xd.grad.abs().max() * 2.0 ** -8
    assert torch.allclose(dw.double(), wd.grad, rtol=1e-2, atol=1e-4) and dw.dtype == w.dtype  # bf16 output
    qy, spt, qyt, _ = R.fp8_rmsnorm_forward(q, s, w, 16, 1e-5)
    assert spt.item() == ((v.abs().max() + 1e-10) / 448).bfloat16().item()
    assert torch.equal(qy.view(torch.uint8), R.cast_fp8(v.bfloat16().float() / spt.float(), E4).view(torch.uint8))
    assert torch.equal(qyt.view(torch.uint8), qy.view(torch.uint8).t())


@pytest.mark.parametrize("affine", [False, True])
def test_layernorm_against_functional_and_autograd(affine):
    M, N = 48, 256
    x = _x(M, N, 22, outliers=False) + 0.3  # a non-zero mean, so that forgetting the mean subtraction shows
    g = _x(M, N, 23, outliers=False) * 0.01
    w = (1 + 0.1 * _x(1, N, 24, outliers=False).float()).reshape(N).bfloat16() if affine else None
    bb = (0.1 * _x(1, N, 25, outliers=False).float()).reshape(N).bfloat16() if affine else None
    q, s = _pg(x)
    xd = R._dequant32(q, s, 16).double().requires_grad_(True)
    wd = w.double().requires_grad_(True) if affine else None
    bd = bb.double().requires_grad_(True) if affine else None
    ref = F.layer_norm(xd, (N,), wd, bd, 1e-5)
    v, mean, rstd = R.layernorm_forward_value(q, s, 16, 1e-5, w, bb)
    assert torch.allclose(v.double(), ref.detach(), rtol=2e-6, atol=2e-7)
    assert torch.allclose(mean.double(), xd.detach().mean(dim=1), rtol=1e-5, atol=1e-7)
    assert torch.allclose(rstd.double(), (xd.detach().var(dim=1, unbiased=False) + 1e-5).rsqrt(), rtol=1e-6)
    ref.backward(g.double())
    out = R.fp8_layernorm_backward(q, s, g, mean, rstd, 16, w)
    dx = out[0] if affine else out
    assert (dx.double() - xd.grad).abs().max() <= xd.grad.abs().max() * 2.0 ** -8
    if affine:
        assert torch.allclose(out[1].double(), wd.grad, rtol=1e-2, atol=1e-4) and out[1].dtype == w.dtype
        assert torch.allclose(out[2].double(), bd.grad, rtol=1e-2, atol=1e-4) and out[2].dtype == w.dtype
    qy, spt, qyt, _, _ = R.fp8_layernorm_forward(q, s, 16, 1e-5, w, bb)
    assert spt.item() == ((v.abs().max() + 1e-10) / 448).bfloat16().item()
    assert torch.equal(qy.view(torch.uint8), R.cast_fp8(v / spt.float(), E4).view(torch.uint8))  # divides the fp32 y
    assert torch.equal(qyt.view(torch.uint8), qy.view(torch.uint8).t())
