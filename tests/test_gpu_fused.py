"""GPU parity: fused SiLU / GELU / mul / add / RMSNorm kernels against the CPU oracle.

mul and add contain no transcendental function: codes, scales and bf16 values must be bit-exact.
SiLU / GELU / RMSNorm / LayerNorm differ from the oracle only through exp / erf / the order of a long sum (a few fp32 ulp
before quantization).  Measured on an MI355X (printed with ``pytest -rP``): FP8 codes differ on 0 .. 2.9e-6 of the elements
(by one code step), bf16 values on 5e-6 .. 1e-5 (by one ulp; two on 1 of 6.3e6 norm gradients), per-tensor scales never.
Bars: codes 1e-5, bf16 values 3e-5, per-tensor scale identical.
Shape: batch 4 x seq 256 x channels 2048, QB 16 (tests/test_fp8_activations.py:218-226 of the reference)."""
import pytest
import torch

from oracle import activation_ref as R

pytestmark = pytest.mark.gpu
E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2
BS, SL, C, QB = 4, 256, 2048, 16


def _rq():
    import coat_amd.activation.real_quantization as rq
    return rq


def rand(seed, scale=1.0, shape=(BS * SL, C)):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).bfloat16()


def pg(x, fp8="E4M3"):
    return R.fp8_quantize(x, QB, fp8)


def b(t):
    return t.cpu().view(torch.uint8)


def _caller():
    import inspect
    return inspect.stack()[2].function


def codes_close(got, want, max_frac=1e-5):
    g, w = b(got).int().flatten(), b(want).int().flatten()
    neq = g != w
    frac = neq.float().mean().item()
    print(f"[measured] {_caller()}: {frac:.3e} of {g.numel()} codes differ (bar {max_frac:.0e})")
    assert frac <= max_frac, f"{frac} of the codes differ"
    if neq.any():
        assert ((g[neq] & 0x7F) - (w[neq] & 0x7F)).abs().max().item() <= 1
        assert (((g[neq] & 0x80) == (w[neq] & 0x80)) | (((g[neq] & 0x7F) + (w[neq] & 0x7F)) <= 1)).all()
    return frac


def bf16_close(got, want, max_frac=3e-5, max_ulp=1):
    g, w = got.cpu().view(torch.int16).int().flatten(), want.view(torch.int16).int().flatten()
    neq = g != w
    frac = neq.float().mean().item()
    ulp = (g[neq] - w[neq]).abs().max().item() if neq.any() else 0
    print(f"[measured] {_caller()}: {frac:.3e} of {g.numel()} bf16 values differ, {ulp} ulp at most (bar {max_frac:.0e}, {max_ulp} ulp)")
    assert frac <= max_frac
    assert ulp <= max_ulp  # neighbouring bf16 values (same sign)


def test_mul_forward_backward_bit_exact(dev):
    rq = _rq()
    x1, x2, g = rand(1), rand(2), rand(3, 0.01)
    (q1, s1), (q2, s2) = pg(x1), pg(x2)
    qy, s, qyt = rq.fp8_mul_forward(q1.to(dev).reshape(BS, SL, C), s1.to(dev).reshape(BS, SL, -1),
                                    q2.to(dev).reshape(BS, SL, C), s2.to(dev).reshape(BS, SL, -1), QB, transpose_output_2d=True)
    wq, ws, wqt = R.fp8_mul_forward(q1, s1, q2, s2, QB)
    assert qy.shape == (BS, SL, C) and qyt.shape == (C, BS * SL) and s.dtype == torch.bfloat16
    assert s.item() == ws.item() and torch.equal(b(qy).reshape(-1, C), b(wq)) and torch.equal(b(qyt), b(wqt))
    y1, (qy2, s2m, qy2t) = rq.fp8_mul_backward(q1.to(dev), s1.to(dev), q2.to(dev), s2.to(dev), g.to(dev), QB, "E5M2",
                                              output_quantized_transpose=True)
    wy1, (wq2, ws2, wq2t) = R.fp8_mul_backward(q1, s1, q2, s2, g, QB, "E5M2", output_quantized_transpose=True)
    assert torch.equal(y1.cpu(), wy1) and s2m.item() == ws2.item() and qy2.dtype == E5
    assert torch.equal(b(qy2), b(wq2)) and torch.equal(b(qy2t), b(wq2t))
    y1b, (y2b, s2b) = rq.fp8_mul_backward(q1.to(dev), s1.to(dev), q2.to(dev), s2.to(dev), g.to(dev), QB, "E5M2")
    wy1b, (wy2b, ws2b) = R.fp8_mul_backward(q1, s1, q2, s2, g, QB, "E5M2")
    assert torch.equal(y1b.cpu(), wy1b) and torch.equal(y2b.cpu(), wy2b) and torch.equal(s2b.cpu(), ws2b)


def test_add_forward_backward_bit_exact(dev):
    rq = _rq()
    x1, x2 = rand(4), rand(5)
    y, (q, s) = rq.fp8_add_Ifp_Ifp_Ofp_Og16(x1.to(dev).reshape(BS, SL, C), x2.to(dev).reshape(BS, SL, C), E4, QB)
    wy, (wq, ws) = R.fp8_add_Ifp_Ifp_Ofp_Og16(x1, x2, E4, QB)
    assert y.shape == (BS, SL, C) and torch.equal(y.cpu().reshape(-1, C), wy)
    assert torch.equal(b(q).reshape(-1, C), b(wq)) and torch.equal(s.cpu().reshape(-1, C // QB), ws)
    y2, (q2, s2, spg) = rq.fp8_add_Ifp_Ifp_Ofp_Opt(x1.to(dev), x2.to(dev), QB, "E5M2")
    wy2, (wq2, ws2, wspg) = R.fp8_add_Ifp_Ifp_Ofp_Opt(x1, x2, QB, "E5M2")
    assert torch.equal(y2.cpu(), wy2) and s2.item() == ws2.item() and torch.equal(spg.cpu(), wspg) and torch.equal(b(q2), b(wq2))


@pytest.mark.parametrize("fp8", ["E4M3", "E5M2"])
def test_silu_forward_backward(dev, fp8):
    rq = _rq()
    x, g = rand(6), rand(7, 0.01)
    q, s = pg(x, fp8)
    y, sy = rq.fp8_silu_forward(q.to(dev), s.to(dev), QB)
    wy, wsy = R.fp8_silu_forward(q, s, QB)
    assert y.dtype == q.dtype
    codes_close(y, wy)
    bf16_close(sy, wsy)
    # fp32 input scales: the output scales are stored as fp32 too (reference silu_fwd.py:166-167), not rounded through bf16
    q32, s32 = R.fp8_quantize(x, QB, fp8, scale_dtype=torch.float32)
    y32, sy32 = rq.fp8_silu_forward(q32.to(dev), s32.to(dev), QB)
    wy32, wsy32 = R.fp8_silu_forward(q32, s32, QB)
    assert sy32.dtype == torch.float32 and wsy32.dtype == torch.float32
    assert torch.allclose(sy32.cpu(), wsy32, rtol=1e-6, atol=0) and (sy32.cpu() != sy32.cpu().bfloat16().float()).any()
    codes_close(y32, wy32)
    gy, gs = rq.fp8_silu_backward(q.to(dev), s.to(dev), g.to(dev), QB, "E5M2")
    wgy, wgs = R.fp8_silu_backward(q, s, g, QB, "E5M2")
    bf16_close(gy, wgy)
    bf16_close(gs, wgs)
    qg, sg, qgt = rq.fp8_silu_backward(q.to(dev), s.to(dev), g.to(dev), QB, "E5M2", output_quantized_transpose=True)
    wqg, wsg, wqgt = R.fp8_silu_backward(q, s, g, QB, "E5M2", output_quantized_transpose=True)
    assert sg.item() == wsg.item() and qg.dtype == E5
    codes_close(qg, wqg)
    assert torch.equal(b(qgt), b(qg).t())


def test_gelu_forward_backward(dev):
    rq = _rq()
    x, g = rand(8), rand(9, 0.01)
    q, s = pg(x)
    qy, sy, qyt = rq.fp8_gelu_forward(q.to(dev), s.to(dev), QB)
    wq, ws, wqt = R.fp8_gelu_forward(q, s, QB)
    assert sy.item() == ws.item()
    codes_close(qy, wq)
    assert torch.equal(b(qyt), b(qy).t())
    qg, sg = rq.fp8_gelu_backward(q.to(dev), s.to(dev), g.to(dev), QB, "E5M2")
    wqg, wsg = R.fp8_gelu_backward(q, s, g, QB, "E5M2")
    assert sg.item() == wsg.item()
    codes_close(qg, wqg)


@pytest.mark.parametrize("N", [2048, 5120, 4096 + 1024 * 8])
def test_rmsnorm_forward_backward(dev, N):
    rq = _rq()
    M = 512
    x, g = rand(10, shape=(M, N)), rand(11, 0.01, shape=(M, N))
    w = (1 + 0.1 * torch.randn(N, generator=torch.Generator().manual_seed(12))).bfloat16()
    q, s = pg(x)
    qy, spt, qyt, (w_, rstd, nw) = rq.fp8_rmsnorm_forward(q.to(dev), s.to(dev), w.to(dev), QB, 1e-5)
    wq, wspt, wqt, wrstd = R.fp8_rmsnorm_forward(q, s, w, QB, 1e-5, accumulate=torch.float64)
    assert torch.allclose(rstd.cpu(), wrstd, rtol=1e-6, atol=0)
    assert spt.item() == wspt.item()
    codes_close(qy, wq)
    assert torch.equal(b(qyt), b(qy).t())
    dx, dw = rq.fp8_rmsnorm_backward(q.to(dev), s.to(dev), g.to(dev), w.to(dev), rstd, QB, nw)
    wdx, wdw = R.fp8_rmsnorm_backward(q, s, g, w, wrstd, QB)
    # dx = (w*dy - xhat*c1)*rstd cancels; the fp32 summation order of c1 shows up as a few bf16 ulp on rare elements
    bf16_close(dx, wdx, 3e-5, max_ulp=2)
    assert dw.dtype == w.dtype and torch.allclose(dw.cpu().float(), wdw.float(), rtol=1e-2, atol=1e-3)  # bf16 output
    # deterministic: the same call again gives the same bits (the reference's lock-ordered dw does not)
    dx2, dw2 = rq.fp8_rmsnorm_backward(q.to(dev), s.to(dev), g.to(dev), w.to(dev), rstd, QB, nw)
    assert torch.equal(dw, dw2) and torch.equal(dx, dx2)


@pytest.mark.parametrize("N,affine", [(2048, False), (5120, False), (4096 + 1024 * 8, False), (2048, True), (5120, True)])
def test_layernorm_forward_backward(dev, N, affine):
    rq = _rq()
    M = 512
    x, g = rand(20, shape=(M, N)) + 0.25, rand(21, 0.01, shape=(M, N))
    w = (1 + 0.1 * torch.randn(N, generator=torch.Generator().manual_seed(22))).bfloat16() if affine else None
    bb = (0.1 * torch.randn(N, generator=torch.Generator().manual_seed(23))).bfloat16() if affine else None
    q, s = pg(x)
    if affine:
        qy, spt, qyt, (w_, b_, mean, rstd, nw) = rq.fp8_layernorm_param_forward(q.to(dev), s.to(dev), w.to(dev), bb.to(dev), QB, 1e-5)
    else:
        qy, spt, qyt, (mean, rstd, nw) = rq.fp8_layernorm_noparam_forward(q.to(dev), s.to(dev), QB, 1e-5)
    wq, wspt, wqt, wmean, wrstd = R.fp8_layernorm_forward(q, s, QB, 1e-5, w, bb, accumulate=torch.float64)
    assert torch.allclose(mean.cpu(), wmean, rtol=1e-5, atol=1e-7)
    assert torch.allclose(rstd.cpu(), wrstd, rtol=2e-6, atol=0)
    assert spt.item() == wspt.item()
    codes_close(qy, wq)
    assert torch.equal(b(qyt), b(qy).t())
    if affine:
        dx, dw, db = rq.fp8_layernorm_param_backward(q.to(dev), s.to(dev), g.to(dev), QB, w.to(dev), bb.to(dev), mean, rstd, nw)
        wdx, wdw, wdb = R.fp8_layernorm_backward(q, s, g, wmean, wrstd, QB, w)
        assert dw.dtype == w.dtype and torch.allclose(dw.cpu().float(), wdw.float(), rtol=1e-2, atol=1e-3)
        assert db.dtype == w.dtype and torch.allclose(db.cpu().float(), wdb.float(), rtol=1e-2, atol=1e-3)
        dx2, dw2, db2 = rq.fp8_layernorm_param_backward(q.to(dev), s.to(dev), g.to(dev), QB, w.to(dev), bb.to(dev), mean, rstd, nw)
        assert torch.equal(dw, dw2) and torch.equal(db, db2) and torch.equal(dx, dx2)
    else:
        dx = rq.fp8_layernorm_noparam_backward(q.to(dev), s.to(dev), g.to(dev), QB, mean, rstd, nw)
        wdx = R.fp8_layernorm_backward(q, s, g, wmean, wrstd, QB)
    # dx = (wdy - (xhat*c1 + c2))*rstd cancels: where the result is below 2^-12 of the tensor's largest gradient the
    # fp32 summation order of c1 / c2 decides its bits, so those elements are held to that absolute bound instead
    big = wdx.float().abs().max()
    small = (wdx.float().abs() < big * 2.0 ** -12) & (dx.cpu().float().abs() < big * 2.0 ** -12)
    bf16_close(torch.where(small.to(dev), torch.zeros_like(dx), dx), torch.where(small, torch.zeros_like(wdx), wdx), 3e-5, max_ulp=2)
    # batched input keeps its leading dimensions
    q3, s3 = q.reshape(4, M // 4, N).to(dev), s.reshape(4, M // 4, N // QB).to(dev)
    if not affine:
        qy3, spt3, qyt3, _ = rq.fp8_layernorm_noparam_forward(q3, s3, QB, 1e-5, transpose_output_2d=True)
        assert qy3.shape == (4, M // 4, N) and qyt3.shape == (N, M) and torch.equal(b(qy3).reshape(M, N), b(qy))


@pytest.mark.parametrize("fp8,QBv", [("E4M3", 16), ("E4M3", 64)])
def test_fused_silu_mul_equals_the_two_kernel_chains(dev, fp8, QBv):
    """coat_fp8_silu_mul_forward / _backward against fp8_silu_forward -> fp8_mul_forward and fp8_mul_backward ->
    fp8_silu_backward (each checked against the oracle above): every output tensor bit for bit."""
    rq = _rq()
    M, N = 384, 1024
    gate, up, g = rand(30, shape=(M, N)), rand(31, shape=(M, N)), rand(32, 0.01, shape=(M, N))
    qg, sg = rq.fp8_quantize(gate.to(dev), QBv, fp8)
    qu, su = rq.fp8_quantize(up.to(dev), QBv, fp8)
    silu_x, silu_s = rq.fp8_silu_forward(qg, sg, QBv)
    mul_x, mul_s, mul_x_t = rq.fp8_mul_forward(silu_x, silu_s, qu, su, QBv, transpose_output_2d=True)
    f_silu_x, f_silu_s, f_mul_x, f_mul_s, f_mul_x_t = rq.fp8_silu_mul_forward(qg, sg, qu, su, QBv, transpose_output_2d=True)
    assert torch.equal(b(f_silu_x), b(silu_x)) and torch.equal(f_silu_s, silu_s)
    assert f_mul_s.item() == mul_s.item() and torch.equal(b(f_mul_x), b(mul_x)) and torch.equal(b(f_mul_x_t), b(mul_x_t))
    gd = g.to(dev)
    g1, (uq, us, uqt) = rq.fp8_mul_backward(silu_x, silu_s, qu, su, gd, QBv, "E5M2", output_quantized_transpose=True)
    gq, gs, gqt = rq.fp8_silu_backward(qg, sg, g1, QBv, "E5M2", output_quantized_transpose=True)
    (f_gq, f_gs, f_gqt), (f_uq, f_us, f_uqt) = rq.fp8_silu_mul_backward(qg, sg, qu, su, silu_x, silu_s, gd, QBv, "E5M2")
    assert f_gs.item() == gs.item() and torch.equal(b(f_gq), b(gq)) and torch.equal(b(f_gqt), b(gqt))
    assert f_us.item() == us.item() and torch.equal(b(f_uq), b(uq)) and torch.equal(b(f_uqt), b(uqt))
    # batched inputs keep their leading dimension
    q3, s3 = qg.reshape(2, M // 2, N), sg.reshape(2, M // 2, N // QBv)
    u3, us3 = qu.reshape(2, M // 2, N), su.reshape(2, M // 2, N // QBv)
    o = rq.fp8_silu_mul_forward(q3, s3, u3, us3, QBv)
    assert o[0].shape == (2, M // 2, N) and o[2].shape == (2, M // 2, N) and torch.equal(b(o[2]).reshape(M, N), b(mul_x))


@pytest.mark.parametrize("QBv", [16, 32])
def test_fused_silu_mul_on_column_slices_and_joined_backward(dev, QBv):
    """gate / up taken as the two column halves of one [M, 2N] projection output (no copies), and the backward that
    writes both gradients side by side: bit for bit the chain of the separate kernels on dense copies, torch.cat,
    max of the group scales and fp8_division_transpose (coat/models/coat_olmo.py:520-528, :594-606)."""
    rq = _rq()
    B, S, N = 2, 96, 512
    M = B * S
    both, g = rand(40, shape=(M, 2 * N)), rand(41, 0.01, shape=(M, N))
    q, s = rq.fp8_quantize(both.to(dev), QBv, "E4M3")
    q3, s3 = q.reshape(B, S, 2 * N), s.reshape(B, S, 2 * N // QBv)
    up_v, gate_v = q3.chunk(2, dim=-1)
    ups_v, gates_v = s3.chunk(2, dim=-1)
    assert not gate_v.is_contiguous()
    up_d, gate_d, ups_d, gates_d = (t.contiguous() for t in (up_v, gate_v, ups_v, gates_v))
    # forward
    silu_x, silu_s = rq.fp8_silu_forward(gate_d, gates_d, QBv)
    mul_x, mul_s, mul_x_t = rq.fp8_mul_forward(silu_x, silu_s, up_d, ups_d, QBv, transpose_output_2d=True)
    f = rq.fp8_silu_mul_forward(gate_v, gates_v, up_v, ups_v, QBv, transpose_output_2d=True)
    assert f[0].shape == (B, S, N) and torch.equal(b(f[0]), b(silu_x)) and torch.equal(f[1], silu_s)
    assert f[3].item() == mul_s.item() and torch.equal(b(f[2]), b(mul_x)) and torch.equal(b(f[4]), b(mul_x_t))
    # backward, joined
    gd = g.to(dev).reshape(B, S, N)
    g1, (ug, ugs) = rq.fp8_mul_backward(silu_x, silu_s, up_d, ups_d, gd, QBv, "E5M2")
    gg, ggs = rq.fp8_silu_backward(gate_d, gates_d, g1, QBv, "E5M2")
    cat = torch.cat([ug, gg], dim=-1)
    smax = torch.max(torch.cat([ugs, ggs]))
    wq, ws, wqt = rq.fp8_division_transpose(cat, QBv, "E5M2", smax)
    jq, js, jqt = rq.fp8_silu_mul_backward_joined(gate_v, gates_v, up_v, ups_v, silu_x, silu_s, gd, QBv, "E5M2")
    assert jq.shape == (B, S, 2 * N) and js.item() == ws.item()
    assert torch.equal(b(jq), b(wq)) and torch.equal(b(jqt), b(wqt))
    # the non-joined backward also takes the slices
    (gq, gs_, gqt), (uq, us_, uqt) = rq.fp8_silu_mul_backward(gate_v, gates_v, up_v, ups_v, silu_x, silu_s, gd, QBv, "E5M2")
    (dq, ds_, dqt), (eq, es_, eqt) = rq.fp8_silu_mul_backward(gate_d, gates_d, up_d, ups_d, silu_x, silu_s, gd, QBv, "E5M2")
    assert gs_.item() == ds_.item() and torch.equal(b(gq), b(dq)) and torch.equal(b(uqt), b(eqt))


@pytest.mark.parametrize("N", [1024, 5120, 4096 + 2048, 8192 + 1024])
def test_rmsnorm_backward_sums_gradients_like_bf16_additions(dev, N):
    """g given as a tuple: identical to adding the bf16 tensors first (the reference's callers do that with torch).  The
    widths take the wave-per-row kernels with 4, 5 and 8 chunks per lane and the block-per-row kernel."""
    rq = _rq()
    M = 96
    x = rand(50, shape=(M, N))
    w = (1 + 0.1 * rand(51, shape=(N,)).float()).bfloat16()
    g1, g2, g3 = rand(52, 0.01, shape=(M, N)), rand(53, 0.01, shape=(M, N)), rand(54, 0.02, shape=(M, N))
    q, s = rq.fp8_quantize(x.to(dev), 16, "E4M3")
    _, _, _, (_, rstd, nw) = rq.fp8_rmsnorm_forward(q, s, w.to(dev), 16, 1e-5, transpose_output_2d=True)
    d1, d2, d3 = g1.to(dev), g2.to(dev), g3.to(dev)
    for gs, summed in (((d1, d2), d1 + d2), ((d1, d2, d3), d1 + d2 + d3), ((d1,), d1)):
        dx_t, dw_t = rq.fp8_rmsnorm_backward(q, s, gs, w.to(dev), rstd, 16, nw)
        dx_s, dw_s = rq.fp8_rmsnorm_backward(q, s, summed, w.to(dev), rstd, 16, nw)
        assert torch.equal(dx_t, dx_s) and torch.equal(dw_t, dw_s)


@pytest.mark.parametrize("M,N,QBv,fp8out", [(96, 1024, 16, "E5M2"), (1504, 4096, 16, "E5M2"), (208, 5120, 16, "E5M2"),
                                            (96, 4096 + 2048, 64, "E4M3"), (64, 8192 + 1024, 16, "E5M2")])
def test_rmsnorm_backward_with_residual_addition_equals_the_two_kernels(dev, M, N, QBv, fp8out):
    """fp8_rmsnorm_backward_add against fp8_rmsnorm_backward followed by fp8_add_Ifp_Ifp_Ofp_Opt, with one, two and three
    gradients: the bf16 sum, the per-group scales, the per-tensor scale, the codes and dw, bit for bit; the addition
    itself against the oracle.  Widths take the 4-, 5- and 8-chunk kernels; the widest falls back to the two kernels."""
    rq = _rq()
    from coat_amd.activation.real_quantization.func_rmsnorm import fp8_rmsnorm_backward_add
    x = rand(70, shape=(M, N))
    w = (1 + 0.1 * rand(71, shape=(N,)).float()).bfloat16().to(dev)
    gs = [rand(72 + i, 0.01 * (i + 1), shape=(M, N)).to(dev) for i in range(3)]
    res = rand(76, 0.02, shape=(M, N))
    res[::5, ::3] *= 30
    res = res.to(dev)
    q, s = rq.fp8_quantize(x.to(dev), QBv, "E4M3")
    _, _, _, (_, rstd, nw) = rq.fp8_rmsnorm_forward(q, s, w, QBv, 1e-5, transpose_output_2d=True)
    for n in (1, 2, 3):
        g = tuple(gs[:n]) if n > 1 else gs[0]
        dx, dw = rq.fp8_rmsnorm_backward(q, s, g, w, rstd, QBv, nw)
        want_y, (want_q, want_s, want_pg) = rq.fp8_add_Ifp_Ifp_Ofp_Opt(res, dx, QBv, fp8out)
        got_y, (got_q, got_s, got_pg), got_dw = fp8_rmsnorm_backward_add(q, s, g, w, rstd, QBv, nw, res, fp8out)
        assert torch.equal(got_y, want_y), (n, "sum")
        assert torch.equal(got_pg.view(torch.int16), want_pg.view(torch.int16)), (n, "group scales")
        assert got_s.dtype == want_s.dtype and got_s.item() == want_s.item(), (n, "tensor scale")
        assert torch.equal(b(got_q), b(want_q)) and torch.equal(got_dw, dw), (n, "codes / dw")
        oy, (oq, os_, opg) = R.fp8_add_Ifp_Ifp_Ofp_Opt(res.cpu(), dx.cpu(), QBv, fp8out)
        assert torch.equal(got_y.cpu(), oy) and torch.equal(got_pg.cpu(), opg) and os_.item() == got_s.item()
        assert torch.equal(b(got_q), oq.view(torch.uint8))


@pytest.mark.parametrize("M,N,QBv,fp8out", [(208, 512, 16, "E5M2"), (1504, 4096, 16, "E5M2"), (64, 4096 + 64, 32, "E4M3"),
                                              (48, 8192 + 128, 128, "E5M2"), (16, 16384, 16, "E5M2")])
def test_layernorm_backward_with_residual_addition_equals_the_two_kernels(dev, M, N, QBv, fp8out):
    """fp8_layernorm_noparam_backward_add against fp8_layernorm_noparam_backward followed by fp8_add_Ifp_Ifp_Ofp_Opt: the
    bf16 sum, the per-group scales, the per-tensor scale and the codes, bit for bit, and the addition itself against the
    oracle.  Widths take the one-, two- and four-chunk kernels, group sizes from one to eight lanes."""
    rq = _rq()
    from coat_amd.activation.real_quantization import fp8_layernorm_noparam_backward_add
    x = rand(80, shape=(M, N))
    g = rand(81, 0.01, shape=(M, N)).to(dev)
    res = rand(82, 0.02, shape=(M, N))
    res[::5, ::3] *= 30
    res = res.to(dev)
    q, s = rq.fp8_quantize(x.to(dev), QBv, "E4M3")
    _, _, _, (mean, rstd, nw) = rq.fp8_layernorm_noparam_forward(q, s, QBv, 1e-5, transpose_output_2d=True)
    dx = rq.fp8_layernorm_noparam_backward(q, s, g, QBv, mean, rstd, nw)
    want_y, (want_q, want_s, want_pg) = rq.fp8_add_Ifp_Ifp_Ofp_Opt(res, dx, QBv, fp8out)
    got_y, (got_q, got_s, got_pg) = fp8_layernorm_noparam_backward_add(q, s, g, QBv, mean, rstd, nw, res, fp8out)
    assert torch.equal(got_y, want_y), "sum"
    assert torch.equal(got_pg.view(torch.int16), want_pg.view(torch.int16)), "group scales"
    assert got_s.dtype == want_s.dtype and got_s.item() == want_s.item(), "tensor scale"
    assert torch.equal(b(got_q), b(want_q)), "codes"
    oy, (oq, os_, opg) = R.fp8_add_Ifp_Ifp_Ofp_Opt(res.cpu(), dx.cpu(), QBv, fp8out)
    assert torch.equal(got_y.cpu(), oy) and torch.equal(got_pg.cpu(), opg) and os_.item() == got_s.item()
    assert torch.equal(b(got_q), oq.view(torch.uint8))


def test_larger_groups_and_float32_scales(dev):
    rq = _rq()
    x1, x2 = rand(13, shape=(128, 512)), rand(14, shape=(128, 512))
    q1, s1 = R.fp8_quantize(x1, 64, "E4M3", torch.float32)
    q2, s2 = R.fp8_quantize(x2, 64, "E4M3", torch.float32)
    qy, s, qyt = rq.fp8_mul_forward(q1.to(dev), s1.to(dev), q2.to(dev), s2.to(dev), 64)
    wq, ws, wqt = R.fp8_mul_forward(q1, s1, q2, s2, 64)
    assert s.item() == ws.item() and torch.equal(b(qy), b(wq)) and torch.equal(b(qyt), b(wqt))


@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("shape,QBv", [((48, 176), 16), ((256, 4096), 32), ((144, 8192 + 64), 16)])
def test_rmsnorm_division_recomputed_equals_division_of_the_stored_tensor(dev, wdtype, shape, QBv):
    """coat_fp8_rmsnorm_division recomputes y from the norm's inputs: same codes, transpose and scale as dividing the
    bf16 tensor that coat_fp8_rmsnorm_forward stores."""
    from coat_amd import _hip
    M, N = shape
    x = rand(41, 1.0, shape)
    q, s = R.fp8_quantize(x, QBv, "E4M3")
    q, s = q.to(dev), s.to(dev)
    w = (torch.ones(N) + 0.1 * torch.randn(N, generator=torch.Generator().manual_seed(5))).to(wdtype).to(dev)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    s_row = torch.empty((M,), dtype=torch.bfloat16, device=dev)
    rstd = torch.empty((M,), dtype=torch.float32, device=dev)
    s_max = torch.zeros(_hip.MAX_WORDS, dtype=torch.float32, device=dev)  # COAT_MAX_WORDS: the slots of the maximum
    lib, st = _hip.lib(), _hip.stream(q.device)
    _hip.check(lib.coat_fp8_rmsnorm_forward(_hip.ptr(q), 0, _hip.ptr(s), _hip.dt(s), _hip.ptr(w), _hip.dt(w), _hip.ptr(y),
                                            _hip.ptr(s_row), _hip.ptr(rstd), _hip.ptr(s_max), M, N, QBv, 1e-5, st), "fwd")
    # statistics-only call: same rstd, row scales and maximum without the bf16 output
    s_row2, rstd2, s_max2 = torch.empty_like(s_row), torch.empty_like(rstd), torch.zeros_like(s_max)
    _hip.check(lib.coat_fp8_rmsnorm_forward(_hip.ptr(q), 0, _hip.ptr(s), _hip.dt(s), _hip.ptr(w), _hip.dt(w), None,
                                            _hip.ptr(s_row2), _hip.ptr(rstd2), _hip.ptr(s_max2), M, N, QBv, 1e-5, st), "stats")
    assert torch.equal(s_row.view(torch.int16), s_row2.view(torch.int16)) and torch.equal(rstd, rstd2)
    assert torch.equal(s_max, s_max2) and s_max.max().item() > 0
    outs = []
    for fused in (False, True):
        qy, qyt = torch.empty((M, N), dtype=torch.uint8, device=dev), torch.empty((N, M), dtype=torch.uint8, device=dev)
        s_out = torch.zeros((), dtype=torch.bfloat16, device=dev)
        if fused:
            _hip.check(lib.coat_fp8_rmsnorm_division(_hip.ptr(q), 0, _hip.ptr(s), _hip.dt(s), _hip.ptr(w), _hip.dt(w),
                                                     _hip.ptr(rstd), _hip.ptr(s_max), _hip.ptr(s_out), _hip.ptr(qy),
                                                     _hip.ptr(qyt), M, N, QBv, st), "rmsnorm_division")
        else:
            _hip.check(lib.coat_fp8_division_from_max(_hip.ptr(y), _hip.dt(y), _hip.ptr(s_max), _hip.ptr(s_out),
                                                      _hip.dt(s_out), _hip.ptr(qy), _hip.ptr(qyt), M, N, 0, st), "division")
        outs.append((qy, qyt, s_out))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    assert outs[0][2].item() == outs[1][2].item() and outs[0][2].item() > 0
    assert torch.equal(outs[1][1], outs[1][0].t().contiguous())


@pytest.mark.parametrize("fp8", ["E4M3", "E5M2"])
@pytest.mark.parametrize("sliced", [False, True])
def test_product_division_recomputed_equals_division_of_the_stored_product(dev, fp8, sliced):
    """coat_fp8_product_division against coat_fp8_mul_forward's stored bf16 product followed by the division, with the
    second factor dense or a column slice of a wider tensor."""
    from coat_amd import _hip
    M, N = 208, 352
    kind = 0 if fp8 == "E4M3" else 1
    a, sa = R.fp8_quantize(rand(51, 1.0, (M, N)), QB, fp8)
    wide, swide = R.fp8_quantize(rand(52, 1.0, (M, 2 * N)), QB, fp8)
    a, sa, wide, swide = a.to(dev), sa.to(dev), wide.to(dev), swide.to(dev)
    if sliced:
        bq, sb, b_pitch, sb_pitch = wide[:, N:], swide[:, N // QB:], 2 * N, 2 * N // QB
    else:
        bq, sb, b_pitch, sb_pitch = wide[:, N:].contiguous(), swide[:, N // QB:].contiguous(), 0, 0
    bd, sbd = wide[:, N:].contiguous(), swide[:, N // QB:].contiguous()
    lib, st = _hip.lib(), _hip.stream(a.device)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    s_max = torch.zeros(_hip.MAX_WORDS, dtype=torch.float32, device=dev)  # COAT_MAX_WORDS: the slots of the maximum
    _hip.check(lib.coat_fp8_mul_forward(_hip.ptr(a), _hip.ptr(sa), _hip.ptr(bd), _hip.ptr(sbd), kind, _hip.dt(sa),
                                        _hip.ptr(y), None, _hip.ptr(s_max), M, N, QB, st), "mul_forward")
    want_q, want_qt = torch.empty((M, N), dtype=torch.uint8, device=dev), torch.empty((N, M), dtype=torch.uint8, device=dev)
    want_s = torch.zeros((), dtype=torch.bfloat16, device=dev)
    _hip.check(lib.coat_fp8_division_from_max(_hip.ptr(y), _hip.dt(y), _hip.ptr(s_max), _hip.ptr(want_s), _hip.dt(want_s),
                                              _hip.ptr(want_q), _hip.ptr(want_qt), M, N, kind, st), "division")
    got_q, got_qt, got_s = torch.empty_like(want_q), torch.empty_like(want_qt), torch.zeros_like(want_s)
    _hip.check(lib.coat_fp8_product_division(_hip.ptr(a), _hip.ptr(sa), _hip.dt(sa), _hip.ptr(bq), _hip.ptr(sb), _hip.dt(sb),
                                             kind, _hip.ptr(s_max), _hip.ptr(got_s), _hip.ptr(got_q), _hip.ptr(got_qt), M, N,
                                             QB, b_pitch, sb_pitch, st), "product_division")
    assert torch.equal(got_q, want_q) and torch.equal(got_qt, want_qt) and got_s.item() == want_s.item() > 0


@pytest.mark.parametrize("wdtype", [None, torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("shape,QBv", [((48, 176), 16), ((272, 4096), 32)])
def test_layernorm_division_recomputed_equals_division_of_the_stored_tensor(dev, wdtype, shape, QBv):
    """coat_fp8_layernorm_division recomputes the fp32 y from the norm's inputs: same codes, transpose and scale as dividing
    the fp32 tensor that coat_fp8_layernorm_forward stores (with and without affine parameters)."""
    from coat_amd import _hip
    M, N = shape
    q, s = R.fp8_quantize(rand(61, 1.0, shape) + 0.25, QBv, "E4M3")
    q, s = q.to(dev), s.to(dev)
    w = b = None
    if wdtype is not None:
        gen = torch.Generator().manual_seed(7)
        w = (torch.ones(N) + 0.1 * torch.randn(N, generator=gen)).to(wdtype).to(dev)
        b = (0.05 * torch.randn(N, generator=gen)).to(wdtype).to(dev)
    wd = -1 if w is None else _hip.dt(w)
    y = torch.empty((M, N), dtype=torch.float32, device=dev)
    s_row = torch.empty((M,), dtype=torch.bfloat16, device=dev)
    mean, rstd = torch.empty((M,), dtype=torch.float32, device=dev), torch.empty((M,), dtype=torch.float32, device=dev)
    s_max = torch.zeros(_hip.MAX_WORDS, dtype=torch.float32, device=dev)  # COAT_MAX_WORDS: the slots of the maximum
    lib, st = _hip.lib(), _hip.stream(q.device)
    _hip.check(lib.coat_fp8_layernorm_forward(_hip.ptr(q), 0, _hip.ptr(s), _hip.dt(s), _hip.ptr(w), _hip.ptr(b), wd,
                                              _hip.ptr(y), _hip.ptr(s_row), _hip.ptr(mean), _hip.ptr(rstd), _hip.ptr(s_max),
                                              M, N, QBv, 1e-5, st), "fwd")
    mean2, rstd2, s_max2 = torch.empty_like(mean), torch.empty_like(rstd), torch.zeros_like(s_max)
    _hip.check(lib.coat_fp8_layernorm_forward(_hip.ptr(q), 0, _hip.ptr(s), _hip.dt(s), _hip.ptr(w), _hip.ptr(b), wd, None,
                                              _hip.ptr(s_row), _hip.ptr(mean2), _hip.ptr(rstd2), _hip.ptr(s_max2), M, N, QBv,
                                              1e-5, st), "stats")
    assert torch.equal(mean, mean2) and torch.equal(rstd, rstd2) and torch.equal(s_max, s_max2)
    want_q, want_qt = torch.empty((M, N), dtype=torch.uint8, device=dev), torch.empty((N, M), dtype=torch.uint8, device=dev)
    want_s = torch.zeros((), dtype=torch.bfloat16, device=dev)
    _hip.check(lib.coat_fp8_division_from_max(_hip.ptr(y), _hip.dt(y), _hip.ptr(s_max), _hip.ptr(want_s), _hip.dt(want_s),
                                              _hip.ptr(want_q), _hip.ptr(want_qt), M, N, 0, st), "division")
    got_q, got_qt, got_s = torch.empty_like(want_q), torch.empty_like(want_qt), torch.zeros_like(want_s)
    _hip.check(lib.coat_fp8_layernorm_division(_hip.ptr(q), 0, _hip.ptr(s), _hip.dt(s), _hip.ptr(w), _hip.ptr(b), wd,
                                               _hip.ptr(mean), _hip.ptr(rstd), _hip.ptr(s_max), _hip.ptr(got_s),
                                               _hip.ptr(got_q), _hip.ptr(got_qt), M, N, QBv, st), "layernorm_division")
    assert torch.equal(got_q, want_q) and torch.equal(got_qt, want_qt) and got_s.item() == want_s.item() > 0


@pytest.mark.parametrize("fp8", ["E4M3", "E5M2"])
@pytest.mark.parametrize("shape,QBv", [((BS, SL, C), 16), ((48, 352), 32), ((7, 64), 16)])
def test_fused_silu_mul_from_bf16_equals_quantize_then_fused_forward(dev, fp8, shape, QBv):
    """One pass over the bf16 gate / up gives the codes and scales of fp8_quantize and everything fp8_silu_mul_forward
    returns, bit for bit (the last shape has no whole 16 x 16 blocks: it raises like the chain, which needs them for the
    transposed output)."""
    rq = _rq()
    gate, up = rand(71, 1.0, shape).to(dev), rand(72, 1.0, shape).to(dev)
    if shape[-2] % 16 != 0:
        with pytest.raises(ValueError):
            rq.fp8_silu_mul_forward_from_bf16(gate, up, QBv, fp8)
        return
    got = rq.fp8_silu_mul_forward_from_bf16(gate, up, QBv, fp8, transpose_output_2d=True)
    gq, gs = rq.fp8_quantize(gate, QBv, fp8)
    uq, us = rq.fp8_quantize(up, QBv, fp8)
    want = (gq, gs, uq, us) + tuple(rq.fp8_silu_mul_forward(gq, gs, uq, us, QBv, transpose_output_2d=True))
    assert len(got) == len(want) == 9
    for i, (a, w) in enumerate(zip(got, want)):
        assert a.shape == w.shape and a.dtype == w.dtype, i
        assert torch.equal(a.view(torch.uint8) if a.dtype in (E4, E5) else a, w.view(torch.uint8) if w.dtype in (E4, E5) else w), i
