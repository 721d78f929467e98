"""GPU parity: FP8 GEMM (MFMA) against the CPU oracle.

Stated tolerance (bf16 output): |C - C_ref| <= 2^-8 max(|C|, |C_ref|) + 2^-14 * sum_k |a||b| * scale, i.e. one bf16
rounding plus the accumulation error of the FP8 MFMA (C_ref from a float64 matmul of the decoded operands).  Measured
accumulation term: 2^-16.5 .. 2^-18.5 of sum |a||b| for e4m3 x e4m3, up to 2^-15.1 with an e5m2 operand (the products of one
instruction are aligned to their largest exponent before they are added, and e5m2 values spread over more binades); the
bar is about three times the worst measured.  Quantize epilogue: compared with quantizing the float64 product; codes differ
on < 4e-3 of the elements (measured 1.1e-3), scales on < 5e-3 (measured 1.6e-3), by one step."""
import pytest
import torch

from oracle import activation_ref as R

pytestmark = pytest.mark.gpu
E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


def _lin():
    from coat_amd.activation.real_quantization import linear
    return linear


def rand_fp8(shape, seed, dtype, scale=1.0):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


GEMM_K = 2.0 ** -14


def check_bf16(c, a, b_rows, sa, sb, bias=None):
    import math
    s = sa.double() * sb.double()
    ref = (a.double() @ b_rows.double().t()) * s
    mag = (a.double().abs() @ b_rows.double().abs().t()) * s
    if bias is not None:
        ref = ref + bias.double()
    c64 = c.cpu().double()
    err = (c64 - ref).abs()
    rounding = torch.maximum(ref.abs(), c64.abs()) * 2.0 ** -8  # half a bf16 ulp of the binade the result lands in
    k = ((err - rounding).clamp_min(0) / mag.clamp_min(1e-300)).max().item()
    print(f"[measured] GEMM {tuple(a.shape)} x {tuple(b_rows.shape)} {a.dtype} {b_rows.dtype}: accumulation term "
          f"2^{math.log2(k) if k > 0 else float('-inf'):.1f} of sum|a||b| (bar 2^-14)")
    assert (err <= rounding + mag * GEMM_K + 1e-30).all(), k


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (512, 768, 512), (300, 200, 272), (64, 48, 16), (1024, 256, 4096)])
@pytest.mark.parametrize("fa,fb", [(E4, E4), (E5, E4), (E4, E5)])
def test_fp8matmul_bf16(dev, M, N, K, fa, fb):
    lin = _lin()
    a, b = rand_fp8((M, K), 1, fa), rand_fp8((N, K), 2, fb)
    sa, sb = torch.tensor(0.02).bfloat16(), torch.tensor(0.013).bfloat16()
    c = lin.fp8matmul(a.to(dev), b.to(dev).t(), False, sa.to(dev), sb.to(dev), 16)
    assert c.dtype == torch.bfloat16 and c.shape == (M, N)
    check_bf16(c, a, b, sa, sb)


@pytest.mark.parametrize("M,N,K,fa", [(4352, 4112, 400, E4), (5000, 4608, 144, E5)])
def test_fp8matmul_more_tiles_than_cus(dev, M, N, K, fa):
    """More 256 x 256 tiles than the chip has CUs: every block walks several tiles with its LDS ring running across the
    tile boundary; ragged last tile row / column and a partial last K-step included."""
    lin = _lin()
    a, b = rand_fp8((M, K), 11, fa), rand_fp8((N, K), 12, E4)
    sa, sb = torch.tensor(0.03).bfloat16(), torch.tensor(0.011).bfloat16()
    bias = torch.randn(N, generator=torch.Generator().manual_seed(13)).bfloat16()
    c = lin.fp8matmul(a.to(dev), b.to(dev).t(), False, sa.to(dev), sb.to(dev), 16, bias.to(dev))
    check_bf16(c, a, b, sa, sb, bias)
    # same operands through the quantizing epilogue: dequantized output within one e4m3 step of the bf16 result
    cq, cs = lin.fp8matmul(a.to(dev), b.to(dev).t(), True, sa.to(dev), sb.to(dev), 16, bias.to(dev))
    deq = cq.cpu().float().reshape(M, N // 16, 16) * cs.cpu().float().unsqueeze(-1)
    gmax = c.cpu().float().reshape(M, N // 16, 16).abs().amax(dim=2, keepdim=True)
    assert ((deq - c.cpu().float().reshape(M, N // 16, 16)).abs() <= gmax * 2.0 ** -3 + 1e-6).all()


def test_fp8matmul_bias_batched_and_rowmajor_b(dev):
    lin = _lin()
    a, b = rand_fp8((4 * 96, 256), 3, E4).reshape(4, 96, 256), rand_fp8((160, 256), 4, E4)
    sa, sb = torch.tensor(0.5).bfloat16(), torch.tensor(0.25).bfloat16()
    bias = torch.randn(160, generator=torch.Generator().manual_seed(5)).bfloat16()
    c = lin.fp8matmul(a.to(dev), b.to(dev).t(), False, sa.to(dev), sb.to(dev), 16, bias.to(dev))
    assert c.shape == (4, 96, 160)
    check_bf16(c.reshape(-1, 160), a.reshape(-1, 256), b, sa, sb, bias)
    # a right operand that is genuinely row-major [K, N]
    bkn = b.view(torch.uint8).t().contiguous().view(E4)
    c2 = lin.fp8matmul(a.to(dev), bkn.to(dev), False, sa.to(dev), sb.to(dev), 16, bias.to(dev))
    assert torch.equal(c2, c)


@pytest.mark.parametrize("M,N,K,QB", [(256, 512, 256, 16), (384, 272, 128, 16), (256, 512, 256, 32), (300, 448, 144, 64),
                                      (384, 288, 128, 32), (4352, 4160, 80, 64)])
def test_fp8matmul_quantized_output(dev, M, N, K, QB):
    """Quantizing epilogue, groups of 16 (every shipped configuration), 32 and 64 columns (the reference's epilogue is
    generic in the group size, linear.py:139-164); ragged last tile row / column, bias in the last case."""
    lin = _lin()
    a, b = rand_fp8((M, K), 6, E4), rand_fp8((N, K), 7, E4)
    sa, sb = torch.tensor(0.02).bfloat16(), torch.tensor(0.02).bfloat16()
    bias = torch.randn(N, generator=torch.Generator().manual_seed(8)).bfloat16() if M > 4000 else None
    cq, cs = lin.fp8matmul(a.to(dev), b.to(dev).t(), True, sa.to(dev), sb.to(dev), QB, None if bias is None else bias.to(dev))
    wq, ws = R.fp8matmul(a, b.t(), True, sa, sb, QB, bias, accumulate=torch.float64)
    assert cq.dtype == E4 and cs.shape == (M, N // QB) and cs.dtype == torch.bfloat16
    g, w = cq.cpu().view(torch.uint8).int(), wq.view(torch.uint8).int()
    neq = g != w
    print(f"[measured] quantizing epilogue {M}x{N}x{K}: {neq.float().mean().item():.3e} of the codes differ (bar 4e-3)")
    assert neq.float().mean().item() < 4e-3
    # where the codes differ, the dequantized values differ by one code step of that magnitude or by the accumulation bound
    dg = R.fp8_dequantize(cq.cpu(), cs.cpu(), QB).double()
    dw = R.fp8_dequantize(wq, ws, QB).double()
    mag = (a.double().abs() @ b.double().abs().t()) * (sa.double() * sb.double())
    if bias is not None:
        mag = mag + bias.double().abs()
    step0 = ws.double().repeat_interleave(QB, dim=1) * 2.0 ** -9  # one step of the subnormal codes of the group
    assert ((dg - dw).abs() <= dw.abs() * 2.0 ** -3 + step0 + mag * 2.0 ** -13 + 1e-12).all()
    sg, sw = cs.cpu().view(torch.int16).int(), ws.view(torch.int16).int()
    print(f"[measured] quantizing epilogue {M}x{N}x{K}: {(sg != sw).float().mean().item():.3e} of the scales differ (bar 5e-3)")
    assert ((sg - sw).abs() <= 1).all() and (sg != sw).float().mean().item() < 5e-3
    # the dequantized product is the product
    deq = R.fp8_dequantize(cq.cpu(), cs.cpu(), QB).double()
    ref = (a.double() @ b.double().t()) * (sa.double() * sb.double())
    if bias is not None:
        ref = ref + bias.double()
    gmax = ref.reshape(M, N // QB, QB).abs().amax(dim=2).repeat_interleave(QB, dim=1)
    assert ((deq - ref).abs() <= gmax * 2.0 ** -4 * 1.05 + 1e-9).all()


def test_linear_forward_backward_and_module(dev):
    """FP8Linear against the oracle's three GEMMs on the same quantized operands (reference test shape scaled down:
    tests/test_fp8_linear.py:151-179), and against the bf16 F.linear within FP8 quantization noise."""
    from coat_amd.activation.real_quantization.fp8linear import FP8Linear
    lin = _lin()
    torch.manual_seed(0)
    B, S, K, N = 2, 256, 512, 768
    x = (torch.randn(B, S, K) * 0.5).bfloat16()
    layer = FP8Linear(K, N, bias=True, device=dev).to(torch.bfloat16)
    layer.train()
    xd = x.to(dev).requires_grad_(True)
    y = layer(xd)
    gy = (torch.randn(B, S, N, generator=torch.Generator().manual_seed(1)) * 0.01).bfloat16()
    y.backward(gy.to(dev))
    # oracle on the CPU
    w, bias = layer.weight.detach().cpu(), layer.bias.detach().cpu()
    qx, sx, qxt = R.fp8_quantize_pertensor_transpose(x.reshape(-1, K), 16, "E4M3")
    qw, sw, qwt = R.fp8_quantize_pertensor_transpose(w, 16, "E4M3")
    check_bf16(y.detach().reshape(-1, N), qx.float(), qw.float(), sx, sw, bias)
    qg, sg, qgt = R.fp8_quantize_pertensor_transpose(gy.reshape(-1, N), 16, "E5M2")
    check_bf16(xd.grad.reshape(-1, K), qg.float(), qwt.float(), sg, sw)
    check_bf16(layer.weight.grad, qgt.float(), qxt.float(), sg, sx)
    assert torch.allclose(layer.bias.grad.cpu().float(), gy.reshape(-1, N).float().sum(0), rtol=2e-2, atol=1e-3)
    # sanity against bf16 linear: relative Frobenius error at the FP8 noise level
    ref = torch.nn.functional.linear(x.float(), w.float(), bias.float())
    rel = (y.detach().cpu().float() - ref).norm() / ref.norm()
    assert rel < 0.06
    layer.eval()
    assert torch.allclose(layer(xd).detach().cpu().float(), ref, rtol=2e-2, atol=2e-2)


def test_fp8matmul_scales_in_different_dtypes(dev):
    """A bf16 activation scale next to an fp32 weight scale (fp32 master weights): each is read in its own dtype and the
    two are multiplied in fp32 (reference linear.py:123-125).  Small integer operands make the accumulation exact, so the
    output must equal bf16(acc * (float(sa) * float(sb))) bit for bit; rounding the fp32 scale to bf16 first would move
    most outputs."""
    lin = _lin()
    g = torch.Generator().manual_seed(9)
    M, N, K = 256, 256, 64
    a = torch.randint(-4, 5, (M, K), generator=g).float().to(E4)
    b = torch.randint(-4, 5, (N, K), generator=g).float().to(E4)
    sa = torch.tensor(0.0234375).bfloat16()            # exactly representable
    base = torch.tensor(0.013).bfloat16().float()
    sb = (base * (1 + 0.97 * 2.0 ** -9)).float()         # just below the midpoint of two bf16 values: rounds back to base
    assert sb.bfloat16().float().item() == base.item() != sb.item()
    acc = a.float() @ b.float().t()                    # |acc| <= 1024: exact in fp32
    want = (acc * (sa.float() * sb)).bfloat16()
    c = lin.fp8matmul(a.to(dev), b.to(dev).t(), False, sa.to(dev), sb.to(dev), 16)
    assert torch.equal(c.cpu(), want)
    wrong = (acc * (sa.float() * sb.bfloat16().float())).bfloat16()
    assert (wrong != want).float().mean().item() > 0.05  # the test would see a bf16-rounded weight scale
    # and the other way round (fp32 first, bf16 second), with the quantizing epilogue
    cq, cs = lin.fp8matmul(a.to(dev), b.to(dev).t(), True, sb.to(dev), sa.to(dev), 16)
    wq, ws = R._quantize_pg(acc * (sb * sa.float()), 16, E4)
    assert torch.equal(cq.cpu().view(torch.uint8), wq.view(torch.uint8)) and torch.equal(cs.cpu(), ws)


@pytest.mark.parametrize("count,M,N,K,fa,fb,quant,qb,with_bias", [
    (3, 512, 512, 256, E4, E4, False, 16, (0, 0, 0)),      # q / k / v forward: 12 tiles, problems change inside a block's walk
    (2, 300, 272, 144, E5, E4, False, 16, (0, 0)),         # ragged tiles, partial last K-step, e5m2 gradients
    (2, 768, 512, 384, E4, E4, True, 16, (0, 0)),          # gate / up forward through the quantizing epilogue
    (4, 2304, 2048, 128, E5, E4, False, 16, (0, 0, 0, 0)), # 4 x 72 tiles: more tiles than CUs, every XCD band spans problems
    (3, 200, 208, 80, E4, E5, True, 16, (0, 0, 0)),        # ragged tiles through the quantizing epilogue (scales stored one by one)
    (3, 300, 272, 144, E4, E4, False, 16, (1, 0, 1)),      # a bias vector in the first and third problem only
    (2, 520, 320, 208, E5, E4, True, 32, (0, 1)),          # e5m2 codes in groups of 32 columns, ragged tiles, one bias
    (3, 264, 448, 96, E4, E4, True, 64, (0, 0, 0)),        # groups of 64 columns
])
def test_grouped_gemm_equals_separate_launches(dev, count, M, N, K, fa, fb, quant, qb, with_bias):
    """coat_fp8_gemm_grouped through the C ABI: every problem's output is bit-identical to coat_fp8_gemm on it, with
    per-problem bias pointers (NULL for some) and with the 16-, 32- and 64-column quantizing epilogues."""
    from coat_amd import _hip
    lib = _hip.lib()
    a = [rand_fp8((M, K), 100 + i, fa).to(dev) for i in range(count)]
    b = [rand_fp8((N, K), 200 + i, fb).to(dev) for i in range(count)]
    sa = [torch.tensor(0.02 + 0.003 * i).bfloat16().to(dev) for i in range(count)]
    sb = [torch.tensor(0.013 - 0.002 * i).float().to(dev) for i in range(count)]
    bias = [torch.randn(N, generator=torch.Generator().manual_seed(300 + i)).bfloat16().to(dev) if with_bias[i] else None
            for i in range(count)]
    any_bias = any(with_bias)
    kind = {E4: 1, E5: 2}[fa] if quant else 0
    odt = fa if quant else torch.bfloat16
    want = [torch.empty((M, N), dtype=odt, device=dev) for _ in range(count)]
    got = [torch.zeros((M, N), dtype=torch.uint8, device=dev).view(odt) if quant else torch.zeros((M, N), dtype=odt, device=dev)
           for _ in range(count)]
    want_s = [torch.empty((M, N // qb), dtype=torch.bfloat16, device=dev) for _ in range(count)] if quant else None
    got_s = [torch.zeros((M, N // qb), dtype=torch.bfloat16, device=dev) for _ in range(count)] if quant else None
    st = _hip.stream(dev)
    for i in range(count):
        _hip.check(lib.coat_fp8_gemm(_hip.ptr(a[i]), _hip.fp8(fa), _hip.ptr(b[i]), _hip.fp8(fb), _hip.ptr(want[i]),
                                     _hip.ptr(want_s[i]) if quant else None, kind, _hip.ptr(sa[i]), _hip.dt(sa[i]),
                                     _hip.ptr(sb[i]), _hip.dt(sb[i]), _hip.ptr(bias[i]), _hip.BF16 if bias[i] is not None else 0,
                                     M, N, K, qb if quant else 0, st), "gemm")
    _hip.check(lib.coat_fp8_gemm_grouped(count, _hip.ptr_array(a), _hip.fp8(fa), _hip.ptr_array(b), _hip.fp8(fb),
                                         _hip.ptr_array(got), _hip.ptr_array(got_s) if quant else None, kind,
                                         _hip.ptr_array(sa), _hip.dt(sa[0]), _hip.ptr_array(sb), _hip.dt(sb[0]),
                                         _hip.ptr_array(bias) if any_bias else None, _hip.BF16 if any_bias else 0,
                                         M, N, K, qb if quant else 0, st), "gemm_grouped")
    for i in range(count):
        assert torch.equal(got[i].view(torch.uint8), want[i].view(torch.uint8)), i
        if quant:
            assert torch.equal(got_s[i].view(torch.int16), want_s[i].view(torch.int16)), i
    # the first problem against the oracle's bound as well
    if not quant:
        check_bf16(got[0], a[0].cpu(), b[0].cpu(), sa[0].cpu(), sb[0].cpu(), bias[0].cpu() if bias[0] is not None else None)


@pytest.mark.parametrize("M,N,K,fa,fb,out,with_bias", [
    (512, 512, 256, E4, E4, "E4M3", False),     # whole tiles, packed scale stores
    (300, 272, 144, E4, E4, "E4M3", True),      # ragged tile rows / columns, partial last K-step, scales stored one by one
    (1100, 1040, 272, E5, E4, "E5M2", False),   # more tiles than one round of a small grid, e5m2 operand and e5m2 codes
    (512, 520, 128, E4, E5, None, False),       # bf16 sum only, rows of N % 16 == 8
    (4352, 2064, 400, E5, E4, None, True),      # more tiles than CUs (the ring runs across tile boundaries)
    (2304, 2048, 128, E4, E4, "E4M3", False),   # 72 whole tiles
])
def test_gemm_with_residual_equals_gemm_then_add(dev, M, N, K, fa, fb, out, with_bias):
    """coat_fp8_gemm_residual against the two kernels it replaces: the bf16 product of coat_fp8_gemm, then the residual
    addition (fp8_add_Ifp_Ifp_Ofp_Og16, or torch's bf16 addition when no FP8 copy is asked for).  Bit-identical sums,
    codes and scales; also with the residual tensor as the output (accumulation in place)."""
    from coat_amd.activation.real_quantization.add_fwd import fp8_add_Ifp_Ifp_Ofp_Og16
    lin = _lin()
    a, b = rand_fp8((M, K), 61, fa).to(dev), rand_fp8((N, K), 62, fb).to(dev)
    sa, sb = torch.tensor(0.021).bfloat16().to(dev), torch.tensor(0.0127).float().to(dev)
    res = (torch.randn(M, N, generator=torch.Generator().manual_seed(63)) * 1.5).bfloat16().to(dev)
    res[::7, ::5] *= 40
    bias = torch.randn(N, generator=torch.Generator().manual_seed(64)).bfloat16().to(dev) if with_bias else None
    prod = lin.fp8matmul(a, b.t(), False, sa, sb, 16, bias)
    if out is None:
        want = prod + res
        got = lin.fp8matmul_add(a, b.t(), res, sa, sb, None, 16, bias)
        assert got.dtype == torch.bfloat16 and torch.equal(got, want)
        # in place through the C ABI: the residual is the output
        from coat_amd import _hip
        acc = res.clone()
        _hip.check(_hip.lib().coat_fp8_gemm_residual(
            _hip.ptr(a), _hip.fp8(fa), _hip.ptr(b), _hip.fp8(fb), _hip.ptr(acc), _hip.ptr(acc), None, None, 0, _hip.ptr(sa),
            _hip.dt(sa), _hip.ptr(sb), _hip.dt(sb), _hip.ptr(bias), _hip.dt(bias) if with_bias else 0, M, N, K,
            _hip.stream(dev)), "gemm_residual in place")
        assert torch.equal(acc, want)
        return
    want_y, (want_q, want_s) = fp8_add_Ifp_Ifp_Ofp_Og16(res, prod, out, 16)
    got_y, (got_q, got_s) = lin.fp8matmul_add(a, b.t(), res, sa, sb, out, 16, bias)
    assert torch.equal(got_y, want_y), "bf16 sum"
    assert got_q.dtype == want_q.dtype and torch.equal(got_q.view(torch.uint8), want_q.view(torch.uint8)), "codes of the sum"
    assert torch.equal(got_s.view(torch.int16), want_s.view(torch.int16)), "group scales of the sum"
    # and the oracle on the same product (the addition itself is bit-exact against the CPU restatement)
    oy, (oq, os_) = R.fp8_add_Ifp_Ifp_Ofp_Og16(res.cpu(), prod.cpu(), out, 16)
    assert torch.equal(got_y.cpu(), oy) and torch.equal(got_q.cpu().view(torch.uint8), oq.view(torch.uint8))
    assert torch.equal(got_s.cpu(), os_)


def test_grouped_linear_wrappers_equal_the_separate_calls(dev):
    """fp8_linear_forward_grouped / fp8_linear_backward_grouped against the per-projection functions, with a bias vector in
    one problem of the C call (bias is per problem) and with projections of different widths (falls back to separate calls)."""
    from coat_amd import _hip
    lin = _lin()
    T, H = 384, 256
    x, xt = rand_fp8((T, H), 1, E4).to(dev), rand_fp8((H, T), 2, E4).to(dev)
    s = torch.tensor(0.031).bfloat16().to(dev)
    ws = [rand_fp8((H, H), 10 + i, E4).to(dev) for i in range(3)]
    wts = [rand_fp8((H, H), 20 + i, E4).to(dev) for i in range(3)]
    sws = [torch.tensor(0.01 * (i + 1)).bfloat16().to(dev) for i in range(3)]
    gs8 = [rand_fp8((T, H), 30 + i, E5).to(dev) for i in range(3)]
    gts = [rand_fp8((H, T), 40 + i, E5).to(dev) for i in range(3)]
    sgs = [torch.tensor(0.002 * (i + 1)).bfloat16().to(dev) for i in range(3)]
    outs = lin.fp8_linear_forward_grouped(x, s, ws, sws, False, 16)
    for o, w, sw in zip(outs, ws, sws):
        assert torch.equal(o, lin.fp8_linear_forward(x, s, w, sw, False, 16))
    outs = lin.fp8_linear_forward_grouped(x, s, ws[:2], sws[:2], True, 16)
    for (q, qs), w, sw in zip(outs, ws, sws):
        wq, wqs = lin.fp8_linear_forward(x, s, w, sw, True, 16)
        assert torch.equal(q.view(torch.uint8), wq.view(torch.uint8)) and torch.equal(qs, wqs)
    dxs, dws = lin.fp8_linear_backward_grouped(xt, s, gs8, sgs, gts, wts, sws, 16)
    for i in range(3):
        dx, dw = lin.fp8_linear_backward(xt, s, gs8[i], sgs[i], gts[i], wts[i], sws[i], 16)
        assert torch.equal(dxs[i], dx) and torch.equal(dws[i], dw)
    # grouped-query shapes: k / v narrower than q -> q in a launch of its own, k and v together; same results, same order
    wk, wv = rand_fp8((H // 4, H), 50, E4).to(dev), rand_fp8((H // 4, H), 51, E4).to(dev)
    outs = lin.fp8_linear_forward_grouped(x, s, [ws[0], wk, wv], sws, False, 16)
    assert outs[0].shape == (T, H) and outs[1].shape == outs[2].shape == (T, H // 4)
    for o, w, sw in zip(outs, (ws[0], wk, wv), sws):
        assert torch.equal(o, lin.fp8_linear_forward(x, s, w, sw, False, 16))
    # bias in the second problem only
    lib = _hip.lib()
    bias = torch.randn(H, generator=torch.Generator().manual_seed(7)).bfloat16().to(dev)
    got = [torch.zeros((T, H), dtype=torch.bfloat16, device=dev) for _ in range(2)]
    _hip.check(lib.coat_fp8_gemm_grouped(2, _hip.ptr_array([x, x]), 0, _hip.ptr_array(ws[:2]), 0, _hip.ptr_array(got), None, 0,
                                         _hip.ptr_array([s, s]), _hip.dt(s), _hip.ptr_array(sws[:2]), _hip.dt(sws[0]),
                                         _hip.ptr_array([None, bias]), _hip.dt(bias), T, H, H, 0, _hip.stream(dev)), "grouped")
    assert torch.equal(got[0], lin.fp8matmul(x, ws[0].t(), False, s, sws[0], 16))
    assert torch.equal(got[1], lin.fp8matmul(x, ws[1].t(), False, s, sws[1], 16, bias))
