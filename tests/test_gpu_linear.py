"""GPU parity: FP8 GEMM (MFMA) against the CPU oracle.

Stated tolerance (bf16 output): |C - C_ref| <= 2^-7 |C_ref| + 2^-14 * sum_k |a||b| * scale, i.e. one bf16 rounding plus
the accumulation error of the FP8 MFMA (measured: <= 2^-17.4 of sum |a||b| for K >= 128, unbiased; the products of one
instruction are aligned to their largest exponent before they are added, so short sums are relatively worse; C_ref from a float64 matmul of
the decoded operands).  Quantize epilogue: codes are
compared where the fp32 accumulators can be expected to agree: mismatch < 1e-2 of the elements, one code step."""
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


def check_bf16(c, a, b_rows, sa, sb, bias=None):
    ref = (a.double() @ b_rows.double().t()) * (sa.double() * sb.double())
    bound = (a.double().abs() @ b_rows.double().abs().t()) * (sa.double() * sb.double()) * 2.0 ** -14
    if bias is not None:
        ref = ref + bias.double()
    err = (c.cpu().double() - ref).abs()
    assert (err <= ref.abs() * 2.0 ** -7 + bound + 1e-30).all(), (err / (ref.abs() + 1e-9)).max().item()


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


@pytest.mark.parametrize("M,N,K", [(256, 512, 256), (384, 272, 128)])
def test_fp8matmul_quantized_output(dev, M, N, K):
    lin = _lin()
    a, b = rand_fp8((M, K), 6, E4), rand_fp8((N, K), 7, E4)
    sa, sb = torch.tensor(0.02).bfloat16(), torch.tensor(0.02).bfloat16()
    cq, cs = lin.fp8matmul(a.to(dev), b.to(dev).t(), True, sa.to(dev), sb.to(dev), 16)
    wq, ws = R.fp8matmul(a, b.t(), True, sa, sb, 16, accumulate=torch.float64)
    assert cq.dtype == E4 and cs.shape == (M, N // 16) and cs.dtype == torch.bfloat16
    g, w = cq.cpu().view(torch.uint8).int(), wq.view(torch.uint8).int()
    neq = g != w
    assert neq.float().mean().item() < 1e-2
    # where the codes differ, the dequantized values differ by one code step of that magnitude or by the accumulation bound
    dg = R.fp8_dequantize(cq.cpu(), cs.cpu(), 16).double()
    dw = R.fp8_dequantize(wq, ws, 16).double()
    mag = (a.double().abs() @ b.double().abs().t()) * (sa.double() * sb.double())
    assert ((dg - dw).abs() <= dw.abs() * 2.0 ** -3 + mag * 2.0 ** -13 + 1e-12).all()
    sg, sw = cs.cpu().view(torch.int16).int(), ws.view(torch.int16).int()
    assert ((sg - sw).abs() <= 1).all() and (sg != sw).float().mean().item() < 1e-2
    # the dequantized product is the product
    deq = R.fp8_dequantize(cq.cpu(), cs.cpu(), 16).double()
    ref = (a.double() @ b.double().t()) * (sa.double() * sb.double())
    gmax = ref.reshape(M, N // 16, 16).abs().amax(dim=2).repeat_interleave(16, dim=1)
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
