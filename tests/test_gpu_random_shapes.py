"""GPU parity on seeded random shapes: ragged tile edges of the quantize / transpose kernels against the CPU oracle,
bit for bit.  Shapes are small multiples of the group size, chosen so that every kernel meets partial tiles in both
directions (tiles are 64 x 128 and 128 x 128)."""
import random

import pytest
import torch

from oracle import activation_ref as R
from test_gpu_quantize import eq_bytes, make_x

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float32, torch.float16]


def _rq():
    import coat_amd.activation.real_quantization as rq
    from coat_amd.activation.real_quantization._quantize_transpose import fp8_quantize_transpose
    rq.fp8_quantize_transpose = fp8_quantize_transpose
    return rq


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_bit_exact(dev, seed):
    rq = _rq()
    rnd = random.Random(1000 + seed)
    QB = rnd.choice([16, 16, 16, 32, 64, 128])
    M = QB * rnd.randint(1, max(1, 400 // QB))
    N = QB * rnd.randint(1, max(1, 400 // QB))
    dtype = rnd.choice(DTYPES)
    fp8 = rnd.choice(["E4M3", "E5M2"])
    x = make_x(M, N, seed, dtype, scale=rnd.choice([1e-3, 1.0, 30.0]))
    xd = x.to(dev)
    what = (seed, M, N, QB, dtype, fp8)

    q, s = rq.fp8_quantize(xd, QB, fp8)
    wq, ws = R.fp8_quantize(x, QB, fp8)
    assert eq_bytes(q, wq) and torch.equal(s.cpu(), ws), what

    (q2, s2), (qt, st) = rq.fp8_quantize_transpose(xd, QB, fp8)
    (_, _), (wqt, wst) = R.fp8_quantize_transpose(x, QB, fp8)
    assert eq_bytes(q2, wq) and torch.equal(s2.cpu(), ws) and eq_bytes(qt, wqt) and torch.equal(st.cpu(), wst), what

    qp, sp, qpt = rq.fp8_quantize_pertensor_transpose(xd, QB, fp8)
    wqp, wsp, wqpt = R.fp8_quantize_pertensor_transpose(x, QB, fp8)
    assert sp.item() == wsp.item() and eq_bytes(qp, wqp) and eq_bytes(qpt, wqpt), what

    only_t, _ = rq.fp8_division_transpose(xd, QB, fp8, sp, only_transposed=True)
    assert eq_bytes(only_t, wqpt), what

    t = rq.fp8_transpose(qp)
    assert eq_bytes(t, wqpt), what

    d = rq.fp8_dequantize(q, s, QB)
    wd = R.fp8_dequantize(wq, ws, QB)
    assert torch.equal(d.cpu(), wd), what


@pytest.mark.parametrize("seed", range(8))
def test_random_grouped_gemm_equals_separate_launches(dev, seed):
    """Seeded random problem counts, shapes (ragged tiles, partial K-steps), operand formats and epilogues: every problem
    of a grouped launch is bit-identical to its own launch."""
    from coat_amd.activation.real_quantization import linear
    rnd = random.Random(7000 + seed)
    count = rnd.choice([2, 3, 4])
    M = rnd.choice([16, 48, 256, 272, 520, 1040])
    N = 16 * rnd.randint(1, 70)
    K = 16 * rnd.randint(1, 40)
    fa = rnd.choice([torch.float8_e4m3fn, torch.float8_e5m2])
    fb = rnd.choice([torch.float8_e4m3fn, torch.float8_e5m2])
    quant = rnd.random() < 0.4
    g = torch.Generator().manual_seed(seed)
    a = [torch.randn(M, K, generator=g).to(fa).to(dev) for _ in range(count)]
    b = [torch.randn(N, K, generator=g).to(fb).to(dev) for _ in range(count)]
    sa = [torch.tensor(rnd.uniform(1e-3, 1e-1)).bfloat16().to(dev) for _ in range(count)]
    sb = [torch.tensor(rnd.uniform(1e-3, 1e-1)).bfloat16().to(dev) for _ in range(count)]
    got = linear.fp8matmul_grouped(a, [x.t() for x in b], quant, sa, sb, 16)
    what = (seed, count, M, N, K, fa, fb, quant)
    for i in range(count):
        want = linear.fp8matmul(a[i], b[i].t(), quant, sa[i], sb[i], 16)
        if quant:
            assert torch.equal(got[i][0].view(torch.uint8), want[0].view(torch.uint8)), what
            assert torch.equal(got[i][1], want[1]), what
        else:
            assert torch.equal(got[i], want), what
