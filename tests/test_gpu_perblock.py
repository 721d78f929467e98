"""GPU parity: the per-block (QB x QB) quantizers against the CPU oracle, codes and scales bit for bit.
Reference: coat/activation/real_quantization/_quantize_perblock.py, _quantize_perblock_transpose.py,
_quantize_perblock_transpose_pergroup.py; the reference's own test is tests/test_fp8_quantize.py:42-48."""
import pytest
import torch

from oracle import activation_ref as R
from test_gpu_quantize import eq_bytes, make_x, special_x

pytestmark = pytest.mark.gpu


def _fns():
    from coat_amd.activation.real_quantization import fp8_quantize_perblock
    from coat_amd.activation.real_quantization._quantize_perblock_transpose import fp8_quantize_perblock_transpose
    from coat_amd.activation.real_quantization._quantize_perblock_transpose_pergroup import \
        fp8_quantize_perblock_transpose_pergroup
    return fp8_quantize_perblock, fp8_quantize_perblock_transpose, fp8_quantize_perblock_transpose_pergroup


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("fp8,QB,M,N,sdt", [("E4M3", 128, 384, 640, torch.float32), ("E4M3", 128, 128, 128, torch.bfloat16),
                                            ("E5M2", 128, 256, 384, torch.float32), ("E4M3", 16, 48, 208, torch.bfloat16),
                                            ("E4M3", 32, 160, 96, torch.float16), ("E5M2", 64, 192, 320, torch.float32),
                                            ("E4M3", 16, 16, 16, torch.float32)])
def test_perblock_family_bit_exact(dev, dtype, fp8, QB, M, N, sdt):
    pb, pbt, pbtg = _fns()
    x = make_x(M, N, 21, dtype)
    if M >= 32 and N >= 128:
        x[:32, :128] = special_x(dtype)
    (wq, ws), (wqt, wst), (wqg, wsg) = R.fp8_quantize_perblock_transpose_pergroup(x, QB, fp8, scale_dtype=sdt)
    xd = x.to(dev)
    q, s = pb(xd, QB, fp8, scale_dtype=sdt)
    assert q.shape == (M, N) and s.shape == (M // QB, N // QB) and s.dtype == sdt and q.dtype == wq.dtype
    assert torch.equal(s.cpu(), ws), "block scales differ"
    assert eq_bytes(q, wq), "block codes differ"
    (q2, s2), (qt, st) = pbt(xd, QB, fp8, scale_dtype=sdt)
    assert eq_bytes(q2, wq) and torch.equal(s2.cpu(), ws)
    assert qt.shape == (N, M) and st.shape == (N // QB, M // QB)
    assert eq_bytes(qt, wqt) and torch.equal(st.cpu(), wst)
    qt1, st1 = pbt(xd, QB, fp8, scale_dtype=sdt, only_transposed=True)
    assert eq_bytes(qt1, wqt) and torch.equal(st1.cpu(), wst)
    (q3, s3), (qt3, st3), (qg, sg) = pbtg(xd, QB, fp8, scale_dtype=sdt)
    assert eq_bytes(q3, wq) and torch.equal(s3.cpu(), ws) and eq_bytes(qt3, wqt) and torch.equal(st3.cpu(), wst)
    assert qg.shape == (M, N) and sg.shape == (M, N // QB)
    assert eq_bytes(qg, wqg) and torch.equal(sg.cpu(), wsg), "per-group part differs"
    (q4, s4), (qt4, st4), (qg4, sg4) = pbtg(xd, QB, fp8, scale_dtype=sdt, only_transposed=True)
    assert q4.shape == (M, N) and s4.shape == (M // QB, N // QB)  # returned uninitialised, as the reference does
    assert eq_bytes(qt4, wqt) and torch.equal(st4.cpu(), wst) and eq_bytes(qg4, wqg) and torch.equal(sg4.cpu(), wsg)


def test_perblock_reference_test_case(dev):
    """tests/test_fp8_quantize.py:42-48: fp32 [4 * 256, 2048], QB 16, e4m3; at least 95 % of the codes and of the scales equal
    those of the test's own torch definition (tests/test_utils.py:53-60, :98-119).  Against the oracle: all of them."""
    pb, _, _ = _fns()
    x = torch.randn(4 * 256, 2048, generator=torch.Generator().manual_seed(0))
    q, s = pb(x.to(dev), 16, torch.float8_e4m3fn)
    tq, ts = R.quantize_tensor_ref_test_perblock(x, 16, "E4M3")
    eq_q = (q.cpu().view(torch.uint8) == tq.view(torch.uint8)).float().mean().item()
    eq_s = (s.cpu() == ts).float().mean().item()
    print(f"equal to the reference test's definition: codes {eq_q:.4f}, scales {eq_s:.4f}")
    assert eq_q >= 0.95 and eq_s >= 0.95
    wq, ws = R.fp8_quantize_perblock(x, 16, "E4M3")
    assert eq_bytes(q, wq) and torch.equal(s.cpu(), ws)


def test_perblock_3d_input_and_errors(dev):
    pb, pbt, _ = _fns()
    x = make_x(2 * 128, 256, 22).reshape(2, 128, 256)
    q, s = pb(x.to(dev), 128, "E4M3", scale_dtype=torch.float32)
    wq, ws = R.fp8_quantize_perblock(x.reshape(-1, 256), 128, "E4M3", scale_dtype=torch.float32)
    assert q.shape == (256, 256) and s.shape == (2, 2)  # "Do not recover to 3D" (rq/_quantize_perblock.py:148)
    assert eq_bytes(q, wq) and torch.equal(s.cpu(), ws)
    with pytest.raises(AssertionError):
        pb(torch.zeros(100, 128, dtype=torch.bfloat16, device=dev), 128, "E4M3")  # M % QB != 0
    with pytest.raises(ValueError):
        pbt(torch.zeros(96, 96, dtype=torch.bfloat16, device=dev), 48, "E4M3")    # QB outside 16 / 32 / 64 / 128


def test_perblock_weight_shape_llama(dev):
    """The DeepSeek-style linear quantizes its weight per 128 x 128 block with fp32 scales
    (coat/activation/deepseek/fp8linear.py:77); [11008, 4096] compared on block rows 0, 40 and 85."""
    pb, _, _ = _fns()
    w = (torch.randn(11008, 4096, generator=torch.Generator().manual_seed(3)) * 0.02).bfloat16()
    q, s = pb(w.to(dev), 128, "E4M3", scale_dtype=torch.float32)
    for b in (0, 40, 85):
        wq, ws = R.fp8_quantize_perblock(w[b * 128:(b + 1) * 128], 128, "E4M3", scale_dtype=torch.float32)
        assert eq_bytes(q[b * 128:(b + 1) * 128], wq) and torch.equal(s[b:b + 1].cpu(), ws)
