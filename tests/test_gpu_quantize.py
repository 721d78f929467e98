"""GPU parity: HIP quantize family (through the Python entry points, i.e. the C ABI) against the CPU oracle.
FP8 codes and scales are compared bit for bit."""
import pytest
import torch

from oracle import activation_ref as R

pytestmark = pytest.mark.gpu

E4, E5 = torch.float8_e4m3fn, torch.float8_e5m2


def _rq():
    import coat_amd.activation.real_quantization as rq
    from coat_amd.activation.real_quantization._quantize_transpose import fp8_quantize_transpose
    rq.fp8_quantize_transpose = fp8_quantize_transpose
    return rq


def make_x(M, N, seed=0, dtype=torch.bfloat16, outliers=True, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, N, generator=g) * scale
    if outliers:
        x[torch.rand(M, N, generator=g) < 0.001] *= 100
    return x.to(dtype)


def special_x(dtype=torch.bfloat16):
    """Rows that exercise zeros, negative zero, denormals, huge values, exact ties and all-equal groups."""
    x = make_x(32, 128, 99, torch.float32)
    x[0] = 0.0
    x[1] = -0.0
    x[2, :16] = 1e-38
    x[2, 16:32] = -1e-40
    x[3] = 3.0e38
    x[3, 5] = -1.0
    x[4] = 448.0
    x[5] = torch.arange(128).float() * 28.0
    x[6, ::2] = -0.0
    x[7] = 1e-12
    x[8, :16] = torch.tensor([i * 0.0625 for i in range(16)])
    if dtype == torch.float16:
        x = x.clamp(-6.0e4, 6.0e4)  # non-finite inputs are outside the contract
    return x.to(dtype)


def eq_bytes(a, b):
    return torch.equal(a.cpu().view(torch.uint8), b.cpu().view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("fp8,QB", [("E4M3", 16), ("E5M2", 16), ("E4M3", 32), ("E4M3", 64), ("E5M2", 128)])
def test_fp8_quantize_bit_exact(dev, dtype, fp8, QB):
    rq = _rq()
    for x in (make_x(96, 256, 1, dtype), special_x(dtype), make_x(3, 128, 2, dtype, scale=1e-3)):
        q, s = rq.fp8_quantize(x.to(dev), QB, fp8)
        wq, ws = R.fp8_quantize(x, QB, fp8)
        assert q.dtype == wq.dtype and s.dtype == torch.bfloat16 and s.shape == ws.shape
        assert torch.equal(s.cpu(), ws), "scales differ"
        assert eq_bytes(q, wq), "codes differ"


def test_fp8_quantize_3d_and_scale_dtype(dev):
    rq = _rq()
    x = make_x(4 * 24, 64, 3).reshape(4, 24, 64)
    q, s = rq.fp8_quantize(x.to(dev), 16, torch.float8_e4m3fn, scale_dtype=torch.float32)
    wq, ws = R.fp8_quantize(x.reshape(-1, 64), 16, "E4M3", torch.float32)
    assert q.shape == (4, 24, 64) and s.shape == (4, 24, 4) and s.dtype == torch.float32
    assert eq_bytes(q.reshape(-1, 64), wq) and torch.equal(s.cpu().reshape(-1, 4), ws)
    e = rq.fp8_quantize(torch.empty(0, 64, dtype=torch.bfloat16, device=dev), 16, "E4M3")
    assert e[0].shape == (0, 64) and e[1].shape == (0, 4)
    with pytest.raises(ValueError):
        rq.fp8_quantize(torch.zeros(4, 40, dtype=torch.bfloat16, device=dev), 16, "E4M3")  # N % QB != 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("fp8,QB,M,N", [("E4M3", 16, 128, 192), ("E5M2", 16, 64, 64), ("E4M3", 32, 96, 160),
                                        ("E4M3", 64, 128, 128), ("E4M3", 16, 16, 16), ("E4M3", 16, 208, 80),
                                        ("E4M3", 128, 384, 640), ("E5M2", 128, 128, 128)])
def test_fp8_quantize_transpose_bit_exact(dev, dtype, fp8, QB, M, N):
    rq = _rq()
    x = make_x(M, N, 4, dtype)
    if M >= 32 and N >= 128:
        x[:32, :128] = special_x(dtype)
    (q, s), (qt, st) = rq.fp8_quantize_transpose(x.to(dev), QB, fp8)
    (wq, ws), (wqt, wst) = R.fp8_quantize_transpose(x, QB, fp8)
    if QB == 128:  # the reference's own test calls it with fp32 scales (tests/test_fp8_quantize.py:57)
        (q32, s32), (qt32, st32) = rq.fp8_quantize_transpose(x.to(dev), QB, fp8, scale_dtype=torch.float32)
        (_, ws32), (_, wst32) = R.fp8_quantize_transpose(x, QB, fp8, scale_dtype=torch.float32)
        assert torch.equal(s32.cpu(), ws32) and torch.equal(st32.cpu(), wst32) and eq_bytes(q32, q) and eq_bytes(qt32, qt)
    assert qt.shape == (N, M) and st.shape == (N, M // QB)
    assert torch.equal(s.cpu(), ws) and eq_bytes(q, wq)
    assert torch.equal(st.cpu(), wst) and eq_bytes(qt, wqt)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("fp8", ["E4M3", "E5M2"])
def test_pertensor_and_division_bit_exact(dev, dtype, fp8):
    rq = _rq()
    x = make_x(80, 176, 5, dtype)
    xd = x.to(dev)
    q, s, spg = rq.fp8_quantize_pertensor(xd, 16, fp8)
    wq, ws, wspg = R.fp8_quantize_pertensor(x, 16, fp8)
    assert s.dtype == torch.bfloat16 and s.numel() == 1 and s.item() == ws.item()
    assert torch.equal(spg.cpu(), wspg) and eq_bytes(q, wq)
    q2, s2, qt = rq.fp8_quantize_pertensor_transpose(xd, 16, fp8)
    assert s2.item() == ws.item() and eq_bytes(q2, wq) and eq_bytes(qt, wq.view(torch.uint8).t().contiguous())
    # scale from abs-max in the input dtype
    q3, s3 = rq.fp8_division(xd, 16, fp8)
    wq3, ws3 = R.fp8_division(x, 16, fp8)
    assert s3.dtype == x.dtype and s3.item() == ws3.item() and eq_bytes(q3, wq3)
    # given scale that is too small: saturation to the largest finite code, no NaN
    small = (ws.float() / 8).to(torch.bfloat16)
    q4, _ = rq.fp8_division(xd, 16, fp8, small.to(dev))
    wq4, _ = R.fp8_division(x, 16, fp8, small)
    assert eq_bytes(q4, wq4) and q4.float().isfinite().all()
    # transposed only, and a CPU-resident scale
    qt5, s5 = rq.fp8_division_transpose(xd, 16, fp8, ws, only_transposed=True)
    assert eq_bytes(qt5, wq.view(torch.uint8).t().contiguous())
    # special values
    sx = special_x(dtype)
    sx[3] = 1.0  # keep the tensor maximum moderate so that the small rows are not all flushed
    q6, s6, qt6 = rq.fp8_quantize_pertensor_transpose(sx.to(dev), 16, fp8)
    wq6, ws6, wqt6 = R.fp8_quantize_pertensor_transpose(sx, 16, fp8)
    assert s6.item() == ws6.item() and eq_bytes(q6, wq6) and eq_bytes(qt6, wqt6)


def test_division_ragged_and_3d(dev):
    rq = _rq()
    x = make_x(7, 37, 6, torch.float32)  # no divisibility needed without the transpose
    s = torch.tensor(0.01, dtype=torch.bfloat16)
    q, _ = rq.fp8_division(x.to(dev), 16, "E4M3", s.to(dev))
    wq, _ = R.fp8_division(x, 16, "E4M3", s)
    assert eq_bytes(q, wq)
    x3 = make_x(2 * 32, 48, 7).reshape(2, 32, 48)
    q3, s3, qt3 = rq.fp8_quantize_pertensor_transpose(x3.to(dev), 16, "E4M3")
    assert q3.shape == (2, 32, 48) and qt3.shape == (2, 24, 64)  # reference reshape (BS, -1, last) of the [48, 64] transpose
    q3b, _, qt3b = rq.fp8_quantize_pertensor_transpose(x3.to(dev), 16, "E4M3", transpose_output_2d=True)
    assert qt3b.shape == (48, 64) and eq_bytes(qt3b, q3b.reshape(64, 48).view(torch.uint8).t().contiguous())


@pytest.mark.parametrize("M,N", [(64, 64), (16, 16), (208, 80), (4096, 1024)])
def test_fp8_transpose(dev, M, N):
    rq = _rq()
    x = torch.randint(0, 256, (M, N), dtype=torch.uint8, generator=torch.Generator().manual_seed(8)).view(E4)
    y = rq.fp8_transpose(x.to(dev))
    assert y.shape == (N, M) and eq_bytes(y, R.fp8_transpose(x))


@pytest.mark.parametrize("fp8,QB", [("E4M3", 16), ("E5M2", 16), ("E4M3", 64)])
def test_fp8_dequantize(dev, fp8, QB):
    rq = _rq()
    x = make_x(48, 128, 9)
    wq, ws = R.fp8_quantize(x, QB, fp8)
    y = rq.fp8_dequantize(wq.to(dev), ws.to(dev), QB)
    assert y.dtype == torch.bfloat16 and torch.equal(y.cpu(), R.fp8_dequantize(wq, ws, QB))


def test_config1_size_properties(dev):
    """The bf16 [4096, 4096] quantize configuration at full size: invariants that need no CPU pass over 16M elements per check."""
    rq = _rq()
    g = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn(4096, 4096, generator=g)
    x[torch.rand(4096, 4096, generator=g) < 0.001] *= 100
    x = x.bfloat16()
    xd = x.to(dev)
    (q, s), (qt, st) = rq.fp8_quantize_transpose(xd, 16, "E4M3")
    q1, s1 = rq.fp8_quantize(xd, 16, "E4M3")
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(s, s1)
    qT, sT = rq.fp8_quantize(xd.t().contiguous(), 16, "E4M3")
    assert torch.equal(qt.view(torch.uint8), qT.view(torch.uint8)) and torch.equal(st, sT)
    # every group's maximum lands on +-448 and dequantization is within half an e4m3 step of the group max
    codes = q1.view(torch.uint8).reshape(4096, 256, 16) & 0x7F
    assert (codes.amax(dim=2) == 0x7E).all()
    deq = rq.fp8_dequantize(q1, s1, 16).float()
    amax = xd.float().reshape(4096, 256, 16).abs().amax(dim=2, keepdim=True)
    err = (deq.reshape(4096, 256, 16) - xd.float().reshape(4096, 256, 16)).abs()
    assert (err <= amax * (2.0 ** -4 + 2.0 ** -7) + 1e-12).all()  # fp8 half step + bf16 rounding of scale and output
    # full-size parity on a slab of rows against the oracle
    wq, ws = R.fp8_quantize(x[:256], 16, "E4M3")
    assert eq_bytes(q1[:256], wq) and torch.equal(s1[:256].cpu(), ws)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_default_division_scale_is_the_device_expression(dev, dtype):
    """(absmax + 1e-10) / fp8max as torch evaluates it on the device (a multiplication by the fp32 reciprocal)."""
    rq = _rq()
    for seed in range(12):
        x = make_x(16, 64, 100 + seed, dtype, scale=0.37 * (seed + 1))
        for fp8 in ("E4M3", "E5M2"):
            _, s = rq.fp8_division(x.to(dev), 16, fp8)
            ws = R.absmax_scale(x, fp8)
            assert s.dtype == dtype and torch.equal(s.cpu().view(torch.int16 if dtype != torch.float32 else torch.int32),
                                                    ws.view(torch.int16 if dtype != torch.float32 else torch.int32))


@pytest.mark.parametrize("sdtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(64, 128), (7, 37)])
def test_division_from_fp32_max_equals_division_by_rounded_scale(dev, sdtype, shape):
    """coat_fp8_division_from_max takes the largest of the maximum's slots (COAT_MAX_WORDS fp32, one slot per 128-byte line),
    rounds it to the scale dtype, divides by that value and stores it."""
    from coat_amd import _hip
    M, N = shape
    x = make_x(M, N, 11, torch.bfloat16).to(dev)
    for m in (0.0123456789, 3.1e-7, 1.0):
        s_max = torch.zeros(_hip.MAX_WORDS, dtype=torch.float32, device=dev)
        s_max[::_hip.MAX_SLOT_STRIDE] = torch.linspace(0.1, 1.0, _hip.MAX_SLOTS, device=dev).roll(5) * m  # largest in slot 4
        s_max[1::_hip.MAX_SLOT_STRIDE] = 7.0  # words between the slots are not part of the maximum
        want_s = torch.tensor(m, dtype=torch.float32, device=dev).to(sdtype)
        tr = M % 16 == 0 and N % 16 == 0
        q, qt = torch.empty((M, N), dtype=torch.uint8, device=dev), torch.empty((N, M), dtype=torch.uint8, device=dev)
        wq, wqt = torch.empty_like(q), torch.empty_like(qt)
        s_out = torch.zeros((), dtype=sdtype, device=dev)
        _hip.check(_hip.lib().coat_fp8_division_from_max(
            _hip.ptr(x), _hip.dt(x), _hip.ptr(s_max), _hip.ptr(s_out), _hip.dt(s_out), _hip.ptr(q),
            _hip.ptr(qt) if tr else None, M, N, 0, _hip.stream(x.device)), "from_max")
        _hip.check(_hip.lib().coat_fp8_division(
            _hip.ptr(x), _hip.dt(x), _hip.ptr(want_s), _hip.dt(want_s), _hip.ptr(wq), _hip.ptr(wqt) if tr else None,
            M, N, 0, _hip.stream(x.device)), "division")
        assert s_out.item() == want_s.item() and torch.equal(q, wq) and (not tr or torch.equal(qt, wqt))
