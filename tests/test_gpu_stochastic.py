"""GPU parity: stochastic-rounding division (the reference's coat/activation/real_quantization/_division.py:96-150
branch) against the CPU oracle, bit for bit: same Philox stream, same perturbation, same FP8 codes."""
import pytest
import torch

from oracle import activation_ref as R
from oracle import stochastic_ref as S
from test_gpu_quantize import eq_bytes, make_x

pytestmark = pytest.mark.gpu


def _rq():
    import coat_amd.activation.real_quantization as rq
    return rq


def tiny_x(dtype):
    """Quotients across zero, both subnormal regimes of the perturbation and the saturating end."""
    x = make_x(32, 64, 5, torch.float32, outliers=False)
    x[0] = 0.0
    x[1] = -0.0
    x[2] = torch.exp2(torch.linspace(-20, 8, 64))
    x[3] = -torch.exp2(torch.linspace(-20, 8, 64))
    x[4] = 1e-30
    x[5] = 440.0 + torch.arange(64) * 0.25
    return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("fp8", ["E4M3", "E5M2"])
def test_division_stochastic_bit_exact(dev, dtype, fp8):
    rq = _rq()
    for x, s in ((make_x(96, 256, 1, dtype), None), (tiny_x(dtype), torch.tensor(1.0, dtype=torch.bfloat16)),
                 (make_x(7, 19, 2, dtype), None)):  # 133 elements: ragged tail of the flat kernel
        sd = None if s is None else s.to(dev)
        q, s_out = rq.fp8_division(x.to(dev), 16, fp8, sd, stochastic=True)
        wq, ws = S.fp8_division_stochastic(x, 16, fp8, s)
        assert torch.equal(s_out.cpu().float(), ws.float())
        assert eq_bytes(q, wq)
        # and it is not the deterministic result
        qd, _ = R.fp8_division(x, 16, fp8, ws)
        if x.numel() > 1000:
            assert not eq_bytes(q, qd)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("fp8", ["E4M3", "E5M2"])
def test_division_transpose_stochastic_bit_exact(dev, dtype, fp8):
    rq = _rq()
    x = make_x(80, 208, 3, dtype)
    q, s, qt = rq.fp8_division_transpose(x.to(dev), 16, fp8, stochastic=True)
    wq, ws, wqt = S.fp8_division_transpose_stochastic(x, 16, fp8)
    assert torch.equal(s.cpu().float(), ws.float())
    assert eq_bytes(q, wq) and eq_bytes(qt, wqt)
    qt2, _ = rq.fp8_division_transpose(x.to(dev), 16, fp8, s, stochastic=True, only_transposed=True)
    assert eq_bytes(qt2, wqt)


def test_callers_pass_the_flag_to_the_division(dev):
    rq = _rq()
    x = make_x(64, 128, 4)
    q, s, s_pg = rq.fp8_quantize_pertensor(x.to(dev), 16, "E4M3", stochastic=True)
    wq, _ = S.fp8_division_stochastic(x, 16, "E4M3", s.cpu())
    assert eq_bytes(q, wq)
    q, s, qt = rq.fp8_quantize_pertensor_transpose(x.to(dev), 16, "E5M2", stochastic=True)
    wq, _, wqt = S.fp8_division_transpose_stochastic(x, 16, "E5M2", s.cpu())
    assert eq_bytes(q, wq) and eq_bytes(qt, wqt)
    x2 = make_x(64, 128, 6)
    y, (q2, s2, _) = rq.fp8_add_Ifp_Ifp_Ofp_Opt(x.to(dev), x2.to(dev), 16, "E4M3", stochastic=True)
    wq2, _ = S.fp8_division_stochastic(y.cpu(), 16, "E4M3", s2.cpu())
    assert eq_bytes(q2, wq2)
    # 3-D input: the noise index is the flat index of the [B*S, C] view
    x3 = make_x(64, 128, 4).reshape(4, 16, 128)
    q3, _ = rq.fp8_division(x3.to(dev), 16, "E4M3", s.to(dev), stochastic=True)
    w3, _ = S.fp8_division_stochastic(x3.reshape(64, 128), 16, "E4M3", s.cpu())
    assert q3.shape == x3.shape and eq_bytes(q3.reshape(64, 128), w3)


def test_stochastic_mean_is_nearer_than_deterministic_bias_bound(dev):
    """The branch adds U[0,1) steps and then rounds to nearest: on average the result sits half a step above the
    input (the reference's behaviour, reproduced).  Checked on a constant between two codes."""
    rq = _rq()
    x = torch.full((256, 256), 1.0625, dtype=torch.float32)  # E4M3 step at 1.0 is 0.125: codes 1.0 and 1.125
    q, _ = rq.fp8_division(x.to(dev), 16, "E4M3", torch.tensor(1.0, device=dev), stochastic=True)
    v = q.float().cpu()
    assert set(v.unique().tolist()) <= {1.0, 1.125, 1.25}
    # x + u*0.125 with u in [0,1): rounds to 1.0 only for u < 0 (never, ties to even at u = 0 -> 1.0), so the mean
    # is about 1.0625 + 0.0625
    assert abs(float(v.mean()) - 1.125) < 0.01


def test_unsupported_combinations_say_why(dev):
    rq = _rq()
    a = torch.zeros(16, 16, dtype=torch.float8_e4m3fn, device=dev)
    one = torch.ones((), dtype=torch.bfloat16, device=dev)
    with pytest.raises(NotImplementedError, match="boundary_check"):
        rq.linear.fp8matmul(a, a.t(), False, one, one, 16, stochastic=True)
