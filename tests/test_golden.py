"""Committed golden fixtures (tests/golden/): hand-written known answers from the OCP FP8 specification, and frozen
outputs of the pinned CPU oracle on small seeded inputs.  CPU tests check the oracle against both; GPU tests check the
HIP path against the committed bytes (bit-exact for codes, scales and the plain AdamW step; the stated tolerances of
tests/test_gpu_adamw.py for the expand step)."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import activation_ref as R
from oracle import adamw_ref as A
from oracle import fp8_codec as C

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
HP = dict(beta1=0.9, beta2=0.95, lr=1e-3, wd=0.1, eps=1e-8)
KEYS_EXP = ["exp_avg", "scale_exp_avg", "expand_exp_avg", "sqrt_minmax_exp_avg",
            "exp_avg_sq", "scale_exp_avg_sq", "expand_exp_avg_sq", "sqrt_minmax_exp_avg_sq"]
KEYS_PLAIN = ["exp_avg", "scale_exp_avg", "exp_avg_sq", "scale_exp_avg_sq"]
FT = {"e4m3": ("E4M3", torch.float8_e4m3fn), "e5m2": ("E5M2", torch.float8_e5m2)}
CE_CASES = {  # name: (ignore_index, lse_square_scale, label_smoothing, reduction, softcap), as tests/golden/make_golden.py
    "plain_mean": (-100, 0.0, 0.0, "mean", None),
    "smooth_z_sum": (-100, 1e-3, 0.1, "sum", None),
    "softcap_mean": (-100, 0.0, 0.0, "mean", 4.0),
}


def known():
    with open(os.path.join(G, "fp8_known_answers.json")) as f:
        return json.load(f)


def bf16_from_bits(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def fp8_from_bytes(a, dt):
    return torch.from_numpy(a.copy()).view(dt)


# ------------------------------------------------------------------------------------------------ CPU: oracle vs fixtures
@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_oracle_codec_known_answers(fmt):
    table = known()[fmt]
    vals = np.array([v for v, _ in table], dtype=np.float32)
    want = np.array([c for _, c in table], dtype=np.uint8)
    assert np.array_equal(C.encode(vals, C.E4M3 if fmt == "e4m3" else C.E5M2), want)
    # the torch-based cast the activation oracle uses gives the same codes
    got = R.cast_fp8(torch.from_numpy(vals), FT[fmt][0]).view(torch.uint8).numpy()
    assert np.array_equal(got, want)
    # decode of every in-range exactly representable entry returns the value
    dec = C.decode(want, C.E4M3 if fmt == "e4m3" else C.E5M2)
    exact = np.abs(vals) <= C.FP8_MAX[C.E4M3 if fmt == "e4m3" else C.E5M2]
    rep = exact & (R.cast_fp8(torch.from_numpy(vals), FT[fmt][0]).float().numpy() == vals)
    assert np.array_equal(dec[rep], vals[rep])


def test_oracle_group_known_answers():
    k = known()
    x = torch.tensor(k["group_e4m3"]["x"]).reshape(1, 16)
    q, s = R.fp8_quantize(x, 16, "E4M3")
    assert s.view(torch.int16).item() & 0xFFFF == k["group_e4m3"]["scale_bf16_bits"]
    assert q.view(torch.uint8).flatten().tolist() == k["group_e4m3"]["codes"]
    q0, s0 = R.fp8_quantize(torch.zeros(1, 16), 16, "E4M3")
    assert s0.view(torch.int16).item() & 0xFFFF == k["group_zero_scale_bf16_bits"] and not q0.view(torch.uint8).any()


def test_oracle_reproduces_quantize_fixture():
    z = np.load(os.path.join(G, "quantize_32x64_bf16.npz"))
    x = bf16_from_bits(z["x_bf16"])
    for name, (ft, dt) in FT.items():
        q, s = R.fp8_quantize(x, 16, ft)
        (_, _), (qt, st) = R.fp8_quantize_transpose(x, 16, ft)
        qp, sp, qpt = R.fp8_quantize_pertensor_transpose(x, 16, ft)
        for got, key in ((q, "q"), (qt, "qt"), (qp, "pt_q"), (qpt, "pt_qt")):
            assert np.array_equal(got.view(torch.uint8).numpy(), z[f"{name}_{key}"]), (name, key)
        for got, key in ((s, "s"), (st, "st"), (sp.reshape(1), "pt_s")):
            assert torch.equal(got, bf16_from_bits(z[f"{name}_{key}"])), (name, key)


@pytest.mark.parametrize("expand", [True, False])
def test_oracle_reproduces_adamw_fixture(expand):
    z = np.load(os.path.join(G, "adamw_expand_1064.npz" if expand else "adamw_plain_1064.npz"))
    keys = KEYS_EXP if expand else KEYS_PLAIN
    p = torch.from_numpy(z["p0"].copy())
    st = A.fresh_state(p, expand)
    for step in (1, 2, 3):
        g = torch.from_numpy(z[f"g{step}"].copy())
        if expand:
            A.adamw_expand_step(p, g, *[st[k] for k in keys], *HP.values(), step, 128, 16)
        else:
            A.adamw_step(p, g, *[st[k] for k in keys], *HP.values(), step, 128)
        assert np.array_equal(p.numpy(), z[f"p{step}"])
        for k in keys:
            got = st[k].view(torch.uint8).numpy() if st[k].dtype == torch.float8_e4m3fn else st[k].numpy()
            assert np.array_equal(got, z[f"{k}{step}"], equal_nan=True), (k, step)


def test_oracle_reproduces_stochastic_fixture():
    from oracle import stochastic_ref as S
    z = np.load(os.path.join(G, "division_stochastic_32x64.npz"))
    x, scale = bf16_from_bits(z["x_bf16"]), bf16_from_bits(z["scale_bf16"]).reshape(())
    for name, (ft, dt) in FT.items():
        q, _, qt = S.fp8_division_transpose_stochastic(x, 16, ft, scale)
        assert np.array_equal(q.view(torch.uint8).numpy(), z[f"{name}_q"])
        assert np.array_equal(qt.view(torch.uint8).numpy(), z[f"{name}_qt"])


def test_oracle_reproduces_cross_entropy_fixture():
    from oracle import cross_entropy_ref as C
    z = np.load(os.path.join(G, "cross_entropy_16x97.npz"))
    x, t = torch.from_numpy(z["x"].copy()), torch.from_numpy(z["target"].copy())
    for name, (ii, lss, ls, red, cap) in CE_CASES.items():
        loss, zl, grad = C.cross_entropy_forward(x, t, ii, lss, ls, red, cap)
        assert abs(loss.item() - float(z[f"{name}_loss"])) <= 1e-12 * abs(float(z[f"{name}_loss"]))
        assert abs(zl.item() - float(z[f"{name}_z"])) <= 1e-12 * max(abs(float(z[f"{name}_z"])), 1e-30)
        assert np.allclose(grad.numpy(), z[f"{name}_grad"], rtol=1e-12, atol=1e-15)


# ------------------------------------------------------------------------------------------------ GPU: HIP path vs fixtures
@pytest.mark.gpu
def test_hip_stochastic_division_matches_fixture(dev):
    import coat_amd.activation.real_quantization as rq
    z = np.load(os.path.join(G, "division_stochastic_32x64.npz"))
    x, scale = bf16_from_bits(z["x_bf16"]).to(dev), bf16_from_bits(z["scale_bf16"]).reshape(()).to(dev)
    for name, (ft, dt) in FT.items():
        q, _, qt = rq.fp8_division_transpose(x, 16, ft, scale, stochastic=True)
        q1, _ = rq.fp8_division(x, 16, ft, scale, stochastic=True)
        for got, key in ((q, "q"), (q1, "q"), (qt, "qt")):
            assert np.array_equal(got.cpu().view(torch.uint8).numpy(), z[f"{name}_{key}"]), (name, key)


@pytest.mark.gpu
def test_hip_cross_entropy_matches_fixture(dev):
    """fp32 logits: loss rtol 2e-6, gradient 2e-6 relative + 3e-7 / divisor (as tests/test_gpu_cross_entropy.py)."""
    from coat_amd.activation.liger.cross_entropy import cross_entropy_forward
    z = np.load(os.path.join(G, "cross_entropy_16x97.npz"))
    t = torch.from_numpy(z["target"].copy())
    for name, (ii, lss, ls, red, cap) in CE_CASES.items():
        x = torch.from_numpy(z["x"].copy()).to(dev)
        loss, zl, grad = cross_entropy_forward(x, t.to(dev), ii, lss, ls, red, cap, True)
        n = float((t != ii).sum()) if red == "mean" else 1.0
        want = torch.from_numpy(z[f"{name}_grad"])
        assert abs(loss.item() - float(z[f"{name}_loss"])) <= 2e-6 * abs(float(z[f"{name}_loss"])), name
        assert abs(zl.item() - float(z[f"{name}_z"])) <= 2e-6 * abs(float(z[f"{name}_z"])) + 1e-12, name
        assert torch.all((grad.double().cpu() - want).abs() <= 2e-6 * want.abs() + 3e-7 / n), name



@pytest.mark.gpu
def test_hip_quantize_matches_fixture(dev):
    import coat_amd.activation.real_quantization as rq
    from coat_amd.activation.real_quantization._quantize_transpose import fp8_quantize_transpose
    z = np.load(os.path.join(G, "quantize_32x64_bf16.npz"))
    x = bf16_from_bits(z["x_bf16"]).to(dev)
    for name, (ft, dt) in FT.items():
        q, s = rq.fp8_quantize(x, 16, ft)
        (q2, s2), (qt, st) = fp8_quantize_transpose(x, 16, ft)
        qp, sp, qpt = rq.fp8_quantize_pertensor_transpose(x, 16, ft)
        for got, key in ((q, "q"), (q2, "q"), (qt, "qt"), (qp, "pt_q"), (qpt, "pt_qt")):
            assert np.array_equal(got.cpu().view(torch.uint8).numpy(), z[f"{name}_{key}"]), (name, key)
        for got, key in ((s, "s"), (s2, "s"), (st, "st"), (sp.reshape(1), "pt_s")):
            assert torch.equal(got.cpu(), bf16_from_bits(z[f"{name}_{key}"])), (name, key)


@pytest.mark.gpu
def test_hip_known_answers(dev):
    import coat_amd.activation.real_quantization as rq
    k = known()
    x = torch.tensor(k["group_e4m3"]["x"]).reshape(1, 16).bfloat16().to(dev)
    q, s = rq.fp8_quantize(x, 16, "E4M3")
    assert s.cpu().view(torch.int16).item() & 0xFFFF == k["group_e4m3"]["scale_bf16_bits"]
    assert q.cpu().view(torch.uint8).flatten().tolist() == k["group_e4m3"]["codes"]
    # single values through the per-tensor division with scale 1: the code of the value itself
    for fmt, (ft, dt) in FT.items():
        vals = torch.tensor([v for v, _ in k[fmt]], dtype=torch.float32)
        want = [c for _, c in k[fmt]]
        pad = (-len(want)) % 16
        xv = torch.nn.functional.pad(vals, (0, pad)).reshape(1, -1).to(dev)
        qd, _ = rq.fp8_division(xv, 16, ft, torch.ones((), dtype=torch.float32, device=dev))
        assert qd.cpu().view(torch.uint8).flatten().tolist()[:len(want)] == want, fmt


@pytest.mark.gpu
def test_hip_adamw_plain_matches_fixture(dev):
    from coat_amd.optimizer import qoptim_cuda as Q
    z = np.load(os.path.join(G, "adamw_plain_1064.npz"))
    p = torch.from_numpy(z["p0"].copy()).to(dev)
    st = {k: v.to(dev) for k, v in A.fresh_state(p.cpu(), False).items()}
    for step in (1, 2, 3):
        g = torch.from_numpy(z[f"g{step}"].copy()).to(dev)
        Q.fp8_adamw_step(p, g, *[st[k] for k in KEYS_PLAIN], *HP.values(), step, 128)
        assert np.array_equal(p.cpu().numpy(), z[f"p{step}"])
        for k in KEYS_PLAIN:
            got = st[k].cpu().view(torch.uint8).numpy() if st[k].dtype == torch.float8_e4m3fn else st[k].cpu().numpy()
            assert np.array_equal(got, z[f"{k}{step}"]), (k, step)


@pytest.mark.gpu
def test_hip_adamw_expand_matches_fixture(dev):
    """Each step starts from the fixture's state of the step before (so errors do not compound) and is held to the
    tolerances stated in tests/test_gpu_adamw.py."""
    from coat_amd.optimizer import qoptim_cuda as Q
    from test_gpu_adamw import compare_expand
    z = np.load(os.path.join(G, "adamw_expand_1064.npz"))
    n = z["p0"].size

    def state_at(step):
        p = torch.from_numpy(z[f"p{step}"].copy())
        if step == 0:
            return p, A.fresh_state(p, True)
        st = {k: (fp8_from_bytes(z[f"{k}{step}"], torch.float8_e4m3fn) if k in ("exp_avg", "exp_avg_sq")
                  else torch.from_numpy(z[f"{k}{step}"].copy())) for k in KEYS_EXP}
        return p, st

    for step in (1, 2, 3):
        p, st = state_at(step - 1)
        pd, std = p.to(dev), {k: v.to(dev) for k, v in st.items()}
        g = torch.from_numpy(z[f"g{step}"].copy()).to(dev)
        Q.fp8_adamw_expand_step(pd, g, *[std[k] for k in KEYS_EXP], *HP.values(), step, 128, 16)
        want_p, want_st = state_at(step)
        compare_expand(pd, std, want_p, want_st, n, tag=f"step {step}")
