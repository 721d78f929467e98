"""GPU parity: the fused FP8 AdamW kernels (through the qoptim_cuda shim / C ABI) against oracle/adamw_ref.c."""
import pytest
import torch

from oracle import adamw_ref as A

pytestmark = pytest.mark.gpu

HP = dict(beta1=0.9, beta2=0.95, lr=3e-4, wd=0.1, eps=1e-8)
KEYS_PLAIN = ("exp_avg", "scale_exp_avg", "exp_avg_sq", "scale_exp_avg_sq")
KEYS_EXP = ("exp_avg", "scale_exp_avg", "expand_exp_avg", "sqrt_minmax_exp_avg",
            "exp_avg_sq", "scale_exp_avg_sq", "expand_exp_avg_sq", "sqrt_minmax_exp_avg_sq")


def _q():
    from coat_amd.optimizer import qoptim_cuda
    return qoptim_cuda


def gpu_step(q, p, g, st, step, expand, hp=HP, expand_min=16):
    if expand:
        q.fp8_adamw_expand_step(p, g, *[st[k] for k in KEYS_EXP], hp["beta1"], hp["beta2"], hp["lr"], hp["wd"],
                                hp["eps"], step, 128, expand_min)
    else:
        q.fp8_adamw_step(p, g, *[st[k] for k in KEYS_PLAIN], hp["beta1"], hp["beta2"], hp["lr"], hp["wd"], hp["eps"],
                         step, 128)


def cpu_step(p, g, st, step, expand, hp=HP, expand_min=16):
    if expand:
        A.adamw_expand_step(p, g, *[st[k] for k in KEYS_EXP], hp["beta1"], hp["beta2"], hp["lr"], hp["wd"], hp["eps"],
                            step, 128, expand_min)
    else:
        A.adamw_step(p, g, *[st[k] for k in KEYS_PLAIN], hp["beta1"], hp["beta2"], hp["lr"], hp["wd"], hp["eps"], step, 128)


def to_dev(st, dev):
    return {k: v.to(dev) for k, v in st.items()}


def grads(n, seed, scale=1e-3):
    return torch.randn(n, generator=torch.Generator().manual_seed(seed)) * scale


@pytest.mark.parametrize("n", [128 * 64, 128 * 9 + 37, 127, 1, 1024 * 3 + 5])
@pytest.mark.parametrize("pdtype", [torch.float32, torch.bfloat16])
def test_plain_step_bit_exact(dev, n, pdtype):
    """No transcendental functions on this path: params, codes and scales must match bit for bit over 3 steps."""
    q = _q()
    p = (torch.randn(n, generator=torch.Generator().manual_seed(0)) * 0.02).to(pdtype)
    st = A.fresh_state(p, expand=False)
    pd, std = p.to(dev), to_dev(st, dev)
    for step in (1, 2, 3):
        g = grads(n, step).to(pdtype)
        cpu_step(p, g, st, step, False)
        gpu_step(q, pd, g.to(dev), std, step, False)
        assert torch.equal(pd.cpu(), p), f"params differ at step {step}"
        for k in KEYS_PLAIN:
            assert torch.equal(std[k].cpu().view(torch.uint8) if std[k].dtype != torch.float32 else std[k].cpu(),
                               st[k].view(torch.uint8) if st[k].dtype != torch.float32 else st[k]), (k, step)


# Smallest fraction of groups whose centre agrees to 1e-5 (tensors of 64 groups or more).  Second moments are sums of
# positive terms: all of them.  A first moment's group minimum is often what is left of beta1*m + (1-beta1)*g after a
# cancellation, and carries the 1e-6 of the dequantized m as a 1e-4 of itself: measured 0.85.
WELL_MIN = {"exp_avg": 0.80, "exp_avg_sq": 0.99}
# Groups whose minimum comes out of such a cancellation: (scale rtol, code mismatch rate, fraction with another k)
# (measured on [11008, 4096] slabs over ten steps: scale 2.1e-3 beyond k times the centre's own difference, codes
# 0 .. 5.4e-5, another exponent on at most 1 of 420 groups)
ILL_BARS = (1e-2, 2e-4, 1e-2)


def compare_expand(pd, std, p, st, n, tag="", p_rtol=2e-6, p_atol=1e-9):
    """Stated tolerances for the expand step (hardware log2/exp2, ~1e-6 relative, against correctly rounded powf).

    params: fp32 rtol 2e-6 (atol 1e-9); bf16 within one bf16 ulp.
    The group minimum Mn is often the result of a cancellation beta1*m + (1-beta1)*g ~ 0, so its absolute error
    is ~1e-6 of the group maximum Mx, not of Mn: the centre c = sqrt(Mx*Mn) is therefore bounded through
    |c^2 - c_ref^2| / c_ref^2 <= 4e-5 * Mx/Mn for every group.  Groups whose c agrees to 1e-5 ("well conditioned":
    every group of a second moment, 85 % of a first moment's; bars WELL_MIN) must have the same exponent k, every one
    of them; the new scale within 6e-6 beyond what the centre's own difference explains (s = (Mx/c)^k / 448, so k times
    it; measured 2.1e-6); codes different on at most 5e-5 of their elements (measured 0 .. 2.6e-5; a tensor too small for
    a rate may have two such elements).  The other groups are held to ILL_BARS.  No code may differ by more than one
    step.  Every measured value is printed (pytest -rP); all bars are checked before the test fails."""
    if p.dtype == torch.float32:
        assert torch.allclose(pd.cpu(), p, rtol=p_rtol, atol=p_atol), tag + " params"
    else:
        assert torch.allclose(pd.cpu().float(), p.float(), rtol=2.0 ** -7, atol=1e-30), tag + " params (bf16 ulp)"
    failures = []
    for name in ("exp_avg", "exp_avg_sq"):
        c_g, c_c = std["sqrt_minmax_" + name].cpu().double(), st["sqrt_minmax_" + name].double()
        k_g, k_c = std["expand_" + name].cpu(), st["expand_" + name]
        s_g, s_c = std["scale_" + name].cpu().double(), st["scale_" + name].double()
        finite_k = (k_c > 0) & torch.isfinite(k_c)
        ratio = torch.where(finite_k, (448 * s_c).pow(2 / k_c.double().clamp_min(1e-3)), torch.ones_like(s_c))
        rel_c2 = (c_g * c_g - c_c * c_c).abs() / (c_c * c_c)
        assert (rel_c2 <= 4e-5 * ratio + 1e-6).all(), (tag, name, "centre", (rel_c2 / ratio).max().item())
        well = ((c_g - c_c).abs() <= 1e-5 * c_c) & finite_k
        ng = k_c.numel()
        well_frac = well.float().mean().item()
        if ng >= 64 and well_frac < WELL_MIN[name]:
            failures.append((tag, name, "well", well_frac))
        pad = ng * 128 - n
        codes_g = torch.nn.functional.pad(std[name].cpu().view(torch.uint8).flatten(), (0, pad)).reshape(ng, 128)
        codes_c = torch.nn.functional.pad(st[name].view(torch.uint8).flatten(), (0, pad)).reshape(ng, 128)
        for cls, groups, s_rtol, code_rate, k_rate in (("well", well, 6e-6, 5e-5, 0.0), ("cancelling", finite_k & ~well, *ILL_BARS)):
            if not groups.any():
                continue
            same = (k_g == k_c) & groups
            k_bad = (groups & ~same).sum().item()
            # s = (Mx / c)^k / 448: a centre that differs by d moves the scale by k * d; what is left is the log2 / exp2 error
            rel_c = (c_g[same] - c_c[same]).abs() / c_c[same]
            s_rel = (s_g[same] - s_c[same]).abs() / s_c[same].abs()
            s_err = (s_rel - k_c[same].double() * rel_c).clamp_min(0).max().item() if same.any() else 0.0
            cg, cc = codes_g[same], codes_c[same]
            neq = cg != cc
            rate = neq.sum().item() / max(1, neq.numel())
            print(f"expand {tag} {name} [{cls}: {groups.sum().item()} of {ng} groups]: k mismatches {k_bad}, "
                  f"scale err beyond k * centre err {s_err:.2e} (raw {s_rel.max().item() if same.any() else 0.0:.2e}), "
                  f"codes {neq.sum().item()} / {neq.numel()} = {rate:.2e}")
            if k_bad > int(k_rate * groups.sum().item() + (1 if k_rate else 0)):
                failures.append((tag, name, cls, "k", k_bad))
            if s_err > s_rtol:
                failures.append((tag, name, cls, "scale", s_err))
            if neq.sum().item() > max(2, int(code_rate * neq.numel())):
                failures.append((tag, name, cls, "codes", neq.sum().item(), neq.numel()))
            if neq.any():  # one code step: neighbouring magnitudes with the same sign (or +0 / -0 against the smallest code)
                a, b = cg[neq].int(), cc[neq].int()
                assert ((a & 0x7F) - (b & 0x7F)).abs().max().item() <= 1, (tag, name, cls, "code step")
                assert (((a & 0x80) == (b & 0x80)) | (((a & 0x7F) + (b & 0x7F)) <= 1)).all(), (tag, name, cls, "code sign")
    assert not failures, failures


@pytest.mark.parametrize("n", [128 * 512, 128 * 9 + 37, 127, 1])
@pytest.mark.parametrize("pdtype", [torch.float32, torch.bfloat16])
def test_expand_step_from_identical_state(dev, n, pdtype):
    q = _q()
    p = (torch.randn(n, generator=torch.Generator().manual_seed(0)) * 0.02).to(pdtype)
    st = A.fresh_state(p, expand=True)
    pd, std = p.to(dev), to_dev(st, dev)
    # A single-element tensor is degenerate for Dynamic Range Expansion (max == min, k = inf): from its second
    # step on the reference algorithm itself stores scale = inf and NaN codes, and what follows depends on the
    # sign bit of a NaN.  Only the steps before that are compared for n == 1.
    for step in ((1, 2) if n == 1 else (1, 2, 3, 4)):
        g = grads(n, step).to(pdtype)
        # each step starts from the oracle's state so that differences do not compound
        pd, std = p.to(dev), to_dev(st, dev)
        cpu_step(p, g, st, step, True)
        gpu_step(q, pd, g.to(dev), std, step, True)
        compare_expand(pd, std, p, st, n, f"step {step}")
    if n >= 128:
        # step 1 from the fresh state has no dequantization error: centre and exponent must be exact
        p1 = (torch.randn(n, generator=torch.Generator().manual_seed(0)) * 0.02).to(pdtype)
        s1 = A.fresh_state(p1, True)
        pd1, sd1 = p1.to(dev), to_dev(s1, dev)
        g = grads(n, 1).to(pdtype)
        cpu_step(p1, g, s1, 1, True)
        gpu_step(q, pd1, g.to(dev), sd1, 1, True)
        assert torch.equal(sd1["sqrt_minmax_exp_avg"].cpu(), s1["sqrt_minmax_exp_avg"])
        assert torch.equal(sd1["sqrt_minmax_exp_avg_sq"].cpu(), s1["sqrt_minmax_exp_avg_sq"])
        assert torch.allclose(pd1.cpu().float(), p1.float(), rtol=2e-6 if pdtype == torch.float32 else 2.0 ** -7, atol=1e-9)


def test_expand_reference_test_case(dev):
    """The reference test's configuration: M 2, N 128, step 1000, lr 0.4 (tests/test_fp8_adamw_expand.py:43-51)."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from test_oracle_adamw import _random_expand_state
    q = _q()
    hp = dict(beta1=0.9, beta2=0.95, lr=0.4, wd=0.1, eps=1e-8)
    n = 256
    gen = torch.Generator().manual_seed(0)
    p = torch.randn(n, generator=gen)
    g = torch.randn(n, generator=gen)
    st = _random_expand_state(n, 1)
    pd, std = p.to(dev), to_dev(st, dev)
    cpu_step(p, g, st, 1000, True, hp)
    gpu_step(q, pd, g.to(dev), std, 1000, True, hp)
    assert torch.allclose(pd.cpu(), p, rtol=1e-4)  # the reference's own bar
    # lr = 0.4: the update is as large as the parameter, so its 1e-6 shows up as an absolute error
    compare_expand(pd, std, p, st, n, "ref case", p_rtol=1e-5, p_atol=2e-6)


def test_expand_zero_handling_matches_reference_tree(dev):
    """Exact zeros take the shuffle-tree path: thread-0 zero survives, partner zeros are skipped,
    all-zero groups stay finite."""
    q = _q()
    hp = dict(beta1=0.0, beta2=0.0, lr=0.0, wd=0.0, eps=1e-8)
    base = torch.linspace(1.0, 2.0, 128)
    cases = []
    for pos in (None, 0, 16, 32, 1, 4, 127, 64, 96):
        g = base.clone()
        if pos is not None:
            g[pos] = 0.0
        cases.append(g)
    cases.append(torch.zeros(128))
    g = torch.cat(cases)
    n = g.numel()
    p = torch.zeros(n)
    st = A.fresh_state(p, True)
    pd, std = p.to(dev), to_dev(st, dev)
    cpu_step(p, g.clone(), st, 1, True, hp)
    gpu_step(q, pd, g.to(dev), std, 1, True, hp)
    for k in ("sqrt_minmax_exp_avg", "sqrt_minmax_exp_avg_sq"):
        assert torch.equal(std[k].cpu(), st[k]), k  # sqrt(Mx)*sqrt(Mn): exact given the same min / max
    compare_expand(pd, std, p, st, n, "zeros")
    # a second step from that state (k = inf / 0 groups exercise the powf special cases)
    g2 = torch.cat([base * 0.5] * (len(cases) - 1) + [torch.zeros(128)])
    pd, std = p.to(dev), to_dev(st, dev)
    cpu_step(p, g2.clone(), st, 2, True, hp)
    gpu_step(q, pd, g2.to(dev), std, 2, True, hp)
    assert torch.isfinite(pd).all()
    compare_expand(pd, std, p, st, n, "zeros step 2")


def test_errors(dev):
    q = _q()
    p = torch.zeros(256, device=dev)
    st = to_dev(A.fresh_state(p.cpu(), True), dev)
    with pytest.raises(RuntimeError, match="Only Support 128"):
        q.fp8_adamw_expand_step(p, p, *[st[k] for k in KEYS_EXP], 0.9, 0.95, 1e-3, 0.1, 1e-8, 1, 64, 16)
    bad = dict(st)
    bad["scale_exp_avg"] = torch.zeros(3, device=dev)
    with pytest.raises(RuntimeError):
        q.fp8_adamw_expand_step(p, p, *[bad[k] for k in KEYS_EXP], 0.9, 0.95, 1e-3, 0.1, 1e-8, 1, 128, 16)


def test_coatadamw_trajectory_and_state_dict(dev):
    """CoatAdamW (drop-in optimizer class) over 10 steps on a [256, 384] weight against the oracle run on
    the CPU with the same gradients, then a state_dict round trip."""
    from coat_amd.optimizer.fp8_adamw import CoatAdamW
    from coat_amd.utils._fp8_quantization_config import QuantizationConfig
    torch.manual_seed(0)
    w0 = torch.randn(256, 384) * 0.02
    for expansion in ("true", "false"):
        w = torch.nn.Parameter(w0.clone().to(dev))
        opt = CoatAdamW([w], lr=3e-4, betas=(0.9, 0.95), weight_decay=0.1, eps=1e-8,
                        qargs=QuantizationConfig(first_order_expansion=expansion, second_order_expansion=expansion))
        p = w0.clone().flatten()
        st = A.fresh_state(p, expansion == "true")
        for step in range(1, 11):
            g = grads(p.numel(), 100 + step)
            w.grad = g.reshape(256, 384).to(dev)
            opt.step()
            cpu_step(p, g, st, step, expansion == "true")
        dp = (w.detach().cpu().flatten() - p).abs()
        if expansion == "false":
            assert dp.max().item() == 0.0  # the plain step is bit-exact, so is its trajectory
        else:
            # a moment that lands one e4m3 code away (about 1e-5 of them per step) moves that element's update by
            # at most one fp8 step of m/denom ~ 1: lr * 2^-3 per step in the worst case; everything else is ulps
            assert dp.max().item() <= 3e-4 * 0.125 * 10 and dp.median().item() <= 1e-8 and (dp > 1e-7).float().mean().item() < 5e-3
        s = opt.state[w]
        assert s["exp_avg"].dtype == torch.float8_e4m3fn and s["scale_exp_avg"].dtype == torch.float32
        assert int(s["step"].item()) == 10 and s["step"].device.type == "cpu"
        if expansion == "false":
            assert "expand_exp_avg" not in s
            assert torch.equal(s["exp_avg"].cpu().view(torch.uint8), st["exp_avg"].view(torch.uint8).reshape(256, 384))
        else:
            m_g = A.dequantize_state(s["exp_avg"].cpu().flatten(), s["scale_exp_avg"].cpu(), s["expand_exp_avg"].cpu(), s["sqrt_minmax_exp_avg"].cpu())
            m_c = A.dequantize_state(st["exp_avg"], st["scale_exp_avg"], st["expand_exp_avg"], st["sqrt_minmax_exp_avg"])
            rel = (m_g - m_c).abs() / m_c.abs().clamp_min(1e-12)
            assert rel.median() < 1e-3 and rel.quantile(0.99) < 0.2  # trajectories stay together to within fp8 steps
        import copy
        sd = copy.deepcopy(opt.state_dict())  # state_dict() hands out the live tensors
        w2 = torch.nn.Parameter(w.detach().clone())
        opt2 = CoatAdamW([w2], lr=3e-4, betas=(0.9, 0.95), weight_decay=0.1, eps=1e-8, qargs=opt.qargs)
        opt2.load_state_dict(sd)
        s2 = opt2.state[w2]
        assert s2["exp_avg"].dtype == torch.float8_e4m3fn and s2["scale_exp_avg"].dtype == torch.float32
        g = grads(p.numel(), 999).reshape(256, 384).to(dev)
        w.grad, w2.grad = g, g.clone()
        opt.step(); opt2.step()
        assert torch.equal(w.detach(), w2.detach())


@pytest.mark.parametrize("expand", [True, False])
@pytest.mark.parametrize("pdtype", [torch.float32, torch.bfloat16])
def test_multi_tensor_step_equals_separate_launches(dev, expand, pdtype):
    """coat_fp8_adamw_expand_step_multi / coat_fp8_adamw_step_multi: 70 tensors (three launches of at most 32), sizes from
    one element over ragged groups to whole waves and an empty tensor in between, three steps: parameters, codes and all
    group vectors bit-identical to one launch per tensor."""
    q = _q()
    sizes = [1, 127, 128, 129, 1024, 1024 * 3 + 5, 4096, 0, 128 * 9 + 37, 128 * 64] * 7
    gen = torch.Generator().manual_seed(5)
    ps = [(torch.randn(n, generator=gen) * 0.02).to(pdtype) for n in sizes]
    keys = KEYS_EXP if expand else KEYS_PLAIN
    single = [(p.to(dev), to_dev(A.fresh_state(p, expand=expand), dev)) for p in ps]
    multi = [(p.to(dev), to_dev(A.fresh_state(p, expand=expand), dev)) for p in ps]
    hp = (HP["beta1"], HP["beta2"], HP["lr"], HP["wd"], HP["eps"])
    for step in (1, 2, 3):
        gs = [(torch.randn(n, generator=gen) * 1e-3).to(pdtype).to(dev) for n in sizes]
        for (p, st), g in zip(single, gs):
            gpu_step(q, p, g, st, step, expand)
        cols = [[st[k] for _, st in multi] for k in keys]
        if expand:
            q.fp8_adamw_expand_step_multi([p for p, _ in multi], gs, *cols, *hp, step, 128, 16)
        else:
            q.fp8_adamw_step_multi([p for p, _ in multi], gs, *cols, *hp, step, 128)
        for i, ((p1, s1), (p2, s2)) in enumerate(zip(single, multi)):
            assert torch.equal(p1, p2), (i, sizes[i], step, "params")
            for k in keys:
                a, b = s1[k], s2[k]
                if a.dtype != torch.float32:
                    a, b = a.view(torch.uint8), b.view(torch.uint8)
                assert torch.equal(a, b) or (torch.equal(a.isnan(), b.isnan()) and torch.equal(a.nan_to_num(), b.nan_to_num())), (i, sizes[i], step, k)


def test_coatadamw_multi_tensor_switch_gives_the_same_trajectory(dev):
    """CoatAdamW buckets the parameters of one dtype and step count into multi-tensor launches; with multi_tensor=False it
    launches once per parameter like the reference.  Same parameters and state after five steps, two dtypes, a parameter
    without gradient and one that joins late (its step count differs, so it gets a bucket of its own)."""
    from coat_amd.optimizer.fp8_adamw import CoatAdamW
    gen = torch.Generator().manual_seed(6)
    shapes = [(64, 128), (300,), (4096,), (17, 33), (1,), (128,)]

    def build():
        g = torch.Generator().manual_seed(7)
        ps = [torch.nn.Parameter((torch.randn(sh, generator=g) * 0.02).to(dev)) for sh in shapes]
        ps += [torch.nn.Parameter((torch.randn(sh, generator=g) * 0.02).bfloat16().to(dev)) for sh in shapes[:3]]
        return ps

    pa, pb = build(), build()
    oa = CoatAdamW(pa, lr=1e-3, weight_decay=0.05)
    ob = CoatAdamW(pb, lr=1e-3, weight_decay=0.05, multi_tensor=False)
    for step in range(5):
        for i, (a, b) in enumerate(zip(pa, pb)):
            if i == 1 or (i == 3 and step < 2):
                a.grad = b.grad = None
                continue
            gr = (torch.randn(a.shape, generator=gen) * 1e-3).to(a.dtype).to(dev)
            a.grad, b.grad = gr, gr.clone()
        oa.step()
        ob.step()
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
        sa, sb = oa.state[a], ob.state[b]
        assert sa.keys() == sb.keys()
        for k in sa:
            x, y = sa[k], sb[k]
            if x.dtype not in (torch.float32,):
                x, y = x.view(torch.uint8), y.view(torch.uint8)
            assert torch.equal(x, y), k
