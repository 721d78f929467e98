"""Pins oracle/adamw_ref.c against things it does not share code with:
the reference test's own torch definition of the step (restated in oracle/adamw_ref.py),
torch.optim.AdamW, and the invariants of Dynamic Range Expansion."""
import math

import torch

from oracle import adamw_ref as A

HP = dict(beta1=0.9, beta2=0.95, lr=0.4, wd=0.1, eps=1e-8)  # tests/test_fp8_adamw_expand.py:43-44


def _random_expand_state(n, seed, k_choices=None):
    """State built the way tests/test_fp8_adamw_expand.py:52-109 builds it: quantize random moments
    per group, then give every group a random exponent i/16 and a random centre."""
    g = torch.Generator().manual_seed(seed)
    ng = (n + 127) // 128
    m = torch.randn(ng * 128, generator=g)
    v = torch.randn(ng * 128, generator=g).abs()
    st = {}
    for name, x in (("exp_avg", m), ("exp_avg_sq", v)):
        B = x.reshape(ng, 128)
        s = (B.abs().amax(dim=1) + 1e-8) / 448
        st[name] = (B / s.unsqueeze(1)).to(torch.float8_e4m3fn).flatten()[:n].contiguous()
        st["scale_" + name] = s.contiguous()
        ks = torch.tensor([i / 16 for i in range(1, 129)]) if k_choices is None else torch.tensor(k_choices)
        st["expand_" + name] = ks[torch.randint(len(ks), (ng,), generator=g)].float().contiguous()
        st["sqrt_minmax_" + name] = torch.randn(ng, generator=g).abs().add(0.05).contiguous()
    return st


def _run_expand(p, gr, st, step, expand_min=16, hp=HP):
    A.adamw_expand_step(p, gr, st["exp_avg"], st["scale_exp_avg"], st["expand_exp_avg"], st["sqrt_minmax_exp_avg"],
                        st["exp_avg_sq"], st["scale_exp_avg_sq"], st["expand_exp_avg_sq"], st["sqrt_minmax_exp_avg_sq"],
                        hp["beta1"], hp["beta2"], hp["lr"], hp["wd"], hp["eps"], step, 128, expand_min)


def test_expand_step_against_reference_tests_definition():
    n = 128 * 64
    gen = torch.Generator().manual_seed(0)
    p = torch.randn(n, generator=gen)
    gr = torch.randn(n, generator=gen)
    st = _random_expand_state(n, 1)
    m_fp = A.dequantize_state(st["exp_avg"], st["scale_exp_avg"], st["expand_exp_avg"], st["sqrt_minmax_exp_avg"]).float()
    v_fp = A.dequantize_state(st["exp_avg_sq"], st["scale_exp_avg_sq"], st["expand_exp_avg_sq"], st["sqrt_minmax_exp_avg_sq"]).float()
    sim = A.simulated_expand_step(p, gr, m_fp, v_fp, step=1000, **HP)
    p_c = p.clone()
    _run_expand(p_c, gr, st, 1000)
    # reference tolerance (tests/test_fp8_adamw_expand.py:296-308): rtol 1e-4 on everything
    assert torch.allclose(sim["params"], p_c, rtol=1e-4, atol=1e-6)
    for name in ("exp_avg", "exp_avg_sq"):
        q, s, k, c = sim[name]
        # the reference test searches k over i/16 with i <= 128, so it caps at 8; the kernel's floor() does not
        assert (k == st["expand_" + name].clamp(max=8.0)).float().mean() >= 0.99  # ties aside
        same_k = k == st["expand_" + name]
        assert same_k.float().mean() >= 0.5
        # rtol 1e-4 is the reference test's bar; a group whose minimum comes from a cancellation
        # beta1*m + (1-beta1)*g ~ 0 amplifies the fp32 rounding of the dequantized input, hence the
        # looser bound on the worst group and the tight one on the median
        rc = (c - st["sqrt_minmax_" + name]).abs() / c
        rs = ((s - st["scale_" + name]).abs() / s)[same_k]
        assert rc.max() < 1e-3 and rc.median() < 1e-6
        assert rs.max() < 1e-3 and rs.median() < 1e-5
        qc = st[name].float().reshape(-1, 128)[same_k]
        eq = (q[same_k] == qc).float().mean().item()
        assert eq >= 0.995, eq  # codes equal except where powf rounding meets an e4m3 rounding boundary
        assert (q[same_k] - qc).abs().max() <= 64  # never more than one step at the top binade


def test_fresh_state_step1_equals_torch_adamw():
    n = 128 * 8 + 37  # ragged tail
    gen = torch.Generator().manual_seed(3)
    p0 = torch.randn(n, generator=gen) * 0.02
    gr = torch.randn(n, generator=gen) * 1e-3
    hp = dict(beta1=0.9, beta2=0.95, lr=3e-4, wd=0.1, eps=1e-8)
    pt = torch.nn.Parameter(p0.clone())
    pt.grad = gr.clone()
    torch.optim.AdamW([pt], lr=hp["lr"], betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1).step()
    for expand in (True, False):
        p = p0.clone()
        st = A.fresh_state(p, expand)
        if expand:
            _run_expand(p, gr, st, 1, hp=hp)
        else:
            A.adamw_step(p, gr, st["exp_avg"], st["scale_exp_avg"], st["exp_avg_sq"], st["scale_exp_avg_sq"],
                         hp["beta1"], hp["beta2"], hp["lr"], hp["wd"], hp["eps"], 1, 128)
        assert torch.allclose(p, pt.detach(), rtol=2e-6, atol=1e-9)
        # m = (1-b1) g and v = (1-b2) g^2 exactly; their quantized images must dequantize back close to them
        m_deq = A.dequantize_state(st["exp_avg"], st["scale_exp_avg"], st.get("expand_exp_avg"), st.get("sqrt_minmax_exp_avg"))
        m_true = ((1 - 0.9) * gr).double()
        # e4m3 has 3 mantissa bits: relative error <= 2^-4 in the expanded domain; expansion by ^k with
        # k>=1 shrinks it, k<1 grows it (k >= 1/2 here), plus subnormal flush of the smallest entries
        rel = ((m_deq - m_true).abs() / m_true.abs().clamp_min(1e-12))
        assert rel.median() < 0.04 and rel.quantile(0.99) < 0.14


def test_dre_invariants():
    n = 128 * 256
    gen = torch.Generator().manual_seed(5)
    p = torch.randn(n, generator=gen) * 0.02
    st = A.fresh_state(p, True)
    hp = dict(beta1=0.9, beta2=0.95, lr=3e-4, wd=0.1, eps=1e-8)
    for step in range(1, 4):
        gr = torch.randn(n, generator=gen) * 1e-3
        _run_expand(p, gr, st, step, hp=hp)
    for name in ("exp_avg", "exp_avg_sq"):
        k, c, s = st["expand_" + name].double(), st["sqrt_minmax_" + name].double(), st["scale_" + name].double()
        assert torch.equal(k * 16, torch.floor(k * 16))  # multiples of 1/expand_min
        codes = st[name].view(torch.uint8).reshape(-1, 128)
        assert ((codes & 0x7F).amax(dim=1) == 0x7E).all()  # the group maximum lands on +-448
        # recover max/min from (c, s, k): Mx/c = (448 s)^(1/k), ratio = (Mx/c)^2
        ratio = (448 * s).pow(1 / k).pow(2)
        assert (ratio.pow(k) <= 448 * 448 / 2 * (1 + 1e-5)).all()
        assert (ratio.pow(k + 1 / 16) > 448 * 448 / 2 * (1 - 1e-5)).all()  # k is the largest admissible multiple
        assert (c > 0).all()


def test_expand_with_unit_exponent_reduces_to_plain_update():
    """k = 1, c = 1 makes the DRE dequantization the identity, so params must follow the plain kernel."""
    n = 128 * 16
    gen = torch.Generator().manual_seed(7)
    p0 = torch.randn(n, generator=gen)
    gr = torch.randn(n, generator=gen)
    st = _random_expand_state(n, 8, k_choices=[1.0])
    for key in ("sqrt_minmax_exp_avg", "sqrt_minmax_exp_avg_sq"):
        st[key].fill_(1.0)
    st2 = {k: v.clone() for k, v in st.items()}
    pe, pp = p0.clone(), p0.clone()
    _run_expand(pe, gr, st, 10)
    A.adamw_step(pp, gr, st2["exp_avg"], st2["scale_exp_avg"], st2["exp_avg_sq"], st2["scale_exp_avg_sq"],
                 HP["beta1"], HP["beta2"], HP["lr"], HP["wd"], HP["eps"], 10, 128)
    assert torch.equal(pe, pp)
    # plain kernel: scale = (max + 1e-20) / 448 and codes = e4m3(m / scale)
    m_new = st2["exp_avg"].float().reshape(-1, 128) * st2["scale_exp_avg"].unsqueeze(1)
    assert ((st2["exp_avg"].view(torch.uint8).reshape(-1, 128) & 0x7F).amax(dim=1) == 0x7E).all()
    assert torch.isfinite(m_new).all()


def test_zero_skipping_minimum_is_order_dependent():
    """fp8_adamw_expand_cuda_kernel.cu:95-101: a zero is skipped only when it arrives from the
    shuffle partner; a zero held by thread 0 survives as the group minimum."""
    hp = dict(beta1=0.0, beta2=0.0, lr=0.0, wd=0.0, eps=1e-8)  # m = g, v = g^2: moments are the gradient itself

    def run(gr):
        p = torch.zeros(128)
        st = A.fresh_state(p, True)
        _run_expand(p, gr.clone(), st, 1, hp=hp)
        return st

    base = torch.linspace(1.0, 2.0, 128)
    st = run(base)
    c_ref = math.sqrt(2.0) * math.sqrt(1.0)
    assert abs(st["sqrt_minmax_exp_avg"].item() - c_ref) < 1e-6
    g1 = base.clone(); g1[16] = 0.0   # arrives from a partner lane: skipped, min stays 1.0
    assert abs(run(g1)["sqrt_minmax_exp_avg"].item() - c_ref) < 1e-6
    g2 = base.clone(); g2[0] = 0.0    # held by thread 0: min = 0 -> Mn = 1e-30
    c2 = run(g2)["sqrt_minmax_exp_avg"].item()
    assert abs(c2 - math.sqrt(2.0) * math.sqrt(1e-30)) < 1e-20
    g3 = base.clone(); g3[32] = 0.0   # lane 0 of warp 1: that warp's result is 0, skipped at block level
    assert abs(run(g3)["sqrt_minmax_exp_avg"].item() - c_ref) < 1e-6


def test_all_zero_group_stays_finite():
    p = torch.ones(256)
    gr = torch.zeros(256)
    gr[128:] = torch.linspace(-1, 1, 128)
    st = A.fresh_state(p, True)
    hp = dict(beta1=0.9, beta2=0.95, lr=1e-3, wd=0.0, eps=1e-8)
    for step in (1, 2, 3):
        _run_expand(p, gr, st, step, hp=hp)
        assert torch.isfinite(p).all()
        assert (st["exp_avg"].view(torch.uint8)[:128] & 0x7F != 0x7F).all()
    assert torch.equal(p[:128], torch.ones(128))  # zero gradient, no decay: untouched


def test_bf16_params_round_once():
    n = 128 * 4
    gen = torch.Generator().manual_seed(11)
    p32 = (torch.randn(n, generator=gen) * 0.02).bfloat16().float()
    gr = (torch.randn(n, generator=gen) * 1e-3).bfloat16()
    hp = dict(beta1=0.9, beta2=0.95, lr=3e-4, wd=0.1, eps=1e-8)
    st_a, st_b = A.fresh_state(p32, True), A.fresh_state(p32, True)
    pa = p32.clone()
    pb = p32.bfloat16()
    _run_expand(pa, gr.float(), st_a, 1, hp=hp)
    _run_expand(pb, gr, st_b, 1, hp=hp)
    assert torch.equal(pb, pa.bfloat16())
    assert torch.equal(st_a["exp_avg"].view(torch.uint8), st_b["exp_avg"].view(torch.uint8))


def test_device_division_and_sqrt_shortcuts_are_exact_on_the_cpu():
    """The plain AdamW kernel replaces two of the compiler's IEEE sequences by shorter ones that must give the same bits:
    sqrt(v) / c2 through the reciprocal of c2 and one FMA correction (the three-operation sequence of div_by_scale), and
    sqrtf through the hardware approximation (within one ulp) and a two-residual correction.  Both are restated in
    oracle/adamw_ref.c with IEEE arithmetic and compared with / and sqrtf: 0 mismatches over every c2 = sqrt(1 - beta2^step)
    of 2000 steps x 2e5 square roots, and over 3e6 second moments x the three possible starting points."""
    L = A.lib()
    gen = torch.Generator().manual_seed(0)
    # second moments as they occur (g^2 scale, spread over 40 binades) and their correctly rounded roots
    v = (torch.rand(200_000, generator=gen) * 2 + 0.5) * torch.pow(2.0, torch.randint(-80, 20, (200_000,), generator=gen).float())
    roots = v.sqrt().contiguous()
    c2 = []
    for beta2 in (0.95, 0.999):
        for step in range(1, 1001):
            c2.append(math.sqrt(1.0 - float(torch.tensor(beta2, dtype=torch.float32).double().pow(float(step)).float())))
    c2 = torch.tensor(c2, dtype=torch.float32).contiguous()
    assert (c2 > 0).all() and (c2 <= 1).all()
    assert L.coat_oracle_count_recip_div_mismatch(roots.data_ptr(), roots.numel(), c2.data_ptr(), c2.numel()) == 0
    x = torch.cat([v, torch.rand(800_000, generator=gen) * 1e-3, torch.rand(2_000_000, generator=gen).pow(8) * 1e-2,
                   torch.tensor([0.0, 2.0 ** -96, 1.0, 4.0, 2.0 ** 60, float("inf")])]).float().contiguous()
    assert L.coat_oracle_count_sqrt_correction_mismatch(x.data_ptr(), x.numel()) == 0


def test_plain_step_trajectory_against_torch_tensor_restatement():
    """The plain step of the C oracle against the reference kernel written a second time with whole-tensor torch operations
    (fp8_adamw_cuda_kernel.cu:37-53, 107-124: dequantize, moments, bias corrections, parameter update, group maximum + 1e-20
    in double, scale = max / 448, codes = e4m3(moment / scale) by torch's own cast).  Six steps from the fresh state on a
    tensor with a ragged last group: parameters, both code tensors and both scale vectors must be bit-identical at every
    step.  (torch's CPU kernels round every + - * / sqrt separately, like the oracle; a dropped term, a wrong bias
    correction or a scale taken from the wrong group shows in the first step.)"""
    n, G = 128 * 5 + 77, 128
    ng = (n + G - 1) // G
    gen = torch.Generator().manual_seed(11)
    p0 = torch.randn(n, generator=gen) * 0.02
    b1, b2, lr, wd, eps = 0.9, 0.95, 3e-4, 0.1, 1e-8
    f32 = lambda x: torch.tensor(x, dtype=torch.float32)
    # oracle state
    p = p0.clone()
    st = A.fresh_state(p, False)
    # restatement state (padded to whole groups; the padding holds zeros and never reaches a stored value)
    pr = p0.clone()
    m8 = torch.zeros(ng * G, dtype=torch.float8_e4m3fn)
    v8 = torch.zeros(ng * G, dtype=torch.float8_e4m3fn)
    sm, sv = st["scale_exp_avg"].clone(), st["scale_exp_avg_sq"].clone()
    for step in range(1, 7):
        gr = torch.randn(n, generator=gen) * (1e-3 * step)
        A.adamw_step(p, gr, st["exp_avg"], st["scale_exp_avg"], st["exp_avg_sq"], st["scale_exp_avg_sq"], b1, b2, lr, wd, eps, step, G)
        g = torch.zeros(ng * G)
        g[:n] = gr
        m = m8.float() * sm.repeat_interleave(G)
        v = v8.float() * sv.repeat_interleave(G)
        m = f32(b1) * m + (f32(1.0) - f32(b1)) * g
        v = f32(b2) * v + ((f32(1.0) - f32(b2)) * g) * g
        c1 = f32(1.0) - torch.pow(f32(b1), f32(float(step)))
        c2 = torch.sqrt(f32(1.0) - torch.pow(f32(b2), f32(float(step))))
        denom = (torch.sqrt(v[:n]) / c2 + f32(eps)) * c1
        update = m[:n] / denom + f32(wd) * pr
        pr = pr - f32(lr) * update
        m[n:] = 0.0
        v[n:] = 0.0
        amax_m = m.abs().reshape(ng, G).amax(dim=1)
        amax_v = v.abs().reshape(ng, G).amax(dim=1)
        sm = ((amax_m.double() + 1e-20).float()) / f32(448.0)
        sv = ((amax_v.double() + 1e-20).float()) / f32(448.0)
        m8 = (m / sm.repeat_interleave(G)).to(torch.float8_e4m3fn)
        v8 = (v / sv.repeat_interleave(G)).to(torch.float8_e4m3fn)
        assert torch.equal(p.view(torch.int32), pr.view(torch.int32)), step
        assert torch.equal(st["scale_exp_avg"].view(torch.int32), sm.view(torch.int32)), step
        assert torch.equal(st["scale_exp_avg_sq"].view(torch.int32), sv.view(torch.int32)), step
        assert torch.equal(st["exp_avg"].view(torch.uint8).flatten()[:n], m8.view(torch.uint8)[:n]), step
        assert torch.equal(st["exp_avg_sq"].view(torch.uint8).flatten()[:n], v8.view(torch.uint8)[:n]), step
