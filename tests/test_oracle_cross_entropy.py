"""Pins oracle/cross_entropy_ref.py against torch's own cross-entropy and against finite differences (CPU)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import cross_entropy_ref as C


def case(BT=12, V=37, seed=0, ignore=3):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(BT, V, generator=g, dtype=torch.float64) * 3
    t = torch.randint(0, V, (BT,), generator=g)
    t[torch.randperm(BT, generator=g)[:ignore]] = -100
    return x, t


@pytest.mark.parametrize("reduction", ["mean", "sum"])
@pytest.mark.parametrize("ls", [0.0, 0.1])
def test_matches_torch_cross_entropy(reduction, ls):
    x, t = case()
    loss, _, grad = C.cross_entropy_forward(x, t, -100, 0.0, ls, reduction)
    xr = x.clone().requires_grad_(True)
    want = F.cross_entropy(xr, t, ignore_index=-100, label_smoothing=ls, reduction=reduction)
    (wg,) = torch.autograd.grad(want, xr)
    assert torch.allclose(loss, want, rtol=1e-12, atol=1e-12)
    assert torch.allclose(grad, wg, rtol=1e-10, atol=1e-12)
    assert torch.all(grad[t == -100] == 0)


def test_other_ignore_index_and_all_ignored():
    x, t = case(ignore=0)
    t[::3] = 5
    loss, _, grad = C.cross_entropy_forward(x, t, 5, 0.0, 0.0, "mean")
    want = F.cross_entropy(x, t, ignore_index=5)
    assert torch.allclose(loss, want, rtol=1e-12)
    assert torch.all(grad[::3] == 0)


def _fd(fn, x, h=1e-6):
    g = torch.zeros_like(x)
    for i in range(x.shape[0]):
        for j in range(x.shape[1]):
            xp, xm = x.clone(), x.clone()
            xp[i, j] += h
            xm[i, j] -= h
            g[i, j] = (fn(xp) - fn(xm)) / (2 * h)
    return g


def test_z_loss_term():
    x, t = case(BT=5, V=11, ignore=1)
    s = 1e-2
    loss, z, grad = C.cross_entropy_forward(x, t, -100, s, 0.0, "mean")
    plain = F.cross_entropy(x, t, ignore_index=-100)
    valid = t != -100
    want_z = s * (torch.logsumexp(x[valid], 1) ** 2).sum() / valid.sum()
    assert torch.allclose(z, want_z, rtol=1e-12)
    assert torch.allclose(loss, plain + want_z, rtol=1e-12)
    fd = _fd(lambda v: C.cross_entropy_forward(v, t, -100, s, 0.0, "mean")[0], x)
    assert torch.allclose(grad, fd, rtol=1e-5, atol=1e-8)


def test_softcap():
    x, t = case(BT=5, V=11, ignore=1)
    cap = 2.5
    loss, _, grad = C.cross_entropy_forward(x, t, -100, 0.0, 0.05, "sum", softcap=cap)
    xr = x.clone().requires_grad_(True)
    want = F.cross_entropy(cap * torch.tanh(xr / cap), t, ignore_index=-100, label_smoothing=0.05, reduction="sum")
    (wg,) = torch.autograd.grad(want, xr)
    assert torch.allclose(loss, want, rtol=1e-12)
    assert torch.allclose(grad, wg, rtol=1e-10, atol=1e-12)
    fd = _fd(lambda v: C.cross_entropy_forward(v, t, -100, 0.0, 0.05, "sum", softcap=cap)[0], x)
    assert torch.allclose(grad, fd, rtol=1e-5, atol=1e-8)
