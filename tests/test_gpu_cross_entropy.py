"""GPU parity: fused cross-entropy (reference coat/activation/liger/cross_entropy.py) against the float64 oracle.

Tolerances (fp32 logits): loss rtol 2e-6 (fp32 sums of BT rows, hardware exp2/log); gradient |d| <= 2e-6 * |ref| +
3e-7 / divisor, i.e. a few fp32 ulps of the softmax probability, which is at most 1 before the division by the count
of non-ignored rows.  bf16 logits: the stored gradient and per-row losses are rounded to bf16, so 2^-8 relative."""
import pytest
import torch

from oracle import cross_entropy_ref as C

pytestmark = pytest.mark.gpu


def _ce():
    import coat_amd.activation.liger.cross_entropy as ce
    return ce


def make(BT, V, seed=0, n_ignore=3, scale=3.0, ignore_index=-100):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(BT, V, generator=g) * scale
    t = torch.randint(0, V, (BT,), generator=g)
    if n_ignore:
        t[torch.randperm(BT, generator=g)[:n_ignore]] = ignore_index
    return x, t


def check(dev, x, t, ignore_index=-100, lss=0.0, ls=0.0, reduction="mean", softcap=None, dtype=torch.float32):
    ce = _ce()
    xd = x.to(dtype).to(dev)
    x_in = xd.float().cpu()  # what the kernel actually saw
    loss, z, xg = ce.cross_entropy_forward(xd, t.to(dev), ignore_index, lss, ls, reduction, softcap, True)
    assert xg.data_ptr() == xd.data_ptr(), "the gradient must be written in place"
    wl, wz, wg = C.cross_entropy_forward(x_in, t, ignore_index, lss, ls, reduction, softcap)
    n = float((t != ignore_index).sum()) if reduction == "mean" else 1.0
    if dtype == torch.float32:
        assert torch.allclose(loss.double().cpu(), wl, rtol=2e-6, atol=1e-7), (loss.item(), wl.item())
        assert torch.allclose(z.double().cpu(), wz, rtol=2e-6, atol=1e-9)
        err = (xg.double().cpu() - wg).abs()
        assert torch.all(err <= 2e-6 * wg.abs() + 3e-7 / n), err.max().item()
    else:
        assert torch.allclose(loss.double().cpu(), wl, rtol=2**-7)
        err = (xg.double().cpu() - wg).abs()
        assert torch.all(err <= 2**-8 * wg.abs() + 1e-6 / n), err.max().item()
    assert torch.all(xg[(t == ignore_index).to(dev)] == 0)
    return loss, xg


@pytest.mark.parametrize("V", [37, 1000, 4096, 5000, 12000, 32000, 40000])
@pytest.mark.parametrize("reduction", ["mean", "sum"])
def test_plain_cross_entropy(dev, V, reduction):
    x, t = make(24, V, seed=V)
    check(dev, x, t, reduction=reduction)


@pytest.mark.parametrize("V", [999, 32000, 50257])
def test_label_smoothing_z_loss_softcap(dev, V):
    x, t = make(16, V, seed=V + 1)
    check(dev, x, t, ls=0.1)
    check(dev, x, t, lss=1e-4)
    check(dev, x, t, ls=0.05, lss=1e-3, reduction="sum")
    check(dev, x, t, softcap=5.0)
    check(dev, x, t, ls=0.1, lss=1e-4, softcap=30.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("V", [1001, 32000, 70000])
def test_half_precision_logits(dev, dtype, V):
    x, t = make(16, V, seed=V + 2)
    check(dev, x, t, dtype=dtype)


def test_other_ignore_index_all_ignored_and_strided_rows(dev):
    ce = _ce()
    x, t = make(16, 512, seed=5, n_ignore=0)
    t[::2] = 7
    check(dev, x, t, ignore_index=7)
    # every row ignored: loss 0, gradient 0
    t[:] = -100
    xd = x.to(dev)
    loss, _, xg = ce.cross_entropy_forward(xd, t.to(dev), -100, 0.0, 0.0, "mean", None, False)
    assert loss.item() == 0.0 and torch.all(xg == 0)
    # rows with a pitch larger than V (a column slice): handled without a copy, the slice holds the gradient
    big = torch.randn(16, 640).to(dev)
    view = big[:, :512]
    keep = big[:, 512:].clone()
    x2, t2 = view.clone().cpu(), make(16, 512, seed=6)[1]
    _, _, g2 = ce.cross_entropy_forward(view, t2.to(dev), -100, 0.0, 0.0, "mean", None, False)
    _, _, wg = C.cross_entropy_forward(x2, t2)
    assert g2.data_ptr() == big.data_ptr()
    assert torch.allclose(g2.double().cpu(), wg, rtol=2e-6, atol=3e-8)
    assert torch.equal(big[:, 512:], keep)


def test_autograd_function_and_causal_lm_loss(dev):
    ce = _ce()
    B, S, V = 2, 33, 1024
    g = torch.Generator().manual_seed(9)
    hidden = torch.randn(B, S, 64, generator=g).to(dev).requires_grad_(True)
    w = (torch.randn(V, 64, generator=g) * 0.2).to(dev).requires_grad_(True)
    labels = torch.randint(0, V, (B, S), generator=g)
    labels[0, :5] = -100
    logits = hidden @ w.t()
    loss = ce.LigerForCausalLMLoss(logits, labels.to(dev), V)
    (loss * 3.0).backward()  # grad_output != 1: the in-place rescale runs
    h2 = hidden.detach().clone().requires_grad_(True)
    w2 = w.detach().clone().requires_grad_(True)
    lg = (h2 @ w2.t()).float()
    want = torch.nn.functional.cross_entropy(lg[:, :-1].reshape(-1, V), labels[:, 1:].reshape(-1).to(dev), ignore_index=-100)
    (want * 3.0).backward()
    assert torch.allclose(loss, want, rtol=1e-5)
    assert torch.allclose(hidden.grad, h2.grad, rtol=1e-4, atol=1e-6)
    assert torch.allclose(w.grad, w2.grad, rtol=1e-4, atol=1e-6)
    # num_items_in_batch: sum reduction divided on the host side
    loss2 = ce.LigerForCausalLMLoss((h2.detach() @ w2.detach().t()), labels.to(dev), V, num_items_in_batch=40)
    n_valid = int((labels[:, 1:] != -100).sum())
    assert torch.allclose(loss2, want.detach() * n_valid / 40, rtol=1e-5)


def test_backward_scale_is_skipped_for_one_and_applied_otherwise(dev):
    ce = _ce()
    x = torch.randn(8, 1000).to(dev)
    ref = x.clone()
    ce.cross_entropy_backward(x, torch.tensor(1.0, device=dev))
    assert torch.equal(x, ref)
    ce.cross_entropy_backward(x, torch.tensor(0.25, device=dev))
    assert torch.equal(x, ref * 0.25)
    xb = torch.randn(8, 1003).to(torch.bfloat16).to(dev)  # ragged row length: scalar path
    refb = xb.clone()
    ce.cross_entropy_backward(xb, torch.tensor(2.0, device=dev, dtype=torch.bfloat16))
    assert torch.equal(xb, refb * 2)
