"""torch-CPU restatement of the reference's fused cross-entropy.  TEST INFRASTRUCTURE ONLY.

Follows coat/activation/liger/cross_entropy.py: the per-row loss of the kernel (:167-198) written as one float64
expression, the gradient obtained from it by autograd instead of the kernel's hand-derived formula (:122-160), and
the host function's reductions (:212-278).

Pin status (tests/test_oracle_cross_entropy.py):
  plain / ignore_index / label_smoothing, mean and sum   == torch.nn.functional.cross_entropy and its autograd
                                                           gradient (library routine)
  lse_square_scale                                        loss - plain loss == scale * mean(logsumexp^2) recomputed
                                                           independently; gradient by central finite differences
  softcap                                                 == plain loss of the capped logits; gradient by the chain
                                                           rule through torch.tanh's autograd and finite differences
"""
import torch


def cross_entropy_forward(x, target, ignore_index=-100, lse_square_scale=0.0, label_smoothing=0.0, reduction="mean",
                          softcap=None):
    """Returns (loss, z_loss, grad): scalars in float64 and d loss / d x in float64, for x [BT, V] and target [BT]."""
    x = x.detach().double().requires_grad_(True)
    V = x.shape[1]
    z = softcap * torch.tanh(x / softcap) if softcap is not None else x
    lse = torch.logsumexp(z, dim=1)
    valid = target != ignore_index
    n = valid.sum().double() if reduction == "mean" else torch.tensor(1.0, dtype=torch.float64)
    safe_t = torch.where(valid, target, torch.zeros_like(target))
    nll = lse - z.gather(1, safe_t[:, None])[:, 0]                      # :172 loss = lse - ori_X_y
    rows = nll
    if label_smoothing > 0:
        eps = label_smoothing / V
        smooth = (-eps * z).sum(dim=1) + label_smoothing * lse           # :183
        rows = nll * (1 - label_smoothing) + smooth                      # :184
    z_rows = lse_square_scale * lse * lse                                # :188
    rows = rows + z_rows
    zero = torch.zeros_like(rows)
    rows = torch.where(valid, rows, zero) / n                            # ignored rows contribute nothing (:79-84)
    z_rows = torch.where(valid, z_rows, zero) / n
    loss = rows.sum()                                                    # :272 torch.sum(loss_1d)
    (grad,) = torch.autograd.grad(loss, x)
    return loss.detach(), z_rows.sum().detach(), grad
