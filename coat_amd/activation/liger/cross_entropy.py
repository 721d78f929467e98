"""Fused cross-entropy of the LM head: loss and, in place of the logits, their gradient.
Reference: coat/activation/liger/cross_entropy.py (kernel :24-198, host :212-411).  Same names, arguments, defaults
and return values; the kernel underneath is coat_amd/csrc/cross_entropy.hip.  Two host synchronisations of the
reference are gone: the count of non-ignored targets stays on the device (reference :240 calls ``.item()``), and the
"is grad_output exactly 1" test of the backward (reference :283, ``torch.equal``) is made by the kernel itself."""
from typing import Optional

import torch

from ... import _hip

_REDUCTION = {"none": 0, "mean": 1, "sum": 2}


def _check_input(_input):
    if _input.dim() != 2:
        raise ValueError(f"expected logits of shape (BT, V), got {tuple(_input.shape)}")
    if not _input.is_cuda:
        raise RuntimeError("coat_amd kernels need tensors on the GPU (got a %s tensor)" % _input.device.type)
    _hip.dt(_input)  # raises on an unsupported dtype


def cross_entropy_forward(_input, target, ignore_index, lse_square_scale, label_smoothing, reduction, softcap,
                          return_z_loss):
    """Returns (loss, z_loss or None, _input); ``_input`` now holds d loss / d logits (reference :212-278)."""
    if return_z_loss not in (True, False, 0, 1):
        raise AssertionError(f"return_z_loss must be True or False. Got: {return_z_loss}")
    if reduction not in _REDUCTION:
        raise ValueError(f"reduction must be 'none', 'mean' or 'sum', got {reduction!r}")
    _check_input(_input)
    BT, V = _input.shape
    if target.shape != (BT,):
        raise ValueError(f"target must have shape ({BT},), got {tuple(target.shape)}")
    # unreduced loss, in the logits' dtype as in the reference (:234-238); every row is written by the kernel
    loss_1d = torch.empty(BT, dtype=_input.dtype, device=_input.device)
    z_loss_1d = torch.empty(BT, dtype=_input.dtype, device=_input.device) if return_z_loss else None
    target = target.to(device=_input.device, dtype=torch.int64).contiguous()
    n_non_ignore = (target != ignore_index).sum()  # int64 scalar on the device
    if _input.stride(-1) != 1:
        _input = _input.contiguous()
    _hip.check(_hip.lib().coat_cross_entropy_forward(
        _hip.ptr(_input), _hip.dt(_input), _input.stride(0), _hip.ptr(target), _hip.ptr(loss_1d), _hip.ptr(z_loss_1d),
        _hip.ptr(n_non_ignore), BT, V, int(ignore_index), float(lse_square_scale), float(label_smoothing),
        _REDUCTION[reduction], float(softcap) if softcap is not None else 0.0, 0 if softcap is None else 1,
        _hip.stream(_input.device)), "cross_entropy_forward")
    loss = torch.sum(loss_1d)
    z_loss = torch.sum(z_loss_1d) if return_z_loss else None
    return loss, z_loss, _input


def cross_entropy_backward(_input, grad_output):
    """_input *= grad_output in place (reference :281-302); untouched when grad_output is exactly 1."""
    _check_input(_input)
    BT, V = _input.shape
    if grad_output.numel() != 1:
        raise ValueError("grad_output must be a scalar")
    g = grad_output.to(_input.device)
    if g.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        g = g.float()
    _hip.check(_hip.lib().coat_cross_entropy_scale_grad(
        _hip.ptr(_input), _hip.dt(_input), _input.stride(0), _hip.ptr(g), _hip.dt(g), BT, V,
        _hip.stream(_input.device)), "cross_entropy_backward")
    return _input


class LigerCrossEntropyFunction(torch.autograd.Function):
    """autograd wrapper with the reference's signature (reference :305-384).  The logits are overwritten by their
    gradient in the forward pass; the backward only rescales them."""

    @staticmethod
    def forward(ctx, _input: torch.Tensor, target: torch.Tensor, ignore_index: int = -100,
                lse_square_scale: float = 0.0, label_smoothing: float = 0.0, reduction: str = "mean",
                softcap: Optional[float] = None, return_z_loss: bool = False):
        loss, z_loss, _input = cross_entropy_forward(_input, target, ignore_index, lse_square_scale, label_smoothing,
                                                     reduction, softcap, return_z_loss)
        ctx.save_for_backward(_input.detach())
        ctx.return_z_loss = return_z_loss
        return loss, z_loss

    @staticmethod
    def backward(ctx, grad_output, grad_ouput2):
        (_input,) = ctx.saved_tensors
        _input = cross_entropy_backward(_input, grad_output)
        return (_input, None, None, None, None, None, None, None)


def liger_fixed_cross_entropy(source, target, num_items_in_batch: int = None, ignore_index: int = -100, **kwargs):
    """Reference :387-393."""
    reduction = "sum" if num_items_in_batch is not None else "mean"
    loss, _ = LigerCrossEntropyFunction.apply(source, target, ignore_index, 0.0, 0.0, reduction)
    if reduction == "sum":
        loss = loss / num_items_in_batch
    return loss


def LigerForCausalLMLoss(logits, labels, vocab_size: int, num_items_in_batch: int = None, ignore_index: int = -100,
                         **kwargs):
    """Shifted next-token loss on fp32 logits (reference :396-411)."""
    logits = logits.float()
    shift_logits = logits[..., :-1, :].contiguous()
    shift_labels = labels[..., 1:].contiguous()
    shift_logits = shift_logits.view(-1, vocab_size)
    shift_labels = shift_labels.view(-1).to(shift_logits.device)
    return liger_fixed_cross_entropy(shift_logits, shift_labels, num_items_in_batch, ignore_index, **kwargs)
