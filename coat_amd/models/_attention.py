"""bf16 scaled-dot-product attention for the decoder layers.

The reference calls the flash-attn library here (coat/models/coat_llama.py:960-971 through transformers).  The forward
of the case the layers use (bf16, causal, no mask, no dropout, head dimension 128) is this library's MFMA kernel
(``coat_attention_forward_bf16``: online softmax, K and V tiles through LDS); its backward is torch's
memory-efficient attention backward, which takes the forward's output and log-sum-exp.  Everything else goes to
``torch.nn.functional.scaled_dot_product_attention`` with the backend order that is fastest on MI355X: on this ROCm
build torch picks its "flash" backend by default, while for the layers' shapes (batch 4, 32 heads, 2048 tokens) its
"memory-efficient" backend runs forward + backward in 1.40 ms against 2.66 ms."""
import math

import torch
import torch.nn.functional as F
from torch.nn.attention import SDPBackend, sdpa_kernel

BACKEND_PRIORITY = [SDPBackend.EFFICIENT_ATTENTION, SDPBackend.FLASH_ATTENTION, SDPBackend.MATH]


def _strides_bshd(t):
    """(batch, token, head) element strides of a [B, heads, S, D] tensor whose last dimension is contiguous."""
    return t.stride(0), t.stride(2), t.stride(1)


def attention_forward(q, k, v, causal=True, scale=None, need_lse=True, out_scale_max=None, out_fp8=None):
    """q [B, H, S, 128], k / v [B, Hkv, S, 128], bf16, any strides with a contiguous last dimension (the transposed views
    of [B, S, H, 128] projections are used where they lie).  Returns (out [B, H, S, 128] laid out as [B, S, H, 128],
    lse fp32 [B, H, S] or None).  ``out_scale_max`` (a ``new_max`` buffer) receives the maximum of the output's group
    scales for the FP8 format ``out_fp8``."""
    from .. import _hip
    B, H, S, D = q.shape
    Hkv = k.shape[1]
    scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
    for t in (q, k, v):
        if t.stride(3) != 1 or any(s % 8 for s in t.stride()[:3]) or t.data_ptr() % 16:
            raise ValueError("attention_forward: the head dimension must be contiguous and rows 16-byte aligned")
    lib, st = _hip.lib(), _hip.stream(q.device)
    out = torch.empty((B, S, H, D), dtype=torch.bfloat16, device=q.device).transpose(1, 2)
    lse = torch.empty((B, H, S), dtype=torch.float32, device=q.device) if need_lse else None
    _hip.check(lib.coat_attention_forward_bf16(_hip.ptr(q), _hip.ptr(k), _hip.ptr(v), _hip.ptr(out), _hip.ptr(lse), B, H, Hkv, S, D,
                                               *_strides_bshd(q), *_strides_bshd(k), *_strides_bshd(v), *_strides_bshd(out),
                                               scale, 1 if causal else 0, _hip.ptr(out_scale_max),
                                               _hip.fp8(out_fp8) if out_scale_max is not None else 0, st), "attention forward")
    return out, lse


class _CausalAttention(torch.autograd.Function):
    """Forward: this library's kernel.  Backward: torch's memory-efficient attention backward on (q, k, v, out, lse)."""

    @staticmethod
    def forward(ctx, q, k, v, out_scale_max=None, out_fp8=None):
        out, lse = attention_forward(q, k, v, causal=True, out_scale_max=out_scale_max, out_fp8=out_fp8)
        ctx.save_for_backward(q, k, v, out, lse)
        return out

    @staticmethod
    def backward(ctx, g):
        q, k, v, out, lse = ctx.saved_tensors
        zero = torch.zeros((), dtype=torch.int64)  # dropout state, unused with dropout_p = 0
        dq, dk, dv, _ = torch.ops.aten._scaled_dot_product_efficient_attention_backward(
            g, q, k, v, None, out, lse, zero, zero, 0.0, [True, True, True, False], True)
        return dq, dk, dv, None, None


def _own_kernel_applies(q, k, v, attn_mask, dropout_p, is_causal):
    return (q.is_cuda and is_causal and attn_mask is None and dropout_p == 0.0 and q.dtype == k.dtype == v.dtype == torch.bfloat16
            and q.dim() == 4 and q.shape[-1] == 128 and k.shape == v.shape and k.shape[1] == q.shape[1]
            and q.shape[2] == k.shape[2] and all(t.stride(3) == 1 and not any(s % 8 for s in t.stride()[:3]) and t.data_ptr() % 16 == 0
                                                   for t in (q, k, v)))


def torch_sdpa(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False):
    """torch's own attention, forward and backward, with the backend order above (what the layers used before this
    library had a forward kernel, and what a plain bf16 torch layer uses)."""
    if not q.is_cuda:
        return F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal)
    with sdpa_kernel(BACKEND_PRIORITY, set_priority=True):
        return F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal)


def sdpa(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False, out_scale_max=None, out_fp8=None):
    """Attention of the decoder layers.  With ``out_scale_max`` (a ``new_max`` buffer) returns (out, filled): the library's
    kernel also merges the maximum of the output's group scales for the FP8 format ``out_fp8`` into the buffer; filled is
    False when torch's attention ran instead and the buffer was left alone."""
    if _own_kernel_applies(q, k, v, attn_mask, dropout_p, is_causal):
        out = _CausalAttention.apply(q, k, v, out_scale_max, out_fp8)
        return out if out_scale_max is None else (out, True)
    out = torch_sdpa(q, k, v, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal)
    return out if out_scale_max is None else (out, False)
