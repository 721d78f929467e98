"""CPU restatement of the attention between the FP8 projections.  TEST INFRASTRUCTURE: imported by tests/, by
__graft_entry__.smoke() and by the cpu_baseline leg of bench.py only; the product never calls it.

The reference hands this step to the flash-attn library through transformers (coat/models/coat_llama.py:960-971, called from
LlamaAttentionWithoutLinear / LlamaFlashAttention2WithoutLinear :981-1074): softmax(q k^T * scale (+ causal mask)) v per
(batch, head) on bf16 q / k / v.  flash-attn is not part of the reference's sources; what is restated here is the
published definition, evaluated in fp32 on the bf16 inputs: the scores, the mask, the row maximum, the exponentials,
their sum and the weighted sum of v, written out step by step, plus the natural log-sum-exp that backward kernels take.

Pinned (tests/test_oracle_attention.py) against torch's own CPU scaled_dot_product_attention in fp32, against
closed forms (a single visible key returns its value row; equal scores return the running mean of v; adding a constant
to all scores changes nothing but the log-sum-exp) and against the definition with grouped-query heads repeated by hand."""
import math

import torch


def attention(q, k, v, causal=True, scale=None):
    """q [B, H, S, D], k / v [B, Hkv, S, D] (any float dtype; H % Hkv == 0: grouped-query heads share k / v).
    Returns (out fp32 [B, H, S, D], lse fp32 [B, H, S], natural logarithm)."""
    B, H, S, D = q.shape
    Hkv = k.shape[1]
    if H % Hkv:
        raise ValueError("heads must be a multiple of kv heads")
    scale = 1.0 / math.sqrt(D) if scale is None else float(scale)
    qf, kf, vf = q.float(), k.float(), v.float()
    if Hkv != H:
        rep = H // Hkv
        kf = kf.repeat_interleave(rep, dim=1)
        vf = vf.repeat_interleave(rep, dim=1)
    s = torch.matmul(qf, kf.transpose(-1, -2)) * scale
    if causal:
        hidden = torch.triu(torch.ones(S, k.shape[2], dtype=torch.bool, device=q.device), diagonal=1)
        s = s.masked_fill(hidden, float("-inf"))
    m = s.max(dim=-1, keepdim=True).values
    p = torch.exp(s - m)
    l = p.sum(dim=-1, keepdim=True)
    out = torch.matmul(p, vf) / l
    return out, (m + torch.log(l)).squeeze(-1)
