"""CPU: oracle/attention_ref.py pinned against torch's scaled_dot_product_attention and closed forms."""
import math

import torch
import torch.nn.functional as F

from oracle import attention_ref as A


def _qkv(B, H, S, D, seed, Hkv=None):
    g = torch.Generator().manual_seed(seed)
    Hkv = H if Hkv is None else Hkv
    return (torch.randn(B, H, S, D, generator=g).bfloat16(), torch.randn(B, Hkv, S, D, generator=g).bfloat16(),
            torch.randn(B, Hkv, S, D, generator=g).bfloat16())


def test_against_torch_sdpa_fp32():
    for causal in (True, False):
        q, k, v = _qkv(2, 3, 77, 64, 1)
        out, lse = A.attention(q, k, v, causal=causal)
        want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=causal)
        assert (out - want).abs().max() < 2e-6
        s = q.float() @ k.float().transpose(-1, -2) / math.sqrt(64)
        if causal:
            s = s.masked_fill(torch.triu(torch.ones(77, 77, dtype=torch.bool), 1), float("-inf"))
        assert (lse - torch.logsumexp(s, -1)).abs().max() < 2e-6
    # a custom scale is the factor on the scores
    q, k, v = _qkv(1, 2, 33, 32, 2)
    out, _ = A.attention(q, k, v, causal=True, scale=0.3)
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True, scale=0.3)
    assert (out - want).abs().max() < 2e-6


def test_closed_forms():
    q, k, v = _qkv(1, 2, 40, 16, 3)
    out, lse = A.attention(q, k, v, causal=True)
    # the first query sees one key: its value row, and log-sum-exp = its score
    assert torch.equal(out[:, :, 0], v.float()[:, :, 0])
    s00 = (q.float()[:, :, 0] * k.float()[:, :, 0]).sum(-1) / 4.0
    assert (lse[:, :, 0] - s00).abs().max() < 1e-6
    # equal scores (k = 0): causal running mean of v, lse = log(number of visible keys)
    out0, lse0 = A.attention(q, torch.zeros_like(k), v, causal=True)
    want = v.float().cumsum(2) / torch.arange(1, 41).view(1, 1, -1, 1)
    assert (out0 - want).abs().max() < 1e-5
    assert (lse0 - torch.log(torch.arange(1, 41).float())).abs().max() < 1e-6
    # a constant added to every score of a query moves only the log-sum-exp: append a dimension that is 1 in k and c_i in q
    c = torch.randn(1, 2, 40, 1).bfloat16()
    q2 = torch.cat([q, c], -1)
    k2 = torch.cat([k, torch.ones(1, 2, 40, 1).bfloat16()], -1)
    out2, lse2 = A.attention(q2, k2, v, causal=True, scale=0.25)
    assert (out2 - out).abs().max() < 2e-5
    assert (lse2 - (lse + 0.25 * c.float().squeeze(-1))).abs().max() < 2e-5


def test_grouped_query_heads_are_repeated():
    q, k, v = _qkv(2, 6, 25, 32, 4, Hkv=2)
    out, lse = A.attention(q, k, v)
    for h in range(6):
        o1, l1 = A.attention(q[:, h:h + 1], k[:, h // 3:h // 3 + 1], v[:, h // 3:h // 3 + 1])
        assert torch.equal(out[:, h:h + 1], o1) and torch.equal(lse[:, h:h + 1], l1)
