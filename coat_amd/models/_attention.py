"""bf16 scaled-dot-product attention for the decoder layers: torch's fused kernels, with the backend order that is
fastest on MI355X.

The reference calls the flash-attn library here (coat/models/coat_llama.py:960-971 through transformers); this build
calls ``torch.nn.functional.scaled_dot_product_attention``.  On this ROCm build torch picks its "flash" backend by
default; for the shapes of the decoder layers (batch 4, 32 heads, 2048 tokens, head dimension 128, causal) its
"memory-efficient" backend runs forward + backward in 1.40 ms against 2.66 ms, so that one is tried first and the
others stay as fallbacks for arguments it does not take.  The mathematics is the same."""
import torch.nn.functional as F
from torch.nn.attention import SDPBackend, sdpa_kernel

BACKEND_PRIORITY = [SDPBackend.EFFICIENT_ATTENTION, SDPBackend.FLASH_ATTENTION, SDPBackend.MATH]


def sdpa(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False):
    if not q.is_cuda:
        return F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal)
    with sdpa_kernel(BACKEND_PRIORITY, set_priority=True):
        return F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal)
