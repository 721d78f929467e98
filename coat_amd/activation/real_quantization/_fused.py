"""Shared marshalling of the fused element-wise entry points (SiLU / GELU / mul / add)."""
import torch

from ... import _hip
from .common import flatten_2d, new_max  # noqa: F401  (re-exported for the fused launchers)


def prep_pg(x, s_x):
    """Flatten a per-group FP8 tensor and its scales to 2-D dense GPU tensors; returns (x2d, s2d, batch)."""
    x, batch = flatten_2d(x)
    s_x, _ = flatten_2d(s_x)
    return _hip.dense(x), _hip.dense(s_x), batch


def prep_bf16(g):
    g, _ = flatten_2d(g)
    if g.dtype != torch.bfloat16:
        g = g.to(torch.bfloat16)
    return _hip.dense(g)
