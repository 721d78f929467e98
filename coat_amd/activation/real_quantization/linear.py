"""Per-tensor-scaled FP8 matmul and the linear forward / backward built on it.
Reference: coat/activation/real_quantization/linear.py:172-302."""
import torch

from ... import _hip
from ._transpose import fp8_transpose
from .common import no_stochastic

_OUT_KIND = {torch.float8_e4m3fn: 1, torch.float8_e5m2: 2}


def _k_contiguous_rows(b):
    """``b`` is the [K, N] right operand.  The kernels (like the reference's callers) want it as the ``.t()``
    view of a row-major [N, K] matrix; a genuinely row-major [K, N] operand is transposed once."""
    bt = b.t()
    if bt.is_contiguous():
        return bt
    return fp8_transpose(b.contiguous(), transpose_output_2d=True)


def fp8matmul(a, b, output_quantize, scale_a, scale_b, QB, bias=None, stochastic=False):
    """a [M, K] fp8 (or [B, S, K]), b [K, N] fp8 -> bf16 [M, N], or (fp8 [M, N], bf16 scales [M, N/QB]) when
    ``output_quantize``; result = (a @ b) * float(scale_a) * float(scale_b) (+ bias)."""
    no_stochastic(stochastic, "the reference's GEMM epilogue loads its noise with boundary_check on a plain "
                  "pointer (linear.py:151-152), which Triton rejects, so there is no behaviour to match")
    batch = None
    if a.dim() == 3:
        batch = a.shape[0]
        a = a.reshape(-1, a.shape[2])
    assert a.shape[1] == b.shape[0], "Incompatible dimensions"
    assert a.is_contiguous(), "Matrix A must be contiguous"
    a = _hip.dense(a)
    bn = _hip.dense(_k_contiguous_rows(b))
    M, K = a.shape
    N = bn.shape[0]
    for s in (scale_a, scale_b):
        if s.numel() != 1:
            raise ValueError("fp8matmul takes per-tensor (single element) scales")
    scale_a = scale_a if scale_a.is_cuda else scale_a.to(a.device)
    scale_b = scale_b if scale_b.is_cuda else scale_b.to(a.device)
    # each scale is read in its own dtype and the two are multiplied in fp32 (reference linear.py:123-125): an fp32
    # weight scale next to a bf16 activation scale is used with all its bits
    if bias is not None:
        bias = _hip.dense(bias)
    if output_quantize:
        c = torch.empty((M, N), device=a.device, dtype=a.dtype)
        scale_c = torch.empty((M, N // QB), device=a.device, dtype=torch.bfloat16)
        kind = _OUT_KIND[a.dtype]
    else:
        c = torch.empty((M, N), device=a.device, dtype=torch.bfloat16)
        scale_c, kind = None, 0
    _hip.check(_hip.lib().coat_fp8_gemm(
        _hip.ptr(a), _hip.fp8(a.dtype), _hip.ptr(bn), _hip.fp8(bn.dtype), _hip.ptr(c), _hip.ptr(scale_c), kind,
        _hip.ptr(scale_a), _hip.dt(scale_a), _hip.ptr(scale_b), _hip.dt(scale_b), _hip.ptr(bias), _hip.dt(bias) if bias is not None else 0,
        M, N, K, QB if output_quantize else 0, _hip.stream(a.device)), "fp8matmul")
    if batch is not None:
        c = c.reshape(batch, -1, N)
        if output_quantize:
            return c, scale_c.reshape(batch, -1, N // QB)
        return c
    return (c, scale_c) if output_quantize else c


def fp8_linear_forward(x, s, w, s_w, output_quantize, QB, bias=None):
    """y = x @ w^T with w [N, K] (reference :253-258)."""
    assert s.numel() == 1, f"X uses per-tensor quantization in linear forward, but the scale shape is {s.shape}"
    assert s_w.numel() == 1, f"W uses per-tensor quantization in linear forward, but the scale shape is {s_w.shape}"
    return fp8matmul(x, w.t(), output_quantize, s, s_w, QB, bias)


def fp8_linear_backward(x_t, s, g, s_g, g_t, w_t, s_w, QB, bias=None, stochastic=False, dgrad_quantize=False):
    """dgrad = g @ w (through w_t [K, N]) and wgrad = g^T @ x (through g_t [N, M] and x_t [K, M]), reference :272-302.
    Returns (dx, dW) or, with dgrad_quantize, (dx fp8, per-group scales, dW)."""
    assert s.numel() == 1, f"X uses per-tensor quantization in linear backward, but the scale shape is {s.shape}"
    assert s_g.numel() == 1, f"G uses per-tensor quantization in linear backward, but the scale shape is {s.shape}"
    assert s_w.numel() == 1, f"W uses per-tensor quantization in linear backward, but the scale shape is {s_w.shape}"
    batch = None
    if g.dim() == 3:
        batch = g.shape[0]
        g = g.reshape(-1, g.shape[-1])
    if dgrad_quantize:
        y, s_y = fp8matmul(g, w_t.t(), True, s_g, s_w, QB, stochastic=stochastic)
    else:
        y = fp8matmul(g, w_t.t(), False, s_g, s_w, QB)
    w_g = fp8matmul(g_t, x_t.t(), False, s_g, s, QB)
    if batch is not None:
        y = y.reshape(batch, -1, y.shape[-1])
        if dgrad_quantize and s_y.numel() > 1:
            s_y = s_y.reshape(batch, -1, s_y.shape[-1])
    return (y, s_y, w_g) if dgrad_quantize else (y, w_g)
