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


def fp8matmul_add(a, b, residual, scale_a, scale_b, fp8type=None, QB=16, bias=None):
    """``fp8matmul(a, b, False, ...)`` followed by the addition of the bf16 tensor ``residual``, in one kernel:
    returns ``y = bf16(float(product) + float(residual))`` and, with ``fp8type``, ``(y, (q, s))`` where q / s are the
    1 x 16 per-group FP8 codes and bf16 scales of the fp32 sum: what ``fp8_add_Ifp_Ifp_Ofp_Og16(residual, product, fp8type,
    16)`` returns (reference add_fwd.py:162-213 after linear.py:172-250), bit for bit.  Falls back to the two kernels for
    shapes the fused epilogue does not take."""
    from .add_fwd import fp8_add_Ifp_Ifp_Ofp_Og16
    from .common import as_fp8_dtype
    lead = a.shape[:-1]
    a2 = a.reshape(-1, a.shape[-1])
    r2 = residual.reshape(-1, residual.shape[-1])
    N = b.shape[1]
    fused = (residual.dtype == torch.bfloat16 and N % 8 == 0 and (fp8type is None or (QB == 16 and N % 16 == 0))
             and tuple(r2.shape) == (a2.shape[0], N))
    if not fused:
        prod = fp8matmul(a2, b, False, scale_a, scale_b, QB, bias)
        if fp8type is None:
            return (prod + r2).reshape(*lead, N)
        y, (q, sq) = fp8_add_Ifp_Ifp_Ofp_Og16(r2, prod, fp8type, QB)
        return y.reshape(*lead, N), (q.reshape(*lead, N), sq.reshape(*lead, N // QB))
    assert a2.shape[1] == b.shape[0], "Incompatible dimensions"
    a2, r2 = _hip.dense(a2), _hip.dense(r2)
    bn = _hip.dense(_k_contiguous_rows(b))
    M, K = a2.shape
    for t in (scale_a, scale_b):
        if t.numel() != 1:
            raise ValueError("fp8matmul takes per-tensor (single element) scales")
    scale_a = scale_a if scale_a.is_cuda else scale_a.to(a2.device)
    scale_b = scale_b if scale_b.is_cuda else scale_b.to(a2.device)
    if bias is not None:
        bias = _hip.dense(bias)
    y = torch.empty((M, N), device=a2.device, dtype=torch.bfloat16)
    q = sq = None
    kind = 0
    if fp8type is not None:
        fp8type = as_fp8_dtype(fp8type)
        q = torch.empty((M, N), device=a2.device, dtype=fp8type)
        sq = torch.empty((M, N // 16), device=a2.device, dtype=torch.bfloat16)
        kind = _OUT_KIND[fp8type]
    _hip.check(_hip.lib().coat_fp8_gemm_residual(
        _hip.ptr(a2), _hip.fp8(a2.dtype), _hip.ptr(bn), _hip.fp8(bn.dtype), _hip.ptr(r2), _hip.ptr(y), _hip.ptr(q), _hip.ptr(sq),
        kind, _hip.ptr(scale_a), _hip.dt(scale_a), _hip.ptr(scale_b), _hip.dt(scale_b), _hip.ptr(bias),
        _hip.dt(bias) if bias is not None else 0, M, N, K, _hip.stream(a2.device)), "fp8matmul_add")
    y = y.reshape(*lead, N)
    if fp8type is None:
        return y
    return y, (q.reshape(*lead, N), sq.reshape(*lead, N // 16))


def fp8_linear_forward_add(x, s, w, s_w, residual, fp8type, QB, bias=None):
    """``fp8_add_Ifp_Ifp_Ofp_Og16(residual, fp8_linear_forward(x, s, w, s_w, False, QB, bias), fp8type, QB)`` in one
    kernel: the projection that closes a residual branch (reference coat_llama.py:440-441, :673-674)."""
    assert s.numel() == 1, f"X uses per-tensor quantization in linear forward, but the scale shape is {s.shape}"
    assert s_w.numel() == 1, f"W uses per-tensor quantization in linear forward, but the scale shape is {s_w.shape}"
    return fp8matmul_add(x, w.t(), residual, s, s_w, fp8type, QB, bias)


_MAX_GROUP = 4  # problems per grouped launch (kMaxGroup of the kernel)


def fp8matmul_grouped(a_list, b_list, output_quantize, scale_a_list, scale_b_list, QB):
    """``[fp8matmul(a, b, output_quantize, sa, sb, QB) for ...]`` with the problems that share a shape and formats (2-D
    ``a``, no bias) in one launch each: the q / k / v or gate / up projections of a layer and their backward products.
    The results are bit-identical to the separate calls; on the persistent grid the problems' tiles form one sequence,
    so a partial last round of tiles is paid once per group.  Problems of different shapes form groups of their own
    (grouped-query attention: k and v share a launch, q takes its own); a problem alone in its group, or one the
    grouped kernel does not take, is a separate call."""
    n = len(a_list)
    assert n == len(b_list) == len(scale_a_list) == len(scale_b_list)

    def signature(i):
        a, b, sa, sb = a_list[i], b_list[i], scale_a_list[i], scale_b_list[i]
        if not (a.dim() == 2 and a.is_contiguous() and b.t().is_contiguous() and sa.numel() == 1 and sb.numel() == 1
                and sa.is_cuda and sb.is_cuda):
            return None
        return (tuple(a.shape), a.dtype, tuple(b.shape), b.dtype, sa.dtype, sb.dtype)

    groups = {}
    for i in range(n):
        sig = signature(i)
        groups.setdefault(sig if sig is not None else ("alone", i), []).append(i)
    out = [None] * n
    for sig, idx in groups.items():
        for at in range(0, len(idx), _MAX_GROUP):
            part = idx[at:at + _MAX_GROUP]
            if len(part) == 1 or sig[0] == "alone":
                for i in part:
                    out[i] = fp8matmul(a_list[i], b_list[i], output_quantize, scale_a_list[i], scale_b_list[i], QB)
            else:
                res = _matmul_group([a_list[i] for i in part], [b_list[i] for i in part], output_quantize,
                                    [scale_a_list[i] for i in part], [scale_b_list[i] for i in part], QB)
                for i, r in zip(part, res):
                    out[i] = r
    return out


def _matmul_group(a_list, b_list, output_quantize, scale_a_list, scale_b_list, QB):
    """One launch for 2 .. 4 problems of one shape, one pair of formats and one pair of scale dtypes."""
    n = len(a_list)
    a_list = [_hip.dense(a) for a in a_list]
    bn_list = [_hip.dense(b.t()) for b in b_list]
    M, K = a_list[0].shape
    N = bn_list[0].shape[0]
    assert K == bn_list[0].shape[1], "Incompatible dimensions"
    dev = a_list[0].device
    if output_quantize:
        c_list = [torch.empty((M, N), device=dev, dtype=a_list[0].dtype) for _ in range(n)]
        cs_list = [torch.empty((M, N // QB), device=dev, dtype=torch.bfloat16) for _ in range(n)]
        kind = _OUT_KIND[a_list[0].dtype]
    else:
        c_list = [torch.empty((M, N), device=dev, dtype=torch.bfloat16) for _ in range(n)]
        cs_list, kind = None, 0
    _hip.check(_hip.lib().coat_fp8_gemm_grouped(
        n, _hip.ptr_array(a_list), _hip.fp8(a_list[0].dtype), _hip.ptr_array(bn_list), _hip.fp8(bn_list[0].dtype),
        _hip.ptr_array(c_list), _hip.ptr_array(cs_list) if cs_list else None, kind,
        _hip.ptr_array(scale_a_list), _hip.dt(scale_a_list[0]), _hip.ptr_array(scale_b_list), _hip.dt(scale_b_list[0]),
        None, 0, M, N, K, QB if output_quantize else 0, _hip.stream(dev)), "fp8matmul_grouped")
    return list(zip(c_list, cs_list)) if output_quantize else c_list


def fp8_linear_forward_grouped(x, s, w_list, s_w_list, output_quantize, QB):
    """``[fp8_linear_forward(x, s, w, s_w, output_quantize, QB) for ...]`` for projections of one input."""
    assert s.numel() == 1, f"X uses per-tensor quantization in linear forward, but the scale shape is {s.shape}"
    n = len(w_list)
    x2 = x.reshape(-1, x.shape[-1]) if x.dim() == 3 else x
    outs = fp8matmul_grouped([x2] * n, [w.t() for w in w_list], output_quantize, [s] * n, s_w_list, QB)
    if x.dim() != 3:
        return outs
    lead = x.shape[:2]
    if output_quantize:
        return [(c.reshape(*lead, -1), cs.reshape(*lead, -1)) for c, cs in outs]
    return [c.reshape(*lead, -1) for c in outs]


def fp8_linear_backward_grouped(x_t, s, g_list, s_g_list, g_t_list, w_t_list, s_w_list, QB):
    """``[fp8_linear_backward(x_t, s, g, s_g, g_t, w_t, s_w, QB) for ...]`` for projections of one input: the dgrads in
    one launch and the wgrads in another.  Returns (list of dx, list of dW)."""
    n = len(g_list)
    assert s.numel() == 1 and all(t.numel() == 1 for t in (*s_g_list, *s_w_list)), "per-tensor scales in linear backward"
    g2 = [g.reshape(-1, g.shape[-1]) if g.dim() == 3 else g for g in g_list]
    dx = fp8matmul_grouped(g2, [w_t.t() for w_t in w_t_list], False, s_g_list, s_w_list, QB)
    dx = [d.reshape(*g.shape[:2], -1) if g.dim() == 3 else d for d, g in zip(dx, g_list)]
    dw = fp8matmul_grouped(g_t_list, [x_t.t()] * n, False, s_g_list, [s] * n, QB)
    return dx, dw


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
