"""torch-CPU restatement of the reference's FP8 activation kernels.  TEST INFRASTRUCTURE ONLY.

Paths are relative to the reference repository root; ``rq/`` abbreviates
``coat/activation/real_quantization/``.  Every function works on 2-D ``[M, N]`` CPU
tensors (the reference flattens 3-D inputs the same way, e.g. rq/_quantize.py:122-126) and
performs every arithmetic step in IEEE fp32 exactly where the kernel does it in fp32.

Definition choices (stated once, used everywhere):
  * group scale  s32 = (max|v| + 1e-10) / fp8max, fp32 (rq/_quantize.py:80-82); the value
    is divided by s32 and the scale is *stored* rounded to bf16 (rq/_quantize.py:86-90).
  * fp32 -> fp8 is round-to-nearest-even with saturation to the largest finite value
    (Triton ``.to(fp8)`` lowers to PTX cvt.rn.satfinite); NaN stays NaN.
  * division is IEEE fp32 division (Triton's tl.fdiv is a fast division and is not a
    reproducible target).
  * exp / erf are torch-CPU's (<= 1 ulp); kernels that contain them are compared within a
    stated mismatch rate, not bit-for-bit.

Pin status (tests/test_oracle_activation.py unless noted):
  cast_fp8                 oracle/fp8_codec.py brute force + torch cast (tests/test_oracle_fp8.py)
  fp8_quantize             closed form on hand-made groups; dequantize(quantize(x)) error bound
                           (half an fp8 step of the group maximum); scale = bf16((amax+1e-10)/448)
                           recomputed in float64; equal-fraction >= 0.95 against the reference
                           test's own definition ``quantize_tensor_ref_test`` (tests/test_utils.py:61-67)
  fp8_quantize_transpose   == fp8_quantize(x.T) (invariant)
  fp8_quantize_perblock*   block maxima and scales recomputed with plain loops in float64; closed form on hand-made
                           blocks; error bound of half an fp8 step of the block maximum; a block as large as the
                           tensor == fp8_division by the fp32 scale; transposed outputs == outputs transposed;
                           per-group part == fp8_quantize; equal-fraction >= 0.95 against the reference test's own
                           definition (tests/test_utils.py:53-60)
  fp8_group_scales, fp8_quantize_pertensor*  per-tensor scale == bf16 of the max group scale
                           (monotone rounding); codes == cast(x / s)
  fp8_division*            transposed output == output.T; absmax scale in the input dtype
  fp8_dequantize           float64 product rounded once
  fp8matmul                float64 matmul of the decoded operands (tests/test_fp8_linear.py:120-124)
  silu/gelu/mul/add/rmsnorm fwd+bwd  torch.nn.functional + autograd on the dequantized inputs
                           (tests/test_fp8_activations.py:50-182, tests/test_fp8_norm.py:92-123)
"""
import math

import torch

SCALE_MIN_THRES = 1e-10  # rq/common.py:20
FP8_MAX_VALUE = {torch.float8_e4m3fn: 448.0, torch.float8_e5m2: 57344.0}  # rq/common.py:22-25
STR2FP8 = {"E4M3": torch.float8_e4m3fn, "E5M2": torch.float8_e5m2}  # rq/common.py:27


def _fp8(fp8type):
    return STR2FP8[fp8type] if isinstance(fp8type, str) else fp8type


def cast_fp8(v32, fp8type):
    """fp32 -> fp8, RNE + satfinite (PTX cvt.rn.satfinite, used by every ``.to(fp8)`` in rq/)."""
    fp8type = _fp8(fp8type)
    mx = FP8_MAX_VALUE[fp8type]
    return torch.clamp(v32.float(), -mx, mx).to(fp8type)  # clamp keeps NaN


def _groups(v32, QB):
    M, N = v32.shape
    return v32.reshape(M, N // QB, QB)


def _group_scale32(v32, QB, fp8type):
    """rq/_quantize.py:79-82: max|v| over each 1xQB group, + 1e-10, / fp8max, all fp32."""
    amax = _groups(v32, QB).abs().amax(dim=2)
    return (amax + SCALE_MIN_THRES) / FP8_MAX_VALUE[_fp8(fp8type)]


def _quantize_pg(v32, QB, fp8type, scale_dtype=torch.bfloat16):
    """rq/_quantize.py:76-91 on an fp32 value tensor: (codes, stored scales)."""
    M, N = v32.shape
    s32 = _group_scale32(v32, QB, fp8type)
    q = cast_fp8((_groups(v32, QB) / s32.unsqueeze(2)).reshape(M, N), fp8type)
    return q, s32.to(scale_dtype)


# ----------------------------------------------------------------------------- quantize family
def fp8_quantize(x, QB, fp8type, scale_dtype=torch.bfloat16):
    """rq/_quantize.py:120-163 (kernel :37-113)."""
    return _quantize_pg(x.float(), QB, fp8type, scale_dtype)


def fp8_quantize_transpose(x, QB, fp8type, scale_dtype=torch.bfloat16):
    """rq/_quantize_transpose.py:175-226: per-group quantize of x and of x^T (kernel :127-137)."""
    x32 = x.float()
    return _quantize_pg(x32, QB, fp8type, scale_dtype), _quantize_pg(x32.t().contiguous(), QB, fp8type, scale_dtype)


def _block_scale32(v32, QB, fp8type):
    """rq/_quantize_perblock.py:72-75: max|v| over each QB x QB block, + 1e-10, / fp8max, all fp32."""
    M, N = v32.shape
    amax = v32.reshape(M // QB, QB, N // QB, QB).abs().amax(dim=(1, 3))
    return (amax + SCALE_MIN_THRES) / FP8_MAX_VALUE[_fp8(fp8type)]


def fp8_quantize_perblock(x, QB, fp8type, scale_dtype=torch.bfloat16):
    """rq/_quantize_perblock.py:107-150 (kernel :33-104): the block is divided by its fp32 scale (:78), the scale is
    stored rounded to ``scale_dtype`` (:82)."""
    v32 = x.float()
    s32 = _block_scale32(v32, QB, fp8type)
    q = cast_fp8(v32 / s32.repeat_interleave(QB, 0).repeat_interleave(QB, 1), fp8type)
    return q, s32.to(scale_dtype)


def fp8_quantize_perblock_transpose(x, QB, fp8type, scale_dtype=torch.bfloat16, only_transposed=False):
    """rq/_quantize_perblock_transpose.py:136-190 (kernel :33-133): the same codes and scales, also transposed (:84-88)."""
    q, s = fp8_quantize_perblock(x, QB, fp8type, scale_dtype)
    q_t, s_t = q.view(torch.uint8).t().contiguous().view(q.dtype), s.t().contiguous()
    return (q_t, s_t) if only_transposed else ((q, s), (q_t, s_t))


def fp8_quantize_perblock_transpose_pergroup(x, QB, fp8type, scale_dtype=torch.bfloat16):
    """rq/_quantize_perblock_transpose_pergroup.py:175-246 (kernel :33-172): per-block pair, its transpose, and the
    1 x QB per-group quantization of the same input (:140-172: row maxima inside the block = groups of QB along N)."""
    (q, s), (q_t, s_t) = fp8_quantize_perblock_transpose(x, QB, fp8type, scale_dtype)
    return (q, s), (q_t, s_t), _quantize_pg(x.float(), QB, fp8type, scale_dtype)


def fp8_group_scales(x, QB, fp8type, scale_dtype=torch.bfloat16):
    """rq/_quantize_pertensor.py:46-103: per-group scales only."""
    return _group_scale32(x.float(), QB, fp8type).to(scale_dtype)


def absmax_scale(x, fp8type):
    """rq/_division.py:178-179: (x.abs().max() + 1e-10) / fp8max evaluated in x's own dtype, on the device.
    torch's device kernel for a tensor divided by a Python number multiplies by the fp32 reciprocal of the number
    (aten/src/ATen/native/cuda/BinaryDivTrueKernel.cu, the CPU-scalar branch); the CPU kernel divides.  The
    reference runs on the device, so the reciprocal form is the one restated here."""
    a = (x.abs().max() + SCALE_MIN_THRES).float()
    inv = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(FP8_MAX_VALUE[_fp8(fp8type)], dtype=torch.float32)
    return (a * inv).to(x.dtype)


def fp8_division(x, QB, fp8type, s_y=None):
    """rq/_division.py:153-207 (kernel :84-113, non-stochastic): q = fp8(x / float(s))."""
    if s_y is None:
        s_y = absmax_scale(x, fp8type)
    return cast_fp8(x.float() / s_y.float(), fp8type), s_y


def fp8_division_transpose(x, QB, fp8type, s_y=None, only_transposed=False):
    """rq/_division_transpose.py:147-210."""
    q, s_y = fp8_division(x, QB, fp8type, s_y)
    q_t = q.view(torch.uint8).t().contiguous().view(q.dtype)
    return (q_t, s_y) if only_transposed else (q, s_y, q_t)


def fp8_quantize_pertensor(x, QB, fp8type, scale_dtype=torch.bfloat16):
    """rq/_quantize_pertensor.py:106-147: group scales -> max -> division."""
    s_pg = fp8_group_scales(x, QB, fp8type, scale_dtype)
    s = s_pg.max()
    q, s = fp8_division(x, QB, fp8type, s)
    return q, s, s_pg


def fp8_quantize_pertensor_transpose(x, QB, fp8type, scale_dtype=torch.bfloat16):
    """rq/_quantize_pertensor_transpose.py:106-150."""
    s = fp8_group_scales(x, QB, fp8type, scale_dtype).max()
    return fp8_division_transpose(x, QB, fp8type, s)


def fp8_transpose(q):
    """rq/_transpose.py:85-115: byte transpose."""
    return q.view(torch.uint8).t().contiguous().view(q.dtype)


def _dequant32(q, s, QB):
    """Shared dequantize prologue of every fused kernel, e.g. rq/silu_fwd.py:100-106."""
    M, N = q.shape
    return (_groups(q.float(), QB) * s.float().unsqueeze(2)).reshape(M, N)


def fp8_dequantize(q, s, QB):
    """rq/_dequantize.py:119-156: bf16(float(q) * float(s))."""
    return _dequant32(q, s, QB).to(torch.bfloat16)


# ----------------------------------------------------------------------------- GEMM
def fp8matmul(a, b, output_quantize, scale_a, scale_b, QB, bias=None, fp8type=None, accumulate=torch.float32):
    """rq/linear.py:172-250 (kernel :61-169).  a [M,K] fp8, b [K,N] fp8 (any strides).

    acc = sum_k a*b (``accumulate`` dtype; the kernel accumulates in fp32 in an unspecified
    order); acc *= float(sa)*float(sb) (:123-127); + bias (:129-131); then bf16 store (:168) or
    1xQB quantize of acc (:139-164) with the output fp8 type = a's type (:187).
    """
    acc = (a.to(accumulate) @ b.to(accumulate)).float()
    acc = acc * (scale_a.float() * scale_b.float())
    if bias is not None:
        acc = acc + bias.float()
    if output_quantize:
        return _quantize_pg(acc, QB, a.dtype if fp8type is None else fp8type)
    return acc.to(torch.bfloat16)


def fp8_linear_forward(x, s, w, s_w, output_quantize, QB, bias=None):
    """rq/linear.py:253-258."""
    return fp8matmul(x, w.t(), output_quantize, s, s_w, QB, bias)


def fp8_linear_backward(x_t, s, g, s_g, g_t, w_t, s_w, QB):
    """rq/linear.py:272-302 without dgrad_quantize: dgrad = g @ w, wgrad = g^T @ x."""
    y = fp8matmul(g, w_t.t(), False, s_g, s_w, QB)
    w_g = fp8matmul(g_t, x_t.t(), False, s_g, s, QB)
    return y, w_g


# ----------------------------------------------------------------------------- activations
def _sigmoid32(x32):
    """rq/silu_fwd.py:109: 1 / (1 + exp(-x)) in fp32."""
    return 1.0 / (1.0 + torch.exp(-x32))


def fp8_silu_forward(q, s, QB):
    """rq/silu_fwd.py:152-198 (kernel :100-122): output fp8 type = input fp8 type (:166)."""
    x = _dequant32(q, s, QB)
    y = _sigmoid32(x) * x
    return _quantize_pg(y, QB, q.dtype, s.dtype)


def silu_backward_value(q, s, g, QB):
    """rq/silu_bwd.py:124-131: (sig + x*sig*(1-sig)) * g, fp32."""
    x = _dequant32(q, s, QB)
    sig = _sigmoid32(x)
    return (sig + x * sig * (1 - sig)) * g.float()


def fp8_silu_backward(q, s, g, QB, fp8type, output_quantized_transpose=False):
    """rq/silu_bwd.py:170-238: bf16 value + per-group scale of the fp32 value (:133-141);
    with output_quantized_transpose the bf16 value is divided by the max scale (:227-230)."""
    v = silu_backward_value(q, s, g, QB)
    y = v.to(torch.bfloat16)
    s_y = _group_scale32(v, QB, fp8type).to(torch.bfloat16)
    if not output_quantized_transpose:
        return y, s_y
    return fp8_division_transpose(y, QB, fp8type, s_y.max())


def fp8_mul_forward(q1, s1, q2, s2, QB):
    """rq/mul_fwd.py:191-254 (kernel :118-163): product -> bf16 + group scales -> max -> division+transpose."""
    v = _dequant32(q1, s1, QB) * _dequant32(q2, s2, QB)
    y = v.to(torch.bfloat16)
    s_y = _group_scale32(v, QB, q1.dtype).to(s1.dtype)
    return fp8_division_transpose(y, QB, q2.dtype, s_y.max())


def fp8_mul_backward(q1, s1, q2, s2, g, QB, fp8type, output_quantized_transpose=False):
    """rq/mul_bwd.py:221-315 (kernel :171-202): g1 = g*x2 -> bf16; g2 = g*x1 -> bf16 + group scales."""
    x1, x2, g32 = _dequant32(q1, s1, QB), _dequant32(q2, s2, QB), g.float()
    y1 = (g32 * x2).to(torch.bfloat16)
    v2 = g32 * x1
    y2 = v2.to(torch.bfloat16)
    s_y2 = _group_scale32(v2, QB, fp8type).to(torch.bfloat16)
    if not output_quantized_transpose:
        return y1, (y2, s_y2)
    return y1, fp8_division_transpose(y2, QB, fp8type, s_y2.max())


def gelu_forward_value(q, s, QB):
    """rq/gelu_fwd.py:108-110: x * (1 + erf(x / sqrt(2))) / 2, fp32."""
    x = _dequant32(q, s, QB)
    cdf = (1.0 + torch.erf(x / torch.tensor(math.sqrt(2.0), dtype=torch.float32))) / 2
    return cdf * x


def fp8_gelu_forward(q, s, QB):
    """rq/gelu_fwd.py:152-203."""
    v = gelu_forward_value(q, s, QB)
    y = v.to(torch.bfloat16)
    s_y = _group_scale32(v, QB, q.dtype).to(s.dtype)
    return fp8_division_transpose(y, QB, q.dtype, s_y.max())


def gelu_backward_value(q, s, g, QB):
    """rq/gelu_bwd.py:124-131: (cdf + x*exp(-x^2/2)/sqrt(2*pi)) * g, fp32."""
    x = _dequant32(q, s, QB)
    cdf = (1.0 + torch.erf(x / torch.tensor(math.sqrt(2.0), dtype=torch.float32))) / 2
    pdf_term = x * torch.exp(-(x * x) / 2) / torch.tensor(math.sqrt(2 * math.pi), dtype=torch.float32)
    return (cdf + pdf_term) * g.float()


def fp8_gelu_backward(q, s, g, QB, fp8type):
    """rq/gelu_bwd.py:173-230: -> max -> fp8_division (no transpose)."""
    v = gelu_backward_value(q, s, g, QB)
    y = v.to(torch.bfloat16)
    s_y = _group_scale32(v, QB, fp8type).to(torch.bfloat16)
    return fp8_division(y, QB, fp8type, s_y.max())


# ----------------------------------------------------------------------------- residual add
def fp8_add_Ifp_Ifp_Ofp_Og16(x1, x2, fp8type, QB):
    """rq/add_fwd.py:162-213 (kernel :107-137): y = x1+x2 -> bf16, and 1xQB quantize of the fp32 sum."""
    v = x1.float() + x2.float()
    return v.to(torch.bfloat16), _quantize_pg(v, QB, fp8type)


def fp8_add_Ifp_Ifp_Ofp_Opt(x1, x2, QB, fp8type):
    """rq/add_bwd.py:147-200: bf16 sum + group scales of the fp32 sum; per-tensor quantize of the bf16 sum."""
    v = x1.float() + x2.float()
    y = v.to(torch.bfloat16)
    s_pg = _group_scale32(v, QB, fp8type).to(torch.bfloat16)
    q, s = fp8_division(y, QB, fp8type, s_pg.max())
    return y, (q, s, s_pg)


# ----------------------------------------------------------------------------- RMSNorm
def rmsnorm_forward_value(q, s, w, QB, eps, accumulate=torch.float32):
    """rq/func_rmsnorm.py:82-102: x=dequant; var=sum(x*x)/N; rstd=1/sqrt(var+eps); y=x*rstd*w (fp32).

    The kernel's tl.sum order is unspecified; ``accumulate=torch.float64`` gives the exactly
    rounded sum used for tolerance statements.
    """
    x = _dequant32(q, s, QB)
    N = x.shape[1]
    var = ((x * x).to(accumulate).sum(dim=1) / N).float()
    rstd = 1.0 / torch.sqrt(var + eps)
    y = (x * rstd.unsqueeze(1)) * w.float().unsqueeze(0)
    return y, rstd


def fp8_rmsnorm_forward(q, s, w, QB, eps, accumulate=torch.float32):
    """rq/func_rmsnorm.py:223-278: row scale (max|y|+1e-10)/fp8max stored bf16 (:105-108), y stored
    bf16 (:111), then max over rows -> division+transpose of the bf16 y (:268-269)."""
    v, rstd = rmsnorm_forward_value(q, s, w, QB, eps, accumulate)
    y = v.to(torch.bfloat16)
    s_row = ((v.abs().amax(dim=1) + SCALE_MIN_THRES) / FP8_MAX_VALUE[q.dtype]).to(torch.bfloat16)
    qy, s_pt, qy_t = fp8_division_transpose(y, QB, q.dtype, s_row.max())
    return qy, s_pt, qy_t, rstd


def fp8_rmsnorm_backward(q, s, g, w, rstd, QB, accumulate=torch.float64):
    """rq/func_rmsnorm.py:281-335 (kernels :121-196, :200-220).

    dx = (w*dy - xhat * mean(xhat*w*dy)) * rstd -> bf16 (:166-173); dw = sum_rows(dy * xhat).
    The reference sums dw in arrival order with partials rounded to w's dtype (:176-196); the
    mathematically intended value (float64 sum rounded once to w's dtype) is what is stated here.
    """
    x = _dequant32(q, s, QB)
    N = x.shape[1]
    dy = g.float()
    xhat = x * rstd.float().unsqueeze(1)
    wdy = w.float().unsqueeze(0) * dy
    c1 = ((xhat * wdy).to(accumulate).sum(dim=1) / N).float()
    dx = ((wdy - xhat * c1.unsqueeze(1)) * rstd.float().unsqueeze(1)).to(torch.bfloat16)
    dw = (dy * xhat).to(accumulate).sum(dim=0).to(w.dtype)
    return dx, dw


# ----------------------------------------------------------------------------- LayerNorm
def layernorm_forward_value(q, s, QB, eps, w=None, b=None, accumulate=torch.float32):
    """rq/func_layernorm_noparam.py:86-113 / rq/func_layernorm_param.py:87-119: x = dequant; mean = sum(x)/N;
    var = sum((x-mean)^2)/N; rstd = 1/sqrt(var+eps); y = (x-mean)*rstd (* w + b), all fp32."""
    x = _dequant32(q, s, QB)
    N = x.shape[1]
    mean = (x.to(accumulate).sum(dim=1) / N).float()
    d = x - mean.unsqueeze(1)
    var = ((d * d).to(accumulate).sum(dim=1) / N).float()
    rstd = 1.0 / torch.sqrt(var + eps)
    y = d * rstd.unsqueeze(1)
    if w is not None:
        y = y * w.float().unsqueeze(0) + b.float().unsqueeze(0)
    return y, mean, rstd


def fp8_layernorm_forward(q, s, QB, eps, w=None, b=None, accumulate=torch.float32):
    """rq/func_layernorm_noparam.py:188-245 / rq/func_layernorm_param.py:243-302: the normalised tensor stays fp32
    (:205), row scale (max|y|+1e-10)/fp8max stored bf16 (:106-112), max over rows, division+transpose of the fp32 y."""
    y, mean, rstd = layernorm_forward_value(q, s, QB, eps, w, b, accumulate)
    s_row = ((y.abs().amax(dim=1) + SCALE_MIN_THRES) / FP8_MAX_VALUE[q.dtype]).to(torch.bfloat16)
    qy, s_pt, qy_t = fp8_division_transpose(y, QB, q.dtype, s_row.max())
    return qy, s_pt, qy_t, mean, rstd


def fp8_layernorm_backward(q, s, g, mean, rstd, QB, w=None, accumulate=torch.float64):
    """rq/func_layernorm_noparam.py:160-185 / rq/func_layernorm_param.py:178-209, :214-240:
    wdy = w*dy (dy without parameters); c1 = sum(xhat*wdy)/N; c2 = sum(wdy)/N; dx = (wdy - (xhat*c1 + c2))*rstd -> bf16;
    dw = sum_rows(dy*xhat), db = sum_rows(dy) (the reference accumulates them under a lock in w's dtype; stated here is
    the float64 sum rounded once)."""
    x = _dequant32(q, s, QB)
    N = x.shape[1]
    dy = g.float()
    xhat = (x - mean.float().unsqueeze(1)) * rstd.float().unsqueeze(1)
    wdy = dy if w is None else w.float().unsqueeze(0) * dy
    c1 = ((xhat * wdy).to(accumulate).sum(dim=1) / N).float()
    c2 = (wdy.to(accumulate).sum(dim=1) / N).float()
    dx = ((wdy - (xhat * c1.unsqueeze(1) + c2.unsqueeze(1))) * rstd.float().unsqueeze(1)).to(torch.bfloat16)
    if w is None:
        return dx
    dw = (dy * xhat).to(accumulate).sum(dim=0).to(w.dtype)
    db = dy.to(accumulate).sum(dim=0).to(w.dtype)
    return dx, dw, db


# ----------------------------------------------------------------------------- the reference tests' own definition
def quantize_tensor_ref_test(x, QB, fp8type):
    """tests/test_utils.py:61-67 ("per_group"): scale = bf16(amax / fp8max) (no 1e-10), and the
    value is divided by the *bf16-rounded* scale.  Differs from the kernel definition above on a
    few percent of codes; the reference accepts >= 95 % equal (tests/test_utils.py:98-119)."""
    fp8type = _fp8(fp8type)
    M, N = x.shape
    g = x.float().reshape(M, N // QB, QB)
    sx = (g.abs().amax(dim=2) / FP8_MAX_VALUE[fp8type]).to(torch.bfloat16)
    q = (g / sx.float().unsqueeze(2)).to(fp8type).reshape(M, N)
    return q, sx


def quantize_tensor_ref_test_perblock(x, QB, fp8type):
    """tests/test_utils.py:53-60 ("per_block"): scale = bf16(amax_block / fp8max) (no 1e-10), the value divided by the
    bf16-rounded scale; >= 95 % equal codes is what the reference's test asks of its kernel (tests/test_fp8_quantize.py:42-48)."""
    fp8type = _fp8(fp8type)
    M, N = x.shape
    g = x.float().reshape(M // QB, QB, N // QB, QB).permute(0, 2, 1, 3)
    sx = (g.abs().amax(dim=(2, 3)) / FP8_MAX_VALUE[fp8type]).to(torch.bfloat16)
    q = (g / sx.float().unsqueeze(2).unsqueeze(3)).to(fp8type)
    return q.permute(0, 2, 1, 3).reshape(M, N), sx
