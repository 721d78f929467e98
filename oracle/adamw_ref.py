"""ctypes binding of oracle/adamw_ref.c and a torch restatement of the reference test's own
simulated optimizer step.  TEST INFRASTRUCTURE ONLY.

``adamw_expand_step`` / ``adamw_step`` mirror the argument order of the reference's pybind entry
points ``qoptim_cuda.fp8_adamw_expand_step`` / ``fp8_adamw_step``
(coat/optimizer/kernels/bindings.cpp:5-8, include/fp8_adamw_expand.h:6-17, include/fp8_adamw.h:6-13)
and mutate CPU tensors in place.

``simulated_expand_step`` restates tests/test_fp8_adamw_expand.py:111-215 — an *independent*
definition of the same step (AdamW written the torch.optim way, the exponent k found by a search
over i/16, fake quantization by (absmax + 1e-8) / 448) — and is what pins the C restatement.
"""
import ctypes
import math
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcoat_oracle.so")
_lib = None


def build(force=False):
    """Compile oracle/adamw_ref.c with the recipe in oracle/Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libcoat_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, f, i, i64 = ctypes.c_void_p, ctypes.c_float, ctypes.c_int, ctypes.c_int64
        L.coat_oracle_adamw_expand.argtypes = [vp, vp, i, vp, vp, vp, vp, vp, vp, vp, vp, f, f, f, f, f, i, i, i64]
        L.coat_oracle_adamw_expand.restype = None
        L.coat_oracle_adamw.argtypes = [vp, vp, i, vp, vp, vp, vp, f, f, f, f, f, i, i64]
        L.coat_oracle_adamw.restype = None
        L.coat_oracle_e4m3_encode.argtypes = [f]
        L.coat_oracle_e4m3_encode.restype = ctypes.c_uint8
        L.coat_oracle_e4m3_decode.argtypes = [ctypes.c_uint8]
        L.coat_oracle_e4m3_decode.restype = f
        L.coat_oracle_count_recip_div_mismatch.argtypes = [vp, i64, vp, i64]
        L.coat_oracle_count_recip_div_mismatch.restype = i64
        L.coat_oracle_count_sqrt_correction_mismatch.argtypes = [vp, i64]
        L.coat_oracle_count_sqrt_correction_mismatch.restype = i64
        _lib = L
    return _lib


def _check(t, dtype=None):
    assert t.device.type == "cpu" and t.is_contiguous()
    if dtype is not None:
        assert t.dtype == dtype, (t.dtype, dtype)
    return t.data_ptr()


def _pdtype(p, g):
    assert p.dtype == g.dtype and p.dtype in (torch.float32, torch.bfloat16)
    return 1 if p.dtype == torch.bfloat16 else 0


def adamw_expand_step(p, g, m8, sm, km, cm, v8, sv, kv, cv, beta1, beta2, lr, wd, eps, step, qgroup_size, expand_min):
    """fp8_adamw_expand_cuda_kernel.cu:205-245 (launcher) + :20-203 (kernel)."""
    assert qgroup_size == 128, "Only Support 128 per-group quantization currently"  # :221
    n = p.numel()
    ng = (n + 127) // 128
    assert sm.numel() == ng and sv.numel() == ng  # :224-225
    f32, e4 = torch.float32, torch.float8_e4m3fn
    lib().coat_oracle_adamw_expand(
        _check(p), _check(g), _pdtype(p, g), _check(m8, e4), _check(sm, f32), _check(km, f32), _check(cm, f32),
        _check(v8, e4), _check(sv, f32), _check(kv, f32), _check(cv, f32),
        beta1, beta2, lr, wd, eps, int(step), int(expand_min), n)


def adamw_step(p, g, m8, sm, v8, sv, beta1, beta2, lr, wd, eps, step, qgroup_size):
    """fp8_adamw_cuda_kernel.cu:127-159 (launcher) + :20-125 (kernel)."""
    assert qgroup_size == 128, "Only Support 128 per-group quantization currently"
    n = p.numel()
    ng = (n + 127) // 128
    assert sm.numel() == ng and sv.numel() == ng
    f32, e4 = torch.float32, torch.float8_e4m3fn
    lib().coat_oracle_adamw(
        _check(p), _check(g), _pdtype(p, g), _check(m8, e4), _check(sm, f32), _check(v8, e4), _check(sv, f32),
        beta1, beta2, lr, wd, eps, int(step), n)


def fresh_state(p, expand=True):
    """coat/optimizer/fp8_adamw.py:117-137: codes 0, scales 0, k = 1, c = 1."""
    ng = (p.numel() + 127) // 128
    st = {
        "exp_avg": torch.zeros(p.shape, dtype=torch.float8_e4m3fn),
        "scale_exp_avg": torch.zeros(ng, dtype=torch.float32),
        "exp_avg_sq": torch.zeros(p.shape, dtype=torch.float8_e4m3fn),
        "scale_exp_avg_sq": torch.zeros(ng, dtype=torch.float32),
    }
    if expand:
        for k in ("expand_exp_avg", "sqrt_minmax_exp_avg", "expand_exp_avg_sq", "sqrt_minmax_exp_avg_sq"):
            st[k] = torch.ones(ng, dtype=torch.float32)
    return st


def dequantize_state(codes, scale, expand=None, sqrt_minmax=None):
    """Inverse map used at the top of the kernel (fp8_adamw_expand_cuda_kernel.cu:44-49), in float64."""
    n = codes.numel()
    ng = scale.numel()
    x = codes.float().double().flatten()
    pad = ng * 128 - n
    x = torch.nn.functional.pad(x, (0, pad)).reshape(ng, 128) * scale.double().unsqueeze(1)
    if expand is not None:
        x = x.sign() * x.abs().pow(1.0 / expand.double().unsqueeze(1)) * sqrt_minmax.double().unsqueeze(1)
    return x.flatten()[:n].reshape(codes.shape)


# ---------------------------------------------------------------------------------------------
def _fake_quant_e4m3(B, epsilon=1e-8):
    """SymmQuantizer.forward for "E4M3" (coat/activation/fake_quantization/quantize_function.py:223-262
    with find_max_min :181-220 and floatExMy_quantize_torch, FloatPointQuantizeTorch.py:22-45).
    B: [groups, 128] float32.  Returns (codes as float values, scale [groups, 1])."""
    absmax = B.abs().amax(dim=1, keepdim=True) + epsilon
    scale = (2 * absmax) / (448 - (-448))
    x = B / scale
    sign, x_abs = x.sign(), x.abs()
    e_bit, m_bit = 4, 3
    Elow, Ehigh, Mhigh = -(2 ** (e_bit - 1)) + 2, 2 ** (e_bit - 1), 2 ** m_bit
    expo = torch.clamp(torch.floor(torch.log2(x_abs)), min=Elow, max=Ehigh)
    mant = x_abs / torch.exp2(expo)
    mant_int = torch.floor(mant)
    mant_frac = torch.round((mant - mant_int) * Mhigh)
    q = sign * (2 ** expo) * (mant_int + mant_frac / Mhigh)
    return q, scale


def simulated_expand_step(params, grads, exp_avg, exp_avg_sq, beta1, beta2, lr, wd, eps, step):
    """tests/test_fp8_adamw_expand.py:111-215.  ``exp_avg`` / ``exp_avg_sq`` are the *dequantized*
    fp32 moments; numel must be a multiple of 128.  Returns a dict with the new params and, for both
    moments, (codes as float values, scale, k, sqrt(min*max)) per group.

    The test increments ``step`` before use (:113) while the kernel uses the step it is given;
    callers pass the step the kernel receives and this function does not increment it.
    """
    power_options = torch.tensor([i / 16 for i in range(1, 129)], dtype=torch.float32)  # :61
    ratio_upperbound = 448 * 448 / 2  # :45-47
    params = params.clone().float()
    m = exp_avg.clone().float().flatten()
    v = exp_avg_sq.clone().float().flatten()
    g = grads.float().flatten()
    params.mul_(1 - lr * wd)  # :116
    m.lerp_(g, 1 - beta1)  # :119
    v.mul_(beta2).addcmul_(g, g, value=1 - beta2)  # :120
    bias_correction1 = 1 - beta1 ** step
    bias_correction2 = 1 - beta2 ** step
    step_size = lr / bias_correction1
    denom = (v.sqrt() / math.sqrt(bias_correction2)).add_(eps)  # :129
    params.addcdiv_(m.reshape(params.shape), denom.reshape(params.shape), value=-step_size)  # :131
    out = {"params": params}
    for name, x in (("exp_avg", m), ("exp_avg_sq", v)):
        B = x.reshape(-1, 128)
        sgn = B.sign()
        bmax, bmin = B.abs().amax(dim=1, keepdim=True), B.abs().amin(dim=1, keepdim=True)  # :141
        sqrt_minmax = (bmax * bmin).sqrt()  # :142
        ratio = bmax / bmin
        idx = (torch.pow(ratio, power_options.unsqueeze(0)) < ratio_upperbound).sum(dim=1)  # :146
        k = power_options[idx - 1].unsqueeze(1)  # :147
        Bk = torch.pow((B / sqrt_minmax).abs(), k) * sgn  # :150-151
        q, scale = _fake_quant_e4m3(Bk)
        out[name] = (q, scale.squeeze(1), k.squeeze(1), sqrt_minmax.squeeze(1))
    return out
