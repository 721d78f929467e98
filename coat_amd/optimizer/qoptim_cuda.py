"""Drop-in for the reference's pybind module ``qoptim_cuda`` (coat/optimizer/kernels/bindings.cpp:5-8).

Same two functions, same positional arguments (include/fp8_adamw.h:6-13, include/fp8_adamw_expand.h:6-17),
torch tensors in, everything updated in place; the work is done by libcoat_hip.so on the tensor's current
stream (the reference launches on the legacy default stream).  Errors the reference raises through
AT_ASSERTM surface as RuntimeError with the same message."""
import torch

from .. import _hip


def _common_checks(params, grads, exp_avg, exp_avg_sq, scales, qgroup_size):
    if qgroup_size != 128:
        raise RuntimeError("Only Support 128 per-group quantization currently")
    if not params.is_cuda:
        raise RuntimeError("qoptim_cuda: params must be on the GPU")
    if grads.dtype != params.dtype:
        raise RuntimeError(f"qoptim_cuda: grads dtype {grads.dtype} differs from params dtype {params.dtype}")
    for name, t in (("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq)):
        if t.dtype != torch.float8_e4m3fn:
            raise RuntimeError(f"expected scalar type Float8_e4m3fn but found {t.dtype} ({name})")
    for t in scales:
        if t.dtype != torch.float32:
            raise RuntimeError(f"expected scalar type Float but found {t.dtype}")
    ngroups = (params.numel() + qgroup_size - 1) // qgroup_size
    if scales[0].numel() != ngroups:
        raise RuntimeError("grid_dim == scale_exp_avg.numel()")
    for t in (params, grads, exp_avg, exp_avg_sq, *scales):
        if not t.is_contiguous():
            raise RuntimeError("qoptim_cuda: tensors must be contiguous")
    return ngroups


def fp8_adamw_expand_step(params, grads, exp_avg, scale_exp_avg, expand_exp_avg, sqrtminmax_exp_avg, exp_avg_sq,
                          scale_exp_avg_sq, expand_exp_avg_sq, sqrtminmax_exp_avg_sq, beta1, beta2, lr, wd, eps, step,
                          qgroup_size, expand_min):
    """Update the quantized optimizer states, use polynomial expander (bindings.cpp:7)."""
    scales = (scale_exp_avg, expand_exp_avg, sqrtminmax_exp_avg, scale_exp_avg_sq, expand_exp_avg_sq,
              sqrtminmax_exp_avg_sq)
    ngroups = _common_checks(params, grads, exp_avg, exp_avg_sq, scales, qgroup_size)
    if scale_exp_avg_sq.numel() != ngroups:
        raise RuntimeError("grid_dim == scale_exp_avg_sq.numel()")
    p = _hip.ptr
    _hip.check(_hip.lib().coat_fp8_adamw_expand_step(
        p(params), p(grads), _hip.dt(params), p(exp_avg), p(scale_exp_avg), p(expand_exp_avg), p(sqrtminmax_exp_avg),
        p(exp_avg_sq), p(scale_exp_avg_sq), p(expand_exp_avg_sq), p(sqrtminmax_exp_avg_sq),
        beta1, beta2, lr, wd, eps, int(step), int(qgroup_size), int(expand_min), params.numel(), ngroups,
        _hip.stream(params.device)), "fp8_adamw_expand_step")


def fp8_adamw_step(params, grads, exp_avg, scale_exp_avg, exp_avg_sq, scale_exp_avg_sq, beta1, beta2, lr, wd, eps,
                   step, qgroup_size):
    """Update the quantized optimizer states (bindings.cpp:6)."""
    ngroups = _common_checks(params, grads, exp_avg, exp_avg_sq, (scale_exp_avg, scale_exp_avg_sq), qgroup_size)
    if scale_exp_avg_sq.numel() != ngroups:
        raise RuntimeError("grid_dim == scale_exp_avg_sq.numel()")
    p = _hip.ptr
    _hip.check(_hip.lib().coat_fp8_adamw_step(
        p(params), p(grads), _hip.dt(params), p(exp_avg), p(scale_exp_avg), p(exp_avg_sq), p(scale_exp_avg_sq),
        beta1, beta2, lr, wd, eps, int(step), int(qgroup_size), params.numel(), ngroups,
        _hip.stream(params.device)), "fp8_adamw_step")
