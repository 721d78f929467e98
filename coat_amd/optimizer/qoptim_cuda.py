"""Drop-in for the reference's pybind module ``qoptim_cuda`` (coat/optimizer/kernels/bindings.cpp:5-8).

``fp8_adamw_expand_step_multi`` / ``fp8_adamw_step_multi`` (no counterpart in the reference) take lists of the same tensors
and step them in one launch per 32 tensors, each tensor bit-identical to its own call.

Same two functions, same positional arguments (include/fp8_adamw.h:6-13, include/fp8_adamw_expand.h:6-17),
torch tensors in, everything updated in place; the work is done by libcoat_hip.so on the tensor's current
stream (the reference launches on the legacy default stream).  Errors the reference raises through
AT_ASSERTM surface as RuntimeError with the same message."""
import ctypes

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


def _pointer_array(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def _multi(expand, params, grads, exp_avg, exp_avg_sq, scale_lists, hyper, step, qgroup_size, expand_min):
    n = len(params)
    if not (len(grads) == len(exp_avg) == len(exp_avg_sq) == n and all(len(l) == n for l in scale_lists)):
        raise RuntimeError("qoptim_cuda: the tensor lists differ in length")
    if n == 0:
        return
    ngroups = []
    for i in range(n):
        if params[i].dtype != params[0].dtype or params[i].device != params[0].device:
            raise RuntimeError("qoptim_cuda: the tensors of one multi-tensor step share dtype and device")
        ngroups.append(_common_checks(params[i], grads[i], exp_avg[i], exp_avg_sq[i], tuple(l[i] for l in scale_lists), qgroup_size))
        if any(l[i].numel() != ngroups[-1] for l in scale_lists):
            raise RuntimeError("grid_dim == scale_exp_avg_sq.numel()")
    numel = (ctypes.c_int64 * n)(*[t.numel() for t in params])
    n_scale = (ctypes.c_int64 * n)(*ngroups)
    arrays = [_pointer_array(l) for l in scale_lists]
    beta1, beta2, lr, wd, eps = hyper
    lib, st = _hip.lib(), _hip.stream(params[0].device)
    if expand:
        sm, km, cm, sv, kv, cv = arrays
        rc = lib.coat_fp8_adamw_expand_step_multi(n, _pointer_array(params), _pointer_array(grads), _hip.dt(params[0]),
                                                  _pointer_array(exp_avg), sm, km, cm, _pointer_array(exp_avg_sq), sv, kv, cv,
                                                  numel, n_scale, beta1, beta2, lr, wd, eps, int(step), int(qgroup_size),
                                                  int(expand_min), st)
    else:
        sm, sv = arrays
        rc = lib.coat_fp8_adamw_step_multi(n, _pointer_array(params), _pointer_array(grads), _hip.dt(params[0]),
                                           _pointer_array(exp_avg), sm, _pointer_array(exp_avg_sq), sv, numel, n_scale,
                                           beta1, beta2, lr, wd, eps, int(step), int(qgroup_size), st)
    _hip.check(rc, "fp8_adamw_expand_step_multi" if expand else "fp8_adamw_step_multi")


def fp8_adamw_expand_step_multi(params, grads, exp_avg, scale_exp_avg, expand_exp_avg, sqrtminmax_exp_avg, exp_avg_sq,
                                scale_exp_avg_sq, expand_exp_avg_sq, sqrtminmax_exp_avg_sq, beta1, beta2, lr, wd, eps, step,
                                qgroup_size, expand_min):
    """``fp8_adamw_expand_step`` on lists of tensors (one dtype, one device, one step count): one launch per 32 tensors."""
    _multi(True, params, grads, exp_avg, exp_avg_sq,
           (scale_exp_avg, expand_exp_avg, sqrtminmax_exp_avg, scale_exp_avg_sq, expand_exp_avg_sq, sqrtminmax_exp_avg_sq),
           (beta1, beta2, lr, wd, eps), step, qgroup_size, expand_min)


def fp8_adamw_step_multi(params, grads, exp_avg, scale_exp_avg, exp_avg_sq, scale_exp_avg_sq, beta1, beta2, lr, wd, eps,
                         step, qgroup_size):
    """``fp8_adamw_step`` on lists of tensors: one launch per 32 tensors."""
    _multi(False, params, grads, exp_avg, exp_avg_sq, (scale_exp_avg, scale_exp_avg_sq), (beta1, beta2, lr, wd, eps), step,
           qgroup_size, 0)
