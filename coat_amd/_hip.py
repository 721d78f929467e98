"""ctypes loader of libcoat_hip.so and the marshalling shared by every Python entry point.

The library is the only compute path: if it is missing or a call is rejected this module raises,
there is no fallback.  Signatures are declared in include/coat_hip.h.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# COAT_HIP_LIB: another build of the same library (an experiment build made with COAT_LIB_OUT=... python -m coat_amd.build)
LIB_PATH = os.environ.get("COAT_HIP_LIB") or os.path.join(_HERE, "libcoat_hip.so")

F32, BF16, F16 = 0, 1, 2
MAX_SLOTS, MAX_SLOT_STRIDE = 16, 32  # COAT_MAX_SLOTS, COAT_MAX_SLOT_STRIDE of include/coat_hip.h
MAX_WORDS = MAX_SLOTS * MAX_SLOT_STRIDE
ABI_VERSION = 5  # COAT_ABI_VERSION of include/coat_hip.h: a library built from another header is refused
E4M3, E5M2 = 0, 1

_DTYPE = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
_FP8 = {torch.float8_e4m3fn: E4M3, torch.float8_e5m2: E5M2}

_vp, _i, _i64, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
_u64 = ctypes.c_uint64

# name -> argument types (all functions return int except the two string getters)
SIGNATURES = {
    "coat_fp8_quantize": [_vp, _i, _vp, _vp, _i, _i64, _i64, _i, _i, _vp],
    "coat_fp8_quantize_transpose": [_vp, _i, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _i, _vp],
    "coat_fp8_quantize_perblock": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _i, _vp],
    "coat_fp8_group_scales": [_vp, _i, _vp, _i, _vp, _i64, _i64, _i, _i, _vp],
    "coat_absmax": [_vp, _i, _vp, _i64, _vp],
    "coat_fp8_division": [_vp, _i, _vp, _i, _vp, _vp, _i64, _i64, _i, _vp],
    "coat_fp8_rmsnorm_division": [_vp, _i, _vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i, _vp],
    "coat_fp8_layernorm_division": [_vp, _i, _vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i, _vp],
    "coat_fp8_silu_mul_forward_bf16": [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i, _vp],
    "coat_fp8_product_division": [_vp, _vp, _i, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _i64, _i64, _i, _i64, _i64, _vp],
    "coat_fp8_division_from_max": [_vp, _i, _vp, _vp, _i, _vp, _vp, _i64, _i64, _i, _vp],
    "coat_fp8_division_stochastic": [_vp, _i, _vp, _i, _vp, _vp, _i64, _i64, _i, _u64, _vp],
    "coat_fp8_transpose": [_vp, _vp, _i64, _i64, _vp],
    "coat_cross_entropy_forward": [_vp, _i, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _f, _f, _i, _f, _i, _vp],
    "coat_cross_entropy_scale_grad": [_vp, _i, _i64, _vp, _i, _i64, _i64, _vp],
    "coat_fp8_dequantize": [_vp, _i, _vp, _i, _vp, _i64, _i64, _i, _vp],
    "coat_fp8_silu_forward": [_vp, _i, _vp, _i, _vp, _vp, _i64, _i64, _i, _vp],
    "coat_fp8_silu_backward": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _vp],
    "coat_fp8_mul_forward": [_vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _i64, _i64, _i, _vp],
    "coat_fp8_mul_backward": [_vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _vp],
    "coat_fp8_gelu_forward": [_vp, _i, _vp, _i, _vp, _vp, _vp, _i64, _i64, _i, _vp],
    "coat_fp8_gelu_backward": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _vp],
    "coat_fp8_add_fwd": [_vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _vp],
    "coat_fp8_add_bwd": [_vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _vp],
    "coat_fp8_rmsnorm_forward": [_vp, _i, _vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i64, _i64, _i, _f, _vp],
    "coat_fp8_rmsnorm_backward": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _vp],
    "coat_fp8_rmsnorm_backward_add": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i64, _i64,
                                      _i, _vp],
    "coat_fp8_rmsnorm_backward_static": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i64, _i64, _i, _vp],
    "coat_fp8_layernorm_forward": [_vp, _i, _vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i, _f, _vp],
    "coat_fp8_layernorm_backward": [_vp, _i, _vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i,
                                    _vp],
    "coat_fp8_layernorm_backward_add": [_vp, _i, _vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i,
                                        _i64, _i64, _i, _vp],
    "coat_fp8_silu_mul_forward": [_vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _i64, _i64, _i, _i64, _i64, _vp],
    "coat_fp8_silu_mul_backward": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i, _i64,
                                   _i64, _i64, _vp],
    "coat_rope_bf16": [_vp, _vp, _vp, _vp, _i64, _f, _vp, _i64, _i, _i, _i, _i, _i64, _i64, _vp, _i, _vp],
    "coat_attention_forward_bf16": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                    _i64, _i64, _i64, _i64, _i64, _f, _i, _vp, _i, _vp],
    "coat_fp8_gemm": [_vp, _i, _vp, _i, _vp, _vp, _i, _vp, _i, _vp, _i, _vp, _i, _i64, _i64, _i64, _i, _vp],
    "coat_fp8_gemm_residual": [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _i, _vp, _i, _i64, _i64, _i64, _vp],
    "coat_fp8_gemm_grouped": [_i, _vp, _i, _vp, _i, _vp, _vp, _i, _vp, _i, _vp, _i, _vp, _i, _i64, _i64, _i64, _i, _vp],
    "coat_fp8_adamw_expand_step": [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _f, _f, _f, _f, _i, _i, _i,
                                   _i64, _i64, _vp],
    "coat_fp8_adamw_step": [_vp, _vp, _i, _vp, _vp, _vp, _vp, _f, _f, _f, _f, _f, _i, _i, _i64, _i64, _vp],
    "coat_fp8_adamw_expand_step_multi": [_i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _f, _f, _f, _f,
                                         _i, _i, _i, _vp],
    "coat_fp8_adamw_step_multi": [_i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _f, _f, _f, _f, _f, _i, _i, _vp],
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built (python -m coat_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"coat_amd: {LIB_PATH} is missing; build it with `python -m coat_amd.build` "
                "(there is no fallback path)")
        L = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes = argtypes
            fn.restype = _i
        L.coat_abi_version.restype = _i
        if L.coat_abi_version() != ABI_VERSION:
            raise RuntimeError(f"coat_amd: {LIB_PATH} has ABI version {L.coat_abi_version()}, this package needs "
                               f"{ABI_VERSION}; rebuild it with `python -m coat_amd.build`")
        L.coat_version.restype = ctypes.c_char_p
        L.coat_status_string.argtypes = [_i]
        L.coat_status_string.restype = ctypes.c_char_p
        _lib = L
    return _lib


def check(status, what):
    if status == 0:
        return
    msg = lib().coat_status_string(status).decode()
    if status in (-1, -2, -3, -5):
        raise ValueError(f"{what}: {msg}")
    raise RuntimeError(f"{what}: {msg}")


def dt(t):
    try:
        return _DTYPE[t.dtype if isinstance(t, torch.Tensor) else t]
    except KeyError:
        raise ValueError(f"unsupported dtype {t.dtype if isinstance(t, torch.Tensor) else t}") from None


def fp8(dtype):
    try:
        return _FP8[dtype]
    except KeyError:
        raise ValueError(f"not an FP8 dtype: {dtype}") from None


def stream(device=None):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def ptr_array(tensors):
    """Host array of device pointers (NULL for None), for entry points that take ``const void* const*``."""
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() if t is not None else None for t in tensors])


def dense(t):
    """Contiguous, 16-byte aligned view or copy of ``t`` on the GPU (the kernels move 16 bytes per lane)."""
    if not t.is_cuda:
        raise RuntimeError("coat_amd kernels need tensors on the GPU (got a %s tensor)" % t.device.type)
    t = t.contiguous()
    if t.data_ptr() % 16 != 0:
        t = t.clone()
    return t
