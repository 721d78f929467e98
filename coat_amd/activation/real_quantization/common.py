"""Constants of the FP8 op library (reference: coat/activation/real_quantization/common.py:20-31)."""
import threading

import torch

SCALE_MIN_THRES = 1e-10

FP8_MAX_VALUE = {
    torch.float8_e4m3fn: 448.0,
    torch.float8_e5m2: 57344.0,
}

convert_str_to_fp8 = {"E4M3": torch.float8_e4m3fn, "E5M2": torch.float8_e5m2}
convert_fp8_to_embit = {
    torch.float8_e4m3fn: (4.0, 3.0),
    torch.float8_e5m2: (5.0, 2.0),
}


def as_fp8_dtype(fp8type):
    """Accepts "E4M3"/"E5M2" or a torch fp8 dtype, as the reference entry points do."""
    if isinstance(fp8type, str):
        return convert_str_to_fp8[fp8type]
    if fp8type not in FP8_MAX_VALUE:
        raise ValueError(f"unsupported fp8 type {fp8type}")
    return fp8type


def flatten_2d(x):
    """3-D [B, S, C] -> 2-D [B*S, C] as every reference launcher does; returns (x2d, batch or None)."""
    if x.dim() == 3:
        return x.reshape(-1, x.shape[-1]), x.shape[0]
    if x.dim() != 2:
        raise ValueError(f"expected a 2-D or 3-D tensor, got shape {tuple(x.shape)}")
    return x, None


def restore(y, batch):
    """Inverse of flatten_2d for an output whose rows follow the input's rows."""
    return y if batch is None else y.reshape(batch, -1, y.shape[-1])


def no_stochastic(stochastic, why):
    """For the two entry points whose stochastic branch does not compile in the reference itself."""
    if stochastic:
        raise NotImplementedError(f"stochastic=True is not available here: {why}")


_MAX_POOL = {}
_MAX_POOL_SIZE = 64
_MAX_POOL_LOCK = threading.Lock()  # host threads may call the entry points together (autograd's backward threads do)


def new_max(device):
    """Zero-initialised buffer for the order-independent device-wide maximum of the group scales: ``_hip.MAX_WORDS`` fp32
    words, 16 slots one 128-byte line apart (include/coat_hip.h, COAT_MAX_WORDS); ``read_max`` gives the maximum.

    Buffers are handed out from a zero-filled pool (one fill kernel per 64 of them instead of one each; a buffer is
    never reused, and the pool lives as long as any of its buffers).  Pools are kept per device and stream, so a buffer
    is always used on the stream that zeroed it."""
    from ... import _hip
    device = torch.device(device)
    if device.type != "cuda":
        return torch.zeros(_hip.MAX_WORDS, dtype=torch.float32, device=device)
    if torch.cuda.is_current_stream_capturing():
        # under graph capture the zero fill has to be a node of the graph (a pool zeroed before the capture would keep the
        # maxima of earlier replays), and memory of the graph's private pool must not be handed out after the capture
        return torch.zeros(_hip.MAX_WORDS, dtype=torch.float32, device=device)
    key = (device.index if device.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(device).cuda_stream)
    with _MAX_POOL_LOCK:  # the slot counter and the dictionary are shared by the threads that use one device and stream
        pool = _MAX_POOL.get(key)
        if pool is None or pool[1] >= _MAX_POOL_SIZE:
            pool = [torch.zeros(_MAX_POOL_SIZE * _hip.MAX_WORDS, dtype=torch.float32, device=device), 0]
            _MAX_POOL[key] = pool
        i = pool[1]
        pool[1] = i + 1
        buf = pool[0]
    return buf[i * _hip.MAX_WORDS:(i + 1) * _hip.MAX_WORDS]


def tag_scale_max(t, buf, fp8type):
    """Producer side of a hand-over: ``buf`` (a ``new_max`` buffer) holds the maximum of the fp32 group scales of the
    bf16 tensor ``t`` for the FP8 format ``fp8type``, merged by the kernel that wrote ``t`` (the RoPE backward, the
    attention forward).  The tag travels with the tensor object, through the autograd engine too."""
    t._coat_scale_max = (buf, fp8type, t._version)
    return t


def known_scale_max(t, fp8type):
    """Consumer side: the tagged buffer if ``t`` still is the tensor its producer wrote (same object, not modified in
    place since, same format), else None, and the caller runs its own scale pass."""
    tag = getattr(t, "_coat_scale_max", None)
    if tag is None:
        return None
    buf, kind, version = tag
    if kind != fp8type or version != t._version or buf.device != t.device or t.dtype != torch.bfloat16:
        return None
    return buf


def scale_max(s):
    """``s.max()`` for a tensor of (non-negative) scales, as a 0-dim tensor of its dtype: the scale with which a tensor
    quantized per tensor was divided is the maximum of the per-group scale tensor that travels with it (reference
    coat/models/coat_llama.py:474, :706).  One pass of the library's abs-max kernel instead of torch's reduction, which
    takes a memset and a kernel of 12 us for these 4 MB and, under HIP graph capture, records a memset node."""
    from ... import _hip
    if not s.is_cuda or s.numel() == 0 or s.dtype not in (torch.bfloat16, torch.float32, torch.float16):
        return s.max()
    s = _hip.dense(s)
    amax = new_max(s.device)
    _hip.check(_hip.lib().coat_absmax(_hip.ptr(s), _hip.dt(s), _hip.ptr(amax), s.numel(), _hip.stream(s.device)), "scale_max")
    return read_max(amax).to(s.dtype)


def read_max(buf):
    """The maximum held by a ``new_max`` buffer, as a 0-dim fp32 tensor (for host-side code; the division kernels read
    the slots themselves)."""
    from ... import _hip
    return buf[::_hip.MAX_SLOT_STRIDE].max()
