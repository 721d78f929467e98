"""OCP FP8 codec in numpy integer arithmetic.  TEST INFRASTRUCTURE ONLY.

The reference stores FP8 as ``torch.float8_e4m3fn`` / ``torch.float8_e5m2``
(coat/activation/real_quantization/common.py:22-26) and converts with Triton's
``.to(fp8)`` (PTX ``cvt.rn.satfinite``: round to nearest even, saturate finite
overflow to the largest normal, NaN stays NaN) or, in the optimizer, with
``static_cast<__nv_fp8_e4m3>(float)`` (cuda_fp8.h: ``__NV_SATFINITE``;
coat/optimizer/kernels/fp8_adamw_expand_cuda_kernel.cu:186-187).

This module is the independent statement of that conversion: it works on the
integer bit pattern of the fp32 input and never calls a library cast.

Pins (tests/test_oracle_fp8.py):
  * ``decode`` against the closed form (-1)^s * 2^(e-bias) * (1 + m/2^mb)
    (subnormals: 2^(1-bias) * m/2^mb) for all 256 codes, and against
    ``torch.Tensor.to(torch.float32)`` from the torch fp8 dtypes.
  * ``encode`` by brute force: for every representable value, every midpoint
    between neighbours and the fp32 numbers next to each midpoint, the result
    must be the nearest representable value computed in float64 with ties to the
    even code; plus agreement with the torch-CPU cast on the whole finite range
    the cast does not turn into NaN / inf.
"""
import numpy as np

E4M3 = "e4m3"
E5M2 = "e5m2"

_FMT = {
    # name: (exponent bits, mantissa bits, bias, max finite code magnitude, nan code magnitude)
    E4M3: (4, 3, 7, 0x7E, 0x7F),
    E5M2: (5, 2, 15, 0x7B, 0x7F),
}

FP8_MAX = {E4M3: 448.0, E5M2: 57344.0}


def decode(codes, fmt):
    """uint8 codes -> float32 values (closed form, no lookup into a library)."""
    eb, mb, bias, _, _ = _FMT[fmt]
    c = np.asarray(codes, dtype=np.uint8).astype(np.int64)
    sign = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> mb) & ((1 << eb) - 1)
    m = c & ((1 << mb) - 1)
    normal = np.ldexp(1.0 + m / float(1 << mb), (e - bias).astype(np.int64))
    sub = np.ldexp(m / float(1 << mb), 1 - bias)
    val = np.where(e == 0, sub, normal)
    if fmt == E4M3:
        val = np.where((c & 0x7F) == 0x7F, np.nan, val)
    else:
        val = np.where((e == 31) & (m == 0), np.inf, val)
        val = np.where((e == 31) & (m != 0), np.nan, val)
    return (sign * val).astype(np.float32)


def encode(x, fmt):
    """float32 -> uint8 codes; round-to-nearest-even, saturate-to-finite, NaN -> 0x7F|sign.

    Integer algorithm on the fp32 bit pattern: rebias the exponent, shift the 23-bit
    mantissa down to ``mb`` bits with RNE (subnormal targets shift further), carry into
    the exponent, clamp to the largest finite code.
    """
    eb, mb, bias, max_code, nan_code = _FMT[fmt]
    xf = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    bits = xf.view(np.uint32).astype(np.int64)
    sign = ((bits >> 24) & 0x80).astype(np.int64)
    mag = bits & 0x7FFFFFFF
    is_nan = mag > 0x7F800000
    e32 = mag >> 23
    m32 = mag & 0x7FFFFF
    # significand with the hidden bit (fp32 subnormals are far below every fp8 subnormal
    # and round to zero; giving them exponent 1 and no hidden bit keeps that exact)
    sig = np.where(e32 == 0, m32, m32 | 0x800000)
    e_unb = np.where(e32 == 0, 1, e32) - 127  # value = sig * 2^(e_unb - 23)
    # target exponent field; values below the smallest normal use the subnormal spacing
    e_t = e_unb + bias
    shift = np.where(e_t >= 1, 23 - mb, 23 - mb + (1 - e_t))
    shift = np.minimum(shift, 40)
    # RNE shift of sig by ``shift`` bits
    half = np.int64(1) << (shift - 1)
    mask = (np.int64(1) << shift) - 1
    q = sig >> shift
    rem = sig & mask
    q = q + ((rem > half) | ((rem == half) & ((q & 1) == 1)))
    # assemble: for normals q has the hidden bit at position mb, so adding ((e_t-1) << mb)
    # lets a mantissa carry roll into the exponent; for subnormal targets the exponent
    # field starts at 0 and a carry produces the smallest normal.
    code = np.where(e_t >= 1, ((e_t - 1) << mb) + q, q)
    code = np.minimum(code, max_code)  # satfinite (also maps +-inf to the largest finite)
    code = np.where(is_nan, nan_code, code)
    return (code | sign).astype(np.uint8)
