"""numpy / torch-CPU restatement of the reference's stochastic-rounding branch.  TEST INFRASTRUCTURE ONLY.

Paths are relative to the reference repository root; ``rq/`` abbreviates
``coat/activation/real_quantization/``.

The branch exists in two reference kernels that can run: per-tensor division (rq/_division.py:96-112)
and division + transpose (rq/_division_transpose.py:103-119).  Both draw ``tl.rand(0, offset)`` with
``offset`` = the element's linear index in the input, pass the quotient through ``_stochastic_rounding``
(rq/_division.py:130-150) and then cast to FP8 with round-to-nearest.  The remaining users of the
``stochastic`` flag either ignore it (rq/silu_bwd.py:171, rq/mul_bwd.py:236-239 allocate noise that the kernel
never reads) or cannot compile with it (rq/linear.py:151-152 passes ``boundary_check`` to a plain pointer
load; rq/func_layernorm_noparam.py:180 names ``e_bit``/``m_bit`` that the kernel never receives).

``tl.rand`` is Triton's (third-party dependency, ``triton>=3.1.0`` in pyproject.toml:16; 3.6.0 installed):
Philox-4x32 with 10 rounds, key = (seed_lo, seed_hi), counter = (offset, 0, 0, 0), first output word, mapped to
[0, 1) by ``uint_to_uniform_float`` (triton/language/random.py).

Pin status (tests/test_oracle_stochastic.py):
  philox4x32_10          the three published Random123 known-answer vectors (all four output words)
  triton_rand            vectors written by Triton's own CPU interpreter (tests/golden/triton_rand_seed0.npz,
                         made by tests/golden/make_golden_triton_rand.py); range [0, 1)
  stochastic_rounding    no vector of the reference's exists; pinned by what the arithmetic fixes: noise 0
                         leaves every value at or above the smallest subnormal unchanged, the result lies in
                         [2^e, 2^(e+1)] of the input's binade, is monotone in the noise, moves the value up by
                         less than one FP8 step of that binade, and the documented oddities (zeros become the
                         smallest subnormal; the step used in [2^-8, 2^-6) for E4M3 is finer than the format's)
                         are reproduced, not repaired
  fp8_division           deterministic branch == oracle/activation_ref.fp8_division when the noise is forced to 0
                         on values already representable
"""
import numpy as np
import torch

from . import activation_ref as R

_M0 = np.uint64(0xD2511F53)  # PHILOX_ROUND_A
_M1 = np.uint64(0xCD9E8D57)  # PHILOX_ROUND_B
_W0 = np.uint32(0x9E3779B9)  # PHILOX_KEY_A
_W1 = np.uint32(0xBB67AE85)  # PHILOX_KEY_B
_MASK = np.uint64(0xFFFFFFFF)

# e_bit, m_bit per format: rq/common.py convert_fp8_to_embit
EM_BITS = {torch.float8_e4m3fn: (4, 3), torch.float8_e5m2: (5, 2)}


def philox4x32_10(c0, c1, c2, c3, k0, k1, rounds=10):
    """Philox-4x32 (Salmon et al., SC'11) as triton/language/random.py:13-42 writes it.  uint32 arrays in and out."""
    c0, c1, c2, c3 = (np.asarray(c, dtype=np.uint32).copy() for c in (c0, c1, c2, c3))
    k0 = np.uint32(k0)
    k1 = np.uint32(k1)
    with np.errstate(over="ignore"):
        for _ in range(rounds):
            p0 = _M0 * c0.astype(np.uint64)  # A * c0
            p1 = _M1 * c2.astype(np.uint64)  # B * c2
            n0 = (p1 >> np.uint64(32)).astype(np.uint32) ^ c1 ^ k0
            n2 = (p0 >> np.uint64(32)).astype(np.uint32) ^ c3 ^ k1
            c1 = (p1 & _MASK).astype(np.uint32)
            c3 = (p0 & _MASK).astype(np.uint32)
            c0, c2 = n0, n2
            k0 = np.uint32((int(k0) + int(_W0)) & 0xFFFFFFFF)
            k1 = np.uint32((int(k1) + int(_W1)) & 0xFFFFFFFF)
    return c0, c1, c2, c3


def triton_randint(seed, offsets):
    """``tl.randint(seed, offset)`` for 32-bit offsets (triton/language/random.py:67-108)."""
    off = np.asarray(offsets).astype(np.uint32)
    z = np.zeros_like(off)
    seed = int(seed)
    return philox4x32_10(off, z, z, z, seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)[0]


def triton_rand(seed, offsets):
    """``tl.rand(seed, offset)``: uniform fp32 in [0, 1) (triton/language/random.py:127-157)."""
    x = triton_randint(seed, offsets).view(np.int32).astype(np.int64)
    x = np.where(x < 0, -x - 1, x)
    return x.astype(np.float32) * np.float32(4.6566127342e-10)


def stochastic_rounding(output, noise, e_bit, m_bit):
    """rq/_division.py:130-150 on fp32 numpy arrays, every step in fp32."""
    out = np.asarray(output, dtype=np.float32)
    noise = np.asarray(noise, dtype=np.float32)
    subnormal_min = np.float32(2.0 ** (2 - 2 ** (e_bit - 1) - m_bit))
    pow2 = (out.view(np.uint32) & np.uint32(0x7F800000)).view(np.float32)
    out_exp = np.maximum(pow2, subnormal_min)
    is_sub = out_exp == subnormal_min
    rescale = np.where(is_sub, np.float32(1.0), np.float32(2.0**m_bit)).astype(np.float32)
    nz = (out_exp * noise) / rescale
    mag = np.abs(out) + nz
    ratio = np.where(is_sub, np.float32(2.0**m_bit), np.float32(2.0)).astype(np.float32)
    mag = np.minimum(np.maximum(mag, out_exp), ratio * out_exp)
    sign = np.where(np.signbit(out), np.float32(-1.0), np.float32(1.0))
    return (sign * mag).astype(np.float32)


def fp8_division_stochastic(x, QB, fp8type, s_y=None, seed=0, noise=None):
    """rq/_division.py:153-207 with ``stochastic=True`` (kernel :84-114).  ``noise`` overrides the Philox draw."""
    fp8 = R._fp8(fp8type)
    if s_y is None:
        s_y = R.absmax_scale(x, fp8type)
    quot = (x.float() / s_y.float()).contiguous()
    if noise is None:
        noise = triton_rand(seed, np.arange(quot.numel(), dtype=np.int64)).reshape(quot.shape)
    e_bit, m_bit = EM_BITS[fp8]
    pert = stochastic_rounding(quot.numpy(), noise, e_bit, m_bit)
    return R.cast_fp8(torch.from_numpy(pert), fp8), s_y


def fp8_division_transpose_stochastic(x, QB, fp8type, s_y=None, only_transposed=False, seed=0):
    """rq/_division_transpose.py:147-210 with ``stochastic=True``: the noise index is the input's linear index."""
    q, s_y = fp8_division_stochastic(x, QB, fp8type, s_y, seed)
    q_t = q.view(torch.uint8).t().contiguous().view(q.dtype)
    return (q_t, s_y) if only_transposed else (q, s_y, q_t)
