"""Pins oracle/stochastic_ref.py (the reference's stochastic-rounding branch,
coat/activation/real_quantization/_division.py:96-150) without a GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import activation_ref as R
from oracle import stochastic_ref as S

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

# Random123 known-answer vectors for philox4x32-10: (counter, key, expected output)
PHILOX_KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((0xFFFFFFFF,) * 4, (0xFFFFFFFF, 0xFFFFFFFF), (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
     (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
]


@pytest.mark.parametrize("ctr,key,want", PHILOX_KAT)
def test_philox_known_answers(ctr, key, want):
    got = S.philox4x32_10(*[np.array([c], dtype=np.uint32) for c in ctr], key[0], key[1])
    assert tuple(int(g[0]) for g in got) == want


def test_rand_matches_tritons_interpreter():
    z = np.load(os.path.join(GOLDEN, "triton_rand_seed0.npz"))
    off = z["offsets"]
    assert np.array_equal(S.triton_randint(0, off).view(np.int32), z["randint_seed0"])
    assert np.array_equal(S.triton_rand(0, off).view(np.uint32), z["rand_seed0"].view(np.uint32))
    seed1 = int(z["seed1"])
    assert np.array_equal(S.triton_randint(seed1, off).view(np.int32), z["randint_seed1"])
    assert np.array_equal(S.triton_rand(seed1, off).view(np.uint32), z["rand_seed1"].view(np.uint32))


def test_rand_range_and_mean():
    u = S.triton_rand(0, np.arange(1 << 20))
    assert u.min() >= 0.0 and u.max() < 1.0
    assert abs(float(u.mean()) - 0.5) < 2e-3
    # the extreme integers map inside [0, 1)
    x = np.array([0x7FFFFFFF, -0x80000000, 0, -1], dtype=np.int64)
    f = np.where(x < 0, -x - 1, x).astype(np.float32) * np.float32(4.6566127342e-10)
    assert f.max() < 1.0 and f.min() == 0.0


@pytest.mark.parametrize("fp8", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_stochastic_rounding_properties(fp8):
    e_bit, m_bit = S.EM_BITS[fp8]
    sub_min = 2.0 ** (2 - 2 ** (e_bit - 1) - m_bit)
    g = torch.Generator().manual_seed(3)
    mag = torch.exp2(torch.empty(20000).uniform_(-12 if e_bit == 4 else -20, 8, generator=g))
    x = (mag * torch.where(torch.rand(20000, generator=g) < 0.5, -1.0, 1.0)).numpy()
    u = torch.rand(20000, generator=g).numpy()
    y = S.stochastic_rounding(x, u, e_bit, m_bit)
    e = np.maximum(np.exp2(np.floor(np.log2(np.abs(x)))).astype(np.float32), np.float32(sub_min))
    normal = e > sub_min
    # sign kept, magnitude never decreases (except the clamp up to the binade floor), stays inside the binade
    assert np.array_equal(np.signbit(y), np.signbit(x))
    assert np.all(np.abs(y) >= np.minimum(np.abs(x), e) - 0)
    assert np.all(np.abs(y)[normal] <= 2 * e[normal])
    assert np.all(np.abs(y)[normal] >= np.abs(x)[normal])
    # the shift is noise * (one FP8 step of the binade) exactly: powers of two times fp32 noise, one rounding in the add
    step = e / np.float32(2.0**m_bit)
    want = np.minimum(np.abs(x)[normal] + (step * u)[normal], 2 * e[normal])
    assert np.array_equal(np.abs(y)[normal], want.astype(np.float32))
    # noise 0 is the identity on everything at or above the smallest subnormal
    big = np.abs(x) >= sub_min
    assert np.array_equal(S.stochastic_rounding(x, np.zeros_like(u), e_bit, m_bit)[big], x[big])
    # monotone in the noise
    y2 = S.stochastic_rounding(x, (u + (1 - u) * np.float32(0.5)).astype(np.float32), e_bit, m_bit)
    assert np.all(np.abs(y2) >= np.abs(y))


def test_stochastic_rounding_small_values_as_the_reference_writes_them():
    # E4M3: smallest subnormal 2^-9.  Below 2^-8 the noise step is 2^-9 and the ceiling 8 * 2^-9;
    # zeros (and anything below 2^-9) are lifted to 2^-9 by the lower clamp, sign of the zero kept.
    x = np.array([0.0, -0.0, 2.0**-12, 2.0**-9, 1.5 * 2.0**-9, 2.0**-8, 1.5 * 2.0**-7], dtype=np.float32)
    y0 = S.stochastic_rounding(x, np.zeros_like(x), 4, 3)
    assert np.array_equal(y0, np.array([2.0**-9, -(2.0**-9), 2.0**-9, 2.0**-9, 1.5 * 2.0**-9, 2.0**-8, 1.5 * 2.0**-7],
                                       dtype=np.float32))
    yh = S.stochastic_rounding(x, np.full_like(x, 0.5), 4, 3)
    want = np.array([2.0**-9, -(2.0**-9), 2.0**-12 + 2.0**-10, 1.5 * 2.0**-9, 2.0**-8, 2.0**-8 + 2.0**-12,
                     1.5 * 2.0**-7 + 2.0**-11], dtype=np.float32)
    want[2] = 2.0**-9  # 2^-12 + 2^-10 < 2^-9: clamped up
    assert np.array_equal(yh, want)


@pytest.mark.parametrize("fp8", ["E4M3", "E5M2"])
def test_division_is_between_floor_and_ceil_and_unbiased_enough(fp8):
    torch.manual_seed(0)
    x = torch.randn(256, 512) * 3
    q, s = S.fp8_division_stochastic(x, 16, fp8)
    qd, _ = R.fp8_division(x, 16, fp8, s)
    quot = x.float() / s.float()
    val = q.float()
    dt = R._fp8(fp8)
    # every result is the round-to-nearest code of a value in [|quot|, |quot| + step): at most one code above
    # the deterministic one, never below it (in magnitude), for values in the normal range
    e_bit, m_bit = S.EM_BITS[dt]
    normal = quot.abs() >= 2.0 ** (3 - 2 ** (e_bit - 1))
    dv = qd.float()
    assert torch.all(val.abs()[normal] >= dv.abs()[normal])
    step = torch.exp2(torch.floor(torch.log2(quot.abs()))) / 2**m_bit
    assert torch.all((val.abs() - quot.abs())[normal] <= 1.5 * step[normal] + 1e-12)
    # forcing the noise to zero gives the deterministic branch wherever the value is not below the smallest subnormal
    q0, _ = S.fp8_division_stochastic(x, 16, fp8, s, noise=np.zeros(x.shape, dtype=np.float32))
    big = quot.abs() >= 2.0 ** (2 - 2 ** (e_bit - 1) - m_bit)
    assert torch.equal(q0.view(torch.uint8)[big], qd.view(torch.uint8)[big])
    # transposed output is the transpose, the noise index being the input's
    qa, _, qt = S.fp8_division_transpose_stochastic(x, 16, fp8, s)
    assert torch.equal(qa.view(torch.uint8), q.view(torch.uint8))
    assert torch.equal(qt.view(torch.uint8), q.view(torch.uint8).t())
