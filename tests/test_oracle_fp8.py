"""Pins oracle/fp8_codec.py (and through it the torch-CPU casts and the C codec in
oracle/adamw_ref.c) by closed forms and brute force."""
import numpy as np
import pytest
import torch

from oracle import adamw_ref, fp8_codec
from oracle.activation_ref import cast_fp8

FMTS = [(fp8_codec.E4M3, torch.float8_e4m3fn, 4, 3, 7), (fp8_codec.E5M2, torch.float8_e5m2, 5, 2, 15)]


def _finite_codes(fmt):
    codes = np.arange(256, dtype=np.uint8)
    vals = fp8_codec.decode(codes, fmt)
    keep = np.isfinite(vals)
    return codes[keep], vals[keep]


@pytest.mark.parametrize("fmt,tdtype,eb,mb,bias", FMTS)
def test_decode_closed_form_and_torch(fmt, tdtype, eb, mb, bias):
    codes = np.arange(256, dtype=np.uint8)
    vals = fp8_codec.decode(codes, fmt)
    # hand-evaluated anchors of the OCP formats
    if fmt == fp8_codec.E4M3:
        assert vals[0x7E] == 448.0 and vals[0x01] == 2.0 ** -9 and vals[0x08] == 2.0 ** -6 and np.isnan(vals[0x7F])
        assert vals[0x38] == 1.0 and vals[0xB8] == -1.0 and vals[0x3C] == 1.5
    else:
        assert vals[0x7B] == 57344.0 and vals[0x01] == 2.0 ** -16 and vals[0x04] == 2.0 ** -14
        assert np.isinf(vals[0x7C]) and np.isnan(vals[0x7D]) and vals[0x3C] == 1.0 and vals[0x3E] == 1.5
    tv = torch.from_numpy(codes).view(tdtype).float().numpy()
    np.testing.assert_array_equal(np.nan_to_num(vals, nan=12345.0), np.nan_to_num(tv, nan=12345.0))


def _nearest_even_f64(x, codes, vals):
    """Brute-force definition: nearest finite value in float64, ties to the even code, saturating."""
    pos = vals >= 0
    pc, pv = codes[pos & (codes < 0x80)], vals[pos & (codes < 0x80)].astype(np.float64)
    order = np.argsort(pv)
    pc, pv = pc[order], pv[order]
    a = np.minimum(np.abs(x.astype(np.float64)), pv[-1])  # saturating
    d = np.abs(a[:, None] - pv[None, :])
    best = d.min(axis=1)
    out = np.empty(len(x), dtype=np.uint8)
    for i in range(len(x)):
        cand = pc[d[i] == best[i]]
        c = cand[0] if len(cand) == 1 else [k for k in cand if k % 2 == 0][0]
        out[i] = c | (0x80 if np.signbit(x[i]) else 0)
    return out


@pytest.mark.parametrize("fmt,tdtype,eb,mb,bias", FMTS)
def test_encode_bruteforce(fmt, tdtype, eb, mb, bias):
    codes, vals = _finite_codes(fmt)
    pv = np.sort(vals[vals >= 0]).astype(np.float32)
    mids = ((pv[:-1].astype(np.float64) + pv[1:].astype(np.float64)) / 2).astype(np.float32)  # exact in fp32
    pts = np.concatenate([pv, mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(np.inf)),
                          np.nextafter(pv, np.float32(np.inf)), np.nextafter(pv[1:], np.float32(0)),
                          np.float32([1e-30, 1e-45, pv[-1] * 1.03, pv[-1] * 1.1, 1e30])])
    pts = np.concatenate([pts, -pts]).astype(np.float32)
    rng = np.random.default_rng(0)
    rnd = (rng.standard_normal(20000) * np.exp(rng.uniform(-12, 12, 20000))).astype(np.float32)
    x = np.concatenate([pts, rnd])
    got = fp8_codec.encode(x, fmt)
    want = _nearest_even_f64(x, codes, vals)
    np.testing.assert_array_equal(got, want)
    # NaN and infinities
    sp = fp8_codec.encode(np.float32([np.nan, np.inf, -np.inf]), fmt)
    assert sp[0] & 0x7F == 0x7F and sp[1] == (0x7E if fmt == fp8_codec.E4M3 else 0x7B) and sp[2] == sp[1] | 0x80


@pytest.mark.parametrize("fmt,tdtype,eb,mb,bias", FMTS)
def test_torch_cast_and_oracle_cast_match_codec(fmt, tdtype, eb, mb, bias):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(200000) * np.exp(rng.uniform(-14, 14, 200000))).astype(np.float32)
    x = np.concatenate([x, np.float32([0.0, -0.0, 448.0, 464.0, 465.0, 57344.0, 61440.0, 7e4, np.inf, -np.inf])])
    want = fp8_codec.encode(x, fmt)
    got = cast_fp8(torch.from_numpy(x), tdtype).view(torch.uint8).numpy()
    np.testing.assert_array_equal(got, want)
    # the raw torch cast agrees wherever it does not overflow (it yields NaN / inf there instead of saturating)
    lim = fp8_codec.FP8_MAX[fmt]
    inr = np.abs(x) <= lim
    raw = torch.from_numpy(x).to(tdtype).view(torch.uint8).numpy()
    np.testing.assert_array_equal(raw[inr], want[inr])
    n = cast_fp8(torch.tensor([float("nan")]), tdtype).view(torch.uint8).item()
    assert n & 0x7F == 0x7F


def test_c_codec_matches_numpy_codec():
    L = adamw_ref.lib()
    codes = np.arange(256, dtype=np.uint8)
    vals = fp8_codec.decode(codes, fp8_codec.E4M3)
    for c in range(256):
        v = L.coat_oracle_e4m3_decode(c)
        assert (np.isnan(v) and np.isnan(vals[c])) or v == vals[c]
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(20000) * np.exp(rng.uniform(-12, 8, 20000))).astype(np.float32)
    pv = np.sort(vals[np.isfinite(vals) & (vals >= 0)])
    mids = ((pv[:-1] + pv[1:]) / 2).astype(np.float32)
    x = np.concatenate([x, pv, mids, -mids, np.nextafter(mids, np.float32(0)), np.float32([np.inf, 1e9, 0.0, -0.0])])
    want = fp8_codec.encode(x, fp8_codec.E4M3)
    got = np.array([L.coat_oracle_e4m3_encode(float(v)) for v in x], dtype=np.uint8)
    np.testing.assert_array_equal(got, want)
    assert L.coat_oracle_e4m3_encode(float("nan")) & 0x7F == 0x7F
