"""Writes the fixtures in this directory.  Run from the repository root:  python tests/golden/make_golden.py

The reference holds no golden vectors for this path and cannot run here (its kernels need CUDA / Triton), so the
fixtures come from two sources, kept apart:

* ``fp8_known_answers.json`` is written BY HAND from the OCP 8-bit floating point specification (bit layouts, bias,
  largest finite value, smallest subnormal, NaN / inf encodings) and from worked group-quantization examples that can be
  checked with pencil and paper.  This script only re-serialises the literal table below; nothing in it is computed by
  the oracle.
* ``*.npz`` files freeze the outputs of the pinned CPU oracle (``oracle/``) on small seeded inputs, so that the HIP path is
  compared with committed bytes and a later edit of the oracle that changes any bit is noticed.

Arrays are plain uint8 / uint16 / float32 (bf16 tensors are stored as their uint16 bit patterns); no pickles.
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))

from oracle import activation_ref as R  # noqa: E402
from oracle import adamw_ref as A  # noqa: E402
from oracle import cross_entropy_ref as C  # noqa: E402
from oracle import stochastic_ref as S  # noqa: E402

# value -> code, by hand from the OCP FP8 specification.  e4m3fn: bias 7, no inf, NaN = S.1111.111, max 448 = 0x7E,
# min subnormal 2^-9 = 0x01.  e5m2: bias 15, inf = S.11111.00, max 57344 = 0x7B, min subnormal 2^-16 = 0x01.
# Ties go to the even code; values beyond the largest finite one saturate (the reference casts with satfinite).
KNOWN = {
    "e4m3": [[0.0, 0x00], [-0.0, 0x80], [1.0, 0x38], [-1.0, 0xB8], [1.125, 0x39], [1.0625, 0x38], [1.1875, 0x3A],
             [448.0, 0x7E], [-448.0, 0xFE], [1000.0, 0x7E], [464.0, 0x7E], [0.001953125, 0x01], [0.0009765625, 0x00],
             [0.0029296875, 0x02], [0.015625, 0x08], [0.017578125, 0x09], [240.0, 0x77], [0.5, 0x30], [3.0, 0x44]],
    "e5m2": [[0.0, 0x00], [1.0, 0x3C], [-1.0, 0xBC], [1.25, 0x3D], [1.125, 0x3C], [1.375, 0x3E], [57344.0, 0x7B],
             [-57344.0, 0xFB], [1.0e6, 0x7B], [1.52587890625e-05, 0x01], [7.62939453125e-06, 0x00], [0.5, 0x38],
             [3.0, 0x42], [49152.0, 0x7A]],
    # one 1 x 16 group, e4m3: amax 448 -> scale (448 + 1e-10) / 448 rounds to 1.0 in fp32; codes are those of the values
    "group_e4m3": {"x": [448.0, -224.0, 1.0, 0.0, 0.5, -0.5, 3.0, 240.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.001953125],
                   "scale_bf16_bits": 0x3F80,
                   "codes": [0x7E, 0xF6, 0x38, 0x00, 0x30, 0xB0, 0x44, 0x77, 0, 0, 0, 0, 0, 0, 0, 0x01]},
    # all-zero group: scale = 1e-10 / 448 (bf16 of 2.2321e-13 = 0x2A7B), codes 0
    "group_zero_scale_bf16_bits": 0x2A7B,
}


def bits16(t):
    return t.view(torch.int16).numpy().view(np.uint16).copy()


def u8(t):
    return t.view(torch.uint8).numpy().copy()


def make_quantize():
    g = torch.Generator().manual_seed(20240)
    x = (torch.randn(32, 64, generator=g) * torch.logspace(-3, 2, 32).unsqueeze(1)).bfloat16()
    x[3, 16:32] = 0  # an all-zero group
    x[5, 0] = 3.0e38  # a group whose scale is huge: its other members quantize to zero / subnormal codes
    out = {"x_bf16": bits16(x)}
    for name, ft in (("e4m3", "E4M3"), ("e5m2", "E5M2")):
        q, s = R.fp8_quantize(x, 16, ft)
        (q2, s2), (qt, st) = R.fp8_quantize_transpose(x, 16, ft)
        assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8))
        qp, sp, _ = R.fp8_quantize_pertensor(x, 16, ft)
        qp2, sp2, qpt = R.fp8_quantize_pertensor_transpose(x, 16, ft)
        out.update({f"{name}_q": u8(q), f"{name}_s": bits16(s), f"{name}_qt": u8(qt), f"{name}_st": bits16(st),
                    f"{name}_pt_q": u8(qp), f"{name}_pt_s": bits16(sp.reshape(1)), f"{name}_pt_qt": u8(qpt)})
    np.savez_compressed(os.path.join(HERE, "quantize_32x64_bf16.npz"), **out)


HP = dict(beta1=0.9, beta2=0.95, lr=1e-3, wd=0.1, eps=1e-8)
KEYS_EXP = ["exp_avg", "scale_exp_avg", "expand_exp_avg", "sqrt_minmax_exp_avg",
            "exp_avg_sq", "scale_exp_avg_sq", "expand_exp_avg_sq", "sqrt_minmax_exp_avg_sq"]
KEYS_PLAIN = ["exp_avg", "scale_exp_avg", "exp_avg_sq", "scale_exp_avg_sq"]


def make_adamw(expand):
    n = 1024 + 40  # a ragged last group
    g = torch.Generator().manual_seed(777)
    p = torch.randn(n, generator=g)
    st = A.fresh_state(p, expand)
    out = {"p0": p.numpy().copy()}
    keys = KEYS_EXP if expand else KEYS_PLAIN
    for step in (1, 2, 3):
        gr = torch.randn(n, generator=g) * 1e-3 * torch.logspace(-2, 1, n)
        out[f"g{step}"] = gr.numpy().copy()
        if expand:
            A.adamw_expand_step(p, gr, *[st[k] for k in keys], *HP.values(), step, 128, 16)
        else:
            A.adamw_step(p, gr, *[st[k] for k in keys], *HP.values(), step, 128)
        out[f"p{step}"] = p.numpy().copy()
        for k in keys:
            out[f"{k}{step}"] = u8(st[k]) if st[k].dtype == torch.float8_e4m3fn else st[k].numpy().copy()
    np.savez_compressed(os.path.join(HERE, "adamw_expand_1064.npz" if expand else "adamw_plain_1064.npz"), **out)


def make_stochastic():
    """Stochastic-rounding division of a [32, 64] tensor by 2^-3: codes for both formats (seed 0, as the reference)."""
    g = torch.Generator().manual_seed(4242)
    x = (torch.randn(32, 64, generator=g) * torch.logspace(-4, 1.5, 32).unsqueeze(1)).bfloat16()
    x[0, :8] = 0.0
    scale = torch.tensor(0.125, dtype=torch.bfloat16)
    out = {"x_bf16": bits16(x), "scale_bf16": bits16(scale.reshape(1))}
    for name, ft in (("e4m3", "E4M3"), ("e5m2", "E5M2")):
        q, _, qt = S.fp8_division_transpose_stochastic(x, 16, ft, scale)
        out[f"{name}_q"] = u8(q)
        out[f"{name}_qt"] = u8(qt)
    np.savez_compressed(os.path.join(HERE, "division_stochastic_32x64.npz"), **out)


CE_CASES = {  # name: (ignore_index, lse_square_scale, label_smoothing, reduction, softcap)
    "plain_mean": (-100, 0.0, 0.0, "mean", None),
    "smooth_z_sum": (-100, 1e-3, 0.1, "sum", None),
    "softcap_mean": (-100, 0.0, 0.0, "mean", 4.0),
}


def make_cross_entropy():
    g = torch.Generator().manual_seed(99)
    x = torch.randn(16, 97, generator=g) * 3
    t = torch.randint(0, 97, (16,), generator=g)
    t[[2, 9]] = -100
    out = {"x": x.numpy().copy(), "target": t.numpy().copy()}
    for name, (ii, lss, ls, red, cap) in CE_CASES.items():
        loss, z, grad = C.cross_entropy_forward(x, t, ii, lss, ls, red, cap)
        out[f"{name}_loss"] = np.float64(loss.item())
        out[f"{name}_z"] = np.float64(z.item())
        out[f"{name}_grad"] = grad.numpy().copy()
    np.savez_compressed(os.path.join(HERE, "cross_entropy_16x97.npz"), **out)


if __name__ == "__main__":
    with open(os.path.join(HERE, "fp8_known_answers.json"), "w") as f:
        json.dump(KNOWN, f, indent=1)
    make_quantize()
    make_adamw(True)
    make_adamw(False)
    make_stochastic()
    make_cross_entropy()
    print("golden fixtures written to", HERE)
