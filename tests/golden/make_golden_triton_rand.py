"""Writes tests/golden/triton_rand_seed0.npz: ``tl.randint`` / ``tl.rand`` as Triton's own CPU interpreter
(TRITON_INTERPRET=1, no GPU) evaluates them, for seed 0 (the seed the reference hard-codes,
coat/activation/real_quantization/_division.py:110) and one 64-bit seed.

Triton is the third-party dependency that owns this arithmetic (triton>=3.1.0 in the reference's
pyproject.toml:16; the vectors were written with the version printed into the file).  Nothing of the
reference is imported.  Run from the repository root:  python tests/golden/make_golden_triton_rand.py
"""
import os

os.environ["TRITON_INTERPRET"] = "1"

import numpy as np  # noqa: E402
import torch  # noqa: E402
import triton  # noqa: E402
import triton.language as tl  # noqa: E402


@triton.jit
def _draw(off_ptr, f_ptr, i_ptr, seed, N: tl.constexpr):
    idx = tl.arange(0, N)
    off = tl.load(off_ptr + idx)
    tl.store(f_ptr + idx, tl.rand(seed, off))
    tl.store(i_ptr + idx, tl.randint(seed, off))


def draw(seed, offsets):
    n = offsets.numel()
    f = torch.empty(n, dtype=torch.float32)
    i = torch.empty(n, dtype=torch.int32)
    _draw[(1,)](offsets, f, i, seed, N=n)
    return f.numpy(), i.numpy()


def main():
    g = torch.Generator().manual_seed(0)
    offsets = torch.cat([
        torch.arange(0, 64, dtype=torch.int32),
        torch.randint(0, 2**31 - 1, (60,), generator=g, dtype=torch.int64).to(torch.int32),
        torch.tensor([2**31 - 1, 4096 * 4096 - 1, 8192 * 11008, 1 << 30], dtype=torch.int32),
    ])
    f0, i0 = draw(0, offsets)
    f1, i1 = draw(0x1234567_89ABCDEF, offsets)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "triton_rand_seed0.npz")
    np.savez(out, offsets=offsets.numpy(), rand_seed0=f0, randint_seed0=i0, seed1=np.int64(0x1234567_89ABCDEF),
             rand_seed1=f1, randint_seed1=i1, triton_version=np.array(triton.__version__))
    print("wrote", out, "triton", triton.__version__)


if __name__ == "__main__":
    main()
