"""GPU checks beyond 2^31 elements per tensor (64-bit indexing): every kernel works on independent rows / groups, so a
slice of the big result must equal, bit for bit, the result of running the same entry point on that slice alone.
The reference stops at 2^31 - 1 elements for the optimizer (int indices, fp8_adamw_expand_cuda_kernel.cu:33-35)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

ROWS, COLS = (1 << 15) + 32, 1 << 16  # 2,149,580,800 elements
PROBES = [(0, 32), (16400, 16432), (ROWS - 32, ROWS)]  # first rows, rows straddling element 2^30, the rows past 2^31


def _rq():
    import coat_amd.activation.real_quantization as rq
    return rq


def _big(dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    x = torch.empty((ROWS, COLS), dtype=torch.bfloat16, device=dev)
    for r0 in range(0, ROWS, 4096):  # in pieces: no 8 GiB fp32 temporary
        r1 = min(r0 + 4096, ROWS)
        x[r0:r1] = torch.randn((r1 - r0, COLS), generator=g, device=dev).bfloat16()
    return x


def _free(dev):
    torch.cuda.synchronize(dev)
    torch.cuda.empty_cache()


def test_quantize_and_division_past_2_31_elements(dev):
    rq = _rq()
    assert ROWS * COLS > 1 << 31
    x = _big(dev, 1)
    q, s = rq.fp8_quantize(x, 16, "E4M3")
    for r0, r1 in PROBES:
        wq, ws = rq.fp8_quantize(x[r0:r1].contiguous(), 16, "E4M3")
        assert torch.equal(q[r0:r1].view(torch.uint8), wq.view(torch.uint8)) and torch.equal(s[r0:r1], ws)
    del q, s
    scale = torch.tensor(0.0117, dtype=torch.bfloat16, device=dev)
    q, _, qt = rq.fp8_division_transpose(x, 16, "E5M2", scale)
    assert qt.shape == (COLS, ROWS)
    for r0, r1 in PROBES:
        wq, _, wqt = rq.fp8_division_transpose(x[r0:r1].contiguous(), 16, "E5M2", scale)
        assert torch.equal(q[r0:r1].view(torch.uint8), wq.view(torch.uint8))
        assert torch.equal(qt[:, r0:r1].view(torch.uint8), wqt.view(torch.uint8))
    del x, q, qt
    _free(dev)


def test_quantize_transpose_past_2_31_elements(dev):
    from coat_amd.activation.real_quantization._quantize_transpose import fp8_quantize_transpose
    x = _big(dev, 2)
    (q, s), (qt, st) = fp8_quantize_transpose(x, 16, "E4M3")
    assert qt.shape == (COLS, ROWS) and st.shape == (COLS, ROWS // 16)
    for r0, r1 in PROBES:
        (wq, ws), (wqt, wst) = fp8_quantize_transpose(x[r0:r1].contiguous(), 16, "E4M3")
        assert torch.equal(q[r0:r1].view(torch.uint8), wq.view(torch.uint8)) and torch.equal(s[r0:r1], ws)
        assert torch.equal(qt[:, r0:r1].view(torch.uint8), wqt.view(torch.uint8))
        assert torch.equal(st[:, r0 // 16:r1 // 16], wst)
    del x, q, s, qt, st
    _free(dev)


def test_quantize_perblock_past_2_31_elements(dev):
    from coat_amd.activation.real_quantization._quantize_perblock_transpose_pergroup import \
        fp8_quantize_perblock_transpose_pergroup
    x = _big(dev, 4)
    (q, s), (qt, st), (qg, sg) = fp8_quantize_perblock_transpose_pergroup(x, 32, "E4M3", scale_dtype=torch.float32)
    assert qt.shape == (COLS, ROWS) and st.shape == (COLS // 32, ROWS // 32) and sg.shape == (ROWS, COLS // 32)
    for r0, r1 in [(0, 32), (16384, 16416), (ROWS - 32, ROWS)]:  # whole rows of 32 x 32 blocks, the middle one at element 2^30
        (wq, ws), (wqt, wst), (wqg, wsg) = fp8_quantize_perblock_transpose_pergroup(x[r0:r1].contiguous(), 32, "E4M3",
                                                                                    scale_dtype=torch.float32)
        assert torch.equal(q[r0:r1].view(torch.uint8), wq.view(torch.uint8)) and torch.equal(s[r0 // 32:r1 // 32], ws)
        assert torch.equal(qt[:, r0:r1].view(torch.uint8), wqt.view(torch.uint8)) and torch.equal(st[:, r0 // 32:r1 // 32], wst)
        assert torch.equal(qg[r0:r1].view(torch.uint8), wqg.view(torch.uint8)) and torch.equal(sg[r0:r1], wsg)
    del x, q, s, qt, st, qg, sg
    _free(dev)


def test_adamw_expand_past_2_31_elements(dev):
    from coat_amd.optimizer import qoptim_cuda
    numel = (1 << 31) + 3 * 4096 + 77  # ragged last group
    ng = (numel + 127) // 128
    g = torch.Generator(device=dev).manual_seed(3)

    def filled(scale):
        t = torch.empty(numel, dtype=torch.float32, device=dev)
        for e0 in range(0, numel, 1 << 28):
            e1 = min(e0 + (1 << 28), numel)
            t[e0:e1] = torch.randn(e1 - e0, generator=g, device=dev) * scale
        return t

    p, grad = filled(0.02), filled(1e-3)

    def state(n, groups):
        return [torch.zeros(n, dtype=torch.float8_e4m3fn, device=dev), torch.zeros(groups, device=dev),
                torch.ones(groups, device=dev), torch.ones(groups, device=dev),
                torch.zeros(n, dtype=torch.float8_e4m3fn, device=dev), torch.zeros(groups, device=dev),
                torch.ones(groups, device=dev), torch.ones(groups, device=dev)]

    hp = (0.9, 0.95, 3e-4, 0.1, 1e-8)
    # the same tail (whole groups from a group boundary on) stepped on its own
    t0 = (ng - 1000) * 128
    p_tail, g_tail = p[t0:].clone(), grad[t0:].clone()
    st_tail = state(numel - t0, 1000)
    p_head, g_head = p[:4096].clone(), grad[:4096].clone()
    st_head = state(4096, 32)
    st = state(numel, ng)
    for step in (1, 2):
        qoptim_cuda.fp8_adamw_expand_step(p, grad, *st, *hp, step, 128, 16)
        qoptim_cuda.fp8_adamw_expand_step(p_tail, g_tail, *st_tail, *hp, step, 128, 16)
        qoptim_cuda.fp8_adamw_expand_step(p_head, g_head, *st_head, *hp, step, 128, 16)
    assert torch.equal(p[t0:], p_tail) and torch.equal(p[:4096], p_head)
    for big, tail, head in zip(st, st_tail, st_head):
        if big.dtype == torch.float8_e4m3fn:
            assert torch.equal(big[t0:].view(torch.uint8), tail.view(torch.uint8))
            assert torch.equal(big[:4096].view(torch.uint8), head.view(torch.uint8))
        else:
            assert torch.equal(big[ng - 1000:], tail) and torch.equal(big[:32], head)
    assert st[0].view(torch.uint8)[t0:].any()  # the tail was really stepped
    del p, grad, st
    _free(dev)
