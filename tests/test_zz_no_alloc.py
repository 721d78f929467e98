"""GPU: the entry point that allocates nothing, coat_fp8_rmsnorm_backward_static, called through the C ABI.

It is coat_fp8_rmsnorm_backward with the weight-gradient partial rows in a device array that lives inside the library
instead of a caller-provided workspace.  With the same number of partial rows the two entry points run the same kernels
in the same order, so dx and dw must be bit-identical.  Two calls in a row, the second on a smaller input (fewer rows and
fewer columns, so that it reads a part of the array the first call filled with other values), then a wide row
(N = 16384, where the array holds 256 partial rows instead of 512)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(dev, M, N, seed, n_grads):
    from coat_amd.activation.real_quantization import fp8_quantize, fp8_rmsnorm_forward
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, N, generator=g).bfloat16().to(dev)
    w = (1 + 0.1 * torch.randn(N, generator=g)).bfloat16().to(dev)
    grads = [(torch.randn(M, N, generator=g) * 1e-2).bfloat16().to(dev) for _ in range(n_grads)]
    qx, sx = fp8_quantize(x, 16, "E4M3")
    _, _, _, (w_, rstd, _) = fp8_rmsnorm_forward(qx, sx, w, 16, 1e-5, transpose_output_2d=True)
    return qx, sx, w_, rstd, grads


def _call_both(dev, M, N, seed, n_grads):
    from coat_amd import _hip
    L = _hip.lib()
    qx, sx, w, rstd, grads = _inputs(dev, M, N, seed, n_grads)
    gp = [_hip.ptr(t) for t in grads] + [None] * (3 - n_grads)
    header_rows = min(512, (512 * 8192) // N)  # coat_rmsnorm_static_partials(N) of include/coat_hip.h
    st = _hip.stream(dev)
    out = []
    for static in (False, True):
        dx = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
        dw = torch.full((N,), float("nan"), dtype=w.dtype, device=dev)
        common = (_hip.ptr(qx), _hip.fp8(qx.dtype), _hip.ptr(sx), _hip.dt(sx), gp[0], gp[1], gp[2], _hip.ptr(w), _hip.dt(w),
                  _hip.ptr(rstd), _hip.ptr(dx), _hip.ptr(dw))
        if static:
            rc = L.coat_fp8_rmsnorm_backward_static(*common, M, N, 16, st)
        else:
            partial = torch.empty((header_rows, N), dtype=torch.float32, device=dev)
            rc = L.coat_fp8_rmsnorm_backward(*common, _hip.ptr(partial), header_rows, M, N, 16, st)
        assert rc == 0, rc
        out.append((dx, dw))
    torch.cuda.synchronize()
    (dx0, dw0), (dx1, dw1) = out
    assert torch.isfinite(dx1.float()).all() and torch.isfinite(dw1.float()).all()
    assert torch.equal(dx0, dx1), (M, N, "dx")
    assert torch.equal(dw0, dw1), (M, N, "dw")
    return dx1, dw1


def test_static_entry_point_equals_the_workspace_entry_point(dev):
    from oracle import activation_ref as R
    # first call: 2048 rows of 4096 (512 partial rows, 4 rows per block), three gradients summed in the kernel
    _call_both(dev, 2048, 4096, 1, 3)
    # second call, smaller in both directions: 304 rows (304 partial rows) of 1024 columns
    dx, dw = _call_both(dev, 304, 1024, 2, 1)
    # and the smaller call is still right against the CPU oracle (dx within 4 bf16 ulp on all but 5e-3, dw to bf16 accuracy)
    qx, sx, w, rstd, grads = _inputs(dev, 304, 1024, 2, 1)
    rdx, rdw = R.fp8_rmsnorm_backward(qx.cpu(), sx.cpu(), grads[0].cpu(), w.cpu(), rstd.cpu(), 16)
    err = (dx.cpu().float() - rdx.float()).abs()
    assert (err <= rdx.float().abs() * 2.0 ** -6 + 1e-8).float().mean().item() > 1 - 5e-3
    assert torch.allclose(dw.cpu().float(), rdw.float(), rtol=1e-2, atol=1e-3)  # bf16 output
    # a wide row: the array holds 256 partial rows of 16384 floats
    _call_both(dev, 512, 16384, 3, 2)
    # and back to the first shape: a third call after other shapes have used the array
    _call_both(dev, 2048, 4096, 4, 2)


def test_static_entry_point_rejects_what_it_cannot_hold(dev):
    from coat_amd import _hip
    L = _hip.lib()
    t = torch.zeros(64, device=dev)
    p = ctypes.c_void_p(t.data_ptr())
    args = (p, 0, p, 1, p, None, None, p, 1, p, p, p)
    assert L.coat_fp8_rmsnorm_backward_static(*args, 16, 32768, 16, None) == -2   # beyond the widest row
    assert L.coat_fp8_rmsnorm_backward_static(*args, 16, 4096 + 8, 16, None) == -2
    assert L.coat_fp8_rmsnorm_backward_static(*args, 0, 4096, 16, None) == 0      # empty: nothing to do
    assert L.coat_fp8_rmsnorm_backward_static(p, 0, p, 1, None, None, None, p, 1, p, p, p, 16, 4096, 16, None) == -1


def test_static_entry_point_under_graph_capture(dev):
    """What the entry point is for: one call recorded into a HIP graph (after a warm-up call outside the capture, which
    performs the once-per-device lookup of the scratch array's address) and replayed on new gradients, with eager work
    of the program between the replays; every replay bit-identical to the workspace entry point run eagerly."""
    from coat_amd import _hip
    L = _hip.lib()
    M, N = 1024, 4096
    qx, sx, w, rstd, grads = _inputs(dev, M, N, 11, 2)
    gen = torch.Generator().manual_seed(12)
    new_grads = [[(torch.randn(M, N, generator=gen) * (1e-2 * (r + 1))).bfloat16().to(dev) for _ in range(2)] for r in range(3)]
    static_g = [g.clone() for g in grads]
    dx = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    dw = torch.empty((N,), dtype=w.dtype, device=dev)
    rows = min(512, (512 * 8192) // N)

    def call_static():
        rc = L.coat_fp8_rmsnorm_backward_static(_hip.ptr(qx), _hip.fp8(qx.dtype), _hip.ptr(sx), _hip.dt(sx), _hip.ptr(static_g[0]),
                                                _hip.ptr(static_g[1]), None, _hip.ptr(w), _hip.dt(w), _hip.ptr(rstd),
                                                _hip.ptr(dx), _hip.ptr(dw), M, N, 16, _hip.stream(dev))
        assert rc == 0, rc

    def eager(gs):
        dx0 = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        dw0 = torch.empty((N,), dtype=w.dtype, device=dev)
        partial = torch.empty((rows, N), dtype=torch.float32, device=dev)
        rc = L.coat_fp8_rmsnorm_backward(_hip.ptr(qx), _hip.fp8(qx.dtype), _hip.ptr(sx), _hip.dt(sx), _hip.ptr(gs[0]), _hip.ptr(gs[1]),
                                         None, _hip.ptr(w), _hip.dt(w), _hip.ptr(rstd), _hip.ptr(dx0), _hip.ptr(dw0),
                                         _hip.ptr(partial), rows, M, N, 16, _hip.stream(dev))
        assert rc == 0, rc
        return dx0, dw0

    side = torch.cuda.Stream(device=dev)  # default priority
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        call_static()  # warm-up: the address lookup happens here, outside the capture
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize(dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call_static()
    torch.cuda.synchronize(dev)
    for gs in new_grads:
        want_dx, want_dw = eager(gs)  # eager work (which also allocates) between the replays
        torch.cuda.synchronize(dev)
        for dst, src in zip(static_g, gs):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize(dev)
        assert torch.equal(dx, want_dx) and torch.equal(dw, want_dw)
