"""The C ABI launches on the stream it is given (torch's current stream), never on the null stream: the same chain run
on a side stream, where every input comes straight out of a long producer kernel sequence on that stream, gives the
results of the default-stream run bit for bit.  (The reference's optimizer extension launches on the legacy default
stream whatever the caller's stream is: no stream argument at coat/optimizer/kernels/fp8_adamw_expand_cuda_kernel.cu:230.)"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _chain(dev):
    import coat_amd.activation.real_quantization as rq
    from coat_amd.activation.real_quantization.linear import fp8matmul
    from coat_amd.optimizer import qoptim_cuda
    g = torch.Generator(device=dev).manual_seed(11)
    a = torch.randn(2048, 2048, generator=g, device=dev).bfloat16()
    w = (torch.randn(2048, 2048, generator=g, device=dev) / 45).bfloat16()
    for _ in range(30):  # a long producer: the consumer below must wait for it through stream order alone
        a = torch.tanh(a @ w) * 3
    out = []
    q, s = rq.fp8_quantize(a, 16, "E4M3")
    out += [q.view(torch.uint8), s]
    qy, sy, qyt, (_, rstd, _) = rq.fp8_rmsnorm_forward(q, s, torch.ones(2048, device=dev, dtype=torch.bfloat16), 16, 1e-5)
    out += [qy.view(torch.uint8), sy, qyt.view(torch.uint8), rstd]
    pq, ps, pqt = rq.fp8_quantize_pertensor_transpose(a, 16, "E5M2")
    out += [pq.view(torch.uint8), ps, pqt.view(torch.uint8)]
    c = fp8matmul(qy, qyt.t(), False, sy, sy, 16)  # [2048, 2048] x [2048, 2048]
    out.append(c)
    p = a.float().clone()
    grad = c.float() * 1e-3
    st = [torch.zeros_like(p, dtype=torch.float8_e4m3fn), torch.zeros(p.numel() // 128, device=dev),
          torch.ones(p.numel() // 128, device=dev), torch.ones(p.numel() // 128, device=dev),
          torch.zeros_like(p, dtype=torch.float8_e4m3fn), torch.zeros(p.numel() // 128, device=dev),
          torch.ones(p.numel() // 128, device=dev), torch.ones(p.numel() // 128, device=dev)]
    for step in (1, 2):
        qoptim_cuda.fp8_adamw_expand_step(p, grad, *st, 0.9, 0.95, 3e-4, 0.1, 1e-8, step, 128, 16)
    out += [p, st[0].view(torch.uint8), st[1], st[4].view(torch.uint8), st[5]]
    return out


def test_entry_points_follow_the_callers_stream(dev):
    want = _chain(dev)
    torch.cuda.synchronize(dev)
    side = torch.cuda.Stream(device=dev)  # default priority
    with torch.cuda.stream(side):
        got = _chain(dev)
    side.synchronize()
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert torch.equal(a, b), f"output {i} differs between the side stream and the default stream"
