"""Benchmark of the FP8 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|adamw|quantize|quantize_transpose|gemm_fwd|...]

Prints ONE JSON line.  The default run (--workload all) times the headline configuration as `value` and adds an `extra`
record for every other leg of the metric (quantize, quantize + transpose, the three GEMMs of the 7B MLP linear, the
SiLU*mul and RMSNorm chains, the 7B and 13B decoder layers), each with its own roofline and CPU baseline.

Headline = one CoatAdamW.step() (Dynamic Range Expansion on) on an fp32 master weight [11008, 4096], grads N(0, 1e-3),
lr 3e-4, betas (0.9, 0.95), wd 0.1, eps 1e-8, starting at step 10 from a moment state produced by nine untimed steps.
A "step" is one pass of the fused kernel over the whole tensor.  `value` is algorithmic GB/s: every distinct input read
once + every output written once (in-place tensors count read + write) divided by the wall-clock per step with inputs
resident in HBM.  `roofline.achieved` uses the kernel's average launch duration: HIP events on the launch stream around
the K back-to-back launches of the timed region, divided by K (per-launch event pairs of a second pass give the spread).
`cpu_baseline` times the CPU oracle (the plain-C AdamW port on every host core; the torch restatements for the other
legs) on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

PROBE_SRC = os.path.join(ROOT, "bench_probe.hip")
PROBE_LIB = os.path.join(ROOT, "libcoat_bench_probe.so")
_probe_lib = None


def build_probe(verbose=True):
    """Compiles bench_probe.hip (the copy / read / fill probe and the clock-probe instances of the GEMM kernel) into
    libcoat_bench_probe.so beside this file.  Measurement code only: nothing of it is part of libcoat_hip.so."""
    import subprocess

    from coat_amd import build as hip_build

    cmd = [hip_build.HIPCC, *hip_build.FLAGS, "-shared", "-I", ROOT, PROBE_SRC, "-o", PROBE_LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on bench_probe.hip:\n" + r.stdout + r.stderr)
    if verbose:
        print(f"[bench] built {PROBE_LIB}")
    return PROBE_LIB


def probe_lib():
    """The measurement library: loaded if it has been built (python -c 'import bench; bench.build_probe()' or
    __graft_entry__.build()), built first otherwise."""
    global _probe_lib
    if _probe_lib is None:
        import ctypes

        if not os.path.exists(PROBE_LIB):
            build_probe()
        L = ctypes.CDLL(PROBE_LIB)
        vp, i64 = ctypes.c_void_p, ctypes.c_int64
        L.bench_hbm_probe.argtypes = [ctypes.c_int, vp, vp, i64, vp]
        L.bench_pattern_probe.argtypes = [ctypes.c_int, vp, vp, vp, i64, i64, vp]
        L.bench_pattern_probe.restype = ctypes.c_int
        L.bench_gemm_clock.argtypes = [vp, ctypes.c_int, vp, vp, vp, vp, i64, i64, i64, vp, vp]
        L.bench_hbm_probe.restype = L.bench_gemm_clock.restype = ctypes.c_int
        _probe_lib = L
    return _probe_lib


def adamw_bytes(numel):
    ngroups = (numel + 127) // 128
    # p r+w (4+4), g r (4), m8 r+w (1+1), v8 r+w (1+1) per element; 6 fp32 group vectors r+w per group
    return numel * 16 + ngroups * 48


def make_adamw_workload(dev, shape, torch, expand=True):
    from coat_amd.optimizer import qoptim_cuda

    numel = shape[0] * shape[1]
    gen = torch.Generator(device="cpu").manual_seed(0)
    p = (torch.randn(shape, generator=gen) * 0.02).to(dev)
    ng = (numel + 127) // 128
    st = [torch.zeros(shape, dtype=torch.float8_e4m3fn, device=dev), torch.zeros(ng, device=dev),
          torch.ones(ng, device=dev), torch.ones(ng, device=dev),
          torch.zeros(shape, dtype=torch.float8_e4m3fn, device=dev), torch.zeros(ng, device=dev),
          torch.ones(ng, device=dev), torch.ones(ng, device=dev)]
    hp = (0.9, 0.95, 3e-4, 0.1, 1e-8)
    grads = []
    for seed in range(1, 5):  # a few distinct gradient tensors, cycled
        g = torch.Generator(device="cpu").manual_seed(seed)
        grads.append((torch.randn(shape, generator=g) * 1e-3).to(dev))

    state = {"step": 0}

    def step():
        state["step"] += 1
        if expand:
            qoptim_cuda.fp8_adamw_expand_step(p, grads[state["step"] % len(grads)], *st, *hp, state["step"], 128, 16)
        else:  # the same step without Dynamic Range Expansion: codes and scales only
            qoptim_cuda.fp8_adamw_step(p, grads[state["step"] % len(grads)], st[0], st[1], st[4], st[5], *hp,
                                       state["step"], 128)

    for _ in range(9):  # steps 1..9: builds a realistic moment state (k, c per group), untimed
        step()
    if expand:
        return step, adamw_bytes(numel), {"workload": "qoptim_cuda.fp8_adamw_expand_step (the call CoatAdamW.step makes) fp32 [11008,4096], DRE on, step 10+, qgroup 128",
                                          "numel": numel, "kernel": "k_fp8_adamw_expand"}
    return step, numel * 16 + ng * 16, {"workload": "qoptim_cuda.fp8_adamw_step fp32 [11008,4096], DRE off, step 10+, qgroup 128",
                                        "numel": numel, "kernel": "k_fp8_adamw_plain"}


def make_adamw_class_workload(dev, shape, torch):
    """The same step through the optimizer class: CoatAdamW.step() on one fp32 parameter [11008, 4096] (the host loop of
    coat/optimizer/fp8_adamw.py:264-515 is then inside the timed region; it ends in the same kernel launch)."""
    from coat_amd.optimizer.fp8_adamw import CoatAdamW
    from coat_amd.utils._fp8_quantization_config import QuantizationConfig

    numel = shape[0] * shape[1]
    gen = torch.Generator(device="cpu").manual_seed(0)
    p = torch.nn.Parameter((torch.randn(shape, generator=gen) * 0.02).to(dev))
    grads = []
    for seed in range(1, 5):  # a few distinct gradient tensors, cycled
        g = torch.Generator(device="cpu").manual_seed(seed)
        grads.append((torch.randn(shape, generator=g) * 1e-3).to(dev))
    opt = CoatAdamW([p], lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1, qargs=QuantizationConfig())
    assert opt.use_expansion, "the headline configuration runs with Dynamic Range Expansion"
    state = {"i": 0}

    def step():
        state["i"] += 1
        p.grad = grads[state["i"] % len(grads)]
        opt.step()

    for _ in range(9):  # steps 1..9: builds a realistic moment state (k, c per group), untimed
        step()
    return step, adamw_bytes(numel), {"workload": "CoatAdamW.step() on one fp32 parameter [11008,4096], DRE on, step 10+, "
                                                  "qgroup 128 (optimizer class host loop + k_fp8_adamw_expand)",
                                      "numel": numel, "kernel": "k_fp8_adamw_expand"}


def make_quantize_workload(dev, torch, transpose, shape=(4096, 4096)):
    from coat_amd.activation.real_quantization import fp8_quantize
    from coat_amd.activation.real_quantization._quantize_transpose import fp8_quantize_transpose

    M, N = shape
    gen = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn(M, N, generator=gen)
    x[torch.rand(M, N, generator=gen) < 0.001] *= 100
    # rotate over buffer sets so that > 512 MB is touched between reuses (the 256 MB Infinity Cache stays cold)
    nset = max(4, min(12, (640 << 20) // (M * N * 2) + 1))
    xs = [x.bfloat16().to(dev).clone() for _ in range(nset)]
    state = {"i": 0}
    fn = fp8_quantize_transpose if transpose else fp8_quantize

    def step():
        state["i"] += 1
        fn(xs[state["i"] % nset], 16, "E4M3")

    nbytes = M * N * 2 + (2 if transpose else 1) * (M * N + M * N // 16 * 2)
    name = "fp8_quantize_transpose" if transpose else "fp8_quantize"
    return step, nbytes, {"workload": f"{name} bf16 [{M},{N}] QB16 e4m3, {nset} rotating inputs", "numel": M * N,
                          "kernel": "k_quantize_transpose" if transpose else "k_quantize_pg"}


def make_perblock_workload(dev, torch, shape):
    """fp8_quantize_perblock_transpose_pergroup (coat/activation/real_quantization/_quantize_perblock_transpose_pergroup.py:175)
    of a bf16 tensor, QB 128, fp32 scales, only_transposed as the DeepSeek-style linear calls it on a gradient
    (coat/activation/deepseek/fp8linear.py:97-99): 2 bytes read, the transposed per-block codes and the per-group codes
    written (1 byte each) plus their scales."""
    from coat_amd.activation.real_quantization._quantize_perblock_transpose_pergroup import \
        fp8_quantize_perblock_transpose_pergroup

    M, N = shape
    gen = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn(M, N, generator=gen) * 1e-2
    nset = max(4, min(12, (640 << 20) // (M * N * 2) + 1))
    xs = [x.bfloat16().to(dev).clone() for _ in range(nset)]
    state = {"i": 0}

    def step():
        state["i"] += 1
        fp8_quantize_perblock_transpose_pergroup(xs[state["i"] % nset], 128, "E4M3", scale_dtype=torch.float32,
                                                 only_transposed=True)

    nbytes = M * N * 4 + (M // 128) * (N // 128) * 4 + M * (N // 128) * 4
    return step, nbytes, {"workload": f"fp8_quantize_perblock_transpose_pergroup bf16 [{M},{N}] QB128 e4m3 fp32 scales, "
                                      f"only_transposed, {nset} rotating inputs", "numel": M * N, "kernel": "k_quantize_perblock"}


def make_gemm_workload(dev, torch, which, grad_format="e5m2"):
    """The three GEMMs of FP8Linear at BASELINE config 3 on the config's own data: X [8192,4096] ~ N(0, 0.02),
    W [11008,4096] ~ N(0, 0.02), grad_out [8192,11008] ~ N(0, 1e-2), bf16, each quantized with its per-tensor scale by
    fp8_quantize_pertensor_transpose (what the module does), and the GEMM gets those codes and scales.
    which = fwd | dgrad | wgrad.  The gradient is e5m2 as the reference's default bobit; grad_format="e4m3" times the
    all-e4m3 variant."""
    from coat_amd.activation.real_quantization._quantize_pertensor_transpose import fp8_quantize_pertensor_transpose
    from coat_amd.activation.real_quantization.linear import fp8matmul

    gfmt = "E5M2" if grad_format == "e5m2" else "E4M3"
    T, K, N = 8192, 4096, 11008
    gen = torch.Generator(device=dev).manual_seed(0)

    def quantized(shape, std, fmt):
        t = (torch.randn(shape, generator=gen, device=dev) * std).bfloat16()
        return fp8_quantize_pertensor_transpose(t, 16, fmt, transpose_output_2d=True)

    qx, sx, qxt = quantized((T, K), 0.02, "E4M3")
    qw, sw, qwt = quantized((N, K), 0.02, "E4M3")
    if which == "fwd":      # Y[T,N] = X[T,K] W[N,K]^T
        a, b, sa, sb, (M_, N_, K_) = qx, qw, sx, sw, (T, N, K)
    else:
        qg, sg, qgt = quantized((T, N), 1e-2, gfmt)
        if which == "dgrad":  # dX[T,K] = G[T,N] Wt[K,N]^T
            a, b, sa, sb, (M_, N_, K_) = qg, qwt, sg, sw, (T, K, N)
        else:                 # dW[N,K] = Gt[N,T] Xt[K,T]^T
            a, b, sa, sb, (M_, N_, K_) = qgt, qxt, sg, sx, (N, K, T)
    a, b = a.contiguous(), b.contiguous()
    del qx, qxt, qw, qwt

    def step():
        fp8matmul(a, b.t(), False, sa, sb, 16)

    flops = 2 * M_ * N_ * K_
    fmt = "e4m3 x e4m3" if which == "fwd" or grad_format == "e4m3" else "e5m2 x e4m3"
    return step, flops, {"workload": f"fp8matmul {which}: [{M_},{K_}] x [{N_},{K_}]^T -> bf16, {fmt}; operands = "
                                     f"per-tensor-quantized X, W ~ N(0,0.02), grad_out ~ N(0,1e-2) with their own scales",
                         "M": M_, "N": N_, "K": K_, "kernel": "k_fp8_gemm"}


def make_linear_workload(dev, torch):
    """The same linear end to end: FP8Linear forward + backward at the Llama-2-7B MLP shape: per-tensor quantization
    (with transposes) of X, W and the output gradient, then the three GEMMs.  Returns (fp8 step, bf16 step, flops)."""
    from coat_amd.activation.real_quantization.fp8linear import FP8Linear

    T, K, N = 8192, 4096, 11008
    torch.manual_seed(0)
    lin = FP8Linear(K, N, bias=False, device=dev).to(torch.bfloat16).train()
    torch.nn.init.normal_(lin.weight, std=0.02)
    ref = torch.nn.Linear(K, N, bias=False, device=dev, dtype=torch.bfloat16)
    ref.weight.data.copy_(lin.weight.data)
    x = (torch.randn(4, 2048, K, device=dev) * 0.02).bfloat16()
    g = (torch.randn(4, 2048, N, device=dev) * 1e-2).bfloat16()

    def run(mod):
        def step():
            mod.weight.grad = None
            xin = x.detach().requires_grad_(True)
            mod(xin).backward(g)
        return step

    return run(lin), run(ref), 3 * 2 * T * K * N, {
        "workload": f"FP8Linear fwd+bwd: X bf16 [4,2048,{K}] x W [{N},{K}], e4m3 per-tensor X/W, e5m2 grad, bf16 outputs",
        "M": T, "N": N, "K": K}


def make_silu_mul_workload(dev, torch):
    """The Llama-2-7B MLP activation: SiLU(gate) * up on bf16 [8192,11008] inputs -> FP8 with 1x16 scales (and the saved FP8
    activations), then the backward chain with a bf16 gradient, as CoatLlamaMLPResidual strings the kernels together
    (coat/models/coat_llama.py:664-766)."""
    import coat_amd.activation.real_quantization as rq

    M, N, QB = 8192, 11008, 16
    gen = torch.Generator(device=dev).manual_seed(0)
    gate = torch.randn(M, N, generator=gen, device=dev).bfloat16()
    up = torch.randn(M, N, generator=gen, device=dev).bfloat16()
    g = (torch.randn(M, N, generator=gen, device=dev) * 1e-2).bfloat16()

    def step():
        # one pass over the bf16 inputs: gate / up / SiLU(gate) as per-group FP8 (saved for backward) + the product's maximum,
        # then the recomputing division; bit-identical to fp8_quantize x 2 followed by fp8_silu_mul_forward
        qg, sg, qu, su, qs, ss, _, _, _ = rq.fp8_silu_mul_forward_from_bf16(gate, up, QB, "E4M3", transpose_output_2d=True)
        rq.fp8_silu_mul_backward(qg, sg, qu, su, qs, ss, g, QB, "E5M2")

    E = M * N
    # forward: read 2 bf16 inputs (4E), write gate / up / silu codes + scales 3(E + E/8), write product q + q^T (2E);
    # backward: read g (2E) + the three saved FP8 tensors 3(E + E/8), write two gradients as q + q^T (4E)
    nbytes = int(4 * E + 3 * (E + E / 8) + 2 * E + 2 * E + 3 * (E + E / 8) + 4 * E)
    return step, nbytes, {"workload": f"SiLU(gate)*up fwd + bwd chain on bf16 [{M},{N}], 1x16 e4m3 / per-tensor e5m2 outputs",
                          "M": M, "N": N, "kernel": "k_silu_mul, k_produced_division_transpose, k_division_transpose"}


def make_rmsnorm_workload(dev, torch):
    """RMSNorm on the FP8 block input [8192,4096] -> FP8 (+ transpose), and its backward."""
    import coat_amd.activation.real_quantization as rq

    M, N, QB = 8192, 4096, 16
    gen = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(M, N, generator=gen, device=dev).bfloat16()
    w = torch.ones(N, device=dev, dtype=torch.bfloat16)
    g = (torch.randn(M, N, generator=gen, device=dev) * 1e-2).bfloat16()
    q, s = rq.fp8_quantize(x, QB, "E4M3")

    def step():
        qy, sy, qyt, (_, rstd, nw) = rq.fp8_rmsnorm_forward(q, s, w, QB, 1e-5, transpose_output_2d=True)
        rq.fp8_rmsnorm_backward(q, s, g, w, rstd, QB, nw)

    E = M * N
    nbytes = int((E + E / 8) + 2 * E + (E + E / 8) + 2 * E + 2 * E)  # fwd: codes+scales in, q + q^T out; bwd: codes+scales, dy in, dx out
    return step, nbytes, {"workload": f"RMSNorm fwd (FP8 in -> per-tensor FP8 + transpose) + bwd on [{M},{N}]",
                          "M": M, "N": N, "kernel": "k_rmsnorm_fwd, k_division_transpose, k_rmsnorm_bwd, k_rmsnorm_dw"}


def make_cross_entropy_workload(dev, torch):
    """LM-head loss of Llama-2 (vocabulary 32000) on 4 x 2048 tokens, fp32 logits as the reference computes it
    (coat/activation/liger/cross_entropy.py:396-411).  One step = loss + in-place gradient, i.e. one read and one
    write of the logits: 8 bytes per logit."""
    from coat_amd.activation.liger.cross_entropy import cross_entropy_forward
    BT, V = 8192, 32000
    torch.manual_seed(0)
    base = torch.randn(BT, V, device=dev)
    work = torch.empty_like(base)
    target = torch.randint(0, V, (BT,), device=dev)

    def step():
        cross_entropy_forward(work, target, -100, 0.0, 0.0, "mean", None, False)

    # the kernel overwrites its input: the logits are restored before every step, outside the timed events
    step.prepare = lambda: work.copy_(base)
    cfg = {"workload": f"cross_entropy fp32 [{BT},{V}], loss + in-place gradient (logits restored by an untimed device "
                       "copy before each step; ms_per_step is the sum of the timed events)",
           "kernel": "k_cross_entropy"}
    return step, 8 * BT * V, cfg


class Bf16DecoderLayer:
    """The same Llama decoder layer in plain bf16 torch (F.linear / F.rms_norm / F.silu / SDPA): the baseline the FP8
    layer has to beat (benchmark/benchmark_llamalayer.py of the reference times HF's LlamaDecoderLayer the same way)."""

    def __init__(self, torch, coat_layer):
        self.torch = torch
        self.p = {n: p.detach().clone().requires_grad_(True) for n, p in coat_layer.named_parameters()}
        self.nh = coat_layer.self_attn.num_heads

    def __call__(self, x):
        import torch.nn.functional as F
        from coat_amd.models._attention import torch_sdpa as sdpa  # torch's fastest backend here, forward and backward
        from coat_amd.models.coat_llama import fused_rotary
        p, torch = self.p, self.torch
        B, S, H = x.shape
        hd = H // self.nh
        h = F.rms_norm(x, (H,), p["input_layernorm.weight"], 1e-5)
        # the same fused RoPE kernel as the FP8 layer uses, so that the comparison is about the FP8 flow only
        q = fused_rotary(F.linear(h, p["BeforeAttention.q_proj.weight"]), self.nh, hd, 10000.0)
        k = fused_rotary(F.linear(h, p["BeforeAttention.k_proj.weight"]), self.nh, hd, 10000.0)
        v = F.linear(h, p["BeforeAttention.v_proj.weight"]).view(B, S, self.nh, hd).transpose(1, 2)
        a = sdpa(q, k, v, is_causal=True).transpose(1, 2).reshape(B, S, H)
        x1 = x + F.linear(a, p["AfterAttention.o_proj.weight"])
        h2 = F.rms_norm(x1, (H,), p["post_attention_layernorm.weight"], 1e-5)
        m = F.silu(F.linear(h2, p["MLPResidual.gate_proj.weight"])) * F.linear(h2, p["MLPResidual.up_proj.weight"])
        return x1 + F.linear(m, p["MLPResidual.down_proj.weight"])


class Bf16OLMoBlock:
    """The OLMo sequential block in plain bf16 torch (non-parametric LayerNorm, fused qkv and up/gate projections,
    SwiGLU), the baseline of --workload olmo_block."""

    def __init__(self, torch, blk):
        self.p = {n: p.detach().clone().requires_grad_(True) for n, p in blk.named_parameters()}
        self.nh, self.fused_dims = blk.config.n_heads, blk.fused_dims

    def __call__(self, x):
        import torch.nn.functional as F
        from coat_amd.models._attention import torch_sdpa as sdpa  # torch's fastest backend here, forward and backward
        from coat_amd.models.coat_llama import fused_rotary
        p = self.p
        B, S, D = x.shape
        hd = D // self.nh
        q, k, v = F.linear(F.layer_norm(x, (D,), None, None, 1e-5), p["BeforeAttention.att_proj.weight"]).split(self.fused_dims, dim=-1)
        q = fused_rotary(q.contiguous(), self.nh, hd, 10000.0)
        k = fused_rotary(k.contiguous(), self.nh, hd, 10000.0)
        v = v.reshape(B, S, self.nh, hd).transpose(1, 2)
        a = sdpa(q, k, v, is_causal=True).transpose(1, 2).reshape(B, S, D)
        x1 = x + F.linear(a, p["AfterAttention.attn_out.weight"])
        up, gate = F.linear(F.layer_norm(x1, (D,), None, None, 1e-5), p["MLPResidual.ff_proj.weight"]).chunk(2, dim=-1)
        return x1 + F.linear(F.silu(gate) * up, p["MLPResidual.ff_out.weight"])


def make_olmo_workload(dev, torch):
    """CoatOLMoSequentialBlock fwd+bwd at the OLMo-7B shape (d_model 4096, 32 heads, mlp_hidden_size 22016),
    batch 4 x seq 2048, random init N(0, 0.02) (coat/models/coat_olmo.py:910-1076)."""
    from coat_amd.activation.real_quantization import Coat_quantize_bgn, Coat_quantize_end
    from coat_amd.models.coat_olmo import CoatOLMoConfig, CoatOLMoSequentialBlock
    from coat_amd.utils._fp8manager import FP8Manager

    D, heads, hidden = 4096, 32, 22016
    B, S = 4, 2048
    torch.manual_seed(0)
    cfg = CoatOLMoConfig(d_model=D, n_heads=heads, mlp_hidden_size=hidden)
    blk = CoatOLMoSequentialBlock(0, cfg)
    for p in blk.parameters():
        torch.nn.init.normal_(p, std=0.02)
    blk = blk.to(dev).to(torch.bfloat16).train()
    bgn, end = Coat_quantize_bgn(blk.qargs), Coat_quantize_end(blk.qargs)
    x = torch.randn(B, S, D, device=dev, dtype=torch.bfloat16)
    gy = torch.randn(B, S, D, device=dev, dtype=torch.bfloat16) * 1e-2
    ref = Bf16OLMoBlock(torch, blk)
    state = {"first": True}

    def step_fp8():
        FP8Manager.is_first_microbatch = state["first"]
        state["first"] = False
        for p in blk.parameters():
            p.grad = None
        h, q, s = bgn(x.detach().requires_grad_(True))
        h, q, s, _ = blk(h, q, s)
        end(h, q, s).backward(gy)

    def step_bf16():
        for p in ref.p.values():
            p.grad = None
        ref(x.detach().requires_grad_(True)).backward(gy)

    gemm_flops = 3 * 2 * B * S * (4 * D * D + D * hidden + D * hidden // 2)
    return step_fp8, step_bf16, gemm_flops, {
        "workload": f"CoatOLMoSequentialBlock fwd+bwd, OLMo-7B shape (d_model {D}, heads {heads}, mlp_hidden_size {hidden}), "
                    f"batch {B} x seq {S}, FP8 linears/activations/LayerNorm, bf16 attention (this library's forward kernel, torch's backward)",
        "tokens": B * S, "gemm_flops": gemm_flops}


def make_layernorm_workload(dev, torch):
    """Non-parametric LayerNorm on the FP8 block input [8192,4096] -> per-tensor FP8 (+ transpose), and its backward
    (coat/activation/real_quantization/func_layernorm_noparam.py:188-297), as the OLMo block calls them."""
    import coat_amd.activation.real_quantization as rq

    M, N, QB = 8192, 4096, 16
    gen = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(M, N, generator=gen, device=dev).bfloat16()
    g = (torch.randn(M, N, generator=gen, device=dev) * 1e-2).bfloat16()
    q, s = rq.fp8_quantize(x, QB, "E4M3")

    def step():
        qy, sy, qyt, (mean, rstd, nw) = rq.fp8_layernorm_noparam_forward(q, s, QB, 1e-5, transpose_output_2d=True)
        rq.fp8_layernorm_noparam_backward(q, s, g, QB, mean, rstd, nw)

    E = M * N
    nbytes = int((E + E / 8) + 2 * E + (E + E / 8) + 2 * E + 2 * E)  # fwd: codes+scales in, q + q^T out; bwd: codes+scales, dy in, dx out
    return step, nbytes, {"workload": f"LayerNorm (no parameters) fwd (FP8 in -> per-tensor FP8 + transpose) + bwd on [{M},{N}]",
                          "M": M, "N": N, "kernel": "k_layernorm_fwd, k_division_transpose, k_layernorm_bwd"}


def make_hbm_probe_workload(dev, torch, kind):
    """What this box's HBM delivers to the simplest kernels on 1 GiB (bench_hbm_probe of bench_probe.hip: one 16-byte access per lane,
    streaming loads): "copy" (1 GiB read + 1 GiB written), "read", "fill".  These are the practical ceilings the
    streaming kernels are compared with next to the nominal 8 TB/s."""
    from coat_amd import _hip
    L = probe_lib()
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src) if kind != "read" else torch.zeros(16, dtype=torch.uint8, device=dev)
    code = {"copy": 0, "read": 1, "fill": 2}[kind]

    def step():
        _hip.check(L.bench_hbm_probe(code, _hip.ptr(src), _hip.ptr(dst), n, _hip.stream(dev)), "hbm_probe")

    return step, (2 * n if kind == "copy" else n), {"workload": f"hbm_probe {kind}: bench_hbm_probe on 1 GiB",
                                                      "kernel": "k_hbm_probe"}


def make_pattern_probe_workload(dev, torch, kind, shape):
    """The access pattern of the per-tensor division kernels with the arithmetic taken out (bench_pattern_probe of
    bench_probe.hip): "narrow" = k_division's (16-byte loads of 2-byte elements, 8-byte stores of 1-byte codes), "tile" =
    k_division_transpose's (128 x 128 tiles, 32 bytes per lane in, 16 bytes into q and 16 into q^T out, no LDS).  Four
    rotating buffer sets, so the memory-side cache holds nothing of the next launch.  The time of these is what the memory
    system allows the real kernels at the same shape."""
    from coat_amd import _hip
    L = probe_lib()
    M, N = shape
    if kind == "tile" and (M % 128 or N % 128):
        raise SystemExit("hbm_tile needs --shape M N with both multiples of 128")
    nset = 4
    xs = [torch.empty(M * N, dtype=torch.bfloat16, device=dev).fill_(1.0) for _ in range(nset)]
    qs = [torch.empty(M * N, dtype=torch.uint8, device=dev) for _ in range(nset)]
    qts = [torch.empty(M * N, dtype=torch.uint8, device=dev) for _ in range(nset)] if kind == "tile" else [None] * nset
    code = {"narrow": 0, "tile": 1}[kind]
    state = {"i": 0}

    def step():
        i = state["i"] = (state["i"] + 1) % nset
        _hip.check(L.bench_pattern_probe(code, _hip.ptr(xs[i]), _hip.ptr(qs[i]), _hip.ptr(qts[i]), M, N, _hip.stream(dev)),
                   "pattern_probe")

    nbytes = M * N * (3 if kind == "narrow" else 4)
    return step, nbytes, {"workload": f"pattern probe {kind}: bench_pattern_probe on 2-byte [{M},{N}], {nset} rotating buffer sets",
                          "kernel": "k_narrow_probe" if kind == "narrow" else "k_tile_probe"}


def make_division_workload(dev, torch, stochastic, transpose=False, shape=(8192, 4096)):
    """Per-tensor division bf16 [8192,4096] (or --shape) -> e5m2 with a given scale, deterministic or with the reference's stochastic
    rounding (coat/activation/real_quantization/_division.py:153-207): 2 bytes read + 1 written per element; with
    ``transpose`` the transposed copy is written too (_division_transpose.py:147-210, 2 + 2 bytes)."""
    import coat_amd.activation.real_quantization as rq

    M, N = shape
    gen = torch.Generator(device=dev).manual_seed(0)
    xs = [torch.randn(M, N, generator=gen, device=dev).bfloat16() for _ in range(max(4, min(6, (400 << 20) // (M * N * 2) + 1)))]
    scale = torch.tensor(0.01, device=dev, dtype=torch.bfloat16)
    it = {"i": 0}

    def step():
        it["i"] = (it["i"] + 1) % len(xs)
        if transpose:
            rq.fp8_division_transpose(xs[it["i"]], 16, "E5M2", scale)
        else:
            rq.fp8_division(xs[it["i"]], 16, "E5M2", scale, stochastic=stochastic)

    name = "fp8_division_transpose" if transpose else "fp8_division"
    return step, (4 if transpose else 3) * M * N, {
        "workload": f"{name} bf16 [{M},{N}] -> e5m2, stochastic={stochastic}", "M": M, "N": N,
        "kernel": "k_division_transpose" if transpose else "k_division"}


def make_layer_workload(dev, torch, size, cache_weights=False):
    """COAT Llama decoder layer fwd+bwd, batch 4 x seq 2048, random init N(0, 0.02)."""
    from coat_amd.activation.real_quantization import Coat_quantize_bgn, Coat_quantize_end
    from coat_amd.models.coat_llama import CoatLlamaConfig, CoatLlamaDecoderLayer
    from coat_amd.utils._fp8manager import FP8Manager

    H, heads, I = (4096, 32, 11008) if size == "7b" else (5120, 40, 13824)
    B, S = 4, 2048
    torch.manual_seed(0)
    # cache_weights: weight_memory_efficient=False, i.e. FP8 weights and their transposes are kept from the first
    # micro-batch on (coat/utils/_fp8_weightcache.py:11-37) instead of being re-quantized in every forward and backward
    cfg = CoatLlamaConfig(hidden_size=H, intermediate_size=I, num_attention_heads=heads,
                          coat_fp8_args={"weight_memory_efficient": not cache_weights})
    layer = CoatLlamaDecoderLayer(cfg, 0)
    for p in layer.parameters():
        if p.dim() == 2:
            torch.nn.init.normal_(p, std=0.02)
    layer = layer.to(dev).to(torch.bfloat16).train()
    bgn, end = Coat_quantize_bgn(layer.qargs), Coat_quantize_end(layer.qargs)
    x = torch.randn(B, S, H, device=dev, dtype=torch.bfloat16)
    gy = torch.randn(B, S, H, device=dev, dtype=torch.bfloat16) * 1e-2
    ref = Bf16DecoderLayer(torch, layer)
    state = {"first": True}

    def step_fp8():
        FP8Manager.is_first_microbatch = state["first"]  # True once, then False (benchmark_llamalayer.py:185-191)
        state["first"] = False
        for p in layer.parameters():
            p.grad = None  # forward + backward only: no accumulation into an existing gradient
        xin = x.detach().requires_grad_(True)
        h, q, s = bgn(xin)
        (h, q, s), = layer(h, q, s)
        end(h, q, s).backward(gy)

    def step_bf16():
        for p in ref.p.values():
            p.grad = None
        xin = x.detach().requires_grad_(True)
        ref(xin).backward(gy)

    gemm_flops = 3 * 2 * B * S * (4 * H * H + 3 * H * I)
    return step_fp8, step_bf16, gemm_flops, {
        "workload": f"CoatLlamaDecoderLayer fwd+bwd, Llama-2-{size.upper()} shape (H {H}, heads {heads}, I {I}), "
                    f"batch {B} x seq {S}, FP8 linears/activations/norms, bf16 attention (this library's forward kernel, torch's backward)"
                    + (", FP8 weights cached across micro-batches" if cache_weights else ""),
        "tokens": B * S, "gemm_flops": gemm_flops}


def host_threads():
    """CPU threads this process may use: the affinity mask, capped at the 16 cores a one-GPU box grants."""
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    return max(1, min(n, 16))


def _median(ts):
    ts = sorted(ts)
    return ts[len(ts) // 2]


def cpu_baseline_adamw(torch):
    """The plain-C oracle on every host core: one thread per core, each stepping its own 4096-group slab of the tensor
    (groups are independent, so this is how a CPU run of the whole tensor would be split), same hyper-parameters, moment
    state built by three oracle steps, about 10 s of wall clock."""
    import threading

    from oracle import adamw_ref as A

    hp = (0.9, 0.95, 3e-4, 0.1, 1e-8)
    n = 128 * 4096  # elements per thread
    T = host_threads()
    keys = ("exp_avg", "scale_exp_avg", "expand_exp_avg", "sqrt_minmax_exp_avg", "exp_avg_sq", "scale_exp_avg_sq",
            "expand_exp_avg_sq", "sqrt_minmax_exp_avg_sq")
    A.lib()
    slabs = []
    for t in range(T):
        gen = torch.Generator().manual_seed(t)
        p = torch.randn(n, generator=gen) * 0.02
        st = A.fresh_state(p, True)
        grads = [torch.randn(n, generator=gen) * 1e-3 for _ in range(4)]
        for step in (1, 2, 3):
            A.adamw_expand_step(p, grads[step % 4], *[st[k] for k in keys], *hp, step, 128, 16)
        slabs.append((p, st, grads))
    reps = [0] * T
    t_end = time.perf_counter() + 10.0

    def work(t):
        p, st, grads = slabs[t]
        step = 3
        while time.perf_counter() < t_end:
            step += 1
            A.adamw_expand_step(p, grads[step % 4], *[st[k] for k in keys], *hp, step, 128, 16)  # ctypes drops the GIL
            reps[t] += 1

    t0 = time.perf_counter()
    threads = [threading.Thread(target=work, args=(t,)) for t in range(T)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    dt = time.perf_counter() - t0
    return {"value": round(adamw_bytes(n) * sum(reps) / dt / 1e9, 4), "unit": "GB/s", "cores": T, "kind": "port",
            "sample": f"oracle/adamw_ref.c, {T} threads, each stepping its own slab of {n} elements (4096 groups) of the "
                      f"tensor, {sum(reps)} slab steps in {dt:.1f} s"}


# HBM / fabric bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs, scaled by what the same
# counters read for a 256 MiB copy).  The counters cannot be read inside this process: the figures come from the separate
# profiling runs recorded under profiles/, not from this run.
MEASURED_TRAFFIC = {
    "adamw": (760.3e6, "profiles/k_fp8_adamw_expand__adamw_11008x4096.txt"),
    "quantize": (52.5e6, "profiles/k_quantize_pg__quantize_4096x4096_bf16.txt"),
    "quantize_transpose": (73.6e6, "profiles/k_quantize_transpose__quantize_transpose_4096x4096_bf16.txt"),
    "gemm_fwd": (696.9e6, "profiles/k_fp8_gemm__llama7b_mlp_8192tok.txt"),
    "gemm_dgrad": (561.4e6, "profiles/k_fp8_gemm__llama7b_mlp_8192tok.txt"),
    "cross_entropy": (2100.3e6, "profiles/k_cross_entropy__llama2_vocab32000_8192tok_fp32.txt"),
    "silu_mul": (2620.2e6, "profiles/k_silu_mul__silu_mul_8192x11008.txt (the five launches of forward + backward together; two passes over the tensors)"),
    "rmsnorm": (332.5e6, "profiles/k_rmsnorm__rmsnorm_8192x4096.txt (the four kernels of forward + backward together)"),
}


def cpu_baseline_quantize(torch, transpose, nbytes):
    """The torch-CPU oracle on the whole [4096,4096] input (same seeded data), all host threads, 3 warm-ups, median of 10."""
    from oracle import activation_ref as R

    gen = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn(4096, 4096, generator=gen)
    x[torch.rand(4096, 4096, generator=gen) < 0.001] *= 100
    x = x.bfloat16()
    fn = R.fp8_quantize_transpose if transpose else R.fp8_quantize
    for _ in range(3):
        fn(x, 16, "E4M3")
    ts = []
    for _ in range(10):
        t0 = time.perf_counter()
        fn(x, 16, "E4M3")
        ts.append(time.perf_counter() - t0)
    return {"value": round(nbytes / _median(ts) / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"the whole bf16 [4096,4096] input, oracle/activation_ref.py ({fn.__name__}), median of 10 runs"}


def cpu_baseline_gemm(torch, which):
    """The oracle's GEMM (fp32 matmul of the decoded FP8 operands, times the two scales, rounded to bf16) on a 1024-row slab of
    the left operand, all host threads, median of 3."""
    from oracle import activation_ref as R

    T, K, N = 8192, 4096, 11008
    M_, N_, K_ = {"fwd": (T, N, K), "dgrad": (T, K, N), "wgrad": (N, K, T)}[which]
    rows = 1024
    gen = torch.Generator().manual_seed(0)
    a = torch.randn(rows, K_, generator=gen).to(torch.float8_e4m3fn)
    b = torch.randn(N_, K_, generator=gen).to(torch.float8_e4m3fn)
    one = torch.tensor(0.01, dtype=torch.bfloat16)
    R.fp8matmul(a, b.t(), False, one, one, 16)
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        R.fp8matmul(a, b.t(), False, one, one, 16)
        ts.append(time.perf_counter() - t0)
    return {"value": round(2 * rows * N_ * K_ / _median(ts) / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": f"oracle/activation_ref.py fp8matmul on {rows} of the {M_} rows of the left operand, median of 3 runs"}


def cpu_baseline_attention(torch):
    """The oracle's attention (oracle/attention_ref.py: fp32 scores, mask, softmax and weighted sum written out) on 4 of the
    128 (batch, head) pairs of the workload, all host threads, median of 3."""
    from oracle import attention_ref

    S, D, heads = 2048, 128, 4
    gen = torch.Generator().manual_seed(0)
    q, k, v = [torch.randn(1, heads, S, D, generator=gen).bfloat16() for _ in range(3)]
    attention_ref.attention(q, k, v)
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        attention_ref.attention(q, k, v)
        ts.append(time.perf_counter() - t0)
    flops = 2 * 2 * heads * S * S * D // 2  # the same count as the GPU leg: the visible half
    return {"value": round(flops / _median(ts) / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle/attention_ref.py on {heads} of the 128 (batch, head) pairs (2048 tokens, head dimension 128), median of 3 runs"}


def cpu_baseline_silu_mul(torch, nbytes_full):
    """The oracle's chain (quantize x 2, SiLU, mul, mul backward, SiLU backward, all with their per-tensor divisions) on a
    256-row slab of the [8192, 11008] inputs, all host threads, median of 3."""
    from oracle import activation_ref as R

    rows, M, N, QB = 256, 8192, 11008, 16
    gen = torch.Generator().manual_seed(0)
    gate, up = torch.randn(rows, N, generator=gen).bfloat16(), torch.randn(rows, N, generator=gen).bfloat16()
    g = (torch.randn(rows, N, generator=gen) * 1e-2).bfloat16()

    def chain():
        qg, sg = R.fp8_quantize(gate, QB, "E4M3")
        qu, su = R.fp8_quantize(up, QB, "E4M3")
        qs, ss = R.fp8_silu_forward(qg, sg, QB)
        R.fp8_mul_forward(qs, ss, qu, su, QB)
        g1, _ = R.fp8_mul_backward(qs, ss, qu, su, g, QB, "E5M2", True)
        R.fp8_silu_backward(qg, sg, g1, QB, "E5M2", True)

    chain()
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        chain()
        ts.append(time.perf_counter() - t0)
    return {"value": round(nbytes_full * rows / M / _median(ts) / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": f"oracle/activation_ref.py chain on {rows} of the {M} rows, median of 3 runs"}


def cpu_baseline_rmsnorm(torch, nbytes_full):
    from oracle import activation_ref as R

    rows, M, N, QB = 1024, 8192, 4096, 16
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(rows, N, generator=gen).bfloat16()
    w = torch.ones(N, dtype=torch.bfloat16)
    g = (torch.randn(rows, N, generator=gen) * 1e-2).bfloat16()
    q, s = R.fp8_quantize(x, QB, "E4M3")

    def chain():
        _, _, _, rstd = R.fp8_rmsnorm_forward(q, s, w, QB, 1e-5)
        R.fp8_rmsnorm_backward(q, s, g, w, rstd, QB, accumulate=torch.float32)

    chain()
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        chain()
        ts.append(time.perf_counter() - t0)
    return {"value": round(nbytes_full * rows / M / _median(ts) / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": f"oracle/activation_ref.py forward + backward on {rows} of the {M} rows, median of 3 runs"}


def cpu_baseline_layer(torch, size):
    """The layer as the chain of the CPU oracle's operations (oracle/layer_ref.py: the reference's call order through
    norm, quantized projections, SiLU * up, residual adds and their backward, fp32 SDPA in between), forward + backward
    on one sequence of 256 tokens with every host core torch uses; ms scaled by tokens to the 4 x 2048 of the GPU run
    (attention, a few per cent of the work, scales worse; the weights' re-quantization does not scale at all)."""
    from oracle import layer_ref

    H, heads, I = (4096, 32, 11008) if size == "7b" else (5120, 40, 13824)
    S = 256
    gen = torch.Generator().manual_seed(0)
    W = {n: (torch.randn(shape, generator=gen) * 0.02).bfloat16() for n, shape in
         (("q", (H, H)), ("k", (H, H)), ("v", (H, H)), ("o", (H, H)), ("gate", (I, H)), ("up", (I, H)), ("down", (H, I)))}
    W["norm1"], W["norm2"] = torch.ones(H).bfloat16(), torch.ones(H).bfloat16()
    x = torch.randn(S, H, generator=gen).bfloat16()
    gy = (torch.randn(S, H, generator=gen) * 1e-2).bfloat16()
    t0 = time.perf_counter()
    layer_ref.decoder_layer_step(x, gy, W, heads, 1)
    ms = (time.perf_counter() - t0) * 1e3
    return {"value": round(ms * 8192 / S, 1), "unit": "ms", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle chain of the layer (oracle/layer_ref.py), forward + backward on 1 x {S} tokens: {ms:.0f} ms, "
                      f"one run, scaled by 8192 / {S} tokens"}


def ramp_clocks(step, seconds, torch):
    """Keep the GPU continuously busy with `step` for `seconds` (untimed) so that the timed region runs at the sustained clock."""
    if seconds <= 0:
        return
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            step()
        torch.cuda.synchronize()


def gemm_clock(dev, torch):
    """The shader clock the FP8 GEMM really runs at.  bench_probe.hip instantiates the library's GEMM kernel with its
    PROBE switch: every block records its duration in shader clocks (s_memtime) and in ticks of the constant 100 MHz
    counter (s_memrealtime); their ratio is the clock.  Operands: the per-tensor-quantized config-3 tensors of the gemm_*
    workloads, and all zeros."""
    from coat_amd import _hip
    from coat_amd.activation.real_quantization._quantize_pertensor_transpose import fp8_quantize_pertensor_transpose

    L = probe_lib()
    probe = torch.zeros(2 * 256, dtype=torch.int64, device=dev)
    T, K, N = 8192, 4096, 11008
    gen = torch.Generator(device=dev).manual_seed(0)

    def quantized(shape, std, fmt):
        t = (torch.randn(shape, generator=gen, device=dev) * std).bfloat16()
        return fp8_quantize_pertensor_transpose(t, 16, fmt, transpose_output_2d=True)

    qx, sx, qxt = quantized((T, K), 0.02, "E4M3")
    qw, sw, qwt = quantized((N, K), 0.02, "E4M3")
    qg, sg, qgt = quantized((T, N), 1e-2, "E5M2")
    cases = (("fwd", qx, qw, sx, sw), ("dgrad", qg, qwt, sg, sw), ("wgrad", qgt, qxt, sg, sx),
             ("dgrad_zero_operands", torch.zeros_like(qg), torch.zeros_like(qwt), sg, sw))
    out = {}
    for name, a, b, sa, sb in cases:
        a, b = a.contiguous(), b.contiguous()
        (M, Kd), Nd = a.shape, b.shape[0]
        c = torch.empty((M, Nd), dtype=torch.bfloat16, device=dev)

        def step():
            _hip.check(L.bench_gemm_clock(_hip.ptr(a), _hip.fp8(a.dtype), _hip.ptr(b), _hip.ptr(c), _hip.ptr(sa), _hip.ptr(sb),
                                          M, Nd, Kd, _hip.ptr(probe), _hip.stream(dev)), "bench_gemm_clock")

        ramp_clocks(step, 2.0, torch)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        ev[0].record()
        for _ in range(50):
            step()
        ev[1].record()
        torch.cuda.synchronize()
        ms = ev[0].elapsed_time(ev[1]) / 50
        p = probe.cpu().view(-1, 2).double()
        tiles = ((M + 255) // 256) * ((Nd + 255) // 256)
        ideal = tiles * ((Kd + 127) // 128) * 2048 / 256  # MFMA clocks per CU if the matrix pipes never waited
        mhz = p[:, 0] / p[:, 1] * 100.0
        out[name] = {"us_per_launch": round(ms * 1e3, 1), "tflops": round(2 * M * Nd * Kd / ms / 1e9, 0),
                     "shader_clock_mhz_mean": round(mhz.mean().item()), "shader_clock_mhz_min": round(mhz.min().item()),
                     "shader_clock_mhz_max": round(mhz.max().item()), "block_shader_clocks_mean": round(p[:, 0].mean().item()),
                     "mfma_clocks_ideal_per_cu": round(ideal), "mfma_busy_of_block_clocks": round(ideal / p[:, 0].mean().item(), 4),
                     "peak_at_this_clock_tflops": round(256 * 8192 * mhz.mean().item() / 1e6, 0)}
    print(json.dumps({"workload": "gemm_clock", "operands": "per-tensor-quantized X, W ~ N(0,0.02), grad_out ~ N(0,1e-2) (config 3)",
                      "gemm": out}))


METRIC = "quantize+AdamW GB/s (% HBM peak); FP8 GEMM TFLOPS; 7B-layer fwd+bwd ms"
LAYER_WORKLOADS = ("layer_7b", "layer_13b", "linear", "olmo_block")


def measure_layer(name, args, dev, torch, cpu):
    if name == "linear":
        step_fp8, step_bf16, gemm_flops, cfg = make_linear_workload(dev, torch)
    elif name == "olmo_block":
        step_fp8, step_bf16, gemm_flops, cfg = make_olmo_workload(dev, torch)
    else:
        step_fp8, step_bf16, gemm_flops, cfg = make_layer_workload(dev, torch, name.split("_")[1], args.cache_weights)

    def time_it(fn):
        ramp_clocks(fn, args.ramp_seconds, torch)
        for _ in range(max(2, args.warmup // 2)):
            fn()
        torch.cuda.synchronize()
        evs = []
        t0 = time.perf_counter()
        for _ in range(args.steps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / args.steps
        ms = sorted(a.elapsed_time(b) for a, b in evs)
        return wall, ms[len(ms) // 2], ms[len(ms) // 5], ms[(4 * len(ms)) // 5]

    wall8, med8, p20, p80 = time_it(step_fp8)
    wall16, med16, _, _ = time_it(step_bf16)
    rec = {
        "value": round(wall8, 4), "unit": "ms", "ms_per_step": round(wall8, 4), "higher_is_better": False,
        "dtype": "fp8", "config": cfg,
        "layer": {"fp8_ms_median": round(med8, 4), "fp8_ms_p20": round(p20, 4), "fp8_ms_p80": round(p80, 4),
                  "bf16_ms_median": round(med16, 4), "bf16_ms_per_step": round(wall16, 4),
                  "speedup_vs_bf16": round(med16 / med8, 4),
                  "fp8_gemm_tflops_equiv": round(gemm_flops / (med8 * 1e-3) / 1e12, 1)},
        "roofline": {"bound": "mfma", "achieved": round(gemm_flops / (med8 * 1e-3) / 1e12, 2), "peak": 5000.0,
                     "unit": "TFLOP/s", "frac": round(gemm_flops / (med8 * 1e-3) / 1e12 / 5000.0, 4), "traffic": None,
                     "note": "GEMM flops of the step over the whole step's time (attention and the FP8 glue kernels included)"},
        "cpu_baseline": cpu_baseline_layer(torch, name.split("_")[1]) if cpu and name.startswith("layer_") else None,
    }
    return rec


def make_attention_workload(dev, torch):
    """The bf16 attention forward of the 7B decoder layer: batch 4, 32 heads, 2048 tokens, head dimension 128, causal; q / k / v
    as the projections leave them ([B, S, H, 128] seen as [B, H, S, 128]).  One step = one launch of the MFMA kernel.  FLOPs: the two products over the visible (lower-triangular) half, 2 * 2 * B * H * S^2 / 2 * 128."""
    from coat_amd.models._attention import attention_forward

    B, H, S, D = 4, 32, 2048, 128
    gen = torch.Generator(device=dev).manual_seed(0)
    q, k, v = [torch.randn(B, S, H, D, generator=gen, device=dev).bfloat16().transpose(1, 2) for _ in range(3)]

    def step():
        attention_forward(q, k, v, causal=True)

    return step, 2 * 2 * B * H * S * S * D // 2, {
        "workload": f"attention forward bf16, causal, batch {B} x {H} heads x {S} tokens x head_dim {D} (k_attn_fwd)",
        "kernel": "k_attn_fwd", "batch": B, "heads": H, "seq": S, "head_dim": D}


def make_stream_workload(name, args, dev, torch):
    if name == "attention":
        return make_attention_workload(dev, torch)
    if name in ("adamw", "adamw_plain"):
        return make_adamw_workload(dev, (11008, 4096), torch, expand=name == "adamw")
    if name == "adamw_class":
        return make_adamw_class_workload(dev, (11008, 4096), torch)
    if name.startswith("gemm"):
        return make_gemm_workload(dev, torch, name.split("_")[1], args.grad_format)
    if name == "cross_entropy":
        return make_cross_entropy_workload(dev, torch)
    if name == "quantize_perblock":
        return make_perblock_workload(dev, torch, tuple(args.shape) if args.shape != [4096, 4096] else (8192, 4096))
    if name in ("hbm_narrow", "hbm_tile"):
        return make_pattern_probe_workload(dev, torch, name.split("_")[1], tuple(args.shape) if args.shape != [4096, 4096] else (8192, 4096))
    if name.startswith("hbm_"):
        return make_hbm_probe_workload(dev, torch, name.split("_")[1])
    if name == "layernorm":
        return make_layernorm_workload(dev, torch)
    if name in ("division", "division_sr", "division_transpose"):
        return make_division_workload(dev, torch, name == "division_sr", transpose=name == "division_transpose",
                                      shape=tuple(args.shape) if args.shape != [4096, 4096] else (8192, 4096))
    if name == "silu_mul":
        return make_silu_mul_workload(dev, torch)
    if name == "rmsnorm":
        return make_rmsnorm_workload(dev, torch)
    return make_quantize_workload(dev, torch, name == "quantize_transpose", tuple(args.shape))


def measure_stream(name, args, dev, torch, cpu):
    """One workload whose step is a short chain of launches: K steps between two synchronisations for `value`, HIP events
    on the launch stream around the same K back-to-back launches for the average launch duration of the roofline."""
    is_gemm = name.startswith("gemm") or name == "attention"  # MFMA-bound legs: `nbytes` holds FLOPs
    step, nbytes, cfg = make_stream_workload(name, args, dev, torch)
    ramp_clocks(step, args.ramp_seconds, torch)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    prepare = getattr(step, "prepare", None)
    # (1) the timed region: exactly K steps between two synchronisations, nothing else in the loop
    wall = region_ms = None
    if not prepare:
        ra, rb = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ra.record()
        for _ in range(args.steps):
            step()
        rb.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        region_ms = ra.elapsed_time(rb)  # HIP events over the timed region: K launches back to back
    # (2) the same K steps again with HIP events around every launch, on the stream the kernels are launched on (torch's
    # current stream): median / p20 / p80 of the launch duration (event records inside loop (1) would add their gaps
    # to the wall clock)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in evs:
        if prepare:
            prepare()
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    kern_ms = sorted(a.elapsed_time(b) for a, b in evs)
    avg_ms = sum(kern_ms) / len(kern_ms) if prepare else region_ms / args.steps
    ms_per_step = avg_ms if prepare else wall * 1e3 / args.steps
    value = nbytes / (ms_per_step * 1e-3) / 1e9
    achieved = nbytes / (avg_ms * 1e-3) / 1e9
    unit, peak, bound = ("TFLOP/s", 2500.0 if name == "attention" else 5000.0, "mfma") if is_gemm else ("GB/s", HBM_PEAK_GBS, "hbm")
    if is_gemm:  # nbytes holds FLOPs for the GEMM workloads; report TFLOP/s
        value, achieved = value / 1e3, achieved / 1e3
    traffic = MEASURED_TRAFFIC.get("adamw" if name == "adamw_class" else name) if args.shape == [4096, 4096] else None
    rec = {
        "value": round(value, 2), "unit": unit, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "dtype": "bf16" if name == "attention" else "fp8" if is_gemm else ("f32" if name.startswith("adamw") else "bf16"), "config": cfg,
        "roofline": {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
                     "frac": round(achieved / peak, 4), "traffic": traffic[0] if traffic else None,
                     "traffic_source": (traffic[1] + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE in a separate run, not this run)") if traffic else None,
                     ("algorithmic_flops_per_launch" if is_gemm else "algorithmic_bytes_per_launch"): nbytes, "kernel_ms_avg": round(avg_ms, 5),
                     "kernel_ms_median": round(kern_ms[len(kern_ms) // 2], 5),
                     "kernel_ms_per_launch_events_avg": round(sum(kern_ms) / len(kern_ms), 5),
                     "kernel_ms_p20": round(kern_ms[len(kern_ms) // 5], 5), "kernel_ms_p80": round(kern_ms[(4 * len(kern_ms)) // 5], 5)},
        "cpu_baseline": None,
    }
    if cpu:
        if name in ("adamw", "adamw_class"):
            rec["cpu_baseline"] = cpu_baseline_adamw(torch)
        elif name in ("quantize", "quantize_transpose") and args.shape == [4096, 4096]:
            rec["cpu_baseline"] = cpu_baseline_quantize(torch, name == "quantize_transpose", nbytes)
        elif name.startswith("gemm"):
            rec["cpu_baseline"] = cpu_baseline_gemm(torch, name.split("_")[1])
        elif name == "silu_mul":
            rec["cpu_baseline"] = cpu_baseline_silu_mul(torch, nbytes)
        elif name == "rmsnorm":
            rec["cpu_baseline"] = cpu_baseline_rmsnorm(torch, nbytes)
        elif name == "attention":
            rec["cpu_baseline"] = cpu_baseline_attention(torch)
    return rec


# the default run: the headline workload (BASELINE configuration 2) plus one record per remaining leg of the metric
EXTRAS = ("quantize", "quantize_transpose", "gemm_fwd", "gemm_dgrad", "gemm_wgrad", "silu_mul", "rmsnorm", "attention", "layer_7b", "layer_13b")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all",
                    choices=["all", "gemm_clock", "adamw", "adamw_class", "adamw_plain", "quantize", "quantize_transpose", "gemm_fwd", "gemm_dgrad",
                             "gemm_wgrad", "linear", "silu_mul", "rmsnorm", "cross_entropy", "layernorm", "division", "division_sr",
                             "division_transpose", "quantize_perblock", "olmo_block", "hbm_copy", "hbm_read", "hbm_fill", "hbm_narrow", "hbm_tile", "layer_7b", "layer_13b", "attention"],
                    help="all (default): the headline AdamW step as `value` plus an `extra` record for every other leg of the metric")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--shape", type=int, nargs=2, default=[4096, 4096], metavar=("M", "N"),
                    help="input shape of the quantize / quantize_transpose workloads (default: the headline [4096, 4096]) and of the division* / hbm_narrow / hbm_tile workloads (default for those: [8192, 4096])")
    ap.add_argument("--cache-weights", action="store_true",
                    help="layer workloads: weight_memory_efficient=False (FP8 weights cached after the first micro-batch)")
    ap.add_argument("--grad-format", default="e5m2", choices=["e5m2", "e4m3"],
                    help="FP8 format of the gradient operand of gemm_dgrad / gemm_wgrad (the reference's default is e5m2)")
    ap.add_argument("--ramp-seconds", type=float, default=1.5,
                    help="untimed continuous run of the step before the W warmup steps: an idle MI355X sits at ~100 MHz and "
                         "takes several hundred ms of load to reach its sustained shader clock, so a few ms of warmup would "
                         "time the kernel on a ramping clock (0 disables)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy a few times (known traffic, to scale rocprofv3 counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus N with N > 1 is not supported "
              "(every kernel on the path is independent per row / per 128-element group)", file=sys.stderr)
        sys.exit(2)

    import torch

    from coat_amd import _hip

    _hip.lib()  # fail loudly if the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.set_num_threads(host_threads())  # the CPU baselines use every core this process may use
    cpu = not args.no_cpu_baseline
    if args.workload == "gemm_clock":
        return gemm_clock(dev, torch)

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    def measure(name):
        fn = measure_layer if name in LAYER_WORKLOADS else measure_stream
        rec = fn(name, args, dev, torch, cpu)
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        return rec

    head = measure("adamw_class" if args.workload == "all" else args.workload)
    out = {"metric": METRIC, "value": head["value"], "unit": head["unit"], "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "ms_per_step": head["ms_per_step"], "higher_is_better": head["higher_is_better"],
           "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"], "data": "synthetic", "config": head["config"]}
    if "layer" in head:
        out["layer"] = head["layer"]
    out["roofline"] = head["roofline"]
    out["cpu_baseline"] = head["cpu_baseline"]
    if args.workload == "all":
        # the other legs of the metric, each timed exactly like a run with --workload <name>
        out["extra"] = {}
        for name in EXTRAS:
            r = measure(name)
            out["extra"][name] = {k: r[k] for k in ("value", "unit", "ms_per_step", "dtype", "roofline", "cpu_baseline") if k in r}
            out["extra"][name]["workload"] = r["config"]["workload"]
            if "layer" in r:
                out["extra"][name]["layer"] = r["layer"]
    print(json.dumps(out))


if __name__ == "__main__":
    main()
