"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares; host-side mirrors of
the reference interface validate their arguments the way the reference does.  No compute calls (no GPU here)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from coat_amd import _hip

    header = open(os.path.join(ROOT, "include", "coat_hip.h")).read()
    declared = set(re.findall(r"\b(coat_[a-z0-9_]+)\s*\(", header))
    declared -= {"coat_status", "coat_dtype", "coat_fp8"}
    declared -= set(re.findall(r"static inline \w+ (coat_[a-z0-9_]+)\s*\(", header))  # header-only helpers
    assert len(declared) >= 11
    L = _hip.lib()
    for name in sorted(declared):
        assert hasattr(L, name), f"{name} declared in include/coat_hip.h but not exported"
    assert set(_hip.SIGNATURES) <= declared
    assert b"gfx950" in L.coat_version()
    abi = int(re.search(r"#define\s+COAT_ABI_VERSION\s+(\d+)", open(os.path.join(ROOT, "include", "coat_hip.h")).read()).group(1))
    assert L.coat_abi_version() == abi == _hip.ABI_VERSION and str(abi).encode() in L.coat_version()
    assert b"128 per-group" in L.coat_status_string(-4)


def test_python_signatures_match_the_header():
    """Every ctypes signature has as many arguments as the header's declaration, with pointers, 64-bit integers, ints
    and floats in the same places (a mismatch would shift every later argument of a call)."""
    from coat_amd import _hip

    header = open(os.path.join(ROOT, "include", "coat_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", " ", header, flags=re.S)
    kinds = {ctypes.c_void_p: "p", ctypes.c_int: "i", ctypes.c_int64: "l", ctypes.c_float: "f", ctypes.c_uint64: "l"}
    for name, argtypes in _hip.SIGNATURES.items():
        m = re.search(r"\bint\s+" + name + r"\s*\(([^)]*)\)\s*;", header)
        assert m, f"{name} not declared as an int function"
        want = ""
        for par in m.group(1).split(","):
            par = " ".join(par.split())
            if "*" in par:
                want += "p"
            elif par.startswith(("int64_t", "uint64_t")):
                want += "l"
            elif par.startswith("float"):
                want += "f"
            else:
                assert par.startswith("int "), (name, par)
                want += "i"
        have = "".join(kinds[t] for t in argtypes)
        assert have == want, f"{name}: ctypes {have} vs header {want}"


def test_argument_validation_without_gpu():
    """Rejected arguments return before any launch, so these run without a GPU."""
    from coat_amd import _hip

    L = _hip.lib()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.c_void_p(ctypes.addressof(buf) & ~15)
    assert L.coat_fp8_quantize(p, 1, p, p, 1, 4, 40, 16, 0, None) == -2  # N % QB
    assert L.coat_fp8_quantize(p, 7, p, p, 1, 4, 64, 16, 0, None) == -3  # dtype
    assert L.coat_fp8_quantize(None, 1, p, p, 1, 4, 64, 16, 0, None) == -1
    assert L.coat_fp8_quantize(p, 1, p, p, 1, 0, 64, 16, 0, None) == 0  # empty
    assert L.coat_fp8_quantize(ctypes.c_void_p(p.value + 2), 1, p, p, 1, 4, 64, 16, 0, None) == -5
    assert L.coat_fp8_quantize_transpose(p, 1, p, p, p, p, 1, 24, 64, 16, 0, None) == -2  # M % QB
    assert L.coat_fp8_transpose(p, p, 8, 64, None) == -2
    assert L.coat_fp8_adamw_step(p, p, 0, p, p, p, p, 0.9, 0.95, 1e-3, 0.1, 1e-8, 1, 64, 256, 2, None) == -4
    assert L.coat_fp8_adamw_step(p, p, 0, p, p, p, p, 0.9, 0.95, 1e-3, 0.1, 1e-8, 1, 128, 256, 3, None) == -2
    with pytest.raises(RuntimeError, match="128 per-group"):
        _hip.check(-4, "x")
    with pytest.raises(ValueError):
        _hip.check(-2, "x")


def test_argument_validation_of_the_remaining_entry_points_without_gpu():
    """Every entry point checks shapes, pointers, alignment and enums before it launches anything."""
    from coat_amd import _hip

    L = _hip.lib()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 15) & ~15)
    odd = ctypes.c_void_p(p.value + 4)
    EINVAL, ESHAPE, EDTYPE, EALIGN = -1, -2, -3, -5
    # per-tensor division family
    assert L.coat_fp8_division(p, 1, p, 1, p, p, 24, 64, 0, None) == ESHAPE            # transpose needs M % 16 == 0
    assert L.coat_fp8_division(p, 1, p, 1, None, None, 16, 64, 0, None) == EINVAL      # no output at all
    assert L.coat_fp8_division(p, 1, p, 1, odd, None, 16, 64, 0, None) == EALIGN
    assert L.coat_fp8_division(p, 1, p, 9, p, None, 16, 64, 0, None) == EDTYPE         # unknown scale dtype
    assert L.coat_fp8_division(p, 1, p, 1, p, None, 16, 64, 5, None) == EINVAL         # unknown fp8 kind
    assert L.coat_fp8_division_from_max(p, 1, p, None, 1, p, None, 16, 64, 0, None) == EINVAL  # nowhere to put the scale
    assert L.coat_fp8_division_stochastic(p, 1, p, 1, p, None, 1 << 17, 1 << 16, 0, 0, None) == ESHAPE  # > 2^32 noise indices
    assert L.coat_fp8_dequantize(p, 0, p, 1, p, 4, 64, 24, None) == ESHAPE
    # per-block quantizers: x, dt, q, s, qt, st, qpg, spg, s_dt, M, N, QB, fp8
    assert L.coat_fp8_quantize_perblock(p, 1, p, p, None, None, None, None, 0, 96, 96, 48, 0, None) == ESHAPE     # QB
    assert L.coat_fp8_quantize_perblock(p, 1, p, p, None, None, None, None, 0, 100, 128, 128, 0, None) == ESHAPE  # M % QB
    assert L.coat_fp8_quantize_perblock(p, 1, p, None, None, None, None, None, 0, 128, 128, 128, 0, None) == EINVAL  # half a pair
    assert L.coat_fp8_quantize_perblock(p, 1, None, None, None, None, None, None, 0, 128, 128, 128, 0, None) == EINVAL  # no output
    assert L.coat_fp8_quantize_perblock(p, 1, p, p, odd, p, None, None, 0, 128, 128, 128, 0, None) == EALIGN
    assert L.coat_fp8_quantize_perblock(p, 1, p, p, None, None, None, None, 9, 128, 128, 128, 0, None) == EDTYPE
    assert L.coat_fp8_quantize_perblock(p, 1, p, p, None, None, None, None, 0, 0, 128, 128, 0, None) == 0         # empty
    # the divisions that recompute their input
    assert L.coat_fp8_rmsnorm_division(p, 0, p, 1, p, 1, p, p, p, p, p, 24, 64, 16, None) == ESHAPE
    assert L.coat_fp8_rmsnorm_division(p, 0, p, 1, p, 1, None, p, p, p, p, 16, 64, 16, None) == EINVAL
    assert L.coat_fp8_rmsnorm_division(p, 0, p, 1, p, 7, p, p, p, p, p, 16, 64, 16, None) == EDTYPE
    assert L.coat_fp8_layernorm_division(p, 0, p, 1, None, None, 1, p, p, p, p, p, p, 16, 64, 16, None) == EINVAL  # w, b missing
    assert L.coat_fp8_layernorm_division(p, 0, p, 1, None, None, -1, p, p, p, p, p, odd, 16, 64, 16, None) == EALIGN
    assert L.coat_fp8_product_division(p, p, 1, p, p, 1, 0, p, p, p, p, 16, 64, 16, 48, 0, None) == ESHAPE  # pitch < N
    assert L.coat_fp8_product_division(p, p, 1, p, p, 4, 0, p, p, p, p, 16, 64, 16, 0, 0, None) == EDTYPE
    # fused activations / norms
    assert L.coat_fp8_silu_forward(p, 0, p, 1, p, p, 4, 40, 16, None) == ESHAPE
    assert L.coat_fp8_silu_mul_forward(p, p, p, p, 0, 1, p, p, None, None, 4, 64, 16, 0, 0, None) == EINVAL  # no maximum word
    assert L.coat_fp8_rmsnorm_forward(p, 0, p, 1, p, 1, None, p, p, p, 4, 32768, 16, 1e-5, None) == ESHAPE   # row too long
    assert L.coat_fp8_rmsnorm_forward(p, 0, p, 1, p, 1, None, None, p, p, 4, 64, 16, 1e-5, None) == EINVAL
    # GEMM
    assert L.coat_fp8_gemm(p, 0, p, 0, p, None, 0, p, 1, p, 1, None, 0, 64, 64, 24, 16, None) == ESHAPE    # K % 16
    assert L.coat_fp8_gemm(p, 0, p, 0, p, None, 1, p, 1, p, 1, None, 0, 64, 64, 64, 16, None) == ESHAPE    # quantized output without scales
    assert L.coat_fp8_gemm(p, 3, p, 0, p, None, 0, p, 1, p, 1, None, 0, 64, 64, 64, 16, None) == EINVAL    # unknown operand format
    assert L.coat_fp8_gemm(p, 0, p, 0, p, None, 0, p, 1, p, 1, None, 0, 0, 64, 64, 16, None) == 0          # empty
    pa = (ctypes.c_void_p * 5)(*[p.value] * 5)      # host arrays of pointers for the grouped GEMM
    pn = (ctypes.c_void_p * 2)(p.value, None)
    po = (ctypes.c_void_p * 2)(p.value, odd.value)
    assert L.coat_fp8_gemm_grouped(0, pa, 0, pa, 0, pa, None, 0, pa, 1, pa, 1, None, 0, 64, 64, 64, 16, None) == EINVAL   # no problem
    assert L.coat_fp8_gemm_grouped(5, pa, 0, pa, 0, pa, None, 0, pa, 1, pa, 1, None, 0, 64, 64, 64, 16, None) == EINVAL   # more than four
    assert L.coat_fp8_gemm_grouped(2, pa, 0, pn, 0, pa, None, 0, pa, 1, pa, 1, None, 0, 64, 64, 64, 16, None) == EINVAL   # second B missing
    assert L.coat_fp8_gemm_grouped(2, pa, 0, pa, 0, po, None, 0, pa, 1, pa, 1, None, 0, 64, 64, 64, 16, None) == EALIGN   # second C misaligned
    assert L.coat_fp8_gemm_grouped(2, pa, 0, pa, 0, pa, pn, 1, pa, 1, pa, 1, None, 0, 64, 64, 64, 16, None) == ESHAPE     # second scale output missing
    assert L.coat_fp8_gemm_grouped(2, pa, 0, pa, 0, pa, None, 0, pa, 1, pa, 1, None, 0, 64, 64, 24, 16, None) == ESHAPE   # K % 16
    assert L.coat_fp8_gemm_grouped(3, pa, 0, pa, 0, pa, None, 0, pa, 1, pa, 1, None, 0, 64, 0, 64, 16, None) == 0         # empty
    # multi-tensor optimizer steps: host arrays of pointers and sizes
    i64 = ctypes.c_int64
    n1, g1, g0 = (i64 * 2)(128, 256), (i64 * 2)(1, 2), (i64 * 2)(1, 3)
    hp = (0.9, 0.95, 1e-3, 0.1, 1e-8, 1)
    assert L.coat_fp8_adamw_expand_step_multi(2, pa, pa, 0, pa, pa, pa, pa, pa, pa, pa, pa, n1, g1, *hp, 64, 16, None) == -4   # group size
    assert L.coat_fp8_adamw_expand_step_multi(2, pa, pa, 0, pa, pa, pa, pa, pa, pa, pa, pa, n1, g0, *hp, 128, 16, None) == ESHAPE  # second scale count
    assert L.coat_fp8_adamw_expand_step_multi(2, pa, pn, 0, pa, pa, pa, pa, pa, pa, pa, pa, n1, g1, *hp, 128, 16, None) == EINVAL  # second gradient missing
    assert L.coat_fp8_adamw_expand_step_multi(2, pa, pa, 0, pa, pa, pa, None, pa, pa, pa, pa, n1, g1, *hp, 128, 16, None) == EINVAL  # no centre array
    assert L.coat_fp8_adamw_expand_step_multi(2, po, pa, 0, pa, pa, pa, pa, pa, pa, pa, pa, n1, g1, *hp, 128, 16, None) == EALIGN  # second parameter misaligned
    assert L.coat_fp8_adamw_expand_step_multi(2, pa, pa, 7, pa, pa, pa, pa, pa, pa, pa, pa, n1, g1, *hp, 128, 16, None) == -3   # dtype
    assert L.coat_fp8_adamw_step_multi(-1, pa, pa, 0, pa, pa, pa, pa, n1, g1, *hp, 128, None) == EINVAL
    assert L.coat_fp8_adamw_step_multi(0, None, None, 0, None, None, None, None, None, None, *hp, 128, None) == 0            # nothing to do
    assert L.coat_fp8_adamw_step_multi(2, pn, pn, 0, pn, pn, pn, pn, (i64 * 2)(0, 0), (i64 * 2)(0, 0), *hp, 128, None) == 0   # only empty tensors
    # fused norm backward + residual addition, attention forward
    assert L.coat_fp8_layernorm_backward_add(p, 0, p, 1, p, None, -1, p, p, None, p, p, p, 1, None, None, None, None, 0, 16, 64, 16, None) == EINVAL  # no residual gradient
    assert L.coat_fp8_layernorm_backward_add(p, 0, p, 1, p, None, -1, p, p, p, p, p, p, 5, None, None, None, None, 0, 16, 64, 16, None) == EINVAL     # unknown output format
    assert L.coat_fp8_layernorm_backward_add(p, 0, p, 1, p, None, -1, p, p, odd, p, p, p, 1, None, None, None, None, 0, 16, 64, 16, None) == EALIGN
    st = [64] * 12
    assert L.coat_attention_forward_bf16(p, p, p, p, None, 1, 4, 4, 64, 64, *st, 0.1, 1, None, 0, None) == ESHAPE   # head dimension
    assert L.coat_attention_forward_bf16(p, p, p, p, None, 1, 4, 3, 64, 128, *st, 0.1, 1, None, 0, None) == EINVAL  # heads % kv_heads
    assert L.coat_attention_forward_bf16(p, p, p, p, None, 1, 4, 4, 64, 128, *st, 0.1, 1, p, 9, None) == EINVAL     # unknown format for the maximum
    assert L.coat_attention_forward_bf16(p, p, p, p, None, 0, 4, 4, 64, 128, *st, 0.1, 1, None, 0, None) == 0       # empty batch
    # RoPE, cross-entropy
    assert L.coat_rope_bf16(p, p, p, p, 8, 1e4, None, 8, 8, 2, 24, 0, 0, 0, None, 0, None) == ESHAPE             # head_dim % 16
    assert L.coat_rope_bf16(p, p, p, p, 8, 1e4, None, 8, 8, 2, 32, 0, 48, 0, None, 0, None) == ESHAPE            # pitch < heads * head_dim
    assert L.coat_rope_bf16(p, p, p, p, 8, 1e4, None, 8, 8, 2, 32, 0, 0, 0, p, 7, None) == EINVAL                # unknown format for the maximum
    assert L.coat_cross_entropy_forward(p, 0, 8, p, p, None, None, 4, 16, -100, 0.0, 0.0, 1, 0.0, 0, None) == EINVAL  # stride < columns
    assert L.coat_cross_entropy_forward(p, 0, 16, p, p, None, None, 4, 16, -100, 0.0, 0.0, 1, 0.0, 0, None) == EINVAL  # mean without a count
    assert L.coat_cross_entropy_forward(p, 0, 16, p, p, None, p, 4, 16, -100, 0.0, 0.0, 7, 0.0, 0, None) == EINVAL


def test_quantization_config_defaults():
    from coat_amd.utils._fp8_quantization_config import QuantizationConfig

    q = QuantizationConfig()
    assert (q.fabit, q.fwbit, q.fobit, q.babit, q.bwbit, q.bobit) == ("E4M3",) * 3 + ("E5M2",) * 3
    assert q.group_size == 16 and q.qgroup_size == 128 and q.expand_min == 16 and q.weight_memory_efficient is True
    assert q.first_order_expansion == "true" and q.epsilon == 1e-10
    q2 = QuantizationConfig(group_size=32, unknown_flag=1)  # unknown keywords are swallowed, as in the reference
    assert q2.group_size == 32 and not hasattr(q2, "unknown_flag")


def test_coatadamw_constructor_and_expansion_switch():
    from coat_amd.optimizer.fp8_adamw import CoatAdamW
    from coat_amd.utils._fp8_quantization_config import QuantizationConfig

    w = torch.nn.Parameter(torch.zeros(4, 4))
    for bad in (dict(lr=-1.0), dict(eps=-1.0), dict(betas=(1.0, 0.9)), dict(betas=(0.9, 1.0)), dict(weight_decay=-0.1)):
        with pytest.raises(ValueError):
            CoatAdamW([w], **bad)
    with pytest.raises(AssertionError):
        CoatAdamW([w], qargs=QuantizationConfig(first_order_expansion="true", second_order_expansion="false"))
    assert CoatAdamW([w]).use_expansion
    assert CoatAdamW([w], qargs=QuantizationConfig(first_order_expansion="expansion", second_order_expansion="expansion")).use_expansion
    # the OLMo YAMLs' spelling "expand" silently selects the plain kernel in the reference too (fp8_adamw.py:293)
    assert not CoatAdamW([w], qargs=QuantizationConfig(first_order_expansion="expand", second_order_expansion="expand")).use_expansion
    opt = CoatAdamW([w])
    w.grad = torch.zeros(4, 4)
    with pytest.raises(RuntimeError):  # CPU tensors are refused loudly, there is no fallback
        opt.step()


def test_dropin_aliases():
    import coat_amd.dropin  # noqa: F401
    import qoptim_cuda
    from coat.activation.real_quantization import fp8_quantize
    from coat.optimizer.fp8_adamw import CoatAdamW

    assert hasattr(qoptim_cuda, "fp8_adamw_expand_step") and callable(fp8_quantize) and CoatAdamW.__name__ == "CoatAdamW"


def test_entry_points_refuse_cpu_tensors():
    from coat_amd.activation.real_quantization import fp8_quantize

    with pytest.raises(RuntimeError, match="GPU"):
        fp8_quantize(torch.zeros(4, 64, dtype=torch.bfloat16), 16, "E4M3")
