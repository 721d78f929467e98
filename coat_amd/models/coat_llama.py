"""COAT Llama decoder layer: FP8 precision flow through norm / linear / activation, bf16 attention.

Drop-in for the layer-level classes of coat/models/coat_llama.py (reference lines :110-766 the three residual
modules and their autograd Functions, :981-1074 the SDPA attention without projections, :1084-1181 the decoder
layer, :1424-1449 make_state_dict_compatible).  Same class names, constructor arguments, forward signatures,
parameter names (``q_proj`` ... ``down_proj``, ``input_layernorm.weight`` ...) and the same tensors saved for backward.

Every tensor that crosses a module boundary or is saved for backward is FP8:
  (hidden bf16, hidden e4m3 per-group, scales)  --BeforeAttention-->  q, k, v bf16  --attention-->  attn bf16
  --AfterAttention-->  (hidden, e4m3, scales)  --MLPResidual-->  (hidden, e4m3, scales)
and in backward the gradient of the FP8 hidden state travels as a per-tensor e5m2 tensor (viewed as e4m3, because
autograd wants forward value and gradient to share a dtype) together with its per-group scale tensor, whose maximum
is the tensor's scale.

This file does not depend on the ``transformers`` package: the configuration is a plain attribute holder and the
rotary embedding / causal SDPA are written out here.  Whole-model classes (CausalLM, HF registration) are out of scope.
"""
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from ._attention import sdpa
from ..activation.real_quantization import (fp8_add_Ifp_Ifp_Ofp_Og16, fp8_add_Ifp_Ifp_Ofp_Opt, fp8_division,
                                            fp8_division_transpose, fp8_linear_backward, fp8_linear_backward_grouped,
                                            fp8_linear_forward, fp8_linear_forward_add, fp8_linear_forward_grouped,
                                            fp8_quantize_pertensor, fp8_quantize_pertensor_transpose,
                                            fp8_rmsnorm_backward, fp8_rmsnorm_backward_add, fp8_rmsnorm_forward,
                                            fp8_silu_mul_backward,
                                            fp8_silu_mul_forward, fp8_transpose)
from ..activation.real_quantization.common import convert_str_to_fp8, new_max, scale_max, tag_scale_max
from ..utils._fp8_quantization_config import QuantizationConfig
from ..utils._fp8_weightcache import FP8CacheWeightModule
from ..utils._fp8manager import FP8Manager

__all__ = [
    "CoatLlamaConfig",
    "CoatLlamaBeforeAttentionResidual",
    "CoatLlamaAfterAttentionResidual",
    "CoatLlamaMLPResidual",
    "CoatLlamaDecoderLayer",
    "LlamaSdpaAttentionWithoutLinear",
    "make_state_dict_compatible",
]

E4M3, E5M2 = torch.float8_e4m3fn, torch.float8_e5m2


class CoatLlamaConfig:
    """The attributes of LlamaConfig that the decoder layer reads, plus ``coat_fp8_args``
    (reference: CoatLlamaConfig(LlamaConfig), :106-107, with the quantization settings carried as a dict, :1092)."""

    model_type = "fp8_llama"

    def __init__(self, hidden_size=4096, intermediate_size=11008, num_attention_heads=32, num_key_value_heads=None,
                 head_dim=None, rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=4096,
                 attention_bias=False, mlp_bias=False, attention_dropout=0.0, hidden_act="silu",
                 _attn_implementation="sdpa", coat_fp8_args=None, **kwargs):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.num_attention_heads = num_attention_heads
        self.num_key_value_heads = num_attention_heads if num_key_value_heads is None else num_key_value_heads
        self.head_dim = hidden_size // num_attention_heads if head_dim is None else head_dim
        self.rms_norm_eps = rms_norm_eps
        self.rope_theta = rope_theta
        self.max_position_embeddings = max_position_embeddings
        self.attention_bias = attention_bias
        self.mlp_bias = mlp_bias
        self.attention_dropout = attention_dropout
        self.hidden_act = hidden_act
        self._attn_implementation = _attn_implementation
        self.coat_fp8_args = dict(coat_fp8_args or {})
        for k, v in kwargs.items():
            setattr(self, k, v)


def _fwobits(qargs):
    return {k: getattr(qargs, k) for k in ("fabit", "fwbit", "fobit", "babit", "bwbit", "bobit")}


def _as_e4m3_input(t, fwobits):
    if fwobits["fabit"] != "E4M3":
        raise ValueError("fabit should be E4M3")
    return t.view(E4M3)


def _as_e5m2_grad(t, fwobits):
    if fwobits["babit"] != "E5M2":
        raise ValueError("babit should be E5M2")
    return t.view(E5M2)


def _forward_weight(origin, cached, scale, qargs, fwobits):
    """FP8 weight for a forward GEMM: the cached copy, or (memory-efficient mode) re-quantized from the master weight
    with the scale cached on the first micro-batch."""
    if qargs.weight_memory_efficient:
        assert cached is None
        return fp8_division(origin, qargs.group_size, fwobits["fwbit"], scale)[0]
    return cached


def _backward_weight_t(saved, scale, qargs, fwobits):
    """Transposed FP8 weight for the dgrad GEMM (``saved`` is the master weight in memory-efficient mode)."""
    if qargs.weight_memory_efficient:
        return fp8_division_transpose(saved, qargs.group_size, fwobits["fwbit"], scale, only_transposed=True)[0]
    return saved


class _ResidualBase(FP8CacheWeightModule):
    def __init__(self, config, qargs, layer_id):
        super().__init__(config, qargs, layer_id)
        self.fwobits = _fwobits(qargs)

    def _prepared(self, names):
        """For each projection: (master weight, fp8, fp8_t, scale) as the autograd Functions expect them."""
        out = []
        with torch.no_grad():
            for name in names:
                w = getattr(self, name).weight
                r = self.prepare_weight(w, name, FP8Manager.is_first_microbatch)
                out += [w, None, None, r] if self.qargs.weight_memory_efficient else [w, r[0], r[1], r[2]]
        return out


# ------------------------------------------------------------------------------------------------ before attention
class CoatLlamaBeforeAttentionResidual(_ResidualBase):
    """Residual branch point + RMSNorm + Q/K/V projections."""

    def __init__(self, config: CoatLlamaConfig, qargs: QuantizationConfig, layer_idx: Optional[int] = None):
        super().__init__(config, qargs, layer_idx)
        self.layer_idx = layer_idx
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = getattr(config, "head_dim", self.hidden_size // self.num_heads)
        self.num_key_value_heads = config.num_key_value_heads
        self.q_proj = nn.Linear(self.hidden_size, self.num_heads * self.head_dim, bias=config.attention_bias)
        self.k_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=config.attention_bias)
        self.v_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=config.attention_bias)

    def forward(self, re_x, x, s, rmsnorm_weight):
        if self.training:
            return _CoatLlamaBeforeAttentionResidual.apply(
                re_x, x, s, *self._prepared(("q_proj", "k_proj", "v_proj")), rmsnorm_weight, self.qargs.group_size,
                self.fwobits, self.layer_id, self.config, self.qargs)
        x = F.rms_norm(re_x, rmsnorm_weight.shape, rmsnorm_weight)
        return re_x, self.q_proj(x), self.k_proj(x), self.v_proj(x)


class _CoatLlamaBeforeAttentionResidual(torch.autograd.Function):
    @staticmethod
    def forward(ctx, re_x, in_x, in_s, w1_origin, w1, w1_t, w1_s, w2_origin, w2, w2_t, w2_s, w3_origin, w3, w3_t, w3_s,
                rmsnorm_weight, group_size, fwobits, layer_id, config, qargs, eps=1e-5):
        in_x = _as_e4m3_input(in_x, fwobits)
        ln_x, ln_s, ln_x_t, ln_utils = fp8_rmsnorm_forward(in_x, in_s, rmsnorm_weight, group_size, eps,
                                                           transpose_output_2d=True)
        # q / k / v projections in one launch (the reference's three fp8_linear_forward calls, :267-269)
        w8s = [_forward_weight(origin, cached, scale, qargs, fwobits)
               for origin, cached, scale in ((w1_origin, w1, w1_s), (w2_origin, w2, w2_s), (w3_origin, w3, w3_s))]
        outs = fp8_linear_forward_grouped(ln_x, ln_s, w8s, [w1_s, w2_s, w3_s], False, group_size)
        del w8s
        ctx.save_for_backward(in_x, in_s, ln_x_t, ln_s)
        if qargs.weight_memory_efficient:
            ctx.weight = w1_origin, w1_s, w2_origin, w2_s, w3_origin, w3_s
        else:
            ctx.weight = w1_t, w1_s, w2_t, w2_s, w3_t, w3_s
        ctx.group_size = group_size
        ctx.ln_utils = ln_utils
        ctx.utils = fwobits, layer_id, config, qargs
        return re_x, outs[0], outs[1], outs[2]

    @staticmethod
    def backward(ctx, fp_grad, query_g, key_g, value_g):
        in_x, in_s, ln_x_t, ln_s = ctx.saved_tensors
        group_size = ctx.group_size
        rms_weight, rstd, num_warps = ctx.ln_utils
        fwobits, layer_id, config, qargs = ctx.utils
        g8s, gss, g8_ts, w_ts = [], [], [], []
        for g, w_saved, w_s in zip((query_g, key_g, value_g), ctx.weight[0::2], ctx.weight[1::2]):
            # the gradients leaving RoPE / attention are bf16: per-tensor e5m2 in both layouts
            g8, gs, g8_t = fp8_quantize_pertensor_transpose(g, group_size, fwobits["babit"], transpose_output_2d=True,
                                                            stochastic=False)
            g8s.append(g8)
            gss.append(gs)
            g8_ts.append(g8_t)
            w_ts.append(_backward_weight_t(w_saved, w_s, qargs, fwobits))
        # the three fp8_linear_backward calls of the reference (:318-326): dgrads in one launch, wgrads in another
        dgrads, wgrads = fp8_linear_backward_grouped(ln_x_t, ln_s, g8s, gss, g8_ts, w_ts, list(ctx.weight[1::2]), group_size)
        del g8s, g8_ts, w_ts
        # fc1_g = dgrads[0] + dgrads[1] + dgrads[2] (reference :328), summed inside the kernel with the same roundings
        # and fp8_add_Ifp_Ifp_Ofp_Opt(fp_grad, in_g) (:331-339) inside the same kernel
        re_g, (in_g, in_sg, in_sg_g16), rms_weight_grad = fp8_rmsnorm_backward_add(
            in_x, in_s, tuple(dgrads), rms_weight, rstd, group_size, num_warps, fp_grad, fwobits["babit"], stochastic=False)
        # the per-group scale tensor is returned as the "gradient" of the forward scales so that shapes match;
        # the consumer takes its maximum, which is the scale in_g was quantized with
        return (re_g, in_g.view(E4M3), in_sg_g16,
                wgrads[0], None, None, None, wgrads[1], None, None, None, wgrads[2], None, None, None,
                rms_weight_grad, None, None, None, None, None, None)


# ------------------------------------------------------------------------------------------------ after attention
class CoatLlamaAfterAttentionResidual(_ResidualBase):
    """Output projection + residual add."""

    def __init__(self, config: CoatLlamaConfig, qargs: QuantizationConfig, layer_id):
        super().__init__(config, qargs, layer_id)
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = getattr(config, "head_dim", self.hidden_size // self.num_heads)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, self.hidden_size, bias=config.attention_bias)

    def forward(self, re_x, in_x):
        if self.training:
            return _CoatLlamaAfterAttentionResidual.apply(re_x, in_x, *self._prepared(("o_proj",)), self.qargs.group_size,
                                                          self.fwobits, self.layer_id, self.config, self.qargs)
        return re_x + self.o_proj(in_x), None, None


class _CoatLlamaAfterAttentionResidual(torch.autograd.Function):
    @staticmethod
    def forward(ctx, re_x, flash_x, w4_origin, w4, w4_t, w4_s, group_size, fwobits, layer_id, config, qargs):
        flash_qx, flash_s, _ = fp8_quantize_pertensor(flash_x, group_size, fwobits["fabit"], want_pg=False)
        w8 = _forward_weight(w4_origin, w4, w4_s, qargs, fwobits)
        # fp8_linear_forward + fp8_add_Ifp_Ifp_Ofp_Og16 of the reference (:440-441): the addition runs in the GEMM epilogue
        fp_x, (out_x, out_s) = fp8_linear_forward_add(flash_qx, flash_s, w8, w4_s, re_x, flash_qx.dtype, group_size)
        # the bf16 attention output is saved (not its FP8 copy): its transpose is re-quantized in backward
        ctx.save_for_backward(flash_x, flash_s)
        ctx.weight = (w4_origin, w4_s) if qargs.weight_memory_efficient else (w4_t, w4_s)
        ctx.group_size = group_size
        ctx.utils = fwobits, layer_id, config, qargs
        return fp_x, out_x.view(E4M3), out_s

    @staticmethod
    def backward(ctx, fp_grad, out_g, out_gs):
        flash_x, flash_s = ctx.saved_tensors
        w_saved, w4_s = ctx.weight
        group_size = ctx.group_size
        fwobits, layer_id, config, qargs = ctx.utils
        out_g = _as_e5m2_grad(out_g, fwobits)
        out_gs_max = scale_max(out_gs)
        out_g_t = fp8_transpose(out_g, transpose_output_2d=True)
        flash_x_t, flash_s = fp8_division_transpose(flash_x, group_size, fwobits["fabit"], flash_s, stochastic=False,
                                                    only_transposed=True)
        w4_t = _backward_weight_t(w_saved, w4_s, qargs, fwobits)
        fc4_g, attn_out_wg = fp8_linear_backward(flash_x_t, flash_s, out_g, out_gs_max, out_g_t, w4_t, w4_s, group_size)
        return fp_grad, fc4_g, attn_out_wg, None, None, None, None, None, None, None, None


# ------------------------------------------------------------------------------------------------ MLP
class CoatLlamaMLPResidual(_ResidualBase):
    """RMSNorm + gate / up projections + SiLU * up + down projection + residual add."""

    def __init__(self, config: CoatLlamaConfig, qargs: QuantizationConfig, layer_id, hidden_size: int):
        super().__init__(config, qargs, layer_id)
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.intermediate_size
        self.gate_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=config.mlp_bias)
        self.up_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=config.mlp_bias)
        self.down_proj = nn.Linear(self.intermediate_size, self.hidden_size, bias=config.mlp_bias)
        assert config.hidden_act == "silu", "We only support silu activation currently"
        self.act_fn = F.silu

    def forward(self, re_x, x, s, rmsnorm_weight):
        if self.training:
            return _CoatLlamaMLPResidual.apply(
                re_x, x, s, *self._prepared(("gate_proj", "up_proj", "down_proj")), rmsnorm_weight,
                self.qargs.group_size, self.fwobits, self.layer_id, self.config, self.qargs)
        x = F.rms_norm(re_x, rmsnorm_weight.shape, rmsnorm_weight)
        x = self.act_fn(self.gate_proj(x)) * self.up_proj(x)
        return re_x + self.down_proj(x), None, None


class _CoatLlamaMLPResidual(torch.autograd.Function):
    @staticmethod
    def forward(ctx, re_x, in_x, in_s, w1_origin, w1, w1_t, w1_s, w2_origin, w2, w2_t, w2_s, w3_origin, w3, w3_t, w3_s,
                rmsnorm_weight, group_size, fwobits, layer_id, config, qargs, eps=1e-5):
        in_x = _as_e4m3_input(in_x, fwobits)
        ln_x, ln_s, ln_x_t, ln_utils = fp8_rmsnorm_forward(in_x, in_s, rmsnorm_weight, group_size, eps,
                                                           transpose_output_2d=True)
        # gate / up projections write per-group FP8 straight from the GEMM epilogue
        # (the reference's two fp8_linear_forward calls, :647-648, in one launch)
        (gate_x, gate_s), (up_x, up_s) = fp8_linear_forward_grouped(
            ln_x, ln_s, [_forward_weight(w1_origin, w1, w1_s, qargs, fwobits), _forward_weight(w2_origin, w2, w2_s, qargs, fwobits)],
            [w1_s, w2_s], True, group_size)
        # one kernel for fp8_silu_forward + fp8_mul_forward of the reference (:664-668), same tensors
        silu_x, silu_s, mul_x, mul_s, mul_x_t = fp8_silu_mul_forward(gate_x, gate_s, up_x, up_s, group_size,
                                                                      transpose_output_2d=True)
        # fp8_linear_forward + fp8_add_Ifp_Ifp_Ofp_Og16 of the reference (:673-674) in one kernel
        fp_x, (out_x, out_s) = fp8_linear_forward_add(mul_x, mul_s, _forward_weight(w3_origin, w3, w3_s, qargs, fwobits),
                                                      w3_s, re_x, mul_x.dtype, group_size)
        ctx.save_for_backward(in_x, in_s, ln_x_t, ln_s, gate_x, gate_s, up_x, up_s, silu_x, silu_s, mul_x_t, mul_s)
        if qargs.weight_memory_efficient:
            ctx.weight = (w1_origin, w1_s, w2_origin, w2_s, w3_origin, w3_s)
        else:
            ctx.weight = (w1_t, w1_s, w2_t, w2_s, w3_t, w3_s)
        ctx.group_size = group_size
        ctx.ln_utils = ln_utils
        ctx.utils = fwobits, layer_id, config, qargs
        return fp_x, out_x.view(E4M3), out_s

    @staticmethod
    def backward(ctx, fp_grad, out_g, out_gs):
        in_x, in_s, ln_x_t, ln_s, gate_x, gate_s, up_x, up_s, silu_x, silu_s, mul_x_t, mul_s = ctx.saved_tensors
        w1_saved, w1_s, w2_saved, w2_s, w3_saved, w3_s = ctx.weight
        group_size = ctx.group_size
        rms_weight, rstd, num_warps = ctx.ln_utils
        fwobits, layer_id, config, qargs = ctx.utils
        out_g = _as_e5m2_grad(out_g, fwobits)
        out_gs_max = scale_max(out_gs)
        # down projection
        out_g_t = fp8_transpose(out_g, transpose_output_2d=True)
        w3_t = _backward_weight_t(w3_saved, w3_s, qargs, fwobits)
        fc3_g, weight3_grad = fp8_linear_backward(mul_x_t, mul_s, out_g, out_gs_max, out_g_t, w3_t, w3_s, group_size)
        del out_g, out_g_t, w3_t
        # element-wise product (1 = gate branch, 2 = up branch) and SiLU
        # one kernel for fp8_mul_backward + fp8_silu_backward of the reference (:741-748), same tensors
        (silu_g, silu_gs, silu_g_t), (mul_g2, mul_gs2, mul_g2_t) = fp8_silu_mul_backward(
            gate_x, gate_s, up_x, up_s, silu_x, silu_s, fc3_g, group_size, fwobits["babit"])
        # gate / up projections
        w1_t = _backward_weight_t(w1_saved, w1_s, qargs, fwobits)
        w2_t = _backward_weight_t(w2_saved, w2_s, qargs, fwobits)
        # (the reference's two fp8_linear_backward calls, :735-740: dgrads in one launch, wgrads in another)
        (fc1_g, fc2_g), (weight1_grad, weight2_grad) = fp8_linear_backward_grouped(
            ln_x_t, ln_s, [silu_g, mul_g2], [silu_gs, mul_gs2], [silu_g_t, mul_g2_t], [w1_t, w2_t], [w1_s, w2_s], group_size)
        # fc_g = fc1_g + fc2_g (reference :742), summed inside the kernel
        # and fp8_add_Ifp_Ifp_Ofp_Opt(fp_grad, in_g) (:745-754) inside the same kernel
        re_g, (in_g, in_sg, in_sg_g16), rms_weight_grad = fp8_rmsnorm_backward_add(
            in_x, in_s, (fc1_g, fc2_g), rms_weight, rstd, group_size, num_warps, fp_grad, fwobits["babit"], stochastic=False)
        return (re_g, in_g.view(E4M3), in_sg_g16,
                weight1_grad, None, None, None, weight2_grad, None, None, None, weight3_grad, None, None, None,
                rms_weight_grad, None, None, None, None, None, None)


# ------------------------------------------------------------------------------------------------ attention (bf16)
class LlamaRMSNorm(nn.Module):
    """Holder of the RMSNorm weight (the normalisation itself runs inside the residual modules)."""

    def __init__(self, hidden_size, eps=1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def forward(self, hidden_states):
        return F.rms_norm(hidden_states, self.weight.shape, self.weight, self.variance_epsilon)


def rotary_cos_sin(position_ids, head_dim, theta, dtype):
    """cos / sin of shape [B, S, head_dim] for the half-rotation layout Llama uses."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=position_ids.device, dtype=torch.float32) / head_dim))
    freqs = position_ids[:, :, None].float() * inv_freq[None, None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def _rotate_half(x):
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin):
    cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    return (q * cos) + (_rotate_half(q) * sin), (k * cos) + (_rotate_half(k) * sin)


_ROPE_TABLES = {}


def rotary_tables(n_pos, head_dim, theta, device):
    """fp32 cos / sin tables [n_pos, head_dim / 2] for the fused RoPE kernel (cached per device and shape)."""
    key = (str(device), int(n_pos), int(head_dim), float(theta))
    if key not in _ROPE_TABLES:
        inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim))
        ang = torch.arange(n_pos, device=device, dtype=torch.float32)[:, None] * inv_freq[None, :]
        _ROPE_TABLES[key] = (ang.cos().contiguous(), ang.sin().contiguous())
    return _ROPE_TABLES[key]


class _FusedRoPE(torch.autograd.Function):
    """x bf16 [B, S, heads * head_dim] -> rotated tensor viewed as [B, heads, S, head_dim]; one HIP kernel per direction
    (``coat_rope_bf16``; the backward pass is the rotation by the negated angle)."""

    @staticmethod
    def forward(ctx, x, cos_tab, sin_tab, pos, heads, head_dim, theta, grad_fp8=None):
        from .. import _hip
        B, S, _ = x.shape
        x = _hip.dense(x)
        y = torch.empty_like(x)
        _hip.check(_hip.lib().coat_rope_bf16(_hip.ptr(x), _hip.ptr(y), _hip.ptr(cos_tab), _hip.ptr(sin_tab), cos_tab.shape[0],
                                             theta, _hip.ptr(pos), B * S, S, heads, head_dim, 0, 0, 0, None, 0,
                                             _hip.stream(x.device)), "rope forward")
        ctx.save_for_backward(cos_tab, sin_tab, pos)
        ctx.dims = (B, S, heads, head_dim, theta)
        ctx.grad_fp8 = grad_fp8
        return y.view(B, S, heads, head_dim).transpose(1, 2)

    @staticmethod
    def backward(ctx, g):
        from .. import _hip
        cos_tab, sin_tab, pos = ctx.saved_tensors
        B, S, heads, head_dim, theta = ctx.dims
        g = _hip.dense(g.transpose(1, 2).to(torch.bfloat16))  # physically [B, S, heads, head_dim]
        dx = torch.empty_like(g)
        # the consumer quantizes this gradient per tensor (reference :318-326): the kernel hands it the scale maximum
        s_max = new_max(g.device) if ctx.grad_fp8 is not None else None
        _hip.check(_hip.lib().coat_rope_bf16(_hip.ptr(g), _hip.ptr(dx), _hip.ptr(cos_tab), _hip.ptr(sin_tab), cos_tab.shape[0],
                                             theta, _hip.ptr(pos), B * S, S, heads, head_dim, 1, 0, 0, _hip.ptr(s_max),
                                             _hip.fp8(ctx.grad_fp8) if s_max is not None else 0,
                                             _hip.stream(g.device)), "rope backward")
        dx = dx.view(B, S, heads * head_dim)
        if s_max is not None:
            tag_scale_max(dx, s_max, ctx.grad_fp8)
        return dx, None, None, None, None, None, None, None


class _FusedQKVRoPE(torch.autograd.Function):
    """qkv bf16 [B, S, Dq + 2 Dkv] (a fused projection's output) -> rotated q [B, heads, S, hd], rotated k
    [B, kv_heads, S, hd] and v [B, kv_heads, S, hd] (a view of qkv).  The kernels read the q / k column slices where
    they lie; the backward writes the two inverse rotations and dv straight into one [B, S, Dq + 2 Dkv] gradient, so
    neither the ``.contiguous()`` copies of the slices nor the concatenation of the three gradients are needed."""

    @staticmethod
    def forward(ctx, qkv, cos_tab, sin_tab, heads, kv_heads, head_dim, theta, grad_fp8=None):
        from .. import _hip
        B, S, W = qkv.shape
        Dq, Dkv = heads * head_dim, kv_heads * head_dim
        assert W == Dq + 2 * Dkv and Dq % 8 == 0 and Dkv % 8 == 0
        qkv = _hip.dense(qkv)
        flat = qkv.view(B * S, W)
        q = torch.empty((B, S, Dq), dtype=qkv.dtype, device=qkv.device)
        k = torch.empty((B, S, Dkv), dtype=qkv.dtype, device=qkv.device)
        lib, st = _hip.lib(), _hip.stream(qkv.device)
        tabs = (_hip.ptr(cos_tab), _hip.ptr(sin_tab), cos_tab.shape[0], theta, None)
        _hip.check(lib.coat_rope_bf16(_hip.ptr(flat[:, :Dq]), _hip.ptr(q), *tabs, B * S, S, heads, head_dim, 0, W, 0, None, 0, st),
                   "rope forward (q of qkv)")
        _hip.check(lib.coat_rope_bf16(_hip.ptr(flat[:, Dq:Dq + Dkv]), _hip.ptr(k), *tabs, B * S, S, kv_heads, head_dim, 0, W,
                                      0, None, 0, st), "rope forward (k of qkv)")
        ctx.save_for_backward(cos_tab, sin_tab)
        ctx.dims = (B, S, heads, kv_heads, head_dim, theta)
        ctx.grad_fp8 = grad_fp8
        v = qkv[..., Dq + Dkv:].view(B, S, kv_heads, head_dim).transpose(1, 2)
        return (q.view(B, S, heads, head_dim).transpose(1, 2), k.view(B, S, kv_heads, head_dim).transpose(1, 2), v)

    @staticmethod
    def backward(ctx, gq, gk, gv):
        from .. import _hip
        cos_tab, sin_tab = ctx.saved_tensors
        B, S, heads, kv_heads, head_dim, theta = ctx.dims
        Dq, Dkv = heads * head_dim, kv_heads * head_dim
        W = Dq + 2 * Dkv
        gq = _hip.dense(gq.transpose(1, 2).to(torch.bfloat16))  # physically [B, S, heads, head_dim]
        gk = _hip.dense(gk.transpose(1, 2).to(torch.bfloat16))
        dqkv = torch.empty((B, S, W), dtype=torch.bfloat16, device=gq.device)
        flat = dqkv.view(B * S, W)
        lib, st = _hip.lib(), _hip.stream(gq.device)
        tabs = (_hip.ptr(cos_tab), _hip.ptr(sin_tab), cos_tab.shape[0], theta, None)
        # the consumer quantizes the fused gradient per tensor (reference coat_olmo.py:318-326 on the fused projection): the
        # three kernels that write its parts merge the maximum of its group scales into one buffer
        s_max = new_max(gq.device) if ctx.grad_fp8 is not None else None
        mx = (_hip.ptr(s_max), _hip.fp8(ctx.grad_fp8) if s_max is not None else 0)
        _hip.check(lib.coat_rope_bf16(_hip.ptr(gq), _hip.ptr(flat[:, :Dq]), *tabs, B * S, S, heads, head_dim, 1, 0, W, *mx, st),
                   "rope backward (q of qkv)")
        _hip.check(lib.coat_rope_bf16(_hip.ptr(gk), _hip.ptr(flat[:, Dq:Dq + Dkv]), *tabs, B * S, S, kv_heads, head_dim, 1, 0,
                                      W, *mx, st), "rope backward (k of qkv)")
        if s_max is not None:
            gv = _hip.dense(gv.transpose(1, 2).to(torch.bfloat16))  # physically [B, S, kv_heads, head_dim]
            _hip.check(lib.coat_rope_bf16(_hip.ptr(gv), _hip.ptr(flat[:, Dq + Dkv:]), *tabs, B * S, S, kv_heads, head_dim, 2, 0,
                                          W, *mx, st), "copy with maximum (v of qkv)")
            tag_scale_max(dqkv, s_max, ctx.grad_fp8)
        else:
            dqkv[..., Dq + Dkv:].copy_(gv.transpose(1, 2).reshape(B, S, Dkv))
        return dqkv, None, None, None, None, None, None, None


def fused_qkv_rotary(qkv, heads, kv_heads, head_dim, theta, grad_fp8=None):
    """RoPE on the q and k parts of a fused projection output qkv [B, S, (heads + 2 kv_heads) * head_dim] (bf16, GPU);
    returns (q [B, heads, S, hd], k [B, kv_heads, S, hd], v [B, kv_heads, S, hd]).  ``grad_fp8`` as in ``fused_rotary``."""
    cos_tab, sin_tab = rotary_tables(qkv.shape[1], head_dim, theta, qkv.device)
    return _FusedQKVRoPE.apply(qkv, cos_tab, sin_tab, heads, kv_heads, head_dim, float(theta), grad_fp8)


def fused_rotary(x, heads, head_dim, theta, position_ids=None, max_positions=None, grad_fp8=None):
    """RoPE on a projection output x [B, S, heads * head_dim] (bf16, on the GPU); returns [B, heads, S, head_dim].
    ``grad_fp8`` (an FP8 dtype): the backward also hands the consumer of x's gradient the maximum of its group scales for
    that format (``common.tag_scale_max``)."""
    B, S, _ = x.shape
    if position_ids is None:
        cos_tab, sin_tab = rotary_tables(S, head_dim, theta, x.device)
        pos = None
    else:
        n_pos = max(int(max_positions or 0), S)
        cos_tab, sin_tab = rotary_tables(n_pos, head_dim, theta, x.device)
        # positions beyond the table are not clamped: the kernel computes their angles itself (no read outside the table)
        pos = position_ids.expand(B, S).reshape(-1).to(torch.int64).contiguous()
    return _FusedRoPE.apply(x, cos_tab, sin_tab, pos, heads, head_dim, float(theta), grad_fp8)


class LlamaSdpaAttentionWithoutLinear(nn.Module):
    """RoPE + causal scaled-dot-product attention on already projected q / k / v (the projections live in the
    Before / AfterAttention modules).  bf16, not part of the FP8 flow."""

    def __init__(self, config: CoatLlamaConfig, layer_idx: Optional[int] = None):
        super().__init__()
        self.config = config
        self.layer_idx = layer_idx
        self.attention_dropout = config.attention_dropout
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = getattr(config, "head_dim", self.hidden_size // self.num_heads)
        self.num_key_value_heads = config.num_key_value_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.rope_theta = config.rope_theta
        # formats in which the neighbouring FP8 modules quantize this module's output (forward) and the gradients of its
        # inputs (backward) per tensor: the kernels here hand them the scale maximum
        qargs = QuantizationConfig(**getattr(config, "coat_fp8_args", {}))
        self._out_fp8 = convert_str_to_fp8[qargs.fabit]
        self._grad_fp8 = convert_str_to_fp8[qargs.babit]

    def forward(self, query_states, key_states, value_states, attention_mask=None, position_ids=None,
                past_key_value=None, output_attentions=False, use_cache=False, cache_position=None,
                position_embeddings=None, **kwargs):
        if past_key_value is not None or use_cache:
            raise NotImplementedError("KV caching is not part of the training path built here")
        bsz, q_len, _ = query_states.size()
        v = value_states.view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        if position_embeddings is None and query_states.is_cuda and query_states.dtype == torch.bfloat16:
            # one fused kernel per tensor and direction instead of mul / neg / cat / add passes
            max_pos = getattr(self.config, "max_position_embeddings", None)
            grad_fp8 = self._grad_fp8 if self.training else None
            q = fused_rotary(query_states, self.num_heads, self.head_dim, self.rope_theta, position_ids, max_pos, grad_fp8)
            k = fused_rotary(key_states, self.num_key_value_heads, self.head_dim, self.rope_theta, position_ids, max_pos,
                             grad_fp8)
        else:
            q = query_states.view(bsz, q_len, self.num_heads, self.head_dim).transpose(1, 2)
            k = key_states.view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
            if position_embeddings is None:
                if position_ids is None:
                    position_ids = torch.arange(q_len, device=q.device).unsqueeze(0).expand(bsz, -1)
                cos, sin = rotary_cos_sin(position_ids, self.head_dim, self.rope_theta, q.dtype)
            else:
                cos, sin = position_embeddings
            q, k = apply_rotary_pos_emb(q, k, cos, sin)
        if self.num_key_value_groups > 1:
            k = k.repeat_interleave(self.num_key_value_groups, dim=1)
            v = v.repeat_interleave(self.num_key_value_groups, dim=1)
        mask = attention_mask
        if mask is not None:
            mask = mask[:, :, :, : k.shape[-2]]
        # in training the next module quantizes this output per tensor (reference :434): the kernel hands it the scale maximum
        out_max = new_max(q.device) if self.training and q.is_cuda else None
        out = sdpa(q, k, v, attn_mask=mask, dropout_p=self.attention_dropout if self.training else 0.0,
                   is_causal=mask is None and q_len > 1, out_scale_max=out_max, out_fp8=self._out_fp8)
        out, used_max = out if out_max is not None else (out, False)
        out = out.transpose(1, 2).contiguous().view(bsz, q_len, -1)
        if used_max:
            tag_scale_max(out, out_max, self._out_fp8)
        return out, None, past_key_value


COAT_LLAMA_ATTENTION_CLASSES = {
    "eager": LlamaSdpaAttentionWithoutLinear,
    "sdpa": LlamaSdpaAttentionWithoutLinear,
    "flash_attention_2": LlamaSdpaAttentionWithoutLinear,  # torch SDPA picks the flash kernel where it can
}


# ------------------------------------------------------------------------------------------------ decoder layer
class CoatLlamaDecoderLayer(nn.Module):
    def __init__(self, config: CoatLlamaConfig, layer_idx: int):
        super().__init__()
        self.layer_idx = layer_idx
        self.hidden_size = config.hidden_size
        self.self_attn = COAT_LLAMA_ATTENTION_CLASSES[config._attn_implementation](config=config, layer_idx=layer_idx)
        self.qargs = QuantizationConfig(**config.coat_fp8_args)
        self.BeforeAttention = CoatLlamaBeforeAttentionResidual(config, self.qargs, layer_idx)
        self.AfterAttention = CoatLlamaAfterAttentionResidual(config, self.qargs, layer_idx)
        self.MLPResidual = CoatLlamaMLPResidual(config, self.qargs, layer_idx, self.hidden_size)
        self.input_layernorm = LlamaRMSNorm(config.hidden_size, eps=config.rms_norm_eps)
        self.post_attention_layernorm = LlamaRMSNorm(config.hidden_size, eps=config.rms_norm_eps)

    def forward(self, hidden_states: torch.Tensor, quant_hidden_states: torch.Tensor, scale_hidden_states: torch.Tensor,
                attention_mask: Optional[torch.Tensor] = None, position_ids: Optional[torch.LongTensor] = None,
                past_key_value=None, output_attentions: Optional[bool] = False, use_cache: Optional[bool] = False,
                cache_position: Optional[torch.LongTensor] = None,
                position_embeddings: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, **kwargs):
        """(hidden bf16 [B,S,H], hidden e4m3 [B,S,H], scales [B,S,H/16]) -> ((hidden, e4m3, scales), [attn], [kv])."""
        residual, query_states, key_states, value_states = self.BeforeAttention(
            hidden_states, quant_hidden_states, scale_hidden_states, self.input_layernorm.weight)
        hidden_states, self_attn_weights, present_key_value = self.self_attn(
            query_states=query_states, key_states=key_states, value_states=value_states, attention_mask=attention_mask,
            position_ids=position_ids, past_key_value=past_key_value, output_attentions=output_attentions,
            use_cache=use_cache, cache_position=cache_position, position_embeddings=position_embeddings, **kwargs)
        hidden_states, quant_hidden_states, scale_hidden_states = self.AfterAttention(residual, hidden_states)
        hidden_states, quant_hidden_states, scale_hidden_states = self.MLPResidual(
            hidden_states, quant_hidden_states, scale_hidden_states, self.post_attention_layernorm.weight)
        outputs = ((hidden_states, quant_hidden_states, scale_hidden_states),)
        if output_attentions:
            outputs += (self_attn_weights,)
        if use_cache:
            outputs += (present_key_value,)
        return outputs


def make_state_dict_compatible(state_dict):
    """Rename the keys of a Hugging Face Llama checkpoint to this layer layout (reference :1424-1449):
    the projections move from ``self_attn`` / ``mlp`` into the three residual modules."""
    moves = {
        "self_attn.q_proj": "BeforeAttention.q_proj",
        "self_attn.k_proj": "BeforeAttention.k_proj",
        "self_attn.v_proj": "BeforeAttention.v_proj",
        "self_attn.o_proj": "AfterAttention.o_proj",
        "mlp.gate_proj": "MLPResidual.gate_proj",
        "mlp.up_proj": "MLPResidual.up_proj",
        "mlp.down_proj": "MLPResidual.down_proj",
    }
    out = {}
    for key, value in state_dict.items():
        for old, new in moves.items():
            if old in key:
                key = key.replace(old, new)
                break
        out[key] = value
    return out
