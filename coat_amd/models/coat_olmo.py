"""COAT OLMo transformer block: the second model family of the reference, same FP8 precision flow as the Llama layer
with a non-parametric LayerNorm, one fused q/k/v projection and one fused up/gate projection whose per-group FP8
output comes straight from the GEMM epilogue.

Drop-in for the block-level classes of coat/models/coat_olmo.py (reference lines :94-245 BeforeAttention, :247-380
AfterAttention, :383-645 MLPResidual, :648-1076 the block).  Same class names, parameter names (``att_proj``,
``attn_out``, ``ff_proj``, ``ff_out``), forward signatures and tensors saved for backward.  The configuration is a plain
attribute holder with OLMo's field names (the reference takes olmo.config.ModelConfig); whole-model classes, FSDP wrap
policies and checkpoint conversion are out of scope.
"""
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from ._attention import sdpa
from ..activation.real_quantization import (fp8_add_Ifp_Ifp_Ofp_Og16, fp8_add_Ifp_Ifp_Ofp_Opt,
                                            fp8_division_transpose, fp8_layernorm_noparam_backward, fp8_layernorm_noparam_backward_add,
                                            fp8_layernorm_noparam_forward, fp8_linear_backward, fp8_linear_forward,
                                            fp8_linear_forward_add,
                                            fp8_quantize_pertensor, fp8_quantize_pertensor_transpose,
                                            fp8_silu_mul_backward_joined, fp8_silu_mul_forward, fp8_transpose)
from ..activation.real_quantization.common import convert_str_to_fp8, new_max, scale_max, tag_scale_max
from ..utils._fp8_quantization_config import QuantizationConfig
from .coat_llama import (E4M3, _as_e4m3_input, _as_e5m2_grad, _backward_weight_t, _forward_weight, _ResidualBase,
                         apply_rotary_pos_emb, fused_qkv_rotary, fused_rotary, rotary_cos_sin)

__all__ = ["CoatOLMoConfig", "CoatOLMoBeforeAttentionResidual", "CoatOLMoAfterAttentionResidual",
           "CoatOLMoMLPResidual", "CoatOLMoSequentialBlock"]


class CoatOLMoConfig:
    """The fields of OLMo's ModelConfig that the block reads (reference: olmo ModelConfig as used at :653-740, :917-945)."""

    def __init__(self, d_model=4096, n_heads=32, n_kv_heads=None, mlp_hidden_size=None, mlp_ratio=4, include_bias=False,
                 rope=True, rope_theta=10000.0, rope_full_precision=True, clip_qkv=None, attention_dropout=0.0,
                 residual_dropout=0.0, activation_type="swiglu", layer_norm_eps=1e-5, norm_after=False,
                 attention_layer_norm=False, init_device=None, coat_fp8_args=None, **kwargs):
        self.d_model, self.n_heads = d_model, n_heads
        self.n_kv_heads = n_kv_heads
        self.mlp_hidden_size, self.mlp_ratio = mlp_hidden_size, mlp_ratio
        self.include_bias = include_bias
        self.rope, self.rope_theta, self.rope_full_precision = rope, rope_theta, rope_full_precision
        self.clip_qkv = clip_qkv
        self.attention_dropout, self.residual_dropout = attention_dropout, residual_dropout
        self.activation_type = activation_type
        self.layer_norm_eps = layer_norm_eps
        self.norm_after = norm_after
        self.attention_layer_norm = attention_layer_norm
        self.init_device = init_device
        self.coat_fp8_args = dict(coat_fp8_args or {})
        for k, v in kwargs.items():
            setattr(self, k, v)

    @property
    def effective_n_kv_heads(self):
        return self.n_heads if self.n_kv_heads is None else self.n_kv_heads


def _layer_norm(x, eps=1e-5):
    return F.layer_norm(x, x.shape[-1:], None, None, eps)


# ------------------------------------------------------------------------------------------------ before attention
class CoatOLMoBeforeAttentionResidual(_ResidualBase):
    """Residual branch point + LayerNorm + the fused q/k/v projection."""

    def __init__(self, config: CoatOLMoConfig, qargs: QuantizationConfig, layer_id, fused_dims: tuple):
        super().__init__(config, qargs, layer_id)
        self.ln_normalized_shape = config.d_model
        self.att_proj = nn.Linear(config.d_model, sum(fused_dims), bias=config.include_bias, device=config.init_device)

    def forward(self, re_x, x, s):
        if self.training:
            return _CoatOLMoBeforeAttentionResidual.apply(re_x, x, s, *self._prepared(("att_proj",)), self.qargs.group_size,
                                                          self.fwobits, self.layer_id, self.config, self.qargs)
        return re_x, self.att_proj(_layer_norm(re_x))


class _CoatOLMoBeforeAttentionResidual(torch.autograd.Function):
    @staticmethod
    def forward(ctx, re_x, in_x, in_s, w1_origin, w1, w1_t, w1_s, group_size, fwobits, layer_id, config, qargs, eps=1e-5):
        in_x = _as_e4m3_input(in_x, fwobits)
        ln_x, ln_s, ln_x_t, ln_utils = fp8_layernorm_noparam_forward(in_x, in_s, group_size, eps, transpose_output_2d=True)
        fc1_x = fp8_linear_forward(ln_x, ln_s, _forward_weight(w1_origin, w1, w1_s, qargs, fwobits), w1_s, False, group_size)
        ctx.save_for_backward(in_x, in_s, ln_x_t, ln_s)
        ctx.weight = (w1_origin, w1_s) if qargs.weight_memory_efficient else (w1_t, w1_s)
        ctx.group_size = group_size
        ctx.ln_utils = ln_utils
        ctx.utils = fwobits, layer_id, config, qargs
        return re_x, fc1_x

    @staticmethod
    def backward(ctx, fp_grad, flash_g):
        in_x, in_s, ln_x_t, ln_s = ctx.saved_tensors
        w_saved, w1_s = ctx.weight
        group_size = ctx.group_size
        mean, rstd, num_warps = ctx.ln_utils
        fwobits, layer_id, config, qargs = ctx.utils
        # the gradient leaving RoPE / attention is bf16: per-tensor e5m2 in both layouts
        flash_g, flash_gs, flash_g_t = fp8_quantize_pertensor_transpose(flash_g, group_size, fwobits["babit"],
                                                                        transpose_output_2d=True, stochastic=False)
        w1_t = _backward_weight_t(w_saved, w1_s, qargs, fwobits)
        fc1_g, att_proj_wg = fp8_linear_backward(ln_x_t, ln_s, flash_g, flash_gs, flash_g_t, w1_t, w1_s, group_size)
        # fp8_layernorm_noparam_backward + fp8_add_Ifp_Ifp_Ofp_Opt(fp_grad, in_g) of the reference, the addition inside the kernel
        re_g, (in_g, in_sg, in_sg_g16) = fp8_layernorm_noparam_backward_add(in_x, in_s, fc1_g, group_size, mean, rstd, num_warps,
                                                                          fp_grad, fwobits["babit"], stochastic=False)
        return re_g, in_g.view(E4M3), in_sg_g16, att_proj_wg, None, None, None, None, None, None, None, None, None


# ------------------------------------------------------------------------------------------------ after attention
class CoatOLMoAfterAttentionResidual(_ResidualBase):
    """Attention output projection + residual add."""

    def __init__(self, config: CoatOLMoConfig, qargs: QuantizationConfig, layer_id):
        super().__init__(config, qargs, layer_id)
        self.attn_out = nn.Linear(config.d_model, config.d_model, bias=config.include_bias, device=config.init_device)

    def forward(self, re_x, in_x):
        if self.training:
            return _CoatOLMoAfterAttentionResidual.apply(re_x, in_x, *self._prepared(("attn_out",)), self.qargs.group_size,
                                                         self.fwobits, self.layer_id, self.config, self.qargs)
        return re_x + self.attn_out(in_x), None, None


class _CoatOLMoAfterAttentionResidual(torch.autograd.Function):
    @staticmethod
    def forward(ctx, re_x, flash_x, w2_origin, w2, w2_t, w2_s, group_size, fwobits, layer_id, config, qargs):
        flash_qx, flash_s, _ = fp8_quantize_pertensor(flash_x, group_size, fwobits["fabit"], want_pg=False)
        # projection + residual addition (fp8_linear_forward then fp8_add_Ifp_Ifp_Ofp_Og16 in the reference) in one kernel
        fp_x, (out_x, out_s) = fp8_linear_forward_add(flash_qx, flash_s, _forward_weight(w2_origin, w2, w2_s, qargs, fwobits),
                                                      w2_s, re_x, flash_qx.dtype, group_size)
        # the bf16 attention output is saved (not its FP8 copy): its transpose is re-quantized in backward (:331)
        ctx.save_for_backward(flash_x, flash_s)
        ctx.weight = (w2_origin, w2_s) if qargs.weight_memory_efficient else (w2_t, w2_s)
        ctx.group_size = group_size
        ctx.utils = fwobits, layer_id, config, qargs
        return fp_x, out_x.view(E4M3), out_s

    @staticmethod
    def backward(ctx, fp_grad, out_g, out_gs):
        flash_x, flash_s = ctx.saved_tensors
        w_saved, w2_s = ctx.weight
        group_size = ctx.group_size
        fwobits, layer_id, config, qargs = ctx.utils
        out_g = _as_e5m2_grad(out_g, fwobits)
        out_gs_max = scale_max(out_gs)
        out_g_t = fp8_transpose(out_g, transpose_output_2d=True)
        flash_x_t, flash_s = fp8_division_transpose(flash_x, group_size, fwobits["fabit"], flash_s, stochastic=False,
                                                    only_transposed=True)
        w2_t = _backward_weight_t(w_saved, w2_s, qargs, fwobits)
        fc2_g, attn_out_wg = fp8_linear_backward(flash_x_t, flash_s, out_g, out_gs_max, out_g_t, w2_t, w2_s, group_size)
        return fp_grad, fc2_g, attn_out_wg, None, None, None, None, None, None, None, None


# ------------------------------------------------------------------------------------------------ MLP
class CoatOLMoMLPResidual(_ResidualBase):
    """LayerNorm + fused up/gate projection + SiLU(gate) * up + output projection + residual add."""

    def __init__(self, config: CoatOLMoConfig, qargs: QuantizationConfig, layer_id, hidden_size: int):
        super().__init__(config, qargs, layer_id)
        assert config.activation_type == "swiglu", "only the SwiGLU block of the reference's FP8 path is built"
        self.ln_normalized_shape = config.d_model
        self.act_output_multiplier = 0.5
        self.ff_proj = nn.Linear(config.d_model, hidden_size, bias=config.include_bias, device=config.init_device)
        self.ff_out = nn.Linear(int(self.act_output_multiplier * hidden_size), config.d_model, bias=config.include_bias,
                                device=config.init_device)

    def forward(self, re_x, x, s):
        if self.training:
            return _CoatOLMoMLPResidual.apply(re_x, x, s, *self._prepared(("ff_proj", "ff_out")), self.qargs.group_size,
                                              self.fwobits, self.layer_id, self.config, self.qargs)
        up, gate = self.ff_proj(_layer_norm(re_x)).chunk(2, dim=-1)
        return re_x + self.ff_out(F.silu(gate) * up), None, None


class _CoatOLMoMLPResidual(torch.autograd.Function):
    @staticmethod
    def forward(ctx, re_x, in_x, in_s, w1_origin, w1, w1_t, w1_s, w2_origin, w2, w2_t, w2_s, group_size, fwobits,
                layer_id, config, qargs, eps=1e-5):
        in_x = _as_e4m3_input(in_x, fwobits)
        ln_x, ln_s, ln_x_t, ln_utils = fp8_layernorm_noparam_forward(in_x, in_s, group_size, eps, transpose_output_2d=True)
        # the fused projection writes per-group FP8 straight from the GEMM epilogue; halves: up first, gate second (:520)
        fc1_x, fc1_s = fp8_linear_forward(ln_x, ln_s, _forward_weight(w1_origin, w1, w1_s, qargs, fwobits), w1_s, True,
                                          group_size)
        # the halves stay column slices of fc1_x / fc1_s (the reference copies them, :522-523); one kernel for
        # fp8_silu_forward + fp8_mul_forward (:525-528), same tensors
        up_x, gate_x = fc1_x.chunk(2, dim=-1)
        up_s, gate_s = fc1_s.chunk(2, dim=-1)
        silu_x, silu_s, mul_x, mul_s, mul_x_t = fp8_silu_mul_forward(gate_x, gate_s, up_x, up_s, group_size,
                                                                    transpose_output_2d=True)
        # projection + residual addition in one kernel, as above
        fp_x, (out_x, out_s) = fp8_linear_forward_add(mul_x, mul_s, _forward_weight(w2_origin, w2, w2_s, qargs, fwobits),
                                                      w2_s, re_x, mul_x.dtype, group_size)
        ctx.save_for_backward(in_x, in_s, ln_x_t, ln_s, gate_x, gate_s, up_x, up_s, silu_x, silu_s, mul_x_t, mul_s)
        if qargs.weight_memory_efficient:
            ctx.weight = (w1_origin, w1_s, w2_origin, w2_s)
        else:
            ctx.weight = (w1_t, w1_s, w2_t, w2_s)
        ctx.group_size = group_size
        ctx.ln_utils = ln_utils
        ctx.utils = fwobits, layer_id, config, qargs
        return fp_x, out_x.view(E4M3), out_s

    @staticmethod
    def backward(ctx, fp_grad, out_g, out_gs):
        in_x, in_s, ln_x_t, ln_s, gate_x, gate_s, up_x, up_s, silu_x, silu_s, mul_x_t, mul_s = ctx.saved_tensors
        w1_saved, w1_s, w2_saved, w2_s = ctx.weight
        group_size = ctx.group_size
        mean, rstd, num_warps = ctx.ln_utils
        fwobits, layer_id, config, qargs = ctx.utils
        out_g = _as_e5m2_grad(out_g, fwobits)
        out_gs_max = scale_max(out_gs)
        out_g_t = fp8_transpose(out_g, transpose_output_2d=True)
        w2_t = _backward_weight_t(w2_saved, w2_s, qargs, fwobits)
        fc2_g, weight2_grad = fp8_linear_backward(mul_x_t, mul_s, out_g, out_gs_max, out_g_t, w2_t, w2_s, group_size)
        del out_g, out_g_t, w2_t
        # one kernel for the reference's fp8_mul_backward + fp8_silu_backward, writing the two bf16 gradients side by
        # side (no torch.cat); the joined tensor is quantized per tensor with the larger of the two maxima (:594-606)
        gateup_g, gateup_gs, gateup_g_t = fp8_silu_mul_backward_joined(gate_x, gate_s, up_x, up_s, silu_x, silu_s, fc2_g,
                                                                       group_size, fwobits["babit"])
        w1_t = _backward_weight_t(w1_saved, w1_s, qargs, fwobits)
        fc1_g, weight1_grad = fp8_linear_backward(ln_x_t, ln_s, gateup_g, gateup_gs, gateup_g_t, w1_t, w1_s, group_size)
        # fp8_layernorm_noparam_backward + fp8_add_Ifp_Ifp_Ofp_Opt(fp_grad, in_g) of the reference, the addition inside the kernel
        re_g, (in_g, in_sg, in_sg_g16) = fp8_layernorm_noparam_backward_add(in_x, in_s, fc1_g, group_size, mean, rstd, num_warps,
                                                                          fp_grad, fwobits["babit"], stochastic=False)
        return (re_g, in_g.view(E4M3), in_sg_g16, weight1_grad, None, None, None, weight2_grad, None, None, None,
                None, None, None, None, None, None)


# ------------------------------------------------------------------------------------------------ the block
class CoatOLMoSequentialBlock(nn.Module):
    """``x + attn_out(attention(att_proj(LN(x))))`` followed by ``x + ff_out(SwiGLU(ff_proj(LN(x))))`` with the hidden
    state carried between the modules as (bf16, e4m3 per-group codes, scales).  Attention (RoPE + causal SDPA) is bf16."""

    def __init__(self, layer_id: int, config: CoatOLMoConfig, qargs: Optional[QuantizationConfig] = None, cache=None):
        super().__init__()
        assert not config.norm_after, "COAT currently does not support PostNorm"
        assert not config.attention_layer_norm, "q/k LayerNorm is not part of the FP8 block built here"
        assert config.d_model % config.n_heads == 0
        self.layer_id = layer_id
        self.config = config
        self.qargs = QuantizationConfig(**config.coat_fp8_args) if qargs is None else qargs
        # formats in which the neighbouring modules quantize the attention output and the fused q / k / v gradient per tensor
        self._out_fp8 = convert_str_to_fp8[self.qargs.fabit]
        self._grad_fp8 = convert_str_to_fp8[self.qargs.babit]
        self.hidden_size = config.mlp_hidden_size if config.mlp_hidden_size is not None else config.mlp_ratio * config.d_model
        head_dim = config.d_model // config.n_heads
        self.fused_dims = (config.d_model, config.effective_n_kv_heads * head_dim, config.effective_n_kv_heads * head_dim)
        self.BeforeAttention = CoatOLMoBeforeAttentionResidual(config, self.qargs, layer_id, self.fused_dims)
        self.AfterAttention = CoatOLMoAfterAttentionResidual(config, self.qargs, layer_id)
        self.MLPResidual = CoatOLMoMLPResidual(config, self.qargs, layer_id, self.hidden_size)

    def attention(self, q, k, v, attention_bias=None):
        B, T, C = q.size()
        dtype = k.dtype
        hd = C // self.config.n_heads
        v = v.view(B, T, self.config.effective_n_kv_heads, hd).transpose(1, 2)
        if self.config.rope and q.is_cuda and dtype == torch.bfloat16:
            # fused kernel, fp32 arithmetic on fp32 tables (what rope_full_precision asks for)
            q = fused_rotary(q, self.config.n_heads, hd, self.config.rope_theta)
            k = fused_rotary(k, self.config.effective_n_kv_heads, hd, self.config.rope_theta)
        else:
            q, k = self._rope_unfused(q, k, hd, dtype)
        return self._sdpa(q, k, v, attention_bias, B, T, C)

    def _rope_unfused(self, q, k, hd, dtype):
        B, T, _ = q.shape
        q = q.view(B, T, self.config.n_heads, hd).transpose(1, 2)
        k = k.view(B, T, self.config.effective_n_kv_heads, hd).transpose(1, 2)
        if self.config.rope:
            pos = torch.arange(T, device=q.device).unsqueeze(0)
            if self.config.rope_full_precision:
                cos, sin = rotary_cos_sin(pos, hd, self.config.rope_theta, torch.float32)
                q, k = apply_rotary_pos_emb(q.float(), k.float(), cos, sin)
                q, k = q.to(dtype), k.to(dtype)
            else:
                cos, sin = rotary_cos_sin(pos, hd, self.config.rope_theta, dtype)
                q, k = apply_rotary_pos_emb(q, k, cos, sin)
        return q, k

    def _sdpa(self, q, k, v, attention_bias, B, T, C):
        if k.size(1) != q.size(1):
            rep = q.size(1) // k.size(1)
            k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
        # in training the next module quantizes this output per tensor: the attention kernel hands it the scale maximum
        out_max = new_max(q.device) if self.training and q.is_cuda else None
        att = sdpa(q, k, v, attn_mask=attention_bias, dropout_p=self.config.attention_dropout if self.training else 0.0,
                   is_causal=attention_bias is None, out_scale_max=out_max, out_fp8=self._out_fp8)
        att, used_max = att if out_max is not None else (att, False)
        att = att.transpose(1, 2).contiguous().view(B, T, C)
        if used_max:
            tag_scale_max(att, out_max, self._out_fp8)
        return att

    def forward(self, x, qx, sx, attention_bias=None, layer_past=None, use_cache=False, max_doc_len=None,
                cu_doc_lens=None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, None]:
        if layer_past is not None or use_cache or max_doc_len is not None or cu_doc_lens is not None:
            raise NotImplementedError("KV caching and document masking are not part of the training path built here")
        x, qkv = self.BeforeAttention(x, qx, sx)
        if self.config.clip_qkv is not None:
            qkv = qkv.clamp(min=-self.config.clip_qkv, max=self.config.clip_qkv)
        if self.config.rope and qkv.is_cuda and qkv.dtype == torch.bfloat16:
            # RoPE reads the q / k column slices of the fused projection where they lie, and its backward writes into the
            # fused gradient (the reference splits, copies, and concatenates the gradients again, :1003-1006)
            B, T, _ = qkv.shape
            C = self.fused_dims[0]
            hd = C // self.config.n_heads
            q, k, v = fused_qkv_rotary(qkv, self.config.n_heads, self.config.effective_n_kv_heads, hd,
                                       self.config.rope_theta, self._grad_fp8 if self.training else None)
            att = self._sdpa(q, k, v, attention_bias, B, T, C)
        else:
            q, k, v = qkv.split(self.fused_dims, dim=-1)
            att = self.attention(q, k, v, attention_bias)
        x, qx, sx = self.AfterAttention(x, att)
        x, qx, sx = self.MLPResidual(x, qx, sx)
        return x, qx, sx, None
