"""CoatAdamW: AdamW whose first and second moments live in FP8 e4m3 with one scale per 128 elements and,
by default, Dynamic Range Expansion (per-group exponent k and centre c).

Drop-in for coat/optimizer/fp8_adamw.py:36-342 of the reference: same constructor, same ``state`` keys
(``step, exp_avg, scale_exp_avg, expand_exp_avg, sqrt_minmax_exp_avg, exp_avg_sq, scale_exp_avg_sq,
expand_exp_avg_sq, sqrt_minmax_exp_avg_sq``; reference :119-137), same state-dict dtype policy
(:231-262).  One fused HIP kernel per parameter tensor does the whole step (``qoptim_cuda`` shim).

Differences, all deliberate:
  * the per-group vectors are always fp32 (the reference allocates them in the parameter dtype, which
    only works for fp32 parameters because its kernel takes ``float*``, :124-137);
  * the kernels run on torch's current stream;
  * ``amsgrad=True`` raises (the reference's branch calls ``torch.zeros(p, ...)`` and cannot run, :133-135).
"""
from collections import defaultdict
from copy import deepcopy
from itertools import chain
from typing import Optional, Tuple

import torch
from torch.optim.optimizer import Optimizer

from ..utils._fp8_quantization_config import QuantizationConfig
from . import qoptim_cuda

convert_str_to_fp8 = {"E4M3": torch.float8_e4m3fn, "E5M2": torch.float8_e5m2}

_EXPAND_KEYS = ("expand_exp_avg", "sqrt_minmax_exp_avg", "expand_exp_avg_sq", "sqrt_minmax_exp_avg_sq")
_STATE_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2, torch.float32)


class CoatAdamW(Optimizer):
    def __init__(
        self,
        params,
        lr: float = 1e-3,
        betas: Tuple[float, float] = (0.9, 0.999),
        eps: float = 1e-8,
        weight_decay: float = 1e-2,
        amsgrad: bool = False,
        qargs: QuantizationConfig = None,
        *,
        fused: Optional[bool] = None,
        multi_tensor: bool = True,
    ):
        # multi_tensor (not in the reference): parameters of one dtype, device and step count share kernel launches
        self.multi_tensor = multi_tensor
        self.qargs = QuantizationConfig() if qargs is None else qargs
        assert self.qargs.first_order_expansion == self.qargs.second_order_expansion, (
            "We expect the first order and second order momentum to use dynamic range expansion at the same time.")
        if not 0.0 <= lr:
            raise ValueError(f"Invalid learning rate: {lr}")
        if not 0.0 <= eps:
            raise ValueError(f"Invalid epsilon value: {eps}")
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError(f"Invalid beta parameter at index 0: {betas[0]}")
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError(f"Invalid beta parameter at index 1: {betas[1]}")
        if not 0.0 <= weight_decay:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")
        if amsgrad:
            raise ValueError("CoatAdamW does not support amsgrad")
        for name in ("first_order_bit", "second_order_bit"):
            if getattr(self.qargs, name) != "E4M3":
                raise ValueError(f"{name} must be E4M3: the optimizer kernels store both moments in e4m3")
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad, fused=fused)
        super().__init__(params, defaults)

    # ------------------------------------------------------------------ state
    @property
    def use_expansion(self) -> bool:
        """Only "expansion" and "true" switch Dynamic Range Expansion on (reference :293)."""
        return self.qargs.first_order_expansion.lower() in ("expansion", "true")

    def __setstate__(self, state):
        super().__setstate__(state)
        for group in self.param_groups:
            group.setdefault("amsgrad", False)
            group.setdefault("fused", None)
            for p in group["params"]:
                p_state = self.state.get(p, {})
                if len(p_state) != 0 and not torch.is_tensor(p_state["step"]):
                    p_state["step"] = torch.tensor(float(p_state["step"]), dtype=torch.float32)

    def _init_state(self, p, expand):
        """Fresh state: codes 0, scales 0, k = 1, c = 1 (reference :117-137)."""
        state = self.state[p]
        ngroups = (p.numel() + self.qargs.qgroup_size - 1) // self.qargs.qgroup_size
        state["step"] = torch.tensor(0.0)  # host tensor: reading it never syncs the device
        for name, bit in (("exp_avg", self.qargs.first_order_bit), ("exp_avg_sq", self.qargs.second_order_bit)):
            state[name] = torch.zeros_like(p, dtype=convert_str_to_fp8[bit], memory_format=torch.contiguous_format)
            state["scale_" + name] = torch.zeros(ngroups, device=p.device, dtype=torch.float32)
            if expand:
                state["expand_" + name] = torch.ones(ngroups, device=p.device, dtype=torch.float32)
                state["sqrt_minmax_" + name] = torch.ones(ngroups, device=p.device, dtype=torch.float32)
        return state

    @torch._disable_dynamo
    def load_state_dict(self, state_dict) -> None:
        """torch's Optimizer.load_state_dict casts every floating-point state tensor to the parameter dtype;
        FP8 codes and fp32 group vectors must keep theirs, so the mapping is redone here with that policy
        (reference :158-262): ``step`` is left alone, every other tensor must be e4m3 / e5m2 / fp32 and is
        only moved to the parameter's device."""
        state_dict = state_dict.copy()
        for pre_hook in self._optimizer_load_state_dict_pre_hooks.values():
            replaced = pre_hook(self, state_dict)
            if replaced is not None:
                state_dict = replaced

        groups, saved_groups = self.param_groups, deepcopy(state_dict["param_groups"])
        if len(groups) != len(saved_groups):
            raise ValueError("loaded state dict has a different number of parameter groups")
        if any(len(g["params"]) != len(s["params"]) for g, s in zip(groups, saved_groups)):
            raise ValueError("loaded state dict contains a parameter group that doesn't match the size of optimizer's group")
        id_map = dict(zip(chain.from_iterable(s["params"] for s in saved_groups),
                          chain.from_iterable(g["params"] for g in groups)))

        def place(param, value, key=None):
            if isinstance(value, torch.Tensor):
                if key == "step":
                    return value
                assert value.dtype in _STATE_DTYPES, f"unexpected optimizer state dtype {value.dtype} for {key}"
                return value.to(device=param.device)
            if isinstance(value, dict):
                return {k: place(param, v, k) for k, v in value.items()}
            return value

        state = defaultdict(dict)
        for k, v in state_dict["state"].items():
            if k in id_map:
                state[id_map[k]] = place(id_map[k], v)
            else:  # a key outside the parameter mapping is kept as it is (torch.optim.Optimizer.load_state_dict does the same)
                state[k] = v
        for g, s in zip(groups, saved_groups):
            s["params"] = g["params"]
        self.__setstate__({"state": state, "param_groups": saved_groups})
        for post_hook in self._optimizer_load_state_dict_post_hooks.values():
            post_hook(self)

    # ------------------------------------------------------------------ step
    @torch.no_grad()
    def step(self, closure=None):
        """Perform a single optimization step."""
        self._cuda_graph_capture_health_check()
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        expand = self.use_expansion
        qgroup_size, expand_min = self.qargs.qgroup_size, self.qargs.expand_min
        for group in self.param_groups:
            beta1, beta2 = group["betas"]
            lr, wd, eps = group["lr"], group["weight_decay"], group["eps"]
            if isinstance(lr, torch.Tensor):
                lr = lr.item()
            # parameters of one dtype, device and step count are stepped together, 32 to a launch (the reference launches
            # once per parameter, :419-515); a parameter alone in its bucket takes the single-tensor entry point
            buckets = {}
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.grad.is_sparse:
                    raise RuntimeError("AdamW does not support sparse gradients")
                state = self.state[p]
                if len(state) == 0:
                    state = self._init_state(p, expand)
                state["step"] += 1
                step = int(state["step"].item())
                grad = p.grad if p.grad.is_contiguous() else p.grad.contiguous()
                if not p.is_contiguous():
                    raise RuntimeError("CoatAdamW needs contiguous parameters (the state is laid out flat)")
                buckets.setdefault((p.dtype, p.device, step), []).append((p, grad, state))
            for (_, _, step), items in buckets.items():
                if len(items) == 1 or not getattr(self, "multi_tensor", True):
                    for p, grad, state in items:
                        if expand:
                            qoptim_cuda.fp8_adamw_expand_step(
                                p, grad, state["exp_avg"], state["scale_exp_avg"], state["expand_exp_avg"],
                                state["sqrt_minmax_exp_avg"], state["exp_avg_sq"], state["scale_exp_avg_sq"],
                                state["expand_exp_avg_sq"], state["sqrt_minmax_exp_avg_sq"],
                                beta1, beta2, lr, wd, eps, step, qgroup_size, expand_min)
                        else:
                            qoptim_cuda.fp8_adamw_step(
                                p, grad, state["exp_avg"], state["scale_exp_avg"], state["exp_avg_sq"],
                                state["scale_exp_avg_sq"], beta1, beta2, lr, wd, eps, step, qgroup_size)
                    continue
                ps, gs, sts = [i[0] for i in items], [i[1] for i in items], [i[2] for i in items]
                col = lambda key: [st[key] for st in sts]  # noqa: E731
                if expand:
                    qoptim_cuda.fp8_adamw_expand_step_multi(
                        ps, gs, col("exp_avg"), col("scale_exp_avg"), col("expand_exp_avg"), col("sqrt_minmax_exp_avg"),
                        col("exp_avg_sq"), col("scale_exp_avg_sq"), col("expand_exp_avg_sq"), col("sqrt_minmax_exp_avg_sq"),
                        beta1, beta2, lr, wd, eps, step, qgroup_size, expand_min)
                else:
                    qoptim_cuda.fp8_adamw_step_multi(
                        ps, gs, col("exp_avg"), col("scale_exp_avg"), col("exp_avg_sq"), col("scale_exp_avg_sq"),
                        beta1, beta2, lr, wd, eps, step, qgroup_size)
        return loss
