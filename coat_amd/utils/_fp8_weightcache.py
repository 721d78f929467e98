"""Per-step cache of weight quantization results (reference: coat/utils/_fp8_weightcache.py:4-37).

On the first micro-batch of an optimizer step the weight's per-tensor scale (memory-efficient mode) or its FP8
copy, transposed FP8 copy and scale (cached mode) are computed and kept on the module; later micro-batches reuse
them, since the master weight does not change between optimizer steps."""
import torch.nn as nn

from ..activation.real_quantization._division import absmax_scale
from ..activation.real_quantization._division_transpose import fp8_division_transpose
from ..activation.real_quantization.common import as_fp8_dtype


class FP8CacheWeightModule(nn.Module):
    def __init__(self, config, qargs, layer_id):
        super().__init__()
        self.config = config
        self.qargs = qargs
        self.layer_id = layer_id

    def prepare_weight(self, weight, weight_name, is_first_microbatch):
        """Memory-efficient mode returns the scale; cached mode returns (weight_fp8, weight_fp8_t, scale)."""
        fwbit = self.fwobits["fwbit"]
        if is_first_microbatch:
            if self.qargs.weight_memory_efficient:
                # only the scale is needed here: one abs-max pass instead of quantizing and discarding the codes
                scale = absmax_scale(weight.detach().contiguous(), as_fp8_dtype(fwbit))
                setattr(self, f"{weight_name}_fp8_scale", scale)
                return scale
            weight_fp8, scale, weight_fp8_t = fp8_division_transpose(weight, self.qargs.group_size, fwbit)
            setattr(self, f"{weight_name}_fp8", weight_fp8)
            setattr(self, f"{weight_name}_fp8_t", weight_fp8_t)
            setattr(self, f"{weight_name}_fp8_scale", scale)
            return weight_fp8, weight_fp8_t, scale
        if self.qargs.weight_memory_efficient:
            return getattr(self, f"{weight_name}_fp8_scale")
        return (getattr(self, f"{weight_name}_fp8"), getattr(self, f"{weight_name}_fp8_t"),
                getattr(self, f"{weight_name}_fp8_scale"))

    def forward(self, x):
        pass
