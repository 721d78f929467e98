"""Quantization settings carried by the models and the optimizer.

Field names and defaults follow coat/utils/_fp8_quantization_config.py:6-80 (the constructor there
also swallows unknown keyword arguments, which HfArgumentParser-based launchers rely on)."""

_FIELDS = (
    # activations / weights / gradients
    ("quantize_model", "true"),
    ("symm", True),
    ("epsilon", 1e-10),
    ("fabit", "E4M3"),
    ("fwbit", "E4M3"),
    ("fobit", "E4M3"),
    ("babit", "E5M2"),
    ("bwbit", "E5M2"),
    ("bobit", "E5M2"),
    ("group_size", 16),
    ("pad_to_multiple_of", 0),
    ("weight_memory_efficient", True),
    # optimizer states
    ("first_order_expansion", "true"),
    ("second_order_expansion", "true"),
    ("first_order_bit", "E4M3"),
    ("second_order_bit", "E4M3"),
    ("qgroup_size", 128),
    ("expand_min", 16),
    # legacy
    ("row_blocksize", -1),
    ("col_blocksize", -1),
)


class QuantizationConfig:
    def __init__(self, *args, **kwargs):
        names = [n for n, _ in _FIELDS]
        if len(args) > len(names):
            raise TypeError(f"QuantizationConfig takes at most {len(names)} positional arguments")
        given = dict(zip(names, args))
        for name, default in _FIELDS:
            if name in given and name in kwargs:
                raise TypeError(f"QuantizationConfig got multiple values for argument {name!r}")
            setattr(self, name, given.get(name, kwargs.get(name, default)))

    def to_dict(self):
        return {n: getattr(self, n) for n, _ in _FIELDS}

    def __repr__(self):
        return "QuantizationConfig(" + ", ".join(f"{k}={v!r}" for k, v in self.to_dict().items()) + ")"

    def __eq__(self, other):
        return isinstance(other, QuantizationConfig) and self.to_dict() == other.to_dict()
