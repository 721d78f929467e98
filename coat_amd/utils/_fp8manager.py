"""Global FP8 execution state (reference: coat/utils/_fp8manager.py:20-25)."""


class FP8Manager:
    """``is_first_microbatch`` is set by the training loop (True on the first micro-batch of an
    optimizer step); weight scales / FP8 weights are refreshed only then."""

    is_first_microbatch = True
