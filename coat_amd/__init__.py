"""coat_amd: MI355X (gfx950) implementation of the FP8 hot path of NVlabs/COAT.

Python entry points keep the reference's names and signatures (``coat_amd.activation.real_quantization``,
``coat_amd.optimizer.fp8_adamw``, ``coat_amd.models.coat_llama``, ``coat_amd.utils``); all compute is in
hand-written HIP kernels behind the C ABI declared in include/coat_hip.h (``coat_amd/libcoat_hip.so``).
``import coat_amd.dropin`` additionally registers the package under the reference's module names
(``coat`` and ``qoptim_cuda``).
"""
__version__ = "0.1.0"
