"""``import coat_amd.dropin`` registers this package under the reference's module names, so code written
against NVlabs/COAT (``from coat.activation.real_quantization import fp8_quantize``, ``import qoptim_cuda``,
``from coat.optimizer.fp8_adamw import CoatAdamW``) runs unchanged on the HIP kernels."""
import importlib
import pkgutil
import sys

import coat_amd
from coat_amd.optimizer import qoptim_cuda as _qoptim


def install():
    sys.modules.setdefault("qoptim_cuda", _qoptim)
    sys.modules.setdefault("coat", coat_amd)
    for info in pkgutil.walk_packages(coat_amd.__path__, prefix="coat_amd."):
        if info.name in ("coat_amd.dropin", "coat_amd.build") or info.name.endswith("libcoat_hip"):
            continue  # the C-ABI shared object sits in the package directory but is not a Python module
        mod = importlib.import_module(info.name)
        sys.modules.setdefault("coat" + info.name[len("coat_amd"):], mod)


install()
