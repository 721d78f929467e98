"""CPU oracle for the FP8 hot path.  TEST INFRASTRUCTURE ONLY.

Everything under ``oracle/`` is a CPU restatement of the reference's algorithms
(NVlabs/COAT), written to be read next to the reference file:line each function
cites.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg
of ``bench.py`` may import it, and only as the checker.  Nothing in ``coat_amd``
imports it; the product path fails loudly when the HIP library is missing.

Modules
  fp8_codec.py       numpy integer-arithmetic OCP FP8 (e4m3fn / e5m2) encoder and
                     decoder; pins the torch-CPU casts the other modules use.
  activation_ref.py  torch-CPU restatement of the quantize / transpose / division /
                     dequantize / GEMM / SiLU / mul / GELU / RMSNorm / add kernels.
  adamw_ref.c        plain-C restatement of the two FP8 AdamW CUDA kernels
                     (with the 32-lane shuffle-tree min/max emulated exactly).
  adamw_ref.py       ctypes binding of adamw_ref.c + a torch restatement of the
                     reference test's own simulated optimizer step.

Pin status is listed per function in each module's header.
"""
