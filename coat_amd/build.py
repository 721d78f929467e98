"""Builds libcoat_hip.so (the C-ABI library of hand-written gfx950 kernels) in-tree with hipcc.

    python -m coat_amd.build            # compile every csrc/*.hip and link coat_amd/libcoat_hip.so

Cross-compiles without a GPU.  Flags that matter for numerics:
  -ffp-contract=off                              no implicit FMA: kernels state every fused operation explicitly
  -Xclang -target-feature -Xclang -packed-fp32-ops   keep the compiler from forming packed-fp32 VALU instructions
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "_obj")
LIB = os.path.join(HERE, "libcoat_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
] + os.environ.get("COAT_HIPCC_FLAGS", "").split()  # extra flags (e.g. -D tuning switches) for experiments


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _compile(src):
    obj = os.path.join(OBJ, os.path.basename(src).replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    return src, obj, r.returncode, r.stdout + r.stderr


def build(verbose=True, jobs=None, lib=None):
    lib = lib or os.environ.get("COAT_LIB_OUT") or LIB
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")))
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, obj, rc, out in ex.map(_compile, srcs):
            # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless
            msgs = [l for l in out.splitlines() if "packed-fp32-ops" not in l and "is not a recognized feature" not in l]
            if rc != 0:
                raise RuntimeError(f"hipcc failed on {src}:\n" + "\n".join(msgs))
            if verbose:
                print(f"[coat_amd.build] compiled {os.path.relpath(src, HERE)}")
                warn = [l for l in msgs if "warning" in l]
                for l in warn[:10]:
                    print("   ", l)
            objs.append(obj)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print(f"[coat_amd.build] linked {lib}")
    return lib


if __name__ == "__main__":
    build()
    sys.exit(0)
