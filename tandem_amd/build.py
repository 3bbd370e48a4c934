"""Builds libtandem_hip.so (the C-ABI library declared in include/tandem_hip.h)
in-tree with hipcc for gfx950. Cross-compiles without a GPU.

    python -m tandem_amd.build
"""

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(CSRC, "libtandem_hip.so")
SOURCES = ["kernels.hip", "abi.hip", "engine.hip", "engine_abi.hip"]

# -ffp-contract=off: no multiply-add is fused unless the source says fma.
# -fhip-fp32-correctly-rounded-divide-sqrt: IEEE division and sqrt (the default; stated).
# -packed-fp32-ops disabled: the compiler must not form v_pk_*_f32 from scalar float code.
FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
         "-fhip-fp32-correctly-rounded-divide-sqrt", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wextra", "-pthread"]


def build(verbose=False, extra=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = [os.path.join(CSRC, s) for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    cmd = [hipcc, *FLAGS, *extra, "-o", LIB, *srcs, "-lrt"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the device-only target feature and says so: harmless
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
