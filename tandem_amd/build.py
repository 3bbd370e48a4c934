"""Builds libtandem_hip.so (the C-ABI library declared in include/tandem_hip.h)
in-tree with hipcc for gfx950, and beside it libtandem_probe.so (include/tandem_probe.h:
the stream-mix measurement kernel that the benchmark and the GPU tests load, kept out of
the plug-in). Cross-compiles without a GPU.

    python -m tandem_amd.build [extra hipcc flags, e.g. -DTDM_NT_MASK=7] [--out=path/to/variant.so]

Every source is compiled to an object of its own, in parallel, then linked.
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(CSRC, "libtandem_hip.so")
SOURCES = ["kernels.hip", "kernels_chain.hip", "abi.hip", "engine.hip", "engine_abi.hip"]
PROBE_LIB = os.path.join(CSRC, "libtandem_probe.so")
PROBE_SOURCES = ["probe.hip"]

# -ffp-contract=off: no multiply-add is fused unless the source says fma.
# -fhip-fp32-correctly-rounded-divide-sqrt: IEEE division and sqrt (the default; stated).
# -packed-fp32-ops disabled: the compiler must not form v_pk_*_f32 from scalar float code.
# -fvisibility=hidden: the library exports the entry points of include/tandem_hip.h and nothing else.
FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off",
         "-fhip-fp32-correctly-rounded-divide-sqrt", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wextra", "-pthread"]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the device-only target feature and says so: harmless
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}): {' '.join(cmd)}\n{out}")
    if verbose and out.strip():
        print(out)


def build(verbose=False, extra=(), out=LIB, sources=None):
    """Compiles every source (always: nothing is reused from an earlier build) and links `out`."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = list(SOURCES if sources is None else sources)
    objdir = os.path.join(CSRC, "_obj", os.path.splitext(os.path.basename(out))[0])
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, os.path.splitext(s)[0] + ".o") for s in srcs]
    jobs = [[hipcc, *FLAGS, *extra, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(srcs, objs)]
    with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1)) as pool:
        list(pool.map(lambda cmd: _run(cmd, verbose), jobs))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-pthread", "-o", out, *objs, "-lrt"], verbose)
    return out


def build_probe(verbose=False, extra=(), out=PROBE_LIB):
    """The measurement library, from the same device headers and with the same flags as the plug-in."""
    return build(verbose, extra, out, PROBE_SOURCES)


if __name__ == "__main__":
    args = sys.argv[1:]
    target = LIB
    for a in list(args):
        if a.startswith("--out="):
            target = os.path.abspath(a[len("--out="):])
            args.remove(a)
    print(build(verbose=True, extra=args, out=target))
    if target == LIB:
        print(build_probe(verbose=True, extra=args))
