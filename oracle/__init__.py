"""CPU oracle for tandem's data-parallel reduction path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package, and only as the checker (or the timed CPU baseline). Nothing under
tandem_amd/ imports it; the HIP path fails loudly when its library is missing
rather than falling back to anything here.

Contents, and what pins each against the reference (tests/test_oracle_*.py):

  ring.fold / expected_*   closed form of the ring's summation order
                           (tandem/comm.py:301-305,336-343).  Pinned by
                           tests/golden/ring_w{2,3,4}.npz and ring_dtypes_w3.npz
                           (outputs of the reference's Python engine), by the
                           independent step-by-step simulator ring.simulate, by
                           the n=2 identity x0/2 + x1/2 and by integer-valued
                           inputs whose sums are exact in any order.  The integer
                           kinds narrower than 64 bits wrap around: pinned by the
                           order-free modular sum (numpy in 64 bits, reduced to the
                           element's width) on inputs that overflow, and by ATen's
                           own add_ on CPU tensors, which is what the reference's
                           engines call for them (tandem/comm.py:276-277).
  adamw.AdamW              tandem/optim.py:16-37.  First and second moments pinned
                           bit for bit by tests/golden/adamw.npz; the parameter
                           update is pinned bit for bit when torch's own CPU sqrt
                           is substituted, and to 1 ulp of the update term with
                           the correctly rounded sqrtf (torch's vectorised CPU
                           sqrt is not correctly rounded on ~0.7% of inputs).
                           float64 and bfloat16 shards (the reference's seven torch
                           operations take any floating dtype): pinned by
                           tests/golden/adamw_dtypes.npz, the reference's ShardedAdamW on
                           such shards (bf16 bit for bit in p, m, v; f64 like fp32), by
                           torch.optim.AdamW(foreach=False) on the CPU, and operation by
                           operation against torch's CPU kernels on inputs where the
                           candidate formulas differ (which scalar is rounded to bf16,
                           what is fused).
  cpu_engine               from-scratch CPU-process engine speaking the Python
                           engine's protocol (tandem/comm.py:172-311); pinned by
                           the same ring fixtures and by tests/golden/train_w*.json.
                           It is also the timed CPU baseline.

oracle/_ref (a build of the reference's own native sources) does not exist: the
reference's C++ engine needs libtorch/ATen + pybind11, its GPU files need nvcc.
"""

import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build():
    """Compiles tandem_oracle.c into oracle/_build/liboracle.so (gcc, seconds)."""
    subprocess.run(["make", "-s", "-B", "-C", _HERE], check=True)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "_build", "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB
