"""AdamW on a flat fp32 shard, on the CPU (TEST INFRASTRUCTURE ONLY).

Follows tandem/optim.py:16-37: the scalars are computed in Python doubles
exactly as written there and rounded to fp32 once when applied to the tensor,
the way torch applies a Python scalar to a float tensor; the per-element
arithmetic is oracle/tandem_oracle.c.
"""

import ctypes

import numpy as np

from . import lib


def _f32(x):
    return float(np.float32(x))


def scalars(step, lr, betas, eps, weight_decay):
    """The fp32 constants of step number `step` (1-based), from the Python-double
    expressions of tandem/optim.py:28-37."""
    beta1, beta2 = betas
    bias_correction1 = 1 - beta1 ** step
    bias_correction2 = 1 - beta2 ** step
    step_size = lr / bias_correction1
    bias_correction2_sqrt = bias_correction2 ** 0.5
    return {
        "use_decay": int(weight_decay != 0),
        "decay": _f32(1 - lr * weight_decay),
        "w1": _f32(1 - beta1),
        "beta2": _f32(beta2),
        "one_m_b2": _f32(1 - beta2),
        "bc2_sqrt": _f32(bias_correction2_sqrt),
        "eps": _f32(eps),
        "neg_step": _f32(-step_size),
    }


def _p(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return ctypes.c_void_p(a.ctypes.data)


class AdamW:
    """Same constructor and update(key, param, grad) as tandem's ShardedAdamW
    (tandem/optim.py:11-16), on numpy fp32 arrays updated in place.

    sqrt: None for the correctly rounded sqrtf, or a callable array -> array
    (tests substitute torch's CPU sqrt to compare bit for bit with fixtures
    produced by torch)."""

    def __init__(self, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, sqrt=None):
        self.lr, self.betas, self.eps, self.weight_decay = lr, betas, eps, weight_decay
        self.state = {}
        self.sqrt = sqrt

    def update(self, key, param, grad):
        if key not in self.state:
            self.state[key] = [0.0, np.zeros_like(param), np.zeros_like(param)]
        st = self.state[key]
        st[0] += 1.0
        step, m, v = st
        n = param.size
        if n == 0:
            return
        s = scalars(step, self.lr, self.betas, self.eps, self.weight_decay)
        f = ctypes.c_float
        L = lib()
        if self.sqrt is None:
            L.orc_adamw_f32(_p(param), _p(grad), _p(m), _p(v), ctypes.c_int64(n), ctypes.c_int(s["use_decay"]),
                            f(s["decay"]), f(s["w1"]), f(s["beta2"]), f(s["one_m_b2"]), f(s["bc2_sqrt"]),
                            f(s["eps"]), f(s["neg_step"]))
            return
        L.orc_adamw_moments_f32(_p(param), _p(grad), _p(m), _p(v), ctypes.c_int64(n), ctypes.c_int(s["use_decay"]),
                                f(s["decay"]), f(s["w1"]), f(s["beta2"]), f(s["one_m_b2"]))
        root = np.ascontiguousarray(self.sqrt(v), dtype=np.float32)
        L.orc_adamw_apply_f32(_p(param), _p(m), _p(root), ctypes.c_int64(n), f(s["bc2_sqrt"]), f(s["eps"]),
                              f(s["neg_step"]))

    def state_bytes(self):
        return sum(a.nbytes + b.nbytes for _, a, b in self.state.values())
