"""AdamW on a flat shard, on the CPU (TEST INFRASTRUCTURE ONLY).

Follows tandem/optim.py:16-37: the scalars are computed in Python doubles
exactly as written there and rounded to fp32 once when applied to the tensor,
the way torch applies a Python scalar to a float tensor; the per-element
arithmetic is oracle/tandem_oracle.c. fp32 shards are numpy float32 arrays;
float64 shards numpy float64 arrays (the scalars stay doubles); bfloat16 and
float16 shards are their bit patterns in numpy uint16 arrays with kind="bf16" /
"f16" (fp32 arithmetic, rounded to the 16-bit type after each of the
reference's torch operations).
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


def _p(a, dtype=np.float32):
    assert a.dtype == dtype and a.flags.c_contiguous
    return ctypes.c_void_p(a.ctypes.data)


def scalars_f64(step, lr, betas, eps, weight_decay):
    """The same constants for float64 shards: a Python double applied to a double tensor is not rounded."""
    beta1, beta2 = betas
    bias_correction1 = 1 - beta1 ** step
    bias_correction2 = 1 - beta2 ** step
    return {"use_decay": int(weight_decay != 0), "decay": 1 - lr * weight_decay, "w1": 1 - beta1, "beta2": beta2,
            "one_m_b2": 1 - beta2, "bc2_sqrt": bias_correction2 ** 0.5, "eps": eps, "neg_step": -(lr / bias_correction1)}


class AdamW:
    """Same constructor and update(key, param, grad) as tandem's ShardedAdamW
    (tandem/optim.py:11-16), on numpy fp32 arrays updated in place.

    sqrt: None for the correctly rounded sqrtf, or a callable array -> array
    (tests substitute torch's CPU sqrt to compare bit for bit with fixtures
    produced by torch)."""

    def __init__(self, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, sqrt=None, kind=None):
        """kind: None (taken from the array: float32 or float64), or "bf16" / "f16" for uint16 arrays of bit patterns."""
        self.lr, self.betas, self.eps, self.weight_decay = lr, betas, eps, weight_decay
        self.state = {}
        self.sqrt = sqrt
        self.kind = kind

    def update(self, key, param, grad):
        if key not in self.state:
            self.state[key] = [0.0, np.zeros_like(param), np.zeros_like(param)]
        st = self.state[key]
        st[0] += 1.0
        step, m, v = st
        n = param.size
        if n == 0:
            return
        if self.kind in ("bf16", "f16") or param.dtype == np.float64:
            return self._update_other(param, grad, m, v, step, n)
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

    def _update_other(self, param, grad, m, v, step, n):
        L = lib()
        if self.kind in ("bf16", "f16"):
            s, f, dt, tag = scalars(step, self.lr, self.betas, self.eps, self.weight_decay), ctypes.c_float, np.uint16, self.kind
        else:
            s, f, dt, tag = scalars_f64(step, self.lr, self.betas, self.eps, self.weight_decay), ctypes.c_double, np.float64, "f64"
        head = (_p(param, dt), _p(grad, dt), _p(m, dt), _p(v, dt), ctypes.c_int64(n), ctypes.c_int(s["use_decay"]),
                f(s["decay"]), f(s["w1"]), f(s["beta2"]), f(s["one_m_b2"]))
        tail = (f(s["bc2_sqrt"]), f(s["eps"]), f(s["neg_step"]))
        if self.sqrt is None:
            getattr(L, f"orc_adamw_{tag}")(*head, *tail)
            return
        getattr(L, f"orc_adamw_moments_{tag}")(*head)
        root = np.ascontiguousarray(self.sqrt(v), dtype=dt)
        getattr(L, f"orc_adamw_apply_{tag}")(_p(param, dt), _p(m, dt), _p(root, dt), ctypes.c_int64(n), *tail)

    def state_bytes(self):
        return sum(a.nbytes + b.nbytes for _, a, b in self.state.values())
