"""AdamW on flat shards of the parameters, for the ZeRO stages: one fused HIP
kernel per shard instead of seven elementwise passes.

Same interface as tandem's ShardedAdamW (tandem/optim.py:11-40 there) and the
same arithmetic, operation for operation: the step's scalars are computed in
Python doubles by the same expressions and applied in the shard's own
arithmetic, as torch does with a Python scalar. fp32 shards: the scalars are
rounded to fp32 once (tdm_k3_adamw). float64: doubles throughout. bfloat16 and
float16: each of the seven operations computes in fp32 and rounds to the type
(tdm_k3_adamw_typed)."""

import ctypes

import torch

from ._lib import (ADAMW_DEVICE_ORDER, ADAMW_HOST_ORDER, AdamwHyper, AdamwScalars, check, dtype_code, lib, require_device_tensor,
                   stream_ptr)

SHARD_DTYPES = (torch.float32, torch.float64, torch.bfloat16, torch.float16)


def step_scalars(step, lr, betas, eps, weight_decay):
    """The constants of step `step` (a float, 1-based), tandem/optim.py:28-37."""
    beta1, beta2 = betas
    bias_correction1 = 1 - beta1 ** step
    bias_correction2 = 1 - beta2 ** step
    step_size = lr / bias_correction1
    bias_correction2_sqrt = bias_correction2 ** 0.5
    s = AdamwScalars()
    s.use_decay = int(weight_decay != 0)
    s.decay = 1 - lr * weight_decay  # ctypes rounds a Python float to fp32 (nearest even) on assignment
    s.w1 = 1 - beta1
    s.beta2 = beta2
    s.one_m_b2 = 1 - beta2
    s.bc2_sqrt = bias_correction2_sqrt
    s.eps = eps
    s.neg_step = -step_size
    s.inv_bc2_sqrt = 1.0 / bias_correction2_sqrt  # torch's GPU `tensor / scalar` multiplies by this
    return s


LINE = 128  # bytes: the kernels write whole cache lines when all of a launch's streams share their distance from one


def zeros_at_phase_of(like, numel=None):
    """A zeroed tensor of `numel` elements (default: as many as `like`) in `like`'s memory
    that starts at the same distance from a 128-byte boundary as `like` does. A shard cut
    out of a flat buffer by tensor_split starts anywhere; the kernels run on 16-byte
    vectors, and on whole cache lines, when all of their streams share that distance (the
    few elements before the boundary are peeled off), so a shard's gradient and optimizer
    state are laid out at the shard's own phase."""
    n = like.numel() if numel is None else int(numel)
    es = like.element_size()
    store = torch.zeros(n + LINE // es, device=like.device, dtype=like.dtype)
    lead = ((like.data_ptr() - store.data_ptr()) % LINE) // es
    return store[lead:lead + n]


def step_hyper(step, lr, betas, eps, weight_decay):
    """The same constants as Python doubles, unrounded, for the entry point that takes the shard's element type."""
    beta1, beta2 = betas
    bias_correction1 = 1 - beta1 ** step
    bias_correction2 = 1 - beta2 ** step
    h = AdamwHyper()
    h.use_decay = int(weight_decay != 0)
    h.decay = 1 - lr * weight_decay
    h.w1 = 1 - beta1
    h.beta2 = beta2
    h.one_m_b2 = 1 - beta2
    h.bc2_sqrt = bias_correction2 ** 0.5
    h.eps = eps
    h.neg_step = -(lr / bias_correction1)
    return h


class ShardedAdamW:
    """order="host" reproduces torch's CPU addcdiv_ (p + (step*m)/d), which is
    what the reference's CPU engine computes; order="device" reproduces torch's
    GPU addcdiv_ kernel (fma(step, m/d, p)), for comparing with
    torch.optim.AdamW run on the GPU itself."""

    def __init__(self, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, order="host"):
        if order not in ("host", "device"):
            raise ValueError(f"unknown update order {order}")
        self.lr, self.betas, self.eps, self.weight_decay = lr, betas, eps, weight_decay
        self.order = ADAMW_HOST_ORDER if order == "host" else ADAMW_DEVICE_ORDER
        self.state = {}  # key -> [step, exp_avg, exp_avg_sq]
        lib()

    def update(self, key, param, grad, copies=()):
        """One step for one shard: `param` and `grad` are same-shaped tensors in GPU
        memory, fp32, float64, bfloat16 or float16 (all but fp32 in host order only);
        `key` names the shard's optimizer state. `copies`:
        further tensors of the same shape (the other ranks' copies of this shard, when
        the ranks are buffers in one memory) that receive the updated parameters in the
        same pass, which makes the all-gather after the step unnecessary."""
        require_device_tensor(param, "ShardedAdamW.update(param)")
        require_device_tensor(grad, "ShardedAdamW.update(grad)")
        for c in copies:
            require_device_tensor(c, "ShardedAdamW.update(copies)")
            if c.dtype != param.dtype or c.shape != param.shape:
                raise ValueError("a copy differs from param in dtype or shape")
        if param.dtype not in SHARD_DTYPES or grad.dtype != param.dtype:
            raise ValueError(f"ShardedAdamW handles fp32, float64, bfloat16 and float16 shards whose gradient has the same dtype (got {param.dtype}, {grad.dtype})")
        if param.dtype != torch.float32 and self.order != ADAMW_HOST_ORDER:
            raise ValueError("order=\"device\" is defined for fp32 shards only")
        if param.shape != grad.shape:
            raise ValueError("param and grad differ in shape")
        if key not in self.state:
            self.state[key] = [0.0, zeros_at_phase_of(param), zeros_at_phase_of(param)]
        st = self.state[key]
        st[0] += 1.0
        step, exp_avg, exp_avg_sq = st
        if param.numel() == 0:
            return
        if param.dtype != torch.float32:
            h = step_hyper(step, self.lr, self.betas, self.eps, self.weight_decay)
            arr = (ctypes.c_void_p * max(1, len(copies)))(*[c.data_ptr() for c in copies])
            check(lib().tdm_k3_adamw_typed(ctypes.c_void_p(param.data_ptr()), ctypes.c_void_p(grad.data_ptr()),
                                           ctypes.c_void_p(exp_avg.data_ptr()), ctypes.c_void_p(exp_avg_sq.data_ptr()),
                                           param.numel(), dtype_code(param.dtype), ctypes.byref(h), self.order, arr, len(copies),
                                           stream_ptr(param.device)))
            return
        s = step_scalars(step, self.lr, self.betas, self.eps, self.weight_decay)
        if copies:
            arr = (ctypes.c_void_p * len(copies))(*[c.data_ptr() for c in copies])
            check(lib().tdm_k3_adamw_gather(ctypes.c_void_p(param.data_ptr()), ctypes.c_void_p(grad.data_ptr()),
                                            ctypes.c_void_p(exp_avg.data_ptr()), ctypes.c_void_p(exp_avg_sq.data_ptr()),
                                            param.numel(), ctypes.byref(s), self.order, arr, len(copies),
                                            stream_ptr(param.device)))
            return
        check(lib().tdm_k3_adamw(ctypes.c_void_p(param.data_ptr()), ctypes.c_void_p(grad.data_ptr()),
                                 ctypes.c_void_p(exp_avg.data_ptr()), ctypes.c_void_p(exp_avg_sq.data_ptr()),
                                 param.numel(), ctypes.byref(s), self.order, stream_ptr(param.device)))

    def begin_step(self, key, param):
        """For a caller that runs the update inside a fused launch of its own
        (Group.zero2_step): creates the shard's state if need be, counts the step, and
        returns (constants, exp_avg, exp_avg_sq, order) for it: the constants rounded to fp32
        for an fp32 shard (AdamwScalars), as doubles for the other shard types (AdamwHyper)."""
        require_device_tensor(param, "ShardedAdamW.begin_step(param)")
        if param.dtype not in SHARD_DTYPES:
            raise ValueError(f"ShardedAdamW handles float32, float64, bfloat16 and float16 shards, not {param.dtype}")
        if param.dtype != torch.float32 and self.order != ADAMW_HOST_ORDER:
            raise ValueError("order='device' is defined for fp32 shards only")
        if key not in self.state:
            self.state[key] = [0.0, zeros_at_phase_of(param), zeros_at_phase_of(param)]
        st = self.state[key]
        st[0] += 1.0
        constants = step_scalars if param.dtype == torch.float32 else step_hyper  # fp32 constants for fp32 shards, doubles otherwise
        return constants(st[0], self.lr, self.betas, self.eps, self.weight_decay), st[1], st[2], self.order

    def state_bytes(self):
        return sum(t.numel() * t.element_size() for _, a, b in self.state.values() for t in (a, b))
