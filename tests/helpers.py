"""Shared by the tests: fixture loading and seeded inputs."""

import json
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def golden_npz(name):
    return np.load(os.path.join(GOLDEN, name))


def golden_json(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


def npz_json(npz, key):
    return json.loads(bytes(npz[key]).decode())


def seeded(seed, rank, n, scale=1.0):
    """The reference tests' seeding idiom (tests/test_comm.py:13-16 there)."""
    g = torch.Generator().manual_seed(seed * 1000 + rank)
    return torch.randn(n, generator=g) * scale


def bits(a):
    """Bit pattern view for exact comparison (distinguishes -0.0 from 0.0, NaNs)."""
    a = np.ascontiguousarray(a)
    return a.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[a.dtype.itemsize])


class OracleShardedAdamW:
    """The oracle's AdamW behind ShardedAdamW's interface, for CPU torch tensors
    (the wrappers' host logic is tested on the CPU with this and the oracle's
    CPU-process group; the product's own optimizer and group are GPU only).
    torch_sqrt=True substitutes torch's CPU sqrt, to compare bit for bit with runs
    that used torch's CPU kernels."""

    def __init__(self, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, torch_sqrt=True):
        self.hyper, self.torch_sqrt, self.inner = (lr, betas, eps, weight_decay), torch_sqrt, None

    def _make(self, dtype):
        from oracle.adamw import AdamW

        # fp32 and float64: torch's vectorised CPU sqrt is not correctly rounded. bfloat16: its root is rounded to 8 bits
        # and comes out the same either way (the exact root never lies near a bfloat16 rounding tie).
        root = (lambda v: torch.from_numpy(v).sqrt().numpy()) if self.torch_sqrt and dtype in (torch.float32, torch.float64) else None
        kind = {torch.bfloat16: "bf16", torch.float16: "f16"}.get(dtype)
        return AdamW(*self.hyper, sqrt=root, kind=kind)

    @staticmethod
    def _array(t):
        t = t.detach()
        return t.view(torch.int16).numpy().view(np.uint16) if t.element_size() == 2 else t.numpy()

    def update(self, key, param, grad):
        assert param.device.type == "cpu" and param.is_contiguous() and grad.is_contiguous() and param.dtype == grad.dtype
        if self.inner is None:
            self.inner = self._make(param.dtype)
        self.inner.update(key, self._array(param), self._array(grad))

    def state_bytes(self):
        return self.inner.state_bytes()

    @property
    def state(self):
        return self.inner.state
