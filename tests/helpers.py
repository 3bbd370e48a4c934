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
    return a.view({2: np.uint16, 4: np.uint32, 8: np.uint64}[a.dtype.itemsize])
