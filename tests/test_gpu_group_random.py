"""A seeded sweep of collectives between process ranks that share the GPU: element type, length,
chunk sizes with empty chunks, views that start anywhere in their allocation (a phase of its own
on every rank), the operation and its variant drawn at random, many in a row on one group so that
staging halves and slots are reused in every combination. Every rank checks its own result bit
for bit against the oracle and the guard elements around its view. Run with -m gpu."""

import os

import numpy as np
import pytest
import torch

from helpers import bits

pytestmark = pytest.mark.gpu
SHIFT = int(os.environ.get("TANDEM_SWEEP_SEED", "0"))  # added to the sweep's seed: other cases of the same kinds

KINDS = {torch.float32: "f32", torch.float64: "f64", torch.float16: "f16", torch.bfloat16: "bf16", torch.int64: "i64",
         torch.int32: "i32", torch.int16: "i16", torch.int8: "i8", torch.uint8: "u8"}
GUARD = 24
TIMEOUT = 60.0


def raw(t):
    t = t.detach().cpu()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def draw(rng, dtype, n):
    if dtype.is_floating_point:
        return torch.from_numpy(rng.standard_normal(n).astype(np.float32)).to(dtype)
    if dtype == torch.int64:
        return torch.from_numpy(rng.integers(-(1 << 50), 1 << 50, n, dtype=np.int64))
    info = torch.iinfo(dtype)
    return torch.from_numpy(rng.integers(info.min, info.max + 1, n, dtype=np.int64)).to(dtype)


def sweep(g, seed, count):
    """Runs on every rank; all ranks draw the same cases. Returns the labels of the cases that came out wrong."""
    from oracle import ring

    dev, w, r = g.device, g.size, g.rank
    rng = np.random.default_rng(seed)
    dtypes = list(KINDS)
    wrong = []
    for k in range(count):
        dtype = dtypes[int(rng.integers(len(dtypes)))]
        kind = KINDS[dtype]
        n = int(rng.choice([0, 1, 3, 17, 255, 1000, 1025, 4099, 10_007, 40_000])) + int(rng.integers(0, 3))
        cuts = np.sort(rng.integers(0, n + 1, w - 1))
        sizes = np.diff(np.concatenate([[0], cuts, [n]])).astype(int).tolist()
        if rng.random() < 0.3:
            i, j = int(rng.integers(w)), int(rng.integers(w))
            if i != j:
                sizes[i] += sizes[j]
                sizes[j] = 0
        starts = [int(rng.integers(0, GUARD)) for _ in range(w)]
        what = str(rng.choice(["all_reduce", "all_reduce", "reduce_scatter", "reduce_scatter_owner", "all_gather", "broadcast"]))
        avg = bool(dtype.is_floating_point and rng.random() < 0.5)
        given = bool(rng.random() < 0.7)  # explicit chunk sizes, or the even split
        root = int(rng.integers(w))
        data = np.random.default_rng([seed, k])
        xs = [draw(data, dtype, n) for _ in range(w)]
        marker = draw(data, dtype, 1)
        xn = [raw(x) for x in xs]
        store = marker.repeat(n + 2 * GUARD).to(dev)
        t = store[starts[r]:starts[r] + n]
        t.copy_(xs[r])
        use = sizes if given else ring.split_sizes(n, w)
        lo = sum(use[:r])
        op = "avg" if avg else "sum"
        if what == "all_reduce":
            g.all_reduce(t, op=op)
            want = ring.expected_all_reduce(xn, avg, kind)
        elif what == "reduce_scatter":
            g.reduce_scatter(t, sizes if given else None, op=op)
            want = ring.expected_reduce_scatter(xn, sizes if given else None, avg, kind)[r]
        elif what == "reduce_scatter_owner":
            g.reduce_scatter(t, sizes if given else None, op=op, partial_sums=False)
            want = ring.expected_reduce_scatter(xn, sizes if given else None, avg, kind)[r]
        elif what == "all_gather":
            g.all_gather(t, sizes if given else None)
            want = ring.expected_all_gather(xn, use)
        else:
            g.broadcast(t, root=root)
            want = xn[root]
        got = raw(t)
        if what == "reduce_scatter_owner":  # only the owner's chunk is promised
            ok = np.array_equal(bits(got[lo:lo + use[r]]), bits(want[lo:lo + use[r]]))
        else:
            ok = np.array_equal(bits(got), bits(want))
        host, m = bits(raw(store)), bits(raw(marker))[0]
        ok = ok and bool((host[:starts[r]] == m).all()) and bool((host[starts[r] + n:] == m).all())
        if not ok:
            wrong.append((k, what, str(dtype), n, sizes if given else None, starts, op, root))
    g.barrier()
    return wrong


@pytest.mark.parametrize("world,algo,count", [(2, "staged", 120), (2, "ring", 120), (3, "staged", 120), (3, "ring", 120), (4, "staged", 120),
                                              (4, "ring", 120), (6, "staged", 60), (8, "ring", 60)])
def test_seeded_sweep_between_processes(world, algo, count, monkeypatch):
    from tandem_amd import launch

    monkeypatch.setenv("TANDEM_HIP_ALGO", algo)
    monkeypatch.setenv("TANDEM_HIP_STAGING_BYTES", "65536")  # a 40,000-element fp64 tensor takes several passes
    for wrong in launch(sweep, world, 31 + world + SHIFT, count, slot_bytes=16384, gpus=[0] * world, timeout=TIMEOUT):
        assert wrong == []
