"""A seeded sweep over what the ring collectives of buffer ranks can be handed at once: world
size, element type, length, explicit chunk sizes with empty chunks, views that start anywhere
inside their allocation (every rank at the same distance from a 16-byte boundary, or not), both
forms of the ring and the single-launch all-reduce. Every result bit for bit against the
oracle, and the guard elements around every view untouched. Run with -m gpu."""

import numpy as np
import pytest
import torch

from helpers import bits

pytestmark = pytest.mark.gpu

KINDS = {torch.float32: "f32", torch.float64: "f64", torch.float16: "f16", torch.bfloat16: "bf16", torch.int64: "i64",
         torch.int32: "i32", torch.int16: "i16", torch.int8: "i8", torch.uint8: "u8"}
GUARD = 24  # elements before and after every view


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


def cases(count, seed):
    rng = np.random.default_rng(seed)
    dtypes = list(KINDS)
    for k in range(count):
        world = int(rng.choice([1, 2, 2, 3, 3, 4, 4, 5, 6, 7, 8]))
        dtype = dtypes[int(rng.integers(len(dtypes)))]
        n = int(rng.choice([0, 1, 2, 7, 31, 257, 1000, 4099, 16_385, 70_001])) + int(rng.integers(0, 3))
        cuts = np.sort(rng.integers(0, n + 1, world - 1)) if world > 1 else np.zeros(0, np.int64)
        sizes = np.diff(np.concatenate([[0], cuts, [n]])).astype(int).tolist()
        if rng.random() < 0.3 and world > 1:  # one more rank with nothing: its elements go to another
            i, j = int(rng.integers(world)), int(rng.integers(world))
            if i != j:
                sizes[i] += sizes[j]
                sizes[j] = 0
        same_phase = rng.random() < 0.6
        first = int(rng.integers(0, GUARD))
        starts = [first if same_phase else int(rng.integers(0, GUARD)) for _ in range(world)]
        yield k, world, dtype, n, sizes, starts, int(rng.integers(1 << 30))


@pytest.mark.parametrize("form", ["steps", "one_launch"])
def test_seeded_sweep(form):
    from oracle import ring
    from tandem_amd import LocalWorld
    from tandem_amd._lib import lib

    assert torch.cuda.is_available(), "these tests need the MI355X"
    dev = torch.device("cuda", 0)
    assert lib().tdm_set_ring_form(0 if form == "steps" else 1) == 0
    try:
        for k, world, dtype, n, sizes, starts, seed in cases(600, 20260):
            kind = KINDS[dtype]
            rng = np.random.default_rng(seed)
            xs = [draw(rng, dtype, n) for _ in range(world)]
            xn = [raw(x) for x in xs]
            marker = draw(rng, dtype, 1)

            def place():
                stores, views = [], []
                for r in range(world):
                    st = marker.repeat(n + 2 * GUARD).to(dev)
                    v = st[starts[r]:starts[r] + n]
                    v.copy_(xs[r])
                    stores.append(st)
                    views.append(v)
                return stores, views

            def guards_intact(stores):
                for r, st in enumerate(stores):
                    host = raw(st)
                    m = raw(marker)[0]
                    assert (bits(host[:starts[r]]) == bits(np.array([m]))[0]).all(), (k, "before", r)
                    assert (bits(host[starts[r] + n:]) == bits(np.array([m]))[0]).all(), (k, "after", r)

            lw = LocalWorld(world)
            label = (k, world, str(dtype), n, sizes, starts)
            for op in (("sum", "avg") if dtype.is_floating_point else ("sum",)):
                avg = op == "avg"
                want = ring.expected_all_reduce(xn, avg, kind)
                for algorithm in ("ring", "fold"):
                    stores, views = place()
                    lw.all_reduce(views, op=op, algorithm=algorithm)
                    for r in range(world):
                        assert np.array_equal(bits(raw(views[r])), bits(want)), (label, op, algorithm, r)
                    guards_intact(stores)
                stores, views = place()
                mine = lw.reduce_scatter(views, sizes, op=op)
                want_rs = ring.expected_reduce_scatter(xn, sizes, avg, kind)
                lo = 0
                for r in range(world):
                    assert np.array_equal(bits(raw(views[r])), bits(want_rs[r])), (label, op, "reduce_scatter", r)
                    assert mine[r].numel() == sizes[r]
                    if sizes[r]:  # (an empty view has no address)
                        assert mine[r].data_ptr() == views[r].data_ptr() + lo * views[r].element_size()
                    lo += sizes[r]
                guards_intact(stores)
            stores, views = place()
            lw.all_gather(views, sizes)
            want = ring.expected_all_gather(xn, sizes)
            for r in range(world):
                assert np.array_equal(bits(raw(views[r])), bits(want)), (label, "all_gather", r)
            guards_intact(stores)
    finally:
        assert lib().tdm_set_ring_form(-1) == 0
