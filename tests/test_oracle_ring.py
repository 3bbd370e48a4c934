"""The ring oracle against the reference engine's own outputs (tests/golden/ring_*.npz),
against an independent message-by-message simulator, and against what the
mathematics fixes (n = 2, integer-valued inputs, linearity in a power of two)."""

import numpy as np
import pytest

from oracle import ring

from helpers import bits, golden_npz, npz_json, seeded


def rank_arrays(npz, world, key):
    return [npz[f"r{r}_{key}"] for r in range(world)]


@pytest.mark.parametrize("world", [2, 3, 4])
def test_all_reduce_matches_reference_engine(world):
    d = golden_npz(f"ring_w{world}.npz")
    xs = rank_arrays(d, world, "in")
    for avg, key in ((False, "ar_sum"), (True, "ar_avg")):
        want = ring.expected_all_reduce(xs, avg)
        for r in range(world):
            assert np.array_equal(bits(d[f"r{r}_{key}"]), bits(want)), (world, key, r)
    tiny = rank_arrays(d, world, "tiny_in")  # fewer elements than ranks
    want = ring.expected_all_reduce(tiny, True)
    for r in range(world):
        assert np.array_equal(bits(d[f"r{r}_tiny_ar_avg"]), bits(want))


@pytest.mark.parametrize("world", [2, 3, 4])
def test_reduce_scatter_whole_buffers_match_reference_engine(world):
    """Not only the owner's chunk: the partial sums left in the other chunks too."""
    d = golden_npz(f"ring_w{world}.npz")
    xs = rank_arrays(d, world, "in")
    cases = npz_json(d, "sizes_json")
    want = ring.expected_reduce_scatter(xs, None, True)
    for r in range(world):
        assert np.array_equal(bits(d[f"r{r}_rs_avg_even"]), bits(want[r]))
    for name, sizes in cases.items():
        for avg, tag in ((True, "avg"), (False, "sum")):
            want = ring.expected_reduce_scatter(xs, sizes, avg)
            for r in range(world):
                assert np.array_equal(bits(d[f"r{r}_rs_{tag}_{name}"]), bits(want[r])), (world, name, tag, r)
        want = ring.expected_all_gather(xs, sizes)
        for r in range(world):
            assert np.array_equal(bits(d[f"r{r}_ag_{name}"]), bits(want)), (world, name, r)


def test_other_dtypes_match_reference_engine():
    d = golden_npz("ring_dtypes_w3.npz")
    for kind in ("f64", "f16", "bf16"):
        xs = [d[f"r{r}_{kind}_in"] for r in range(3)]
        if kind != "f64":
            xs = [x.view(np.uint16) for x in xs]
        for avg, key in ((False, "ar_sum"), (True, "ar_avg")):
            want = ring.expected_all_reduce(xs, avg, kind)
            for r in range(3):
                got = d[f"r{r}_{kind}_{key}"]
                assert np.array_equal(bits(got), bits(want)), (kind, key, r)


@pytest.mark.parametrize("world", [1, 2, 3, 4, 5, 7])
@pytest.mark.parametrize("kind", ["f32", "f64", "bf16", "f16"])
def test_closed_form_equals_message_simulator(world, kind):
    n = 1003
    xs = [seeded(5, r, n).numpy() for r in range(world)]
    if kind == "f64":
        xs = [x.astype(np.float64) * 1.0000001 for x in xs]
    elif kind == "f16":
        xs = [x.astype(np.float16).view(np.uint16) for x in xs]
    elif kind == "bf16":
        xs = [(x.view(np.uint32) >> 16).astype(np.uint16) for x in xs]
    sizes = [0] * world
    sizes[0] = 7
    sizes[-1] += n - 7
    for avg in (False, True):
        sim = ring.simulate(xs, "all_reduce", None, avg, kind, piece_elems=61)
        want = ring.expected_all_reduce(xs, avg, kind)
        for r in range(world):
            assert np.array_equal(bits(sim[r]), bits(want)), (world, kind, avg, r)
        if world == 1:
            continue
        for sz in (None, sizes):
            sim = ring.simulate(xs, "reduce_scatter", sz, avg, kind, piece_elems=16)
            want = ring.expected_reduce_scatter(xs, sz, avg, kind)
            for r in range(world):
                assert np.array_equal(bits(sim[r]), bits(want[r])), (world, kind, avg, r)
    sim = ring.simulate(xs, "all_gather", sizes if world > 1 else None, False, kind)
    want = ring.expected_all_gather(xs, sizes if world > 1 else None)
    for r in range(world):
        assert np.array_equal(bits(sim[r]), bits(want))


def test_two_ranks_is_half_plus_half():
    xs = [seeded(0, r, 4099).numpy() for r in range(2)]
    want = xs[0] / np.float32(2) + xs[1] / np.float32(2)
    assert np.array_equal(bits(ring.expected_all_reduce(xs, True)), bits(want))


@pytest.mark.parametrize("world", [2, 3, 4])
def test_integer_valued_inputs_sum_exactly(world):
    # the reference tests' own expectation (tests/test_comm.py:23-26 there)
    import torch

    for n in (0, 1, 5, 64, 1000, 4099):
        xs = []
        for r in range(world):
            g = torch.Generator().manual_seed(r)
            xs.append(torch.randint(-100, 100, (n,), generator=g).to(torch.float32).numpy())
        want = sum(x.astype(np.float64) for x in xs) if n else np.zeros(0)
        got = ring.expected_all_reduce(xs, False)
        assert np.array_equal(got.astype(np.float64), want)
        xi = [x.astype(np.int64) for x in xs]
        assert np.array_equal(ring.expected_all_reduce(xi, False, "i64"), want.astype(np.int64))


@pytest.mark.parametrize("kind", ["i32", "i16", "i8", "u8"])
@pytest.mark.parametrize("world", [2, 3, 4, 8])
def test_narrow_integer_sums_wrap_around(kind, world):
    """Full-range inputs, so most sums overflow. Two independent statements of the result: the
    sum in 64 bits reduced to the element's width (order-free), and ATen's add_ applied in the
    ring's order on CPU tensors, which is what the reference's engines do for these dtypes
    (tandem/comm.py:276-277; tandem/csrc/collectives.cpp:254-256)."""
    import torch

    dt = ring.KINDS[kind]
    info = np.iinfo(dt)
    rng = np.random.default_rng(world * 10 + len(kind))
    for n in (0, 1, 5, 1000, 4099):
        xs = [rng.integers(info.min, int(info.max) + 1, n, dtype=np.int64).astype(dt) for _ in range(world)]
        modular = sum(x.astype(np.int64) for x in xs).astype(dt) if n else np.zeros(0, dt)  # astype keeps the low bits
        got = ring.expected_all_reduce(xs, False, kind)
        assert got.dtype == dt and np.array_equal(got, modular)
        sizes = [n // world] * world
        sizes[0] += n - sum(sizes)
        outs = ring.expected_reduce_scatter(xs, sizes, False, kind)
        sim = ring.simulate(xs, "reduce_scatter", sizes, False, kind, piece_elems=7)
        lo = 0
        for c, size in enumerate(sizes):
            acc = torch.from_numpy(xs[(c + 1) % world][lo:lo + size].copy())
            for k in range(2, world + 1):
                r = (c + k) % world
                acc = torch.from_numpy(xs[r][lo:lo + size].copy()).add_(acc)  # into.add_(slot) on rank r
                assert np.array_equal(outs[r][lo:lo + size], acc.numpy()), (kind, world, n, c, k)
            lo += size
        for r in range(world):
            assert np.array_equal(outs[r], sim[r])
    with pytest.raises(ValueError):
        ring.expected_all_reduce([np.zeros(4, dt)] * 2, True, kind)


def test_power_of_two_scaling_commutes_with_the_ring():
    # scaling every input by 2^k scales every partial sum exactly (no overflow here)
    xs = [seeded(9, r, 777).numpy() for r in range(4)]
    a = ring.expected_reduce_scatter(xs, None, True)
    b = ring.expected_reduce_scatter([x * np.float32(8) for x in xs], None, True)
    for r in range(4):
        assert np.array_equal(bits(a[r] * np.float32(8)), bits(b[r]))


def test_world_three_divides_truly():
    # x / 3 and x * (1/3) differ on about a third of fp32 values; the fixtures hold the former
    d = golden_npz("ring_w3.npz")
    x = d["r0_in"]
    recip = x * (np.float32(1) / np.float32(3))
    true = x / np.float32(3)
    assert (bits(recip) != bits(true)).mean() > 0.1
    lo, hi = ring.chunk_bounds(x.shape[0], 3)[2]  # chunk 2 on rank 0 holds rank 0's bare x / 3
    got = d["r0_rs_avg_even"][lo:hi]
    assert np.array_equal(bits(got), bits(true[lo:hi]))


def test_bad_sizes_are_rejected():
    with pytest.raises(ValueError):
        ring.chunk_bounds(10, 3, [5, 5])
    with pytest.raises(ValueError):
        ring.chunk_bounds(10, 2, [5, 6])


def test_split_sizes_match_reference():
    from helpers import golden_json

    for key, want in golden_json("plans.json")["split_sizes"].items():
        n, w = map(int, key.split("/"))
        assert ring.split_sizes(n, w) == want
