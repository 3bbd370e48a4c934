"""K1 / K4 on the GPU, through the C ABI, against the CPU oracle and the fixtures
written by the reference's Python engine. Bit-exact: every comparison is on bit
patterns. Run with -m gpu on an MI355X."""

import numpy as np
import pytest
import torch

from helpers import bits, golden_npz, npz_json, seeded

pytestmark = pytest.mark.gpu

KINDS = {torch.float32: "f32", torch.float64: "f64", torch.float16: "f16", torch.bfloat16: "bf16", torch.int64: "i64",
         torch.int32: "i32", torch.int16: "i16", torch.int8: "i8", torch.uint8: "u8"}


def to_np(t):
    t = t.detach().cpu()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def from_np(a, dtype, dev):
    if dtype in (torch.float16, torch.bfloat16):
        return torch.from_numpy(a.view(np.int16).copy()).view(dtype).to(dev)
    return torch.from_numpy(np.array(a, copy=True)).to(dev)


@pytest.fixture(params=["steps", "one_launch"], autouse=True)
def ring_form(request):
    """Every test here runs with the ring collectives as W-1 launches and as one launch
    (world sizes 2..8 have the second form; views whose phases differ between the ranks take the steps either way)."""
    from tandem_amd._lib import lib

    assert lib().tdm_set_ring_form(0 if request.param == "steps" else 1) == 0
    yield request.param
    assert lib().tdm_set_ring_form(-1) == 0


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return torch.device("cuda", 0)


def inputs(world, n, dtype, seed=0):
    xs = []
    for r in range(world):
        if dtype == torch.int64:
            g = torch.Generator().manual_seed(seed * 1000 + r)
            xs.append(torch.randint(-1000, 1000, (n,), generator=g))
        elif not dtype.is_floating_point:  # the narrower integers over their whole range: most sums wrap around
            g, info = torch.Generator().manual_seed(seed * 1000 + r), torch.iinfo(dtype)
            xs.append(torch.randint(info.min, info.max + 1, (n,), generator=g).to(dtype))
        else:
            xs.append(seeded(seed, r, n).to(dtype))
    return xs


@pytest.mark.parametrize("world", [2, 3, 4])
def test_fixtures_of_the_reference_engine(dev, world):
    """Same inputs as the reference run; outputs must equal the reference's, on
    every rank, for the whole buffer (partial sums included)."""
    from tandem_amd import LocalWorld

    d = golden_npz(f"ring_w{world}.npz")
    lw = LocalWorld(world)
    xs = [d[f"r{r}_in"] for r in range(world)]

    def fresh():
        return [torch.from_numpy(x.copy()).to(dev) for x in xs]

    for op, key in (("sum", "ar_sum"), ("avg", "ar_avg")):
        for algorithm in ("ring", "fold"):
            bufs = fresh()
            lw.all_reduce(bufs, op=op, algorithm=algorithm)
            for r in range(world):
                assert np.array_equal(bits(to_np(bufs[r])), bits(d[f"r{r}_{key}"])), (key, algorithm, r)
    bufs = fresh()
    lw.reduce_scatter(bufs, None, op="avg")
    for r in range(world):
        assert np.array_equal(bits(to_np(bufs[r])), bits(d[f"r{r}_rs_avg_even"]))
    for name, sizes in npz_json(d, "sizes_json").items():
        for op in ("avg", "sum"):
            bufs = fresh()
            mine = lw.reduce_scatter(bufs, sizes, op=op)
            lo = 0
            for r in range(world):
                want = d[f"r{r}_rs_{op}_{name}"]
                assert np.array_equal(bits(to_np(bufs[r])), bits(want)), (name, op, r)
                assert np.array_equal(bits(to_np(mine[r])), bits(want[lo:lo + sizes[r]]))
                lo += sizes[r]
        bufs = fresh()
        lw.all_gather(bufs, sizes)
        for r in range(world):
            assert np.array_equal(bits(to_np(bufs[r])), bits(d[f"r{r}_ag_{name}"])), (name, r)
    bufs = [torch.from_numpy(d[f"r{r}_tiny_in"].copy()).to(dev) for r in range(world)]
    lw.all_reduce(bufs, op="avg")
    for r in range(world):
        assert np.array_equal(bits(to_np(bufs[r])), bits(d[f"r{r}_tiny_ar_avg"]))


def test_fixtures_other_dtypes(dev):
    from tandem_amd import LocalWorld

    d = golden_npz("ring_dtypes_w3.npz")
    lw = LocalWorld(3)
    for kind, dtype in (("f64", torch.float64), ("f16", torch.float16), ("bf16", torch.bfloat16)):
        for op, key in (("sum", "ar_sum"), ("avg", "ar_avg")):
            bufs = [from_np(d[f"r{r}_{kind}_in"].view(np.uint16) if kind != "f64" else d[f"r{r}_{kind}_in"], dtype, dev)
                    for r in range(3)]
            lw.all_reduce(bufs, op=op)
            for r in range(3):
                assert np.array_equal(bits(to_np(bufs[r])), bits(d[f"r{r}_{kind}_{key}"])), (kind, key, r)


@pytest.mark.parametrize("world", [1, 2, 3, 4, 5, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16, torch.bfloat16, torch.int64])
def test_against_oracle(dev, world, dtype):
    """The sizes the reference tests use (tests/test_comm.py:10, test_engine_cuda.py:34
    there) plus sizes that cross the kernel's tile and vector boundaries."""
    from oracle import ring
    from tandem_amd import LocalWorld

    kind = KINDS[dtype]
    lw = LocalWorld(world)
    for n in (0, 1, 5, 64, 1000, 4099, 10_007, 65_536 + 3):
        xs = inputs(world, n, dtype)
        xn = [to_np(x) for x in xs]
        ops = ("sum",) if dtype == torch.int64 else ("sum", "avg")
        for op in ops:
            want = ring.expected_all_reduce(xn, op == "avg", kind)
            for algorithm in ("ring", "fold"):
                bufs = [x.to(dev) for x in xs]
                lw.all_reduce(bufs, op=op, algorithm=algorithm)
                for r in range(world):
                    assert np.array_equal(bits(to_np(bufs[r])), bits(want)), (world, dtype, n, op, algorithm, r)
            sizes = [n // world] * world
            sizes[-1] += n - sum(sizes)
            sizes = sizes[1:] + sizes[:1]  # uneven, and empty when n < world
            bufs = [x.to(dev) for x in xs]
            lw.reduce_scatter(bufs, sizes, op=op)
            want = ring.expected_reduce_scatter(xn, sizes, op == "avg", kind)
            for r in range(world):
                assert np.array_equal(bits(to_np(bufs[r])), bits(want[r])), (world, dtype, n, op, r)
        bufs = [x.to(dev) for x in xs]
        lw.all_gather(bufs, sizes)
        want = ring.expected_all_gather(xn, sizes)
        for r in range(world):
            assert np.array_equal(bits(to_np(bufs[r])), bits(want))


@pytest.mark.parametrize("world", [2, 3, 4, 8])
@pytest.mark.parametrize("dtype", [torch.int32, torch.int16, torch.int8, torch.uint8])
def test_integer_sums_wrap_around(dev, world, dtype):
    """The integer types narrower than 64 bits: sums wrap around as ATen's add_ does (what the
    reference's engines call for them: tandem/comm.py:276-277, tandem/csrc/collectives.cpp:254-256
    there), partial sums included; averaging them is refused. Also from views that start off the
    16-byte grid, where 1-byte elements have up to 15 head elements."""
    from oracle import ring
    from tandem_amd import LocalWorld

    kind = KINDS[dtype]
    lw = LocalWorld(world)
    for n, shift in ((0, 0), (1, 0), (5, 3), (1000, 0), (4099, 1), (65_536 + 3, 0), (65_536 + 35, 13)):
        xs = inputs(world, n, dtype, seed=3)
        xn = [to_np(x) for x in xs]
        def on_device():
            if shift == 0:
                return [x.to(dev) for x in xs]
            backing = [torch.zeros(n + 64, dtype=dtype, device=dev) for _ in xs]
            views = [b[shift:shift + n] for b in backing]
            for v, x in zip(views, xs):
                v.copy_(x)
            return views
        want = ring.expected_all_reduce(xn, False, kind)
        assert np.array_equal(want, sum(x.astype(np.int64) for x in xn).astype(want.dtype) if n else want)  # the order-free modular sum
        for algorithm in ("ring", "fold"):
            bufs = on_device()
            lw.all_reduce(bufs, algorithm=algorithm)
            for r in range(world):
                assert np.array_equal(to_np(bufs[r]), want), (world, dtype, n, shift, algorithm, r)
        sizes = [n // world] * world
        sizes[-1] += n - sum(sizes)
        sizes = sizes[1:] + sizes[:1]
        bufs = on_device()
        lw.reduce_scatter(bufs, sizes)
        want = ring.expected_reduce_scatter(xn, sizes, False, kind)
        for r in range(world):
            assert np.array_equal(to_np(bufs[r]), want[r]), (world, dtype, n, shift, r)
        bufs = on_device()
        lw.all_gather(bufs, sizes)
        want = ring.expected_all_gather(xn, sizes)
        for r in range(world):
            assert np.array_equal(to_np(bufs[r]), want)
    with pytest.raises(ValueError, match="cannot be averaged"):
        lw.all_reduce([torch.zeros(8, dtype=dtype, device=dev) for _ in range(world)], op="avg")


def test_unaligned_views_and_special_values(dev):
    """Views that start 4 bytes into an allocation (no 16-byte alignment, and
    ranks that disagree on their phase), denormals, signed zeros, infinities."""
    from oracle import ring
    from tandem_amd import LocalWorld

    world, n = 4, 9001
    lw = LocalWorld(world)
    special = torch.tensor([0.0, -0.0, 1e-45, -1e-45, 1e-39, 3e38, -3e38, float("inf"), float("-inf"), float("nan"),
                            1.17549435e-38, 2e-38], dtype=torch.float32)
    xs = []
    for r in range(world):
        x = seeded(2, r, n)
        x[r:r + special.numel()] = special
        x[100:110] = 1e-40 * (r + 1)
        xs.append(x)
    xn = [x.numpy() for x in xs]
    # every rank the same distance from a 16-byte boundary (the kernels peel a head and run on vectors), and ranks
    # that disagree (element by element)
    for shifts in ([1, 1, 1, 1], [2, 2, 2, 2], [3, 3, 3, 3], [0, 1, 2, 3], [3, 0, 0, 1]):
        for op in ("sum", "avg"):
            for algorithm in ("ring", "fold"):
                store = [torch.zeros(n + 8, device=dev) for _ in range(world)]
                bufs = [store[r][shifts[r]:shifts[r] + n] for r in range(world)]
                for b, x in zip(bufs, xs):
                    b.copy_(x)
                lw.all_reduce(bufs, op=op, algorithm=algorithm)
                want = ring.expected_all_reduce(xn, op == "avg")
                for r in range(world):
                    got = to_np(bufs[r])
                    nan = np.isnan(want)
                    assert np.array_equal(np.isnan(got), nan)
                    assert np.array_equal(bits(got)[~nan], bits(want)[~nan]), (shifts, op, algorithm, r)
                    # nothing outside the view was touched
                    assert float(store[r][:shifts[r]].abs().sum()) == 0 and float(store[r][shifts[r] + n:].abs().sum()) == 0


@pytest.mark.parametrize("world", [2, 3, 4])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_nan_and_infinity_in_16_bit_collectives(dev, world, dtype):
    """The stated policy: a NaN result of a 16-bit sum or average is the type's canonical quiet NaN
    (bf16 0x7fc0, f16 0x7e00), whatever the sign and payload of the NaNs that went in; infinities keep
    their sign, inf + -inf is that NaN. Inputs carry NaNs of both signs and several payloads and both
    infinities at different places on different ranks. Every all-reduce result has passed through an
    addition, so it is compared bit for bit with the oracle, NaNs included; a bare reduce_scatter leaves
    chunks no arithmetic touched (their NaNs keep the bits they came with), so there the NaN positions
    and all other bits are compared."""
    from oracle import ring
    from tandem_amd import LocalWorld

    kind = KINDS[dtype]
    canonical = 0x7fc0 if dtype == torch.bfloat16 else 0x7e00
    inf = 0x7f80 if dtype == torch.bfloat16 else 0x7c00
    nans = [canonical, canonical | 0x8000, inf | 1, inf | 0x8001, 0x7fff, 0xffff]
    n = 3 * 2048 + 77
    lw = LocalWorld(world)
    xn = []
    for r in range(world):
        x = to_np(seeded(9, r, n).to(dtype)).copy()
        for k, pattern in enumerate(nans):  # every NaN pattern on every rank, each at a place of its own
            x[(7 * r + 13 * k) % n] = pattern
            x[2048 + world * k + r] = pattern
        x[100 + r] = inf                    # +inf on one rank only
        x[200 + r] = inf | 0x8000           # -inf on one rank only
        x[300] = inf if r % 2 == 0 else inf | 0x8000  # +inf and -inf meet: NaN
        x[301] = inf                        # +inf on every rank: +inf
        xn.append(x)
    for op in ("sum", "avg"):
        want = ring.expected_all_reduce(xn, op == "avg", kind)
        is_nan = (want & 0x7fff) > inf
        assert is_nan.sum() >= 2 * len(nans) and np.all(want[is_nan] == canonical)
        assert is_nan[300] and want[301] == inf and not is_nan[100] and not is_nan[200]
        for algorithm in ("ring", "fold"):
            bufs = [from_np(x, dtype, dev) for x in xn]
            lw.all_reduce(bufs, op=op, algorithm=algorithm)
            for r in range(world):
                assert np.array_equal(to_np(bufs[r]), want), (world, dtype, op, algorithm, r)
        bufs = [from_np(x, dtype, dev) for x in xn]
        lw.reduce_scatter(bufs, None, op=op)
        wants = ring.expected_reduce_scatter(xn, None, op == "avg", kind)
        for r in range(world):
            got, w = to_np(bufs[r]), wants[r]
            nan = (w & 0x7fff) > inf
            assert np.array_equal((got & 0x7fff) > inf, nan), (world, dtype, op, r)
            assert np.array_equal(got[~nan], w[~nan]), (world, dtype, op, r)


@pytest.mark.parametrize("world", [2, 3])
def test_two_byte_elements_off_the_vector_grid(dev, world):
    """bf16 views 1..7 elements past a 16-byte boundary, the same on every rank: up to seven head elements are
    peeled before the vectors start. Reduce-scatter with its partial sums, all-gather and both all-reduces."""
    from oracle import ring
    from tandem_amd import LocalWorld

    lw = LocalWorld(world)
    n = 20_011
    xs = [seeded(7, r, n).to(torch.bfloat16) for r in range(world)]
    xn = [to_np(x) for x in xs]
    for shift in (1, 3, 4, 7):
        def views():
            store = [torch.zeros(n + 16, dtype=torch.bfloat16, device=dev) for _ in range(world)]
            bufs = [st[shift:shift + n] for st in store]
            for b, x in zip(bufs, xs):
                b.copy_(x)
            return store, bufs

        for algorithm in ("ring", "fold"):
            store, bufs = views()
            lw.all_reduce(bufs, op="avg", algorithm=algorithm)
            want = ring.expected_all_reduce(xn, True, "bf16")
            for r in range(world):
                assert np.array_equal(bits(to_np(bufs[r])), bits(want)), (shift, algorithm, r)
                assert float(store[r][:shift].float().abs().sum()) == 0 and float(store[r][shift + n:].float().abs().sum()) == 0
        store, bufs = views()
        lw.reduce_scatter(bufs, None, op="avg")
        want = ring.expected_reduce_scatter(xn, None, True, "bf16")
        for r in range(world):
            assert np.array_equal(bits(to_np(bufs[r])), bits(want[r])), (shift, r)


def test_unit_gather(dev):
    from tandem_amd import LocalWorld

    for world, numel in ((2, 7_087_872), (4, 10_007), (3, 2)):
        lw = LocalWorld(world)
        sizes = [numel // world + (1 if q < numel % world else 0) for q in range(world)]
        shards = [seeded(4, q, sizes[q]).to(dev) for q in range(world)]
        fulls = [torch.full((numel,), -7.0, device=dev) for _ in range(world)]
        lw.unit_gather(fulls, shards, sizes)
        want = torch.cat(shards)
        for f in fulls:
            assert torch.equal(f, want)
    # a shard that already lies in place is left alone
    lw = LocalWorld(2)
    full = torch.arange(10, dtype=torch.float32, device=dev)
    other = torch.full((4,), 5.0, device=dev)
    second = full.clone()
    lw.unit_gather([full, second], [full[:6], other], [6, 4])
    assert torch.equal(full, torch.tensor([0, 1, 2, 3, 4, 5, 5, 5, 5, 5.0], device=dev))
    assert torch.equal(second, full)


@pytest.mark.parametrize("world", [1, 2, 3, 5, 8, 9, 12])
def test_unit_gather_for_every_rank_at_once(dev, world):
    """One launch fills all the ranks' full buffers (up to 8 ranks; beyond, a launch per rank): other element types,
    shards and full buffers that start anywhere in their allocations, an empty shard, and nothing written outside."""
    from tandem_amd import LocalWorld

    lw = LocalWorld(world)
    rng = np.random.default_rng(world)
    for dtype in (torch.float32, torch.bfloat16, torch.int8, torch.float64):
        for numel in (0, 5, 4099, 70_001):
            cuts = np.sort(rng.integers(0, numel + 1, world - 1))
            sizes = np.diff(np.concatenate([[0], cuts, [numel]])).astype(int).tolist()
            if world > 2:
                sizes[1] += sizes[2]
                sizes[2] = 0
            starts = [int(rng.integers(0, 16)) for _ in range(2 * world)]
            data = [torch.from_numpy(rng.integers(-100, 100, m)).to(dtype) for m in sizes]
            shard_store = [torch.full((m + 32,), 9, dtype=dtype, device=dev) for m in sizes]
            shards = [st[starts[q]:starts[q] + sizes[q]] for q, st in enumerate(shard_store)]
            for sh, x in zip(shards, data):
                sh.copy_(x)
            full_store = [torch.full((numel + 32,), 7, dtype=dtype, device=dev) for _ in range(world)]
            fulls = [st[starts[world + r]:starts[world + r] + numel] for r, st in enumerate(full_store)]
            lw.unit_gather(fulls, shards, sizes)
            want = torch.cat(data) if numel else torch.zeros(0, dtype=dtype)
            for r in range(world):
                assert torch.equal(fulls[r].cpu(), want), (world, dtype, numel, sizes, r)
                lo = starts[world + r]
                host = full_store[r].cpu()
                assert bool((host[:lo] == 7).all()) and bool((host[lo + numel:] == 7).all()), (world, dtype, numel, r)
            for q in range(world):
                assert torch.equal(shards[q].cpu(), data[q])


def test_bad_arguments_raise(dev):
    from tandem_amd import LocalWorld, _lib

    lw = LocalWorld(2)
    a, b = torch.zeros(8, device=dev), torch.zeros(8, device=dev)
    with pytest.raises(ValueError):
        lw.reduce_scatter([a, b], [4, 5])
    with pytest.raises(ValueError):
        lw.all_reduce([a, b], op="max")
    with pytest.raises(ValueError):
        lw.all_reduce([a, torch.zeros(8)])  # a CPU tensor: no CPU path
    with pytest.raises(ValueError):
        lw.all_reduce([a, b[::2]])
    with pytest.raises(ValueError):
        lw.all_reduce([a.long(), b.long()], op="avg")
    # overlapping destination and source are refused by the launcher itself
    pairs = (_lib.Pair * 1)()
    pairs[0].dst, pairs[0].src, pairs[0].count = a.data_ptr(), a.data_ptr() + 8, 4
    assert _lib.lib().tdm_k1_reduce_step(pairs, 1, 0, 2, 1, 1, 0, None) == 1
    assert b"overlap" in _lib.lib().tdm_last_error()


def test_full_size_properties(dev):
    """The benchmark's largest case: four ranks x 64 Mi fp32 (256 MiB each). The
    oracle is too slow for all of it, so: every rank ends with the same bits,
    integer-valued inputs sum exactly, a power-of-two scaling of the inputs
    scales the result exactly, and a strided sample is checked against the
    oracle."""
    from oracle import ring
    from tandem_amd import LocalWorld

    world, n = 4, 64 << 20
    lw = LocalWorld(world)
    gens = [torch.Generator(device=dev).manual_seed(10 + r) for r in range(world)]
    xs = [torch.randn(n, device=dev, generator=g) * 1e-2 for g in gens]
    bufs = [x.clone() for x in xs]
    lw.all_reduce(bufs, op="avg", algorithm="ring")
    folded = [x.clone() for x in xs]
    lw.all_reduce(folded, op="avg", algorithm="fold")
    assert torch.equal(bufs[3].view(torch.int32), folded[1].view(torch.int32))  # one launch, same bits
    del folded
    for r in range(1, world):
        assert torch.equal(bufs[0].view(torch.int32), bufs[r].view(torch.int32))
    scaled = [x * 16.0 for x in xs]
    lw.all_reduce(scaled, op="avg")
    assert torch.equal((bufs[0] * 16.0).view(torch.int32), scaled[0].view(torch.int32))
    # a sample of 1 Mi elements per chunk against the oracle
    bounds = ring.chunk_bounds(n, world)
    for c, (lo, hi) in enumerate(bounds):
        sl = slice(lo + 12345, lo + 12345 + (1 << 20))
        sample = [x[sl].cpu().numpy() for x in xs]
        want = ring.fold(sample, c, 0, 1 << 20, True)
        assert np.array_equal(bits(to_np(bufs[0][sl])), bits(want)), c
    del scaled
    ints = [torch.randint(-100, 100, (n,), device=dev, generator=g).float() for g in gens]
    exact = sum(i.double() for i in ints)
    lw.all_reduce(ints, op="sum")
    assert torch.equal(ints[2].double(), exact)


@pytest.mark.parametrize("world", [2, 4])
def test_collectives_replayed_from_a_hip_graph(dev, world):
    """The single-process collectives make no allocation, copy or host wait, so a caller
    may capture them into a HIP graph (a ring pass at a small size is six launches of a
    few microseconds each). Every replay, with eager work and a host wait between the
    replays, must give the eager result's bits."""
    from oracle import ring
    from tandem_amd import LocalWorld

    lw = LocalWorld(world)
    n = 16 * 1024 + 37
    ins = [[seeded(60 + k, r, n) * 1e-2 for r in range(world)] for k in range(4)]
    bufs = [torch.empty(n, device=dev) for _ in range(world)]
    other = [torch.empty(n, device=dev) for _ in range(world)]

    def ring_pass(b):
        lw.reduce_scatter(b, op="avg")
        lw.all_gather(b)

    def fold(b):
        lw.all_reduce(b, "avg", algorithm="fold")

    for run in (ring_pass, fold):
        for b, x in zip(bufs, ins[0]):
            b.copy_(x)
        run(bufs)  # warm-up outside the capture
        torch.cuda.synchronize(dev)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run(bufs)
        for k in range(1, 4):
            want = ring.expected_all_reduce([x.numpy() for x in ins[k]], True)
            for b, o, x in zip(bufs, other, ins[k]):
                b.copy_(x)
                o.copy_(x)
            graph.replay()
            run(other)  # the same call made eagerly, behind the replay on the same stream
            torch.cuda.synchronize(dev)
            for r in range(world):
                assert np.array_equal(bits(bufs[r].cpu().numpy()), bits(want)), (run.__name__, k, r)
                assert torch.equal(bufs[r].view(torch.int32), other[r].view(torch.int32)), (run.__name__, k, r)
