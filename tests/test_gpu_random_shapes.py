"""A seeded sweep over what the ring collectives of buffer ranks can be handed at once: world
size, element type, length, explicit chunk sizes with empty chunks, views that start anywhere
inside their allocation (every rank at the same distance from a 16-byte boundary, or not), both
forms of the ring and the single-launch all-reduce. Every result bit for bit against the
oracle, and the guard elements around every view untouched. Run with -m gpu."""

import os

import numpy as np
import pytest
import torch

from helpers import bits

pytestmark = pytest.mark.gpu
SHIFT = int(os.environ.get("TANDEM_SWEEP_SEED", "0"))  # added to every sweep's seed: other cases of the same kinds

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
        for k, world, dtype, n, sizes, starts, seed in cases(600, 20260 + SHIFT):
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


def bucket_cases(count, seed):
    rng = np.random.default_rng(seed)
    dtypes = list(KINDS)
    for k in range(count):
        world = int(rng.integers(1, 9))
        dtype = dtypes[int(rng.integers(len(dtypes)))]
        numels = [int(rng.choice([1, 2, 3, 7, 33, 255, 1024, 4097, 9000])) + int(rng.integers(0, 2)) for _ in range(int(rng.integers(1, 13)))]
        order = rng.permutation(len(numels)).tolist()
        buckets, at = [], 0
        while at < len(order):
            take = int(rng.integers(1, 5))
            buckets.append(order[at:at + take])
            at += take
        starts = [[int(rng.integers(0, GUARD)) for _ in numels] for _ in range(world)]  # every tensor of every rank at a phase of its own
        yield k, world, dtype, numels, buckets, starts, bool(rng.random() < 0.4), bool(rng.random() < 0.5), int(rng.integers(1 << 30))


def test_seeded_sweep_of_bucket_tables():
    """The table-driven fold (DDP's buckets in one launch): random tensor lists cut into random buckets, world sizes
    1..8, every element type, tensors that start anywhere in their allocations, in place or into other tensors, through
    the table on the device and through the entry point that allocates nothing. Per bucket: the ring all-reduce of the
    flattened bucket."""
    from oracle import ring
    from tandem_amd import LocalWorld

    assert torch.cuda.is_available(), "these tests need the MI355X"
    dev = torch.device("cuda", 0)
    for k, world, dtype, numels, buckets, starts, elsewhere, static, seed in bucket_cases(150, 77 + SHIFT):
        kind = KINDS[dtype]
        rng = np.random.default_rng(seed)
        grads = [[draw(rng, dtype, n) for n in numels] for _ in range(world)]
        marker = draw(rng, dtype, 1)

        def place(fill):
            stores, views = [], []
            for r in range(world):
                row_s, row_v = [], []
                for i, n in enumerate(numels):
                    st = marker.repeat(n + 2 * GUARD).to(dev)
                    v = st[starts[r][i]:starts[r][i] + n]
                    if fill:
                        v.copy_(grads[r][i])
                    row_s.append(st)
                    row_v.append(v)
                stores.append(row_s)
                views.append(row_v)
            return stores, views

        stores, views = place(True)
        out_stores, outs = place(False) if elsewhere else (stores, views)
        table = LocalWorld(world).bucket_table(views, buckets, outs if elsewhere else None)
        average = dtype.is_floating_point
        (table.run_static if static else table.run)(average=average)
        label = (k, world, str(dtype), numels, buckets, elsewhere, static)
        for b in buckets:
            flat = [np.concatenate([raw(grads[r][i]) for i in b]) for r in range(world)]
            want = ring.expected_all_reduce(flat, average, kind)
            off = 0
            for i in b:
                for r in range(world):
                    assert np.array_equal(bits(raw(outs[r][i])), bits(want[off:off + numels[i]])), (label, i, r)
                    if elsewhere:
                        assert np.array_equal(bits(raw(views[r][i])), bits(raw(grads[r][i]))), (label, "source changed", i, r)
                off += numels[i]
        m = bits(raw(marker))[0]
        for r in range(world):
            for i, n in enumerate(numels):
                host = bits(raw(out_stores[r][i]))
                lo = starts[r][i]
                assert (host[:lo] == m).all() and (host[lo + n:] == m).all(), (label, "guard", i, r)


def test_seeded_sweep_of_adamw_shards():
    """K3 on shards of random length whose parameter and gradient views start at phases of their own
    (0..3 elements past a 16-byte boundary), random hyper-parameters (both lerp branches, with and
    without decay), a few steps each: parameters and both moments bit for bit the oracle's."""
    from oracle.adamw import AdamW as Oracle
    from tandem_amd import ShardedAdamW

    assert torch.cuda.is_available(), "these tests need the MI355X"
    dev = torch.device("cuda", 0)
    rng = np.random.default_rng(4242 + SHIFT)
    for k in range(80):
        n = int(rng.choice([0, 1, 3, 4, 5, 127, 128, 129, 1000, 4097, 33_333, 70_000])) + int(rng.integers(0, 2))
        kw = dict(lr=float(10 ** rng.uniform(-4, -1.5)), betas=(float(rng.choice([0.0, 0.3, 0.5, 0.9])), float(rng.choice([0.7, 0.95, 0.999]))),
                  eps=float(rng.choice([1e-8, 1e-6])), weight_decay=float(rng.choice([0.0, 0.01, 0.1, 0.5])))
        ps, gs = int(rng.integers(0, 4)), int(rng.integers(0, 4))
        ours, ref = ShardedAdamW(**kw), Oracle(**kw)
        p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
        pstore = torch.full((n + 8,), 7.0, device=dev)
        p = pstore[ps:ps + n]
        p.copy_(torch.from_numpy(p0))
        pn = p0.copy()
        steps = int(rng.integers(1, 5))
        for _ in range(steps):
            g0 = (rng.standard_normal(n) * 1e-3).astype(np.float32)
            g0[: n // 7] = 0.0
            gstore = torch.full((n + 8,), -3.0, device=dev)
            g = gstore[gs:gs + n]
            g.copy_(torch.from_numpy(g0))
            ours.update("k", p, g)
            ref.update("k", pn, g0)
            assert np.array_equal(g.cpu().numpy(), g0) and float(gstore[:gs].sum()) == -3.0 * gs  # the gradient is only read
        label = (k, n, kw, ps, gs, steps)
        assert np.array_equal(bits(p.cpu().numpy()), bits(pn)), label
        if n:
            _, m, v = ours.state["k"]
            assert np.array_equal(bits(m.cpu().numpy()), bits(ref.state["k"][1])), label
            assert np.array_equal(bits(v.cpu().numpy()), bits(ref.state["k"][2])), label
        host = pstore.cpu().numpy()
        assert (host[:ps] == 7.0).all() and (host[ps + n:] == 7.0).all(), label


def test_seeded_sweep_of_zero2_steps():
    """ZeRO-2 for a whole group on one GPU over random parameter lists, world sizes 1..8 and bucket sizes: the three
    ways through a step (ring steps + AdamW + ring all-gather; the fold + AdamW writing every copy; everything in one
    launch) must leave the same bits in every rank's parameters and optimizer state, two steps running."""
    from tandem_amd.local import LocalZeRO2

    assert torch.cuda.is_available(), "these tests need the MI355X"
    dev = torch.device("cuda", 0)
    rng = np.random.default_rng(9 + SHIFT)
    kw = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    for k in range(40):
        world = int(rng.integers(1, 9))
        numels = [int(rng.choice([1, 2, 5, 64, 257, 1024, 3001, 8192])) + int(rng.integers(0, 2)) for _ in range(int(rng.integers(1, 10)))]
        bucket_bytes = int(rng.choice([64, 1024, 4096, 1 << 20]))
        n = sum(numels)
        zs = [LocalZeRO2(world, numels, dev, bucket_bytes=bucket_bytes, **kw) for _ in range(3)]
        p0 = torch.from_numpy((rng.standard_normal(n) * 0.02).astype(np.float32)).to(dev)
        for z in zs:
            for b in z.bufs:
                b.copy_(p0)
        for step in range(2):
            for r in range(world):
                g = torch.from_numpy((rng.standard_normal(n) * 1e-3).astype(np.float32)).to(dev)
                for z in zs:
                    z.staging[r].copy_(g)
            zs[0].reduce_grads("ring"); zs[0].step(fused_gather=False); zs[0].zero_grad()
            zs[1].reduce_grads("fold"); zs[1].step(); zs[1].zero_grad()
            zs[2].reduce_and_step(); zs[2].zero_grad()
        label = (k, world, numels, bucket_bytes)
        for other in zs[1:]:
            for r in range(world):
                assert torch.equal(zs[0].bufs[r].view(torch.int32), other.bufs[r].view(torch.int32)), label
                if zs[0].grad_shards[r].numel():
                    for i in (1, 2):
                        assert torch.equal(zs[0].opts[r].state["flat"][i].view(torch.int32), other.opts[r].state["flat"][i].view(torch.int32)), (label, r, i)
        for r in range(1, world):
            assert torch.equal(zs[2].bufs[0].view(torch.int32), zs[2].bufs[r].view(torch.int32)), label


def _raw_any(t):
    t = t.detach().cpu()
    return t.view(torch.int16).numpy().view(np.uint16).copy() if t.element_size() == 2 else t.numpy().copy()


def test_seeded_sweep_of_adamw_shards_of_other_dtypes():
    """The same sweep over float64, bfloat16 and float16 shards (tdm_k3_adamw_typed): random lengths, parameter,
    gradient and state views at phases of their own (so that some launches peel to the cache line, some to the vector,
    some go element by element), random hyper-parameters with an eps and gradients that the 16-bit types can hold, now
    and then with copies written in the same pass: parameters, both moments and every copy bit for bit the oracle's."""
    from oracle.adamw import AdamW as Oracle
    from tandem_amd import ShardedAdamW

    assert torch.cuda.is_available(), "these tests need the MI355X"
    dev = torch.device("cuda", 0)
    rng = np.random.default_rng(777 + SHIFT)
    kinds = {torch.float64: None, torch.bfloat16: "bf16", torch.float16: "f16"}
    for k in range(90):
        dtype = [torch.float64, torch.bfloat16, torch.float16][k % 3]
        per_line = 128 // torch.empty(0, dtype=dtype).element_size()
        n = int(rng.choice([1, 3, 7, 8, 9, 63, 64, 65, 127, 1000, 4097, 33_333])) + int(rng.integers(0, 2))
        kw = dict(lr=float(10 ** rng.uniform(-4, -2)), betas=(float(rng.choice([0.0, 0.3, 0.5, 0.9])), float(rng.choice([0.7, 0.95, 0.999]))),
                  eps=float(rng.choice([1e-4, 1e-3])), weight_decay=float(rng.choice([0.0, 0.01, 0.1])))
        ncopies = int(rng.choice([0, 0, 1, 3]))
        same = bool(rng.integers(0, 2))  # every stream at one phase, or phases of their own
        phases = [int(rng.integers(0, per_line))] * (4 + ncopies) if same else [int(rng.integers(0, per_line)) for _ in range(4 + ncopies)]
        pad = 2 * per_line
        stores = [torch.full((n + 2 * pad,), -7.0, dtype=dtype, device=dev) for _ in range(4 + ncopies)]
        views = [s_[pad + ph:pad + ph + n] for s_, ph in zip(stores, phases)]
        p0 = torch.from_numpy(rng.standard_normal(n) * 0.05).to(dtype)
        views[0].copy_(p0)
        ours, ref = ShardedAdamW(**kw), Oracle(**kw, kind=kinds[dtype])
        ours.state["k"] = [0.0, views[2].zero_(), views[3].zero_()]
        pn = _raw_any(p0)
        steps = int(rng.integers(1, 4))
        for _ in range(steps):
            g0 = torch.from_numpy(rng.standard_normal(n) * 3e-2).to(dtype)
            g0[: n // 7] = 0.0
            views[1].copy_(g0)
            ours.update("k", views[0], views[1], views[4:])
            ref.update("k", pn, _raw_any(g0))
        label = (k, str(dtype), n, kw, phases, ncopies, steps)
        assert np.array_equal(bits(_raw_any(views[0])), bits(pn)), label
        assert np.array_equal(bits(_raw_any(views[2])), bits(ref.state["k"][1])), label
        assert np.array_equal(bits(_raw_any(views[3])), bits(ref.state["k"][2])), label
        for c in views[4:]:
            assert np.array_equal(bits(_raw_any(c)), bits(pn)), label
        for s_, ph in zip(stores, phases):
            assert float((s_[:pad + ph].double() + 7.0).abs().sum()) == 0 and float((s_[pad + ph + n:].double() + 7.0).abs().sum()) == 0, label


def test_seeded_sweep_of_zero2_steps_of_other_dtypes():
    """The three ways through a ZeRO-2 step over float64, bfloat16 and float16 models, random parameter lists, world
    sizes 1..8 and bucket sizes: ring steps + AdamW + all-gather, the fold + AdamW writing every copy, and everything in
    one launch (tdm_k23_zero2_step_typed) must leave the same bits in every rank's parameters and optimizer state."""
    from tandem_amd.local import LocalZeRO2

    assert torch.cuda.is_available(), "these tests need the MI355X"
    dev = torch.device("cuda", 0)
    rng = np.random.default_rng(31 + SHIFT)
    kw = dict(lr=1e-3, betas=(0.9, 0.95), eps=1e-4, weight_decay=0.1)
    for k in range(36):
        dtype = [torch.float64, torch.bfloat16, torch.float16][k % 3]
        world = int(rng.integers(1, 9))
        numels = [int(rng.choice([1, 2, 5, 64, 257, 1024, 3001, 8192])) + int(rng.integers(0, 2)) for _ in range(int(rng.integers(1, 10)))]
        bucket_bytes = int(rng.choice([64, 1024, 4096, 1 << 20]))
        n = sum(numels)
        zs = [LocalZeRO2(world, numels, dev, bucket_bytes=bucket_bytes, dtype=dtype, **kw) for _ in range(3)]
        p0 = torch.from_numpy(rng.standard_normal(n) * 0.05).to(dtype).to(dev)
        for z in zs:
            for b in z.bufs:
                b.copy_(p0)
        for step in range(2):
            for r in range(world):
                g = torch.from_numpy(rng.standard_normal(n) * 3e-2).to(dtype).to(dev)
                for z in zs:
                    z.staging[r].copy_(g)
            zs[0].reduce_grads("ring"); zs[0].step(fused_gather=False); zs[0].zero_grad()
            zs[1].reduce_grads("fold"); zs[1].step(); zs[1].zero_grad()
            zs[2].reduce_and_step(); zs[2].zero_grad()
        label = (k, str(dtype), world, numels, bucket_bytes)
        for other in zs[1:]:
            for r in range(world):
                assert np.array_equal(bits(_raw_any(zs[0].bufs[r])), bits(_raw_any(other.bufs[r]))), label
                if zs[0].grad_shards[r].numel():
                    for i in (1, 2):
                        assert np.array_equal(bits(_raw_any(zs[0].opts[r].state["flat"][i])), bits(_raw_any(other.opts[r].state["flat"][i]))), (label, r, i)
        for r in range(1, world):
            assert np.array_equal(bits(_raw_any(zs[2].bufs[0])), bits(_raw_any(zs[2].bufs[r]))), label
        assert np.isfinite(zs[2].bufs[0].double().cpu().numpy()).all(), label
