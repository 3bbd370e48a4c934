"""The ZeRO-2 step with every rank on one GPU (LocalZeRO2) against the oracle:
per-bucket ring reduce-scatter with the reference's bucket_sizes, add into the
gradient shard, sharded AdamW, all-gather. Bit-exact at a reduced size; at the
benchmark's full size (85,842,432 parameters, world 4) through properties and a
sampled comparison. Run with -m gpu."""

import math

import numpy as np
import pytest
import torch

from helpers import bits, golden_json, seeded

pytestmark = pytest.mark.gpu
KW = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)


def oracle_zero2(world, numels, bucket_bytes, params0, grads_per_step):
    """The same step written with the oracle only: numpy buffers per rank."""
    from oracle import ring
    from oracle.adamw import AdamW
    from tandem_amd.buckets import FlatLayout, zero_buckets

    lay = [FlatLayout(numels, world, r) for r in range(world)]
    bufs = [params0.copy() for _ in range(world)]
    opts = [AdamW(**KW) for _ in range(world)]
    for grads in grads_per_step:
        shards = [np.zeros(l.hi - l.lo, np.float32) for l in lay]
        for a, b, _ in zero_buckets(numels, 4, bucket_bytes):
            sizes = lay[0].bucket_sizes(a, b)
            outs = ring.expected_reduce_scatter([g[a:b] for g in grads], sizes, True)
            lo = a
            for c, m in enumerate(sizes):
                if m:
                    at = lo - lay[c].lo
                    shards[c][at:at + m] += outs[c][lo - a:lo - a + m]
                lo += m
        for r in range(world):
            opts[r].update("flat", bufs[r][lay[r].lo:lay[r].hi], shards[r])
        full = ring.expected_all_gather(bufs, lay[0].sizes)
        bufs = [full.copy() for _ in range(world)]
    return bufs, opts


@pytest.mark.parametrize("algorithm", ["fold", "ring", "fused"])
@pytest.mark.parametrize("world", [2, 4, 3])
def test_small_model_bit_exact_with_oracle(world, algorithm):
    from tandem_amd.local import LocalZeRO2

    dev = torch.device("cuda", 0)
    plan = golden_json("plans.json")
    numels = [math.prod(s) for _, s in plan["small_params"]]
    n = sum(numels)
    p0 = (seeded(1, 0, n) * 0.02).numpy()
    steps = 5
    grads = [[(seeded(10 + s, r, n) * 1e-3).numpy() for r in range(world)] for s in range(steps)]
    for g in grads[0]:
        g[:7] = [0.0, -0.0, 1e-45, -1e-45, 0.0, -0.0, 0.0]  # signed zeros survive only as the reference's add_ leaves them
    z = LocalZeRO2(world, numels, dev, bucket_bytes=4 << 10, **KW)
    for b in z.bufs:
        b.copy_(torch.from_numpy(p0))
    for s in range(steps):
        for r in range(world):
            z.staging[r].copy_(torch.from_numpy(grads[s][r]))
        if algorithm == "fused":  # reduce-scatter, add, AdamW and all-gather as one launch
            assert z._step_table is not None and z._shards_zero
            z.reduce_and_step()
        else:
            z.reduce_grads(algorithm)
            z.step(fused_gather=algorithm == "fold")  # the update writes every rank's copy, or a ring all-gather follows
        z.zero_grad()
    want, opts = oracle_zero2(world, numels, 4 << 10, p0, grads)
    for r in range(world):
        assert np.array_equal(bits(z.bufs[r].cpu().numpy()), bits(want[r])), (world, r)
        assert np.array_equal(bits(z.opts[r].state["flat"][1].cpu().numpy()), bits(opts[r].state["flat"][1]))
        assert np.array_equal(bits(z.opts[r].state["flat"][2].cpu().numpy()), bits(opts[r].state["flat"][2]))


@pytest.mark.parametrize("one_allocation", [False, True])
@pytest.mark.parametrize("algorithm", ["fold", "ring", "fused"])
def test_shards_that_start_off_the_16_byte_grid(algorithm, one_allocation):
    """World 3 over a flat buffer of odd length: tensor_split puts the second and third shard
    1 and 2 elements past a multiple of four (tandem/zero.py:29-54 there: shards start
    anywhere). Gradient shards and optimizer state sit at their shard's phase, so every
    launch peels a head and runs on vectors; five steps against the oracle, bit for bit."""
    from tandem_amd.local import LocalZeRO2

    dev = torch.device("cuda", 0)
    world, numels = 3, [4099, 10_007, 33, 5001, 1, 12_288, 782]
    n = sum(numels)
    z = LocalZeRO2(world, numels, dev, bucket_bytes=16 << 10, one_allocation=one_allocation, **KW)
    assert sorted(l.lo % 4 for l in z.layouts) == [0, 1, 2], [l.lo for l in z.layouts]
    if one_allocation:  # every buffer inside the one pool, none overlapping
        lo, hi = z._pool.data_ptr(), z._pool.data_ptr() + 4 * z._pool.numel()
        parts = z.bufs + z.staging + z.grad_shards + [t for o in z.opts for t in o.state["flat"][1:]]
        spans = sorted((t.data_ptr(), t.data_ptr() + 4 * t.numel()) for t in parts)
        assert spans[0][0] >= lo and spans[-1][1] <= hi and all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
    for r, l in enumerate(z.layouts):  # the layout this test is about
        phase = z.bufs[r][l.lo:l.hi].data_ptr() % 128
        assert phase == 4 * (l.lo % 32)
        assert z.grad_shards[r].data_ptr() % 128 == phase
        assert z.opts[r].state["flat"][1].data_ptr() % 128 == z.opts[r].state["flat"][2].data_ptr() % 128 == phase
    p0 = (seeded(2, 0, n) * 0.02).numpy()
    steps = 5
    grads = [[(seeded(20 + s, r, n) * 1e-3).numpy() for r in range(world)] for s in range(steps)]
    for b in z.bufs:
        b.copy_(torch.from_numpy(p0))
    for s in range(steps):
        for r in range(world):
            z.staging[r].copy_(torch.from_numpy(grads[s][r]))
        if algorithm == "fused":
            assert z._step_table is not None and z._shards_zero
            z.reduce_and_step()
        else:
            z.reduce_grads(algorithm)
            z.step(fused_gather=algorithm == "fold")
        z.zero_grad()
    want, opts = oracle_zero2(world, numels, 16 << 10, p0, grads)
    for r in range(world):
        assert np.array_equal(bits(z.bufs[r].cpu().numpy()), bits(want[r])), r
        assert np.array_equal(bits(z.opts[r].state["flat"][1].cpu().numpy()), bits(opts[r].state["flat"][1]))
        assert np.array_equal(bits(z.opts[r].state["flat"][2].cpu().numpy()), bits(opts[r].state["flat"][2]))


def _raw(t):
    t = t.detach().cpu()
    return t.view(torch.int16).numpy().view(np.uint16).copy() if t.element_size() == 2 else t.numpy().copy()


@pytest.mark.parametrize("algorithm", ["fold", "ring", "fused"])
@pytest.mark.parametrize("world", [2, 4, 3])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float64])
def test_other_shard_dtypes_bit_exact_with_oracle(dtype, world, algorithm):
    """The ZeRO-2 step over bfloat16 and float64 models (the reference's classes and its seven-operation AdamW take
    any floating dtype, tandem/zero.py:69-170, tandem/optim.py:28-37): per-bucket ring reduce-scatter in the type's own
    rounding, the add into the zeroed gradient shard, the typed AdamW, the all-gather; by ring steps, by the fold and as
    ONE launch (tdm_k23_zero2_step_typed). Four steps against the oracle, bit for bit in every rank's parameters and in
    both moments; world 3 puts the shards off the 16-byte grid."""
    from oracle import ring
    from oracle.adamw import AdamW
    from tandem_amd.buckets import FlatLayout, zero_buckets
    from tandem_amd.local import LocalZeRO2

    dev = torch.device("cuda", 0)
    kind = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float64: "f64"}[dtype]
    es = 8 if kind == "f64" else 2
    numels = [4099, 10_007, 33, 5001, 1, 12_288, 782]
    n = sum(numels)
    steps = 4
    kw = dict(lr=1e-3, betas=(0.9, 0.95), eps=1e-6, weight_decay=0.1)
    p0 = (seeded(3, 0, n).double() * 0.02).to(dtype)
    scale = 1e-3 if kind != "f16" else 2e-2  # float16 holds the squares of these; smaller ones only as subnormals or zero
    grads = [[(seeded(30 + s, r, n).double() * scale).to(dtype) for r in range(world)] for s in range(steps)]
    for g in grads[0]:
        g[:4] = torch.tensor([0.0, -0.0, 1e-30, -1e-30], dtype=torch.float64).to(dtype)
    z = LocalZeRO2(world, numels, dev, bucket_bytes=16 << 10, dtype=dtype, **kw)
    assert z.bufs[0].dtype == dtype and z.opts[0].state["flat"][1].dtype == dtype
    for b in z.bufs:
        b.copy_(p0)
    for s in range(steps):
        for r in range(world):
            z.staging[r].copy_(grads[s][r])
        if algorithm == "fused":
            assert z._step_table is not None and z._shards_zero
            z.reduce_and_step()
        else:
            z.reduce_grads(algorithm)
            z.step(fused_gather=algorithm == "fold")
        z.zero_grad()
    # the same step written with the oracle only
    lay = [FlatLayout(numels, world, r) for r in range(world)]
    bufs = [_raw(p0) for _ in range(world)]
    opts = [AdamW(**kw, kind=kind if kind != "f64" else None) for _ in range(world)]
    for s in range(steps):
        gs = [_raw(g) for g in grads[s]]
        shards = [np.zeros(l.hi - l.lo, bufs[0].dtype) for l in lay]
        for a, b, _ in zero_buckets(numels, es, 16 << 10):
            sizes = lay[0].bucket_sizes(a, b)
            outs = ring.expected_reduce_scatter([g[a:b] for g in gs], sizes, True, kind)
            lo = a
            for c, m in enumerate(sizes):
                if m:
                    mine = outs[c][lo - a:lo - a + m].copy()
                    if kind != "f64":
                        mine[mine == 0x8000] = 0  # 0 + (-0) = +0, as grad_shard.add_(mine) leaves it; nothing else changes
                    else:
                        mine = 0.0 + mine
                    shards[c][lo - lay[c].lo:lo - lay[c].lo + m] = mine
                lo += m
        for r in range(world):
            opts[r].update("flat", bufs[r][lay[r].lo:lay[r].hi], shards[r])
        full = ring.expected_all_gather(bufs, lay[0].sizes)
        bufs = [full.copy() for _ in range(world)]
    for r in range(world):
        assert np.array_equal(bits(_raw(z.bufs[r])), bits(bufs[r])), (dtype, world, algorithm, r)
        assert np.array_equal(bits(_raw(z.opts[r].state["flat"][1])), bits(opts[r].state["flat"][1])), (dtype, world, algorithm, r)
        assert np.array_equal(bits(_raw(z.opts[r].state["flat"][2])), bits(opts[r].state["flat"][2])), (dtype, world, algorithm, r)


def test_full_size_step():
    """85,842,432 parameters, world 4, 25 MiB buckets, the reference's bucket_sizes
    (plans.json), one step. The ring's steps and the fold leave the same gradient
    shards; the averaged gradient equals the oracle's ring-order fold on a sample of
    every fifth bucket's chunks; every rank ends with the same parameters; one whole
    shard equals the oracle's AdamW. (The twenty steps of the configuration, against
    torch.optim.AdamW and the oracle, are test_config_4_twenty_steps below.)"""
    from oracle import ring
    from oracle.adamw import AdamW
    from tandem_amd.local import LocalZeRO2

    dev = torch.device("cuda", 0)
    plan = golden_json("plans.json")
    numels = [math.prod(s) for _, s in plan["medium_params"]]
    world, n = 4, sum(numels)
    assert n == 85_842_432
    z = LocalZeRO2(world, numels, dev, **KW)
    assert [[a, b] for a, b, _ in z.buckets] == plan["medium_zero_25MiB_w4"]["ranges"]
    gen = torch.Generator(device=dev).manual_seed(0)
    p0 = torch.randn(n, device=dev, generator=gen) * 0.02
    for b in z.bufs:
        b.copy_(p0)
    grads = []
    for r in range(world):
        g = torch.randn(n, device=dev, generator=gen) * 1e-3
        z.staging[r].copy_(g)
        grads.append(g)
    z.reduce_grads("ring")
    ring_shards = [g.clone() for g in z.grad_shards]
    z.zero_grad()
    for r in range(world):
        z.staging[r].copy_(grads[r])
    z.reduce_grads("fold")
    for r in range(world):  # one launch, same bits as the ring steps
        assert torch.equal(ring_shards[r].view(torch.int32), z.grad_shards[r].view(torch.int32))
    del ring_shards
    # the averaged gradient in ring order, sampled per bucket chunk
    lay = z.layouts
    for a, b, _ in z.buckets[::5]:
        sizes = lay[0].bucket_sizes(a, b)
        lo = a
        for c, m in enumerate(sizes):
            if m:
                k = min(m, 50_000)
                sample = [g[lo:lo + k].cpu().numpy() for g in grads]
                # chunk c of this bucket: fold ending at rank c
                want = ring.fold(sample, c, 0, k, True) + np.float32(0)
                got = z.grad_shards[c][lo - lay[c].lo:lo - lay[c].lo + k].cpu().numpy()
                assert np.array_equal(bits(got), bits(want)), (a, b, c)
            lo += m
    shards_before = [g.clone() for g in z.grad_shards]
    z.step()
    for r in range(1, world):
        assert torch.equal(z.bufs[0].view(torch.int32), z.bufs[r].view(torch.int32))
    # one shard against the oracle's AdamW, whole
    r = 2
    pn = p0[lay[r].lo:lay[r].hi].cpu().numpy().copy()
    AdamW(**KW).update("k", pn, shards_before[r].cpu().numpy())
    assert np.array_equal(bits(z.bufs[0][lay[r].lo:lay[r].hi].cpu().numpy()), bits(pn))


def test_config_4_twenty_steps():
    """The configuration as stated: the 85,842,432-parameter GPT, world 4 on one GPU,
    16 buckets of up to 25 MiB, reduce-scatter into 21,460,608-element shards, AdamW
    (lr 3e-4, betas 0.9/0.95, eps 1e-8, wd 0.1) for TWENTY steps with fresh seeded
    gradients each step, all-gather; as the reference checks its ZeRO against torch's
    AdamW end to end (tests/test_zero.py:46-66 there). Both forms of the step run side
    by side, reduce_grads() + step() and reduce_and_step() (one launch), in both
    operation orders. One whole shard is followed on the side, fed every step with the
    oracle's ring-order fold of that step's four gradients (which the kernels' own
    gradient shard must equal bit for bit):
      order="device": torch.optim.AdamW([shard], foreach=False, fused=False) on the GPU;
                      parameters and both moments bit for bit;
      order="host":   the oracle's AdamW (the reference's operation order on the CPU);
                      parameters and both moments bit for bit.
    After step 20 every rank holds the same buffer in every run, and the one-launch form
    equals the two-kernel form in every buffer and both moments of every rank."""
    from oracle import ring
    from oracle.adamw import AdamW
    from tandem_amd.local import LocalZeRO2

    dev = torch.device("cuda", 0)
    plan = golden_json("plans.json")
    numels = [math.prod(s) for _, s in plan["medium_params"]]
    world, n, steps, watched = 4, sum(numels), 20, 2
    assert n == 85_842_432
    runs = {(order, form): LocalZeRO2(world, numels, dev, order=order, **KW)
            for order in ("device", "host") for form in ("two_kernels", "one_launch")}
    lay = runs["host", "two_kernels"].layouts
    lo, hi = lay[watched].lo, lay[watched].hi
    assert hi - lo == 21_460_608 and len(runs["host", "two_kernels"].buckets) == 16
    p0 = torch.randn(n, device=dev, generator=torch.Generator(device=dev).manual_seed(4)) * 0.02
    for z in runs.values():
        for b in z.bufs:
            b.copy_(p0)
    torch_p = torch.nn.Parameter(p0[lo:hi].clone())
    torch_opt = torch.optim.AdamW([torch_p], foreach=False, fused=False, **KW)
    oracle_p = p0[lo:hi].cpu().numpy().copy()
    oracle_opt = AdamW(**KW)
    del p0
    for step in range(steps):
        shard_grads = []
        for r in range(world):
            g = torch.randn(n, device=dev, generator=torch.Generator(device=dev).manual_seed(1000 * step + r)) * 1e-3
            for z in runs.values():
                z.staging[r].copy_(g)
            shard_grads.append(g[lo:hi].cpu().numpy())
        del g
        # the watched shard's gradient as the reference leaves it: the ring's order for chunk `watched`, added into a zeroed shard
        mine = np.float32(0.0) + ring.fold(shard_grads, watched, 0, hi - lo, True)
        for (order, form), z in runs.items():
            if form == "one_launch":
                assert z._step_table is not None and z._shards_zero
                z.reduce_and_step()
            else:
                z.reduce_grads()
                assert np.array_equal(bits(z.grad_shards[watched].cpu().numpy()), bits(mine)), (step, order)
                z.step()
            z.zero_grad()
        torch_p.grad = torch.from_numpy(mine).to(dev)
        torch_opt.step()
        oracle_opt.update("k", oracle_p, mine)
    want = {"device": (torch_p.detach().cpu().numpy(), torch_opt.state[torch_p]["exp_avg"].cpu().numpy(),
                       torch_opt.state[torch_p]["exp_avg_sq"].cpu().numpy()),
            "host": (oracle_p, oracle_opt.state["k"][1], oracle_opt.state["k"][2])}
    assert not np.array_equal(bits(want["device"][0]), bits(want["host"][0]))  # the two orders do differ over twenty steps
    for (order, form), z in runs.items():
        what = (order, form)
        assert z.opts[watched].state["flat"][0] == float(steps), what
        for r in range(1, world):
            assert torch.equal(z.bufs[0].view(torch.int32), z.bufs[r].view(torch.int32)), what + (r,)
        p, m, v = want[order]
        assert np.array_equal(bits(z.bufs[0][lo:hi].cpu().numpy()), bits(p)), what
        assert np.array_equal(bits(z.opts[watched].state["flat"][1].cpu().numpy()), bits(m)), what
        assert np.array_equal(bits(z.opts[watched].state["flat"][2].cpu().numpy()), bits(v)), what
    for order in ("device", "host"):
        a, b = runs[order, "two_kernels"], runs[order, "one_launch"]
        assert torch.equal(a.bufs[0].view(torch.int32), b.bufs[0].view(torch.int32)), order
        for r in range(world):
            for i in (1, 2):
                assert torch.equal(a.opts[r].state["flat"][i].view(torch.int32), b.opts[r].state["flat"][i].view(torch.int32)), (order, r, i)


def test_full_size_step_in_one_launch():
    """The same 85,842,432-parameter step as reduce_and_step(): one launch must leave
    every rank's parameters and every rank's optimizer state with the bits that
    reduce_grads() + step() leave, over three steps."""
    from tandem_amd.local import LocalZeRO2

    dev = torch.device("cuda", 0)
    plan = golden_json("plans.json")
    numels = [math.prod(s) for _, s in plan["medium_params"]]
    world, n = 4, sum(numels)
    apart, fused = LocalZeRO2(world, numels, dev, **KW), LocalZeRO2(world, numels, dev, **KW)
    gen = torch.Generator(device=dev).manual_seed(3)
    p0 = torch.randn(n, device=dev, generator=gen) * 0.02
    for z in (apart, fused):
        for b in z.bufs:
            b.copy_(p0)
    del p0
    for step in range(3):
        for r in range(world):
            g = torch.randn(n, device=dev, generator=gen) * 1e-3
            g[:4] = torch.tensor([0.0, -0.0, 1e-45, -1e-45], device=dev)
            apart.staging[r].copy_(g)
            fused.staging[r].copy_(g)
        del g
        apart.reduce_grads()
        apart.step()
        apart.zero_grad()
        fused.reduce_and_step()
        fused.zero_grad()
    for r in range(world):
        assert torch.equal(apart.bufs[r].view(torch.int32), fused.bufs[r].view(torch.int32)), r
        for i in (1, 2):
            assert torch.equal(apart.opts[r].state["flat"][i].view(torch.int32), fused.opts[r].state["flat"][i].view(torch.int32)), (r, i)
        assert apart.opts[r].state["flat"][0] == fused.opts[r].state["flat"][0] == 3.0
        assert float(fused.grad_shards[r].abs().sum()) == 0.0


@pytest.mark.parametrize("average", [1, 0])
@pytest.mark.parametrize("world", [1, 2, 3, 4, 5, 6, 7, 8])
def test_one_launch_step_through_the_c_abi(world, average):
    """tdm_k23_zero2_step on its own, at every world size it is built for: segments of
    odd lengths (one element, a tile and a bit, several tiles), each owned by a different
    chunk, once 16-byte aligned and once 4 bytes off (a peeled head, then vectors), two steps. Host
    order against the oracle's fold + AdamW; device order against the oracle's fold fed
    to the separate AdamW kernel in device order."""
    import ctypes

    from oracle import ring
    from oracle.adamw import AdamW
    from tandem_amd import _lib
    from tandem_amd._lib import check, lib, stream_ptr
    from tandem_amd.optim import ShardedAdamW, step_scalars

    dev = torch.device("cuda", 0)
    counts = [1, 3, 4099, 10007, 0, 4 * 4096 + 4, 2048]
    for shift in (0, 1):
        for order in ("host", "device"):
            nseg = len(counts)
            total = sum(counts) + 8 * nseg + 8
            grads_h = [(seeded(40 + shift, r, total) * 1e-3).numpy() for r in range(world)]
            for g in grads_h:
                g[shift:shift + 4] = [0.0, -0.0, 1e-45, -1e-45]
            p_h = (seeded(50, 0, total) * 0.02).numpy()
            grads = [torch.from_numpy(g).to(dev) for g in grads_h]
            params = [torch.from_numpy(p_h).to(dev) for _ in range(world)]
            m, v = torch.zeros(total, device=dev), torch.zeros(total, device=dev)
            segs = (_lib.StepSeg * nseg)()
            spans, at = [], shift
            for k, n in enumerate(counts):
                spans.append((at, at + n, k % world))
                for r in range(world):
                    segs[k].grad[r] = grads[r].data_ptr() + at * 4
                    segs[k].param[r] = params[r].data_ptr() + at * 4
                segs[k].exp_avg, segs[k].exp_avg_sq = m.data_ptr() + at * 4, v.data_ptr() + at * 4
                segs[k].count, segs[k].chunk = n, k % world
                at += -(-n // 4) * 4 + 4  # keeps every segment's start at the same offset from 16-byte alignment
            ntiles = lib().tdm_k23_table_tiles(segs, nseg)
            tile = lib().tdm_table_tile_bytes() // 4
            head = (4 - shift) % 4  # elements before the next 16-byte boundary: peeled off, the rest runs on vectors
            assert ntiles == sum(-(-(n - head if n > head else n) // tile) for n in counts)
            image = torch.empty(lib().tdm_k23_table_bytes(segs, nseg), dtype=torch.uint8)
            check(lib().tdm_k23_table_build(segs, nseg, world, ctypes.c_void_p(image.data_ptr())))
            table = image.to(dev)
            # expectation
            want_p, want_m, want_v = p_h.copy(), np.zeros(total, np.float32), np.zeros(total, np.float32)
            oracle_opts = {k: AdamW(**KW) for k in range(nseg)}
            device_opt = ShardedAdamW(order="device", **KW)
            dp = torch.from_numpy(p_h).to(dev)
            for step in (1.0, 2.0):
                s = step_scalars(step, KW["lr"], KW["betas"], KW["eps"], KW["weight_decay"])
                check(lib().tdm_k23_zero2_step(ctypes.c_void_p(table.data_ptr()), ntiles, world, average, ctypes.byref(s),
                                               _lib.ADAMW_HOST_ORDER if order == "host" else _lib.ADAMW_DEVICE_ORDER,
                                               stream_ptr(dev)))
                for k, (lo, hi, c) in enumerate(spans):
                    if hi == lo:
                        continue
                    mine = np.float32(0.0) + ring.fold(grads_h, c, lo, hi, bool(average))
                    if order == "host":
                        o = oracle_opts[k]
                        o.update("s", want_p[lo:hi], mine)
                        want_m[lo:hi], want_v[lo:hi] = o.state["s"][1], o.state["s"][2]
                    else:
                        device_opt.update(k, dp[lo:hi], torch.from_numpy(mine).to(dev))
            torch.cuda.synchronize(dev)
            if order == "device":
                want_p = dp.cpu().numpy()
                for k, (lo, hi, _) in enumerate(spans):
                    if hi > lo:
                        want_m[lo:hi] = device_opt.state[k][1].cpu().numpy()
                        want_v[lo:hi] = device_opt.state[k][2].cpu().numpy()
            what = (world, average, shift, order)
            for r in range(world):  # every rank's copy, and nothing outside the segments touched
                assert np.array_equal(bits(params[r].cpu().numpy()), bits(want_p)), what + (r,)
            assert np.array_equal(bits(m.cpu().numpy()), bits(want_m)), what
            assert np.array_equal(bits(v.cpu().numpy()), bits(want_v)), what


@pytest.mark.parametrize("world", [1, 2, 3, 4, 5, 6, 7, 8])
def test_one_segment_in_the_launch_equals_the_table(world):
    """tdm_k23_zero2_step_segment (the segment travels in the kernel's arguments: what a
    process rank runs over its shard) against tdm_k23_zero2_step over a one-row table,
    which the test above pins to the oracle: same bits in every buffer, aligned and not,
    sum and average, both orders."""
    import ctypes

    from tandem_amd import _lib
    from tandem_amd._lib import check, lib, stream_ptr
    from tandem_amd.optim import step_scalars

    dev = torch.device("cuda", 0)
    n = 3 * 4096 + 1031
    for shift, average, order, chunk in ((0, 1, _lib.ADAMW_HOST_ORDER, world - 1), (1, 0, _lib.ADAMW_DEVICE_ORDER, 0),
                                         (0, 0, _lib.ADAMW_HOST_ORDER, world // 2), (3, 1, _lib.ADAMW_DEVICE_ORDER, world // 3)):
        grads = [(seeded(70 + shift, r, n + 8) * 1e-3).to(dev) for r in range(world)]
        p0 = (seeded(71, 0, n + 8) * 0.02).to(dev)
        results = []
        for entry in ("table", "segment"):
            params = [p0.clone() for _ in range(world)]
            m, v = torch.zeros(n + 8, device=dev), torch.zeros(n + 8, device=dev)
            seg = (_lib.StepSeg * 1)()
            for r in range(world):
                seg[0].grad[r] = grads[r].data_ptr() + shift * 4
                seg[0].param[r] = params[r].data_ptr() + shift * 4
            seg[0].exp_avg, seg[0].exp_avg_sq = m.data_ptr() + shift * 4, v.data_ptr() + shift * 4
            seg[0].count, seg[0].chunk = n, chunk
            if entry == "table":
                ntiles = lib().tdm_k23_table_tiles(seg, 1)
                image = torch.empty(lib().tdm_k23_table_bytes(seg, 1), dtype=torch.uint8)
                check(lib().tdm_k23_table_build(seg, 1, world, ctypes.c_void_p(image.data_ptr())))
                table = image.to(dev)
            for step in (1.0, 2.0):
                s = step_scalars(step, KW["lr"], KW["betas"], KW["eps"], KW["weight_decay"])
                if entry == "table":
                    check(lib().tdm_k23_zero2_step(ctypes.c_void_p(table.data_ptr()), ntiles, world, average, ctypes.byref(s), order,
                                                   stream_ptr(dev)))
                else:
                    check(lib().tdm_k23_zero2_step_segment(seg, world, average, ctypes.byref(s), order, stream_ptr(dev)))
            torch.cuda.synchronize(dev)
            results.append([t.cpu() for t in params + [m, v]])
        for a, b in zip(*results):
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (world, shift, average, order)
        assert not torch.equal(results[0][0], p0.cpu())  # the step did happen
