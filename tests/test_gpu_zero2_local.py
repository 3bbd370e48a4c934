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


def test_full_size_step():
    """85,842,432 parameters, world 4, 25 MiB buckets, the reference's bucket_sizes
    (plans.json). Properties: every rank ends with the same parameters; each rank's
    shard equals a sampled oracle evaluation; the step matches torch.optim.AdamW on
    the GPU when run in torch's GPU op order."""
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
