"""The benchmark's configurations at their STATED sizes, checked (bench.py only times them):
the DDP bucket path over the 85.8M-parameter GPT's 149 gradients (world 2, 16 buckets of
25 MiB, 161 segments), ZeRO-3 over the same model between two processes with a batch of
8 x 512 tokens, and the reference's own CPU-runnable case, all_reduce(avg) of 1,048,576
seeded N(0,1) elements per rank between two processes, on every path the hip backend has.
After tests/test_engine_cuda.py:84-127 and tests/test_zero.py:38-66 of the reference.
Run with -m gpu."""

import math

import numpy as np
import pytest
import torch

from helpers import bits, golden_json, seeded

pytestmark = pytest.mark.gpu
TIMEOUT = 120.0


# ---------------------------------------------------------------- config 3: the bucket path
def medium_plan():
    plan = golden_json("plans.json")
    names = [n for n, _ in plan["medium_params"]]
    numels = [math.prod(s) for _, s in plan["medium_params"]]
    buckets = [[names.index(n) for n in b] for b in plan["medium_ddp_25MiB"]]
    return numels, buckets


def test_bucket_path_over_the_85m_gpt():
    """LocalWorld(2).bucket_table over the reference's own bucket plan (tests/golden/plans.json,
    written by tandem/ddp.py:56-68 there). Every element of every gradient on both ranks must be
    g0/2 + g1/2 (two ranks: any order gives the same bits), in place and out of place; and for
    every bucket its first, its last and the segment that straddles the ring's chunk boundary
    are compared with the oracle's fold, which also pins the chunk each segment was given."""
    from oracle import ring
    from tandem_amd import LocalWorld
    from tandem_amd.buckets import fold_segments

    dev = torch.device("cuda", 0)
    numels, buckets = medium_plan()
    assert sum(numels) == 85_842_432 and len(numels) == 149 and len(buckets) == 16
    assert sorted(i for b in buckets for i in b) == list(range(149))
    world = 2
    grads = []
    for r in range(world):
        gen = torch.Generator(device=dev).manual_seed(1000 + r)
        grads.append([torch.randn(m, device=dev, generator=gen) * 1e-3 for m in numels])
    want = [a * 0.5 + b * 0.5 for a, b in zip(*grads)]  # x / 2 is exact, and so is the order at two ranks
    lw = LocalWorld(world)
    outs = [[torch.full_like(t, 7.0) for t in row] for row in grads]
    table = lw.bucket_table(grads, buckets, outs)
    assert table.nseg == 161 and table.elements == 85_842_432
    table.run(True)
    torch.cuda.synchronize()
    for r in range(world):
        for i in range(149):
            assert torch.equal(outs[r][i].view(torch.int32), want[i].view(torch.int32)), (r, i)
    # the oracle on sampled segments: first, last, and the one that crosses the chunk boundary
    for b, members in enumerate(buckets):
        sizes = [numels[i] for i in members]
        segs = fold_segments(sizes, world)
        flat = [np.concatenate([grads[r][i].cpu().numpy() for i in members]) for r in range(world)]
        starts = np.cumsum([0] + sizes)
        crossing = [k for k in range(1, len(segs)) if segs[k][0] == segs[k - 1][0]]  # one tensor cut in two
        for k in sorted({0, len(segs) - 1, *crossing, *(c - 1 for c in crossing)}):
            pos, off, count, chunk = segs[k]
            lo = int(starts[pos]) + off
            take = min(count, 40_000)
            for a in sorted({lo, lo + count - take}):
                expect = ring.fold(flat, chunk, a, a + take, True)
                got = outs[1][members[pos]][a - int(starts[pos]):a - int(starts[pos]) + take].cpu().numpy()
                assert np.array_equal(bits(got), bits(expect)), (b, k)
        del flat
    # in place: the same table over the gradients themselves
    lw.bucket_table(grads, buckets).run(True)
    torch.cuda.synchronize()
    for r in range(world):
        for i in range(149):
            assert torch.equal(grads[r][i].view(torch.int32), want[i].view(torch.int32)), (r, i)


# ---------------------------------------------------------------- config 5: ZeRO-3, two processes, the 85.8M GPT
def checksums(t):
    """Two 64-bit sums over the bit patterns: enough to tell two 343 MB buffers apart
    without sending them through a file."""
    v = t.detach().reshape(-1).view(torch.int32).to(torch.int64)
    weights = (torch.arange(v.numel(), device=v.device, dtype=torch.int64) % 65521) + 1
    return [int(v.sum()), int((v * weights).sum())]


def medium_rank(g, strategy):
    from tandem_amd import ShardedAdamW
    from tandem_amd.data import synthetic
    from tandem_amd.model import GPT, Config
    from tandem_amd.zero import FSDP, ZeRO

    torch.backends.cuda.enable_flash_sdp(False)
    torch.backends.cuda.enable_mem_efficient_sdp(False)
    torch.backends.cuda.matmul.allow_tf32 = False
    cfg = Config.preset("medium")
    torch.manual_seed(0)
    text = synthetic(100_000)
    model = GPT(cfg).to(g.device)
    opt = ShardedAdamW(lr=3e-4, betas=(0.9, 0.95), weight_decay=0.1)
    out = {}
    if strategy == "zero3":
        z = FSDP(model, g, opt)
        out["units"] = [u.layout.numel for u in z.units]
        # every unit's gathered parameters against the shards themselves, brought together another way:
        # an ordinary all_gather through the engine's staging instead of the direct arena reads
        same = []
        for u in z.units:
            through_staging = torch.zeros(u.layout.numel, device=g.device)
            through_staging[u.layout.lo:u.layout.hi] = u.shard
            g.all_gather(through_staging, u.layout.sizes)
            same.append(bool(torch.equal(u.gathered_copy().view(torch.int32), through_staging.view(torch.int32))))
        out["gather_equals_cat_of_shards"] = same
        seen = []  # what each unit's forward found in its full buffer, against the same cat of shards
        for u in z.units:
            def look(module, args, u=u):
                seen.append((u.index, checksums(u.full)))
            u.module.register_forward_pre_hook(look)  # after FSDP's own hook, which has gathered by then
        before = z.full_parameters()
        out["start"] = checksums(before)
    else:
        z = ZeRO(model, g, 2, opt)
    x, y = text.batch(0, 8, cfg.seq, rank=g.rank, world=g.size, device=g.device)
    g.barrier()
    torch.cuda.synchronize()
    g.trace = []
    g.tracing = True
    loss = z(x, y)
    loss.backward()
    torch.cuda.synchronize()
    g.tracing = False
    spans = list(g.trace)
    out["loss"] = loss.item()
    out["gathers"] = sum(1 for name, *_ in spans if name == "gather_unit")
    out["comm_bytes"] = sum(nbytes for name, _, _, nbytes in spans if name != "barrier")
    if strategy == "zero3":
        out["max_live"], out["live_after_backward"] = z.max_live, z.live
        sizes = [0]
        for n in out["units"]:
            sizes.append(sizes[-1] + n)
        out["forward_saw_the_shards"] = [cs == checksums(before[sizes[k]:sizes[k + 1]]) for k, cs in seen]
        out["forward_order"] = [k for k, _ in seen]
        del before
    z.step()
    z.zero_grad()
    w = z.full_parameters() if strategy == "zero3" else torch.cat([p.detach().reshape(-1) for p in model.parameters()])
    torch.cuda.synchronize()
    out["weights_checksums"] = checksums(w)
    if g.rank == 0:
        out["weights"] = w.cpu()
    if strategy == "zero3":
        out["live"] = z.live
    return out


def test_zero3_over_the_85m_gpt_between_two_processes():
    """One training step of FSDP over GPT(Config.preset("medium")), batch 8 x 512 from synthetic()
    split over two processes that share the GPU. Every unit's gather equals the concatenation of
    the two shards, in set-up and as each unit's forward found it; at most three units whole at
    once and none afterwards; 27 gathers and the reference's byte count per step
    (bench/t4/2026-10-02.jsonl:22 there: 1,029,316,608); both ranks end with the same weights,
    and those equal a ZeRO-2 run of the same model on the same batch bit for bit (two ranks:
    the average has one order)."""
    from tandem_amd import launch

    z3 = launch(medium_rank, 2, "zero3", gpus=[0, 0], timeout=TIMEOUT)
    plan = golden_json("plans.json")
    for r, out in enumerate(z3):
        assert out["units"] == plan["medium_units"] and len(out["units"]) == 14
        assert all(out["gather_equals_cat_of_shards"]), (r, out["gather_equals_cat_of_shards"])
        assert out["forward_order"] == list(range(14)) and all(out["forward_saw_the_shards"]), r
        assert out["max_live"] <= 3 and out["live_after_backward"] == 0 and out["live"] == 0, r
        assert out["gathers"] == 27, (r, out["gathers"])
        assert out["comm_bytes"] == 1_029_316_608, (r, out["comm_bytes"])
        assert math.isfinite(out["loss"]) and 5.0 < out["loss"] < 6.5  # ln 256 = 5.545: an untrained byte model
    assert z3[0]["start"] == z3[1]["start"]
    assert z3[0]["weights_checksums"] == z3[1]["weights_checksums"], "the ranks drifted apart"
    assert z3[0]["weights"].numel() == 85_842_432
    z2 = launch(medium_rank, 2, "zero2", gpus=[0, 0], timeout=TIMEOUT)
    assert z2[0]["weights_checksums"] == z2[1]["weights_checksums"]
    for r in range(2):
        assert z3[r]["loss"] == z2[r]["loss"], r
    assert torch.equal(z3[0]["weights"].view(torch.int32), z2[0]["weights"].view(torch.int32))


# ---------------------------------------------------------------- config 1: 4 MB per rank, two processes
def config1_rank(g, direct):
    n = 1_048_576
    x = seeded(0, g.rank, n).to(g.device)  # N(0, 1), generator seeded with seed * 1000 + rank (tests/test_comm.py:13-16 there)
    if direct:
        t = g.shared_empty(n)
        t.copy_(x)
        g.all_reduce(t, op="avg", direct=True)
    else:
        t = x.clone()
        g.all_reduce(t, op="avg")
    torch.cuda.synchronize()
    return t.cpu()


@pytest.mark.parametrize("path", ["staged", "small", "ring", "direct"])
def test_config_1_all_reduce_on_every_path(path, monkeypatch):
    """The reference's own CPU-runnable configuration as the hip backend runs it: launch(..., 2),
    all_reduce(avg) of randn(1_048_576) seeded per rank, result x0/2 + x1/2 bit for bit on both
    ranks, through the staged passes, the one-handshake form for small tensors, the slot ring
    (two chunks of 2 MiB, one piece each) and arena to arena."""
    from tandem_amd import launch

    if path == "staged":
        monkeypatch.setenv("TANDEM_HIP_SMALL_BYTES", "0")  # 4 MB would otherwise take the one-handshake form
    elif path == "ring":
        monkeypatch.setenv("TANDEM_HIP_ALGO", "ring")
    res = launch(config1_rank, 2, path == "direct", gpus=[0, 0], timeout=TIMEOUT)
    x0, x1 = seeded(0, 0, 1_048_576), seeded(0, 1, 1_048_576)
    want = x0 / 2 + x1 / 2
    for r in range(2):
        assert np.array_equal(bits(res[r].numpy()), bits(want.numpy())), (path, r)
