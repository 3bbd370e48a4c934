"""Host logic of DDP / ZeRO-1/2 / FSDP on the CPU: the product's wrappers driven by
the oracle's CPU-process group and the oracle's AdamW must reproduce, bit for
bit, the training runs the reference itself produced (tests/golden/train_w*.json:
losses of every step and a digest of the final weights, world sizes 2, 3, 4),
and, at world 2, torch's own DistributedDataParallel + AdamW over gloo (what the
reference's tests/test_ddp.py and tests/test_zero.py check)."""

import hashlib
import os
import tempfile

import pytest
import torch

from helpers import OracleShardedAdamW, golden_json
from oracle.cpu_engine import cpu_launch
from tandem_amd.data import synthetic
from tandem_amd.ddp import DDP
from tandem_amd.model import GPT, Config
from tandem_amd.zero import FSDP, ZeRO

CFG = Config(seq=32, layers=2, heads=2, dim=32)


def sha(t):
    return hashlib.sha256(t.detach().contiguous().numpy().tobytes()).hexdigest()


def train_rank(g, strategy, bucket_bytes, steps, batch, accumulate=1, zero_every=1):
    torch.manual_seed(0)
    text = synthetic(20_000)
    model = GPT(CFG)
    losses, extra = [], {}
    if strategy == "ddp":
        z = DDP(model, g, bucket_bytes=bucket_bytes)
        opt = torch.optim.AdamW(model.parameters(), lr=3e-3, weight_decay=0.1, foreach=False)
    else:
        sopt = OracleShardedAdamW(lr=3e-3, weight_decay=0.1)
        stage = int(strategy[-1])
        z = ZeRO(model, g, stage, sopt, bucket_bytes) if stage < 3 else FSDP(model, g, sopt)
    for step in range(steps):
        for micro in range(accumulate):
            x, y = text.batch(step * accumulate + micro, batch, CFG.seq, rank=g.rank, world=g.size)
            if strategy == "ddp" and micro < accumulate - 1:
                with z.no_sync():
                    loss = z(x, y)
                    (loss / accumulate).backward()
            else:
                loss = z(x, y)
                (loss / accumulate).backward()
            losses.append(loss.item())
        last = (step + 1) % zero_every == 0
        if strategy == "ddp":
            opt.step()
            if last:
                opt.zero_grad()
        else:
            z.step()
            if last:
                z.zero_grad()
    if strategy == "zero3":
        w = z.full_parameters()
        extra = {"max_live": z.max_live, "live": z.live}
    else:
        w = torch.cat([p.detach().reshape(-1) for p in model.parameters()])
        if strategy == "zero2":
            assert all(p.grad is None for p in model.parameters())  # only shard gradients are kept
    if strategy != "ddp":
        extra["state_bytes"] = sopt.state_bytes()
    return {"losses": losses, "sha256": sha(w), "first8": w[:8].tolist(), "last8": w[-8:].tolist(), "numel": w.numel(),
            "weights": w if g.size == 2 else None, **extra}


@pytest.mark.parametrize("world", [2, 3, 4])
@pytest.mark.parametrize("strategy", ["ddp", "zero1", "zero2", "zero3"])
def test_reproduces_the_reference_training_runs(world, strategy):
    want = golden_json(f"train_w{world}.json")
    got = cpu_launch(train_rank, world, strategy, want["bucket_bytes"], want["steps"], want["batch"], slot_bytes=1024)
    for r in range(world):
        ref = want[strategy][r]
        assert got[r]["losses"] == ref["losses"], (world, strategy, r)
        assert got[r]["first8"] == ref["first8"] and got[r]["last8"] == ref["last8"]
        assert got[r]["sha256"] == ref["sha256"], (world, strategy, r)
        if strategy == "zero3":
            # at most the running unit, the prefetched one and the head are whole at once
            assert got[r]["max_live"] == ref["max_live"] <= 3 and got[r]["live"] == 0
        if strategy != "ddp":
            assert got[r]["state_bytes"] <= 2 * 4 * (got[r]["numel"] // world + 1)


@pytest.mark.parametrize("world", [2, 3])
def test_reproduces_the_reference_runs_with_two_backward_passes_a_step(world):
    """tests/golden/train_accumulating.json: the reference's own runs with two micro-batches before every step. Its ZeRO
    and FSDP add every backward pass into their gradient (shard) until zero_grad() (tandem/zero.py:139-153,165-170,
    306-317), its DDP skips the all-reduce under no_sync() (tandem/ddp.py:79-87): same losses, same weights, bit for bit.
    The fixture's second half: one backward pass a step, but zero_grad() only after every second step."""
    want = golden_json("train_accumulating.json")
    for strategy in ("ddp", "zero1", "zero2", "zero3"):
        got = cpu_launch(train_rank, world, strategy, want["bucket_bytes"], want["steps"], want["batch"], want["micro_batches"], slot_bytes=1024)
        for r in range(world):
            ref = want[str(world)][strategy][r]
            assert got[r]["losses"] == ref["losses"], (world, strategy, r)
            assert got[r]["first8"] == ref["first8"] and got[r]["last8"] == ref["last8"], (world, strategy, r)
            assert got[r]["sha256"] == ref["sha256"], (world, strategy, r)
        # and a step() that is not followed by zero_grad(): the next backward adds to what is there
        got = cpu_launch(train_rank, world, strategy, want["bucket_bytes"], want["steps"], want["batch"], 1, 2, slot_bytes=1024)
        for r in range(world):
            ref = want["zero_grad_every_second_step"][str(world)][strategy][r]
            assert got[r]["losses"] == ref["losses"], (world, strategy, r, "zero_grad every second step")
            assert got[r]["sha256"] == ref["sha256"], (world, strategy, r, "zero_grad every second step")


def fsdp_rank_without_prefetch(g, batch):
    torch.manual_seed(0)
    text = synthetic(20_000)
    z = FSDP(GPT(CFG), g, OracleShardedAdamW(lr=3e-3, weight_decay=0.1), prefetch=False)
    losses = []
    for step in range(3):
        x, y = text.batch(step, batch, CFG.seq, rank=g.rank, world=g.size)
        loss = z(x, y)
        loss.backward()
        losses.append(loss.item())
        z.step()
        z.zero_grad()
    return {"losses": losses, "sha256": sha(z.full_parameters()), "max_live": z.max_live, "live": z.live}


@pytest.mark.parametrize("world", [2, 3])
def test_fsdp_without_prefetch_as_the_reference_runs_it(world):
    """FSDP(prefetch=False) in the reference: the same weights, and no more units whole at once than it has."""
    want = golden_json("train_accumulating.json")
    got = cpu_launch(fsdp_rank_without_prefetch, world, want["batch"], slot_bytes=1024)
    for r in range(world):
        ref = want["fsdp_without_prefetch"][str(world)][r]
        assert got[r]["losses"] == ref["losses"] and got[r]["sha256"] == ref["sha256"], (world, r)
        assert got[r]["max_live"] == ref["max_live"] and got[r]["live"] == ref["live"] == 0, (world, r, got[r]["max_live"], ref["max_live"])


def train_rank_typed(g, strategy, bucket_bytes, steps, batch, dtype_name):
    torch.manual_seed(0)
    text = synthetic(20_000)
    model = GPT(CFG).to(getattr(torch, dtype_name))
    losses = []
    if strategy == "ddp":
        z = DDP(model, g, bucket_bytes=bucket_bytes)
        opt = torch.optim.AdamW(model.parameters(), lr=3e-3, weight_decay=0.1, foreach=False)
    else:
        sopt = OracleShardedAdamW(lr=3e-3, weight_decay=0.1)
        stage = int(strategy[-1])
        z = ZeRO(model, g, stage, sopt, bucket_bytes) if stage < 3 else FSDP(model, g, sopt)
    for step in range(steps):
        x, y = text.batch(step, batch, CFG.seq, rank=g.rank, world=g.size)
        loss = z(x, y)
        loss.backward()
        losses.append(loss.item())
        if strategy == "ddp":
            opt.step()
            opt.zero_grad()
        else:
            z.step()
            z.zero_grad()
    w = z.full_parameters() if strategy == "zero3" else torch.cat([p.detach().reshape(-1) for p in model.parameters()])
    assert w.dtype == getattr(torch, dtype_name)
    return {"losses": losses, "sha256": sha(w.view(torch.int16) if w.element_size() == 2 else w), "first8": w[:8].double().tolist(),
            "last8": w[-8:].double().tolist()}


@pytest.mark.parametrize("world", [2, 3])
@pytest.mark.parametrize("dtype_name", ["bfloat16", "float64"])
def test_reproduces_the_reference_runs_on_bfloat16_and_float64_models(dtype_name, world):
    """tests/golden/train_dtypes.json: the reference's DDP, ZeRO-1/2 and FSDP over its own engine with the model in
    bfloat16 and in float64 (its wrappers, collectives and ShardedAdamW take any floating type). The product's wrappers
    over the oracle's group and the oracle's typed AdamW must give the same losses and the same weights, bit for bit:
    the composition of the typed ring (every addition rounded to the type) and the typed update, end to end."""
    want = golden_json("train_dtypes.json")
    for strategy in ("ddp", "zero1", "zero2", "zero3"):
        got = cpu_launch(train_rank_typed, world, strategy, want["bucket_bytes"], want["steps"], want["batch"], dtype_name, slot_bytes=1024)
        for r in range(world):
            ref = want[dtype_name][str(world)][strategy][r]
            assert got[r]["losses"] == ref["losses"], (dtype_name, world, strategy, r)
            assert got[r]["first8"] == ref["first8"] and got[r]["last8"] == ref["last8"], (dtype_name, world, strategy, r)
            assert got[r]["sha256"] == ref["sha256"], (dtype_name, world, strategy, r)


def torch_rank(rank, world, init, out, accumulate):
    import torch.distributed as dist
    from torch.nn.parallel import DistributedDataParallel

    torch.set_num_threads(1)
    dist.init_process_group("gloo", init_method=f"file://{init}", rank=rank, world_size=world)
    torch.manual_seed(0)
    text = synthetic(20_000)
    model = GPT(CFG)
    ddp = DistributedDataParallel(model)
    opt = torch.optim.AdamW(model.parameters(), lr=3e-3, weight_decay=0.1, foreach=False)
    losses = []
    for step in range(6):
        for micro in range(accumulate):
            x, y = text.batch(step * accumulate + micro, 8, CFG.seq, rank=rank, world=world)
            if micro < accumulate - 1:
                with ddp.no_sync():
                    loss = ddp(x, y)
                    (loss / accumulate).backward()
            else:
                loss = ddp(x, y)
                (loss / accumulate).backward()
            losses.append(loss.item())
        opt.step()
        opt.zero_grad()
    torch.save((losses, torch.cat([p.detach().reshape(-1) for p in model.parameters()])), f"{out}.{rank}")
    dist.destroy_process_group()


def run_torch_ddp(accumulate=1):
    import torch.multiprocessing as mp

    with tempfile.TemporaryDirectory() as d:
        mp.spawn(torch_rank, args=(2, os.path.join(d, "init"), os.path.join(d, "out"), accumulate), nprocs=2)
        return [torch.load(os.path.join(d, f"out.{r}")) for r in range(2)]


def test_two_ranks_match_torch_ddp_and_adamw_bit_for_bit():
    """With 2 ranks the average is (a / 2) + (b / 2) in any order, so DDP and all
    three ZeRO stages must equal torch DDP + torch AdamW: every loss, every weight."""
    ref = run_torch_ddp()
    for strategy, bucket in (("ddp", 64 << 10), ("zero1", 4 << 10), ("zero2", 4 << 10), ("zero3", 4 << 10)):
        ours = cpu_launch(train_rank, 2, strategy, bucket, 6, 8, slot_bytes=512)
        for r in range(2):
            assert ours[r]["losses"] == ref[r][0], (strategy, r)
            assert torch.equal(ours[r]["weights"], ref[r][1]), (strategy, r)


def test_gradient_accumulation_matches_torch_ddp():
    ref = run_torch_ddp(accumulate=2)
    ours = cpu_launch(train_rank, 2, "ddp", 1 << 20, 6, 8, 2, slot_bytes=4096)
    assert ours[0]["losses"] == ref[0][0]
    assert torch.equal(ours[0]["weights"], ref[0][1])


def test_wrappers_refuse_a_group_without_the_gather_helpers():
    class Bare:
        size, rank = 1, 0

    with pytest.raises(TypeError, match="pack"):
        DDP(GPT(CFG), Bare())
    with pytest.raises(TypeError, match="pack"):
        ZeRO(GPT(CFG), Bare(), 2)
    with pytest.raises(ValueError):
        ZeRO(GPT(CFG), Bare(), 3)


class _Arenas:
    """What ShardHome and DDP ask of a group's arenas, on the CPU: the allocator of tandem_amd.Group.shared_empty
    (256-byte aligned, a new arena when `grow` is given and the tensor does not fit) over plain tensors."""

    ARENA_LIMIT = (1 << 31) - 4096

    def __init__(self, rank, size):
        self.rank, self.size = rank, size
        self.arenas, self.used = [], 0

    def shared_empty(self, numel, dtype=torch.float32, grow=None):
        es = torch.empty(0, dtype=dtype).element_size()
        need = numel * es
        at = -(-self.used // 256) * 256
        if not self.arenas or at + need > self.arenas[-1].numel():
            assert grow is not None or not self.arenas
            self.arenas.append(torch.zeros(max(need, min(int(grow or 0), self.ARENA_LIMIT)), dtype=torch.uint8))
            at = 0
        self.used = at + need
        return self.arenas[-1][at:at + need].view(dtype)

    def arena_offset(self, t):
        for k, a in enumerate(self.arenas):
            off = t.data_ptr() - a.data_ptr()
            if 0 <= off and off + t.numel() * t.element_size() <= a.numel():
                return (k << 31) + off
        return None


@pytest.mark.parametrize("seed", range(8))
def test_shard_home_lays_units_out_in_slabs(seed, monkeypatch):
    """Every unit's shard lies inside one slab, no two shards of a rank overlap, a slab ends before the limit unless one
    unit alone is longer, and every rank computes the same places for every rank."""
    import random

    from tandem_amd.fsdp import ShardHome

    rng = random.Random(seed)
    world = rng.choice([2, 3, 4, 8])
    monkeypatch.setattr(ShardHome, "SLAB_BYTES", rng.choice([4096, 16384, 1 << 20]))
    units = []
    for _ in range(rng.randrange(1, 20)):
        total = rng.choice([0, 1, 7, 1000, 5000, 40_000])
        units.append([total // world + (1 if q < total % world else 0) for q in range(world)])
    homes = []
    before = rng.choice([0, 0, 3, 499])  # something of the group's own before the shards: the same on every rank
    for r in range(world):
        g = _Arenas(r, world)
        if before:
            g.shared_empty(before)
        homes.append((ShardHome(g, units, torch.float32), g))
    cap = ShardHome.SLAB_BYTES // 4
    for r, (home, g) in enumerate(homes):
        spans = []
        for k, sizes in enumerate(units):
            shard = home.shard(k, sizes[r])
            assert shard.numel() == sizes[r]
            offs = home.peer_offsets(k)
            assert offs == homes[0][0].peer_offsets(k)  # the same on every rank
            if sizes[r]:
                assert g.arena_offset(shard) == offs[r] and offs[r] % 128 == 0
                spans.append((offs[r], offs[r] + 4 * sizes[r]))
        spans.sort()
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
        for slab in home.slabs:
            alone = any(max(-(-s // 32) * 32 for s in sizes) >= slab.numel() for sizes in units)
            assert slab.numel() <= cap or alone


class _ArenaGroup(_Arenas):
    def broadcast(self, t, root=0, async_op=False):
        return t

    def pack(self, flat, pieces):
        for at, t in pieces:
            flat[at:at + t.numel()] = t.reshape(-1)


@pytest.mark.parametrize("slab_bytes", [2048, 8192, 1 << 30])
def test_ddp_carves_its_buckets_from_slabs(slab_bytes, monkeypatch):
    """DDP(direct=True): every bucket lies inside one arena, buckets do not overlap, and a rebuild in another order
    carves the slabs that are there again instead of asking for more."""
    monkeypatch.setattr(DDP, "SLAB_BYTES", slab_bytes)
    torch.manual_seed(0)
    model = torch.nn.Sequential(*[torch.nn.Linear(17, 17) for _ in range(6)], torch.nn.Linear(17, 3))
    g = _ArenaGroup(0, 2)
    z = DDP(model, g, bucket_bytes=1024, direct=True)

    def check():
        spans = []
        for b in z.buckets:
            off = g.arena_offset(b.flat)
            assert off is not None and off % 256 == 0
            spans.append((off, off + 4 * b.flat.numel()))
            assert sum(p.numel() for p in b.params) == b.flat.numel()
        spans.sort()
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
        assert sorted(id(p) for b in z.buckets for p in b.params) == sorted(id(p) for p in z.params)

    check()
    arenas = len(g.arenas)
    assert arenas >= (3 if slab_bytes == 2048 else 1)
    z._build(list(z.params))  # the order in which the gradients turned out to arrive
    check()
    assert len(g.arenas) <= arenas + 1


class _FailingGroup:
    """One rank whose second all_reduce fails when waited for on the host; a wait that only orders the stream
    (what tandem_amd.Group offers as Work.wait(stream_ordered=True)) returns without a word, as it does on the GPU
    when the collective has not run yet."""

    size, rank, stream_ordered_waits = 1, 0, True

    class _Work:
        def __init__(self, group, fails):
            self.group, self.fails = group, fails

        def wait(self, stream_ordered=False):
            self.group.waits.append("stream" if stream_ordered else "host")
            if self.fails and not stream_ordered:
                raise RuntimeError("all_reduce: rank 1 did not answer in time")

    def __init__(self):
        self.calls, self.waits = 0, []

    def broadcast(self, t, root=0, async_op=False):
        return t

    def pack(self, flat, pieces):
        for off, t in pieces:
            flat[off:off + t.numel()].copy_(t.reshape(-1))

    def all_reduce(self, t, op="sum", async_op=False, **_):
        self.calls += 1
        return self._Work(self, fails=self.calls == 2)

    def all_gather(self, t, sizes=None, async_op=False, **_):
        work = self._Work(self, fails=False)
        return work if async_op else work.wait()


def test_a_failed_bucket_raises_from_backward_before_any_step():
    """DDP's default waits for its buckets on the host at the end of backward, as the reference's does
    (tandem/ddp.py:111-115): a bucket whose all-reduce fails raises from that backward, so no optimizer step is
    taken on gradients that were never reduced. Ordering only the stream is opt-in, and then this backward returns."""
    torch.manual_seed(0)
    text = synthetic(5_000)
    x, y = text.batch(0, 4, CFG.seq)
    g = _FailingGroup()
    z = DDP(GPT(CFG), g, bucket_bytes=4 << 10)
    assert z.stream_ordered is False and len(z.buckets) > 2
    before = [p.detach().clone() for p in z.module.parameters()]
    with pytest.raises(RuntimeError, match="did not answer"):
        z(x, y).backward()
    assert set(g.waits) == {"host"}
    assert all(torch.equal(a, b) for a, b in zip(before, z.module.parameters()))
    g = _FailingGroup()
    z = DDP(GPT(CFG), g, bucket_bytes=4 << 10, stream_ordered=True)
    z(x, y).backward()  # the failure is the next collective's to raise (tests/test_gpu_group.py)
    assert set(g.waits) == {"stream"}


def test_zero_waits_for_its_all_gather_on_the_host_unless_asked():
    torch.manual_seed(0)
    text = synthetic(5_000)
    x, y = text.batch(0, 4, CFG.seq)
    for ordered, want in ((False, "host"), (True, "stream")):
        g = _FailingGroup()
        g.calls = 10  # nothing fails here
        z = ZeRO(GPT(CFG), g, 1, OracleShardedAdamW(lr=3e-3, weight_decay=0.1), 4 << 10, stream_ordered=ordered)
        z(x, y).backward()
        g.waits.clear()
        z.step()
        assert g.waits == [want], (ordered, g.waits)


def test_make_sync_has_the_references_shape():
    """Group.make_sync(ctx, size, slots) -> (full, free, barrier), as the reference's launcher calls it
    (tandem/comm.py:175-181,537 there); the Group takes the tuple or the barrier alone."""
    import multiprocessing as mp

    from tandem_amd import Group

    full, free, barrier = Group.make_sync(mp.get_context("spawn"), 3, 2)
    assert len(full) == len(free) == 9 and barrier.parties == 3
    assert not full[0].acquire(block=False) and free[0].acquire(block=False) and free[0].acquire(block=False)
    assert not free[0].acquire(block=False)
