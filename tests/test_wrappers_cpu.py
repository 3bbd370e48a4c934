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


def train_rank(g, strategy, bucket_bytes, steps, batch, accumulate=1):
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
        if strategy == "ddp":
            opt.step()
            opt.zero_grad()
        else:
            z.step()
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
