"""End to end on the GPU: processes sharing the MI355X through Group(backend="hip")
train the small GPT with DDP, ZeRO-1, ZeRO-2 and FSDP. With 2 ranks the average is
(a / 2) + (b / 2) in any order, so all four strategies (and one process that
computes both ranks' gradients itself) must agree bit for bit: every loss, every
weight. Mirrors tests/test_ddp.py, tests/test_zero.py and
tests/test_engine_cuda.py:100-127 of the reference. Run with -m gpu."""

import pytest
import torch

pytestmark = pytest.mark.gpu

STEPS, BATCH = 4, 8
LR, WD = 3e-3, 0.1
TIMEOUT = 90.0


def cfg():
    from tandem_amd.model import Config

    return Config(seq=32, layers=2, heads=2, dim=32)


def deterministic():
    torch.backends.cuda.enable_flash_sdp(False)
    torch.backends.cuda.enable_mem_efficient_sdp(False)
    torch.backends.cuda.matmul.allow_tf32 = False


def train_rank(g, strategy, bucket_bytes, steps, batch, accumulate=1, zero_every=1):
    from tandem_amd import ShardedAdamW
    from tandem_amd.data import synthetic
    from tandem_amd.ddp import DDP
    from tandem_amd.model import GPT
    from tandem_amd.zero import FSDP, ZeRO

    deterministic()
    c = cfg()
    torch.manual_seed(0)
    text = synthetic(20_000)
    model = GPT(c).to(g.device)
    extra = {}
    # a trailing "d": buckets and flat buffers in the shared arenas, collectives arena to arena;
    # "f": that, and ZeRO-2's reduce-scatters, update and all-gather as one launch per rank
    if strategy.startswith("ddp"):
        z = DDP(model, g, bucket_bytes=bucket_bytes, direct=strategy.endswith("d"))
        opt = torch.optim.AdamW(model.parameters(), lr=LR, weight_decay=WD, foreach=False, fused=False)
    else:
        sopt = ShardedAdamW(lr=LR, weight_decay=WD, order="device")  # torch's GPU op order, to compare with torch.optim.AdamW
        stage = int(strategy[4])
        if stage < 3:
            z = ZeRO(model, g, stage, sopt, bucket_bytes, direct=strategy[-1] in "df", fused_step=strategy.endswith("f"))
            assert z.direct == (strategy[-1] in "df") and z.fused_step == strategy.endswith("f")
        else:  # "zero3": shards in the shared arena, gathered directly; "zero3s": staged through the slots
            z = FSDP(model, g, sopt, direct=not strategy.endswith("s"))
            assert z._direct == (not strategy.endswith("s"))
    losses = []
    for step in range(steps):
        for micro in range(accumulate):
            x, y = text.batch(step * accumulate + micro, batch, c.seq, rank=g.rank, world=g.size, device=g.device)
            if micro < accumulate - 1 and strategy.startswith("ddp"):  # accumulate locally, reduce with the last micro-batch
                with z.no_sync():
                    loss = z(x, y)
                    (loss / accumulate).backward()
            else:
                loss = z(x, y)
                (loss / accumulate).backward() if accumulate > 1 else loss.backward()
        losses.append(loss.item())
        if strategy.startswith("ddp"):
            opt.step()
            opt.zero_grad()
        else:
            z.step()
            if (step + 1) % zero_every == 0:
                z.zero_grad()
    if strategy.startswith("zero3"):
        w = z.full_parameters()
        extra = {"max_live": z.max_live, "live": z.live}
    else:
        w = torch.cat([p.detach().reshape(-1) for p in model.parameters()])
    if not strategy.startswith("ddp"):
        # what the reference's tests/test_zero.py:35-36,54 asks of the sharded strategies: two moments for this rank's shard
        # only, and from stage 2 on no full gradients left behind by a backward
        numel = sum(p.numel() for p in model.parameters())
        extra["state_ok"] = sopt.state_bytes() <= 2 * 4 * (numel // g.size + len(list(model.parameters())))
        if int(strategy[4]) >= 2:
            extra["no_full_grads"] = all(p.grad is None for p in model.parameters())
    torch.cuda.synchronize()
    return {"losses": losses, "weights": w.cpu(), **extra}


def train_rank_small_slabs(g, strategy, bucket_bytes, steps, batch):
    """The same run with slabs so small that the buckets (the shards) spread over several arenas."""
    from tandem_amd.ddp import DDP
    from tandem_amd.fsdp import ShardHome

    DDP.SLAB_BYTES, ShardHome.SLAB_BYTES = 24 << 10, 8 << 10
    out = train_rank(g, strategy, bucket_bytes, steps, batch)
    out["arenas"] = g.arena_count
    return out


def one_process(world, accumulate=1, zero_every=1):
    """Both ranks' gradients computed in this process, averaged as (a/2) + (b/2),
    torch AdamW on the GPU."""
    from tandem_amd.data import synthetic
    from tandem_amd.model import GPT

    deterministic()
    dev = torch.device("cuda", 0)
    c = cfg()
    torch.manual_seed(0)
    text = synthetic(20_000)
    model = GPT(c).to(dev)
    opt = torch.optim.AdamW(model.parameters(), lr=LR, weight_decay=WD, foreach=False, fused=False)
    losses = [[] for _ in range(world)]
    kept = None
    for step in range(STEPS):
        grads = []
        for r in range(world):
            for micro in range(accumulate):
                x, y = text.batch(step * accumulate + micro, BATCH, c.seq, rank=r, world=world, device=dev)
                loss = model(x, y)
                (loss / accumulate).backward() if accumulate > 1 else loss.backward()
            losses[r].append(loss.item())
            grads.append([p.grad.clone() for p in model.parameters()])
            opt.zero_grad()
        for i, p in enumerate(model.parameters()):
            mean = grads[0][i] / world + grads[1][i] / world
            p.grad = mean if kept is None else kept[i] + mean  # what a gradient shard holds when it was not zeroed
        opt.step()
        kept = None if (step + 1) % zero_every == 0 else [p.grad.clone() for p in model.parameters()]
        opt.zero_grad()
    return losses, torch.cat([p.detach().reshape(-1) for p in model.parameters()]).cpu()


def test_buckets_and_shards_spread_over_several_arenas():
    """An arena is one exported allocation of under 2 GiB: larger models take several. Forced here with tiny slabs."""
    from tandem_amd import launch

    ref_losses, ref_w = one_process(2)
    for s in ("ddpd", "zero3"):
        res = launch(train_rank_small_slabs, 2, s, 4 << 10, STEPS, BATCH, slot_bytes=4096, gpus=[0, 0], timeout=TIMEOUT)
        for r in range(2):
            assert res[r]["arenas"] >= 3, (s, res[r]["arenas"])
            assert res[r]["losses"] == ref_losses[r], (s, r)
            assert torch.equal(res[r]["weights"], ref_w), (s, r)


def test_two_ranks_all_strategies_agree_bit_for_bit():
    from tandem_amd import launch

    runs = {s: launch(train_rank, 2, s, 4 << 10, STEPS, BATCH, slot_bytes=4096, gpus=[0, 0], timeout=TIMEOUT)
            for s in ("ddp", "ddpd", "zero1", "zero1d", "zero2", "zero2d", "zero2f", "zero3", "zero3s")}
    ref_losses, ref_w = one_process(2)
    for s, res in runs.items():
        assert torch.equal(res[0]["weights"], res[1]["weights"]), f"{s}: the ranks drifted apart"
        for r in range(2):
            assert res[r]["losses"] == ref_losses[r], (s, r)
            assert torch.equal(res[r]["weights"], ref_w), (s, r)
    for s in ("zero3", "zero3s"):
        assert runs[s][0]["max_live"] <= 3 and runs[s][0]["live"] == 0
    for s, res in runs.items():
        if not s.startswith("ddp"):
            assert all(x["state_ok"] for x in res), f"{s}: optimizer state beyond this rank's shard"
            assert all(x.get("no_full_grads", True) for x in res), f"{s}: full gradients were kept"


def train_rank_typed(g, strategy, dtype_name, steps, batch):
    """The small GPT in bfloat16 or float64 under every strategy, stepped by ShardedAdamW in the reference's operation
    order (the reference's wrappers and its optimizer take any floating dtype). DDP has no sharded optimizer of its own:
    it applies the same per-element update to every parameter after its buckets are reduced, which is what the sharded
    strategies compute shard by shard."""
    from tandem_amd import ShardedAdamW
    from tandem_amd.data import synthetic
    from tandem_amd.ddp import DDP
    from tandem_amd.model import GPT
    from tandem_amd.zero import FSDP, ZeRO

    deterministic()
    dtype = getattr(torch, dtype_name)
    c = cfg()
    torch.manual_seed(0)
    text = synthetic(20_000)
    model = GPT(c).to(g.device).to(dtype)
    sopt = ShardedAdamW(lr=LR, weight_decay=WD)
    if strategy.startswith("ddp"):
        z = DDP(model, g, bucket_bytes=4 << 10, direct=strategy.endswith("d"))
    elif strategy.startswith("zero3"):
        z = FSDP(model, g, sopt, direct=not strategy.endswith("s"))
    else:
        fused = strategy.endswith("f")  # reduce-scatters, AdamW and all-gather as one launch per rank
        z = ZeRO(model, g, int(strategy[4]), sopt, 4 << 10, direct=strategy.endswith("d") or fused, fused_step=fused)
    losses = []
    for step in range(steps):
        x, y = text.batch(step, batch, c.seq, rank=g.rank, world=g.size, device=g.device)
        loss = z(x, y)
        loss.backward()
        losses.append(loss.item())
        if strategy.startswith("ddp"):
            with torch.no_grad():
                for i, p in enumerate(model.parameters()):
                    sopt.update(i, p.data.view(-1), p.grad.reshape(-1).contiguous())
            for p in model.parameters():
                p.grad = None
        else:
            z.step()
            z.zero_grad()
    w = z.full_parameters() if strategy.startswith("zero3") else torch.cat([p.detach().reshape(-1) for p in model.parameters()])
    torch.cuda.synchronize()
    assert w.dtype == dtype and all(m.dtype == dtype for _, m, _ in sopt.state.values())
    return {"losses": losses, "weights": w.cpu()}


@pytest.mark.parametrize("dtype_name", ["bfloat16", "float64"])
def test_bf16_and_f64_models_all_strategies_agree(dtype_name):
    """Two ranks, a bfloat16 and a float64 model: DDP, ZeRO-1, ZeRO-2 (also with its step as one launch per rank) and FSDP, through the slots and arena to arena, must
    end with the same weights bit for bit and see the same losses (at two ranks the average is (a/2) + (b/2) in any order,
    and the update is per element), and the model must learn. What the kernels compute for these types is pinned against
    the oracle elsewhere; this is the wrappers carrying the dtype through buckets, shards, optimizer state and gathers."""
    from tandem_amd import launch

    runs = {s: launch(train_rank_typed, 2, s, dtype_name, STEPS, BATCH, slot_bytes=4096, gpus=[0, 0], timeout=TIMEOUT)
            for s in ("ddp", "ddpd", "zero1", "zero1d", "zero2", "zero2d", "zero2f", "zero3", "zero3s")}
    ref = runs["ddp"]
    assert ref[0]["losses"][-1] < ref[0]["losses"][0]
    for s, res in runs.items():
        assert torch.equal(res[0]["weights"].view(torch.uint8), res[1]["weights"].view(torch.uint8)), f"{s}: the ranks drifted apart"
        for r in range(2):
            assert res[r]["losses"] == ref[r]["losses"], (s, r, dtype_name)
            assert torch.equal(res[r]["weights"].view(torch.uint8), ref[0]["weights"].view(torch.uint8)), (s, r, dtype_name)


def test_four_ranks_stay_in_step():
    """World 4: the ring's order now matters and is pinned elsewhere (kernels against
    the oracle, host logic against the reference's runs on the CPU); here the ranks
    must end with identical weights, the model must learn, and FSDP must never hold
    more than three units whole."""
    from tandem_amd import launch

    kept = {}
    for s in ("ddp", "ddpd", "zero1", "zero1d", "zero2", "zero2d", "zero2f", "zero3", "zero3s"):
        res = launch(train_rank, 4, s, 4 << 10, 6, 8, slot_bytes=1024, gpus=[0] * 4, timeout=TIMEOUT)
        kept[s] = res[0]
        for r in range(1, 4):
            assert torch.equal(res[0]["weights"], res[r]["weights"]), (s, r)
        mean_first = sum(res[r]["losses"][0] for r in range(4)) / 4
        mean_last = sum(res[r]["losses"][-1] for r in range(4)) / 4
        assert mean_last < mean_first, s
        if s.startswith("zero3"):
            assert all(x["max_live"] <= 3 and x["live"] == 0 for x in res)
    # arena to arena or through the slots: the same sums in the same order, so the same bits
    for direct, ring in (("ddpd", "ddp"), ("zero2d", "zero2"), ("zero2f", "zero2"), ("zero1d", "zero1")):
        assert kept[direct]["losses"] == kept[ring]["losses"], direct
        assert torch.equal(kept[direct]["weights"], kept[ring]["weights"]), direct


def test_gradient_accumulation_matches_one_process():
    """DDP.no_sync (tests/test_ddp.py:115-119 in the reference): two micro-batches, the
    first accumulated locally inside the buckets, the sum reduced with the second."""
    from tandem_amd import launch

    ref_losses, ref_w = one_process(2, accumulate=2)
    for s in ("ddp", "ddpd"):
        res = launch(train_rank, 2, s, 4 << 10, STEPS, BATCH, 2, slot_bytes=4096, gpus=[0, 0], timeout=TIMEOUT)
        for r in range(2):
            assert res[r]["losses"] == ref_losses[r], (s, r)
            assert torch.equal(res[r]["weights"], ref_w), (s, r)


def test_zero2_accumulation_with_and_without_the_fused_step():
    """ZeRO-2 accumulates by reducing every backward into the gradient shard. With
    fused_step the first backward is only packed; the second one must first reduce it
    the ordinary way, and the step after is the ordinary one: the same bits as without,
    at two ranks and (where the ring's order matters) at four."""
    from tandem_amd import launch

    for world, slot in ((2, 4096), (4, 1024)):
        runs = {s: launch(train_rank, world, s, 4 << 10, 4, 8, 2, slot_bytes=slot, gpus=[0] * world, timeout=TIMEOUT)
                for s in ("zero2", "zero2d", "zero2f")}
        for s in ("zero2d", "zero2f"):
            for r in range(world):
                assert runs[s][r]["losses"] == runs["zero2"][r]["losses"], (world, s, r)
                assert torch.equal(runs[s][r]["weights"], runs["zero2"][0]["weights"]), (world, s, r)


def test_stream_ordered_wait_gives_the_same_weights(monkeypatch):
    """TANDEM_HIP_WAIT=stream: wait() parks the training stream on a word the engine sets
    behind the collective's last kernel, and the host runs ahead. Same bits."""
    from tandem_amd import launch

    monkeypatch.setenv("TANDEM_HIP_WAIT", "stream")
    ref_losses, ref_w = one_process(2)
    for s in ("ddp", "ddpd", "zero2", "zero2f", "zero3"):
        res = launch(train_rank, 2, s, 4 << 10, STEPS, BATCH, slot_bytes=4096, gpus=[0, 0], timeout=TIMEOUT)
        for r in range(2):
            assert res[r]["losses"] == ref_losses[r], (s, r)
            assert torch.equal(res[r]["weights"], ref_w), (s, r)


def test_step_without_zero_grad_keeps_the_old_gradients():
    """tandem's ZeRO-2 zeroes its gradient shard only in zero_grad() (tandem/zero.py:165-170
    in the reference): a step() followed by another backward steps on the SUM of both
    gradients. The one-launch step never fills the shard, so it has to catch up here. Two
    ranks: equal to one process that keeps the gradients; four ranks: equal to the
    ordinary path, where the ring's order matters."""
    from tandem_amd import launch

    ref_losses, ref_w = one_process(2, zero_every=2)
    for s in ("zero2", "zero2d", "zero2f"):
        res = launch(train_rank, 2, s, 4 << 10, STEPS, BATCH, 1, 2, slot_bytes=4096, gpus=[0, 0], timeout=TIMEOUT)
        for r in range(2):
            assert res[r]["losses"] == ref_losses[r], (s, r)
            assert torch.equal(res[r]["weights"], ref_w), (s, r)
    runs = {s: launch(train_rank, 4, s, 4 << 10, 5, 8, 1, 3, slot_bytes=1024, gpus=[0] * 4, timeout=TIMEOUT) for s in ("zero2", "zero2f")}
    for r in range(4):
        assert runs["zero2f"][r]["losses"] == runs["zero2"][r]["losses"], r
        assert torch.equal(runs["zero2f"][r]["weights"], runs["zero2"][0]["weights"]), r


def mixed_dtypes(g, direct):
    """DDP over a model whose parameters are fp32 and bf16: a bucket ends where the dtype changes (tandem/ddp.py:56-68 in the
    reference), and every gradient must come out as g0/2 + g1/2 in its own dtype."""
    from tandem_amd.ddp import DDP

    class Mixed(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = torch.nn.Linear(48, 64)
            self.b = torch.nn.Linear(64, 64).to(torch.bfloat16)
            self.c = torch.nn.Linear(64, 8)

        def forward(self, x):
            return self.c(self.b(self.a(x).to(torch.bfloat16)).float())

    deterministic()
    dev = g.device
    torch.manual_seed(0)
    model = Mixed().to(dev)
    x = torch.randn(16, 48, device=dev, generator=torch.Generator(device=dev).manual_seed(10 + g.rank))
    model(x).square().mean().backward()
    local = [p.grad.clone() for p in model.parameters()]
    want = []
    for t in local:  # every rank's gradient, then the mean as the ring forms it at two ranks
        both = torch.empty(2 * t.numel(), device=dev, dtype=t.dtype)
        both[g.rank * t.numel():(g.rank + 1) * t.numel()] = t.reshape(-1)
        g.all_gather(both)
        want.append((both[:t.numel()] / 2 + both[t.numel():] / 2).view_as(t))
    model.zero_grad()
    z = DDP(model, g, bucket_bytes=8 << 10, direct=direct)
    dtypes = [b.flat.dtype for b in z.buckets]
    z(x).square().mean().backward()
    torch.cuda.synchronize()
    same = all(p.grad.dtype == w.dtype and torch.equal(p.grad.view(torch.int16 if w.dtype == torch.bfloat16 else torch.int32),
                                                        w.view(torch.int16 if w.dtype == torch.bfloat16 else torch.int32))
               for p, w in zip(model.parameters(), want))
    return same, [str(d) for d in dtypes]


@pytest.mark.parametrize("direct", [False, True])
def test_ddp_over_parameters_of_two_dtypes(direct):
    from tandem_amd import launch

    for same, dtypes in launch(mixed_dtypes, 2, direct, slot_bytes=4096, gpus=[0, 0], timeout=TIMEOUT):
        assert same
        assert "torch.bfloat16" in dtypes and "torch.float32" in dtypes and len(dtypes) >= 3
