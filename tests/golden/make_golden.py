"""Writes the golden fixtures in this directory by running the reference
implementation (tandem's Python engine, CPU processes) on small seeded inputs.

Run once, in the build container only, where the reference is mounted:

    python tests/golden/make_golden.py [/root/reference] [only: ring adamw adamw_dtypes plans data train train_dtypes train_accumulating]

The fixtures are data only (inputs, expected outputs, digests). They pin the
parts of the path that no test of the reference pins by itself:

  ring_w{2,3,4}.npz   floating-point summation order of the ring at world
                      sizes 2, 3 and 4 (all_reduce sum/avg, reduce_scatter with
                      even, uneven, empty and one-owner chunk sizes, including
                      the partial sums left in the other chunks; all_gather).
  ring_dtypes_w3.npz  fp64 / fp16 / bf16 all_reduce at world 3.
  adamw.npz           ShardedAdamW.update, 20 steps, the benchmark's hyper-parameters.
  adamw_dtypes.npz    the same update on bfloat16, float16 and float64 shards (the reference's
                      seven torch operations take any floating dtype), both lerp branches.
  plans.json          DDP / ZeRO bucket packing, shard sizes, bucket_sizes and the
                      GPT's parameter registration order and unit sizes.
  data.json           digests of synthetic() and Text.batch().
  train_*.json        losses and weight digests of DDP / ZeRO-1/2/3 training
                      runs (CPU, tiny GPT) at world sizes 2, 3 and 4.
  train_dtypes.json   the same runs with the model in bfloat16 and in float64, world sizes 2 and 3.
  train_accumulating.json   the same runs with two backward passes before every step, world sizes 2 and 3.

Nothing here is loaded by the library; tests read the fixtures only.
"""

import hashlib
import json
import os
import sys

sys.dont_write_bytecode = True  # the reference tree is read-only: leave no __pycache__ in it

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, REF)
HERE = os.path.dirname(os.path.abspath(__file__))

from tandem import launch  # noqa: E402
from tandem.data import synthetic  # noqa: E402
from tandem.ddp import DDP  # noqa: E402
from tandem.model import GPT, Config  # noqa: E402
from tandem.optim import ShardedAdamW  # noqa: E402
from tandem.zero import FSDP, ZeRO, _Flat, _split_sizes  # noqa: E402

N = 517  # odd: tensor_split gives uneven chunks
SLOT = 256  # bytes: every chunk travels as several pieces


def sha(t):
    return hashlib.sha256(t.detach().contiguous().cpu().numpy().tobytes()).hexdigest()


def rank_input(seed, rank, n, scale=1.0):
    g = torch.Generator().manual_seed(seed * 1000 + rank)
    return torch.randn(n, generator=g) * scale


def size_cases(n, w):
    uneven = [n // w] * w
    uneven[-1] += n - sum(uneven)
    uneven = uneven[1:] + uneven[:1]  # the rotation tests/test_comm.py uses
    holes = [0] * w
    holes[w - 1] = n  # ZeRO-2's usual case: one owner
    split = [0] * w
    split[0], split[1] = 5, n - 5  # a bucket that straddles a shard boundary
    empty_first = [0] + [n // (w - 1)] * (w - 1)
    empty_first[-1] += n - sum(empty_first)
    return {"uneven": uneven, "one_owner": holes, "straddle": split, "empty_first": empty_first}


def ring_rank(g, n):
    r, w = g.rank, g.size
    out = {}
    x = rank_input(0, r, n)
    out["in"] = x.clone()
    t = x.clone()
    g.all_reduce(t)
    out["ar_sum"] = t
    t = x.clone()
    g.all_reduce(t, op="avg")
    out["ar_avg"] = t
    t = x.clone()
    g.reduce_scatter(t, None, op="avg")
    out["rs_avg_even"] = t
    for name, sizes in size_cases(n, w).items():
        t = x.clone()
        g.reduce_scatter(t, sizes, op="avg")
        out[f"rs_avg_{name}"] = t
        t = x.clone()
        g.reduce_scatter(t, sizes, op="sum")
        out[f"rs_sum_{name}"] = t
        t = x.clone()
        g.all_gather(t, sizes)
        out[f"ag_{name}"] = t
    tiny = rank_input(7, r, w - 1)  # fewer elements than ranks: empty chunks from tensor_split
    out["tiny_in"] = tiny.clone()
    g.all_reduce(tiny, op="avg")
    out["tiny_ar_avg"] = tiny
    return {k: v.numpy() for k, v in out.items()}


def dtype_rank(g, n):
    out = {}
    for name, dt in (("f64", torch.float64), ("f16", torch.float16), ("bf16", torch.bfloat16)):
        x = rank_input(3, g.rank, n).to(dt)
        out[f"{name}_in"] = x.clone()
        t = x.clone()
        g.all_reduce(t)
        out[f"{name}_ar_sum"] = t
        t = x.clone()
        g.all_reduce(t, op="avg")
        out[f"{name}_ar_avg"] = t
    # 16-bit floats are stored as their bit patterns
    return {k: (v.view(torch.int16) if v.element_size() == 2 else v).numpy() for k, v in out.items()}


def write_ring():
    for w in (2, 3, 4):
        res = launch(ring_rank, w, N, slot_bytes=SLOT)
        flat = {"sizes_json": np.frombuffer(json.dumps(size_cases(N, w)).encode(), dtype=np.uint8)}
        for r, d in enumerate(res):
            for k, v in d.items():
                flat[f"r{r}_{k}"] = v
        np.savez_compressed(os.path.join(HERE, f"ring_w{w}.npz"), **flat)
    res = launch(dtype_rank, 3, 131, slot_bytes=64)
    flat = {}
    for r, d in enumerate(res):
        for k, v in d.items():
            flat[f"r{r}_{k}"] = v
    np.savez_compressed(os.path.join(HERE, "ring_dtypes_w3.npz"), **flat)


def write_adamw():
    n, steps = 1531, 20
    torch.set_num_threads(1)
    g = torch.Generator().manual_seed(11)
    p = torch.randn(n, generator=g) * 0.02
    p[:4] = torch.tensor([0.0, -0.0, 1e-30, -3e-39])  # zeros and a denormal
    out = {"p0": p.clone().numpy()}
    opt = ShardedAdamW(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    grads = []
    for s in range(steps):
        gs = torch.Generator().manual_seed(100 + s)
        gr = torch.randn(n, generator=gs) * 1e-3
        gr[:2] = 0.0
        grads.append(gr.numpy().copy())
        opt.update("k", p, gr)
        if s in (0, 1, steps - 1):
            _, m, v = opt.state["k"]
            out[f"p{s + 1}"], out[f"m{s + 1}"], out[f"v{s + 1}"] = p.clone().numpy(), m.clone().numpy(), v.clone().numpy()
    out["grads"] = np.stack(grads)
    # no weight decay, default betas: the other branch of update()
    p2 = torch.from_numpy(out["p0"]).clone()
    opt2 = ShardedAdamW(lr=1e-3, weight_decay=0.0)
    for s in range(3):
        opt2.update("k", p2, torch.from_numpy(grads[s]))
    out["nowd_p3"] = p2.numpy()
    out["hyper_json"] = np.frombuffer(json.dumps({
        "main": {"lr": 3e-4, "betas": [0.9, 0.95], "eps": 1e-8, "weight_decay": 0.1, "steps": steps},
        "nowd": {"lr": 1e-3, "betas": [0.9, 0.999], "eps": 1e-8, "weight_decay": 0.0, "steps": 3},
    }).encode(), dtype=np.uint8)
    np.savez_compressed(os.path.join(HERE, "adamw.npz"), **out)


def write_adamw_dtypes():
    """ShardedAdamW.update on bf16, f16 and f64 tensors: 20 steps with the benchmark's hyper-parameters, and 3 steps
    of the other branches (beta1 < 0.5, no weight decay). 16-bit tensors are stored as bit patterns."""
    n, steps = 773, 20
    torch.set_num_threads(1)
    out = {}

    def raw(t):
        return (t.view(torch.int16) if t.element_size() == 2 else t).numpy().copy()

    hyper = {"main": {"lr": 3e-4, "betas": [0.9, 0.95], "eps": 1e-8, "weight_decay": 0.1, "steps": steps},
             "other": {"lr": 1e-2, "betas": [0.3, 0.7], "eps": 1e-6, "weight_decay": 0.0, "steps": 3}}
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16), ("f64", torch.float64)):
        g = torch.Generator().manual_seed(21)
        p0 = (torch.randn(n, generator=g, dtype=torch.float64) * 0.02).to(dt)
        p0[:4] = torch.tensor([0.0, -0.0, 1e-30, -3e-39], dtype=torch.float64).to(dt)
        grads = []
        for s in range(steps):
            gr = (torch.randn(n, generator=torch.Generator().manual_seed(200 + s), dtype=torch.float64) * 1e-3).to(dt)
            gr[:2] = 0.0
            grads.append(gr)
        out[f"{name}_p0"] = raw(p0)
        out[f"{name}_grads"] = np.stack([raw(gr) for gr in grads])
        for case, h in hyper.items():
            p = p0.clone()
            opt = ShardedAdamW(lr=h["lr"], betas=tuple(h["betas"]), eps=h["eps"], weight_decay=h["weight_decay"])
            for s in range(h["steps"]):
                opt.update("k", p, grads[s])
                if s in (0, h["steps"] - 1):
                    _, m, v = opt.state["k"]
                    assert m.dtype == dt and v.dtype == dt
                    out[f"{name}_{case}_p{s + 1}"], out[f"{name}_{case}_m{s + 1}"], out[f"{name}_{case}_v{s + 1}"] = raw(p), raw(m), raw(v)
    out["hyper_json"] = np.frombuffer(json.dumps(hyper).encode(), dtype=np.uint8)
    np.savez_compressed(os.path.join(HERE, "adamw_dtypes.npz"), **out)


def names_of(model):
    return {p: n for n, p in model.named_parameters()}


def ddp_buckets(model, bucket_bytes):
    """The reference's packing rule, run on parameters without storage."""
    d = DDP.__new__(DDP)
    torch.nn.Module.__init__(d)
    d.bucket_bytes = bucket_bytes
    params = [p for p in model.parameters() if p.requires_grad]
    d._make_buckets(list(reversed(params)))
    nm = names_of(model)
    return [[nm[p] for p in b.params] for b in d.buckets]


def zero_buckets(model, bucket_bytes, world):
    """ZeRO.__init__'s packing loop needs a group; its two ingredients (the
    _Flat offsets and the greedy rule) are exercised through _Flat and a
    one-rank ZeRO instance built on meta tensors."""

    class OneRank:
        size, rank = 1, 0

        def broadcast(self, t, root=0):
            return t

    z = ZeRO(model, OneRank(), stage=2, optimizer=ShardedAdamW(), bucket_bytes=bucket_bytes)
    params = [p for p in model.parameters() if p.requires_grad]
    flat = _Flat(params, world, 0)
    return {
        "ranges": [[b.a, b.b] for b in z.buckets],
        "counts": [len(b.params) for b in z.buckets],
        "bucket_sizes": [flat.bucket_sizes(b.a, b.b) for b in z.buckets],
        "shard_sizes": flat.sizes,
    }


def write_plans():
    out = {}
    with torch.device("meta"):
        medium = GPT(Config.preset("medium"))
        small = GPT(Config(seq=32, layers=2, heads=2, dim=32))
    out["medium_params"] = [[n, list(p.shape)] for n, p in medium.named_parameters()]
    out["medium_units"] = [sum(p.numel() for p in m.parameters()) for m in medium.units()]
    out["small_params"] = [[n, list(p.shape)] for n, p in small.named_parameters()]
    out["medium_ddp_25MiB"] = ddp_buckets(medium, 25 << 20)
    out["small_ddp_64KiB"] = ddp_buckets(small, 64 << 10)
    out["small_ddp_4KiB"] = ddp_buckets(small, 4 << 10)
    out["medium_zero_25MiB_w4"] = zero_buckets(medium, 25 << 20, 4)
    with torch.device("meta"):
        small = GPT(Config(seq=32, layers=2, heads=2, dim=32))
    out["small_zero_4KiB_w3"] = zero_buckets(small, 4 << 10, 3)
    out["split_sizes"] = {f"{n}/{w}": _split_sizes(n, w) for n in (0, 1, 5, 10, 10007, 85842432) for w in (1, 2, 3, 4, 7)}
    with open(os.path.join(HERE, "plans.json"), "w") as f:
        json.dump(out, f, indent=0)


def write_data():
    text = synthetic(20_000)
    x, y = text.batch(3, 8, 32, rank=1, world=2)
    torch.manual_seed(0)
    model = GPT(Config(seq=32, layers=2, heads=2, dim=32))
    w = torch.cat([p.detach().reshape(-1) for p in model.parameters()])
    out = {
        "synthetic_20000_sha256": hashlib.sha256(text.data.to(torch.uint8).numpy().tobytes()).hexdigest(),
        "synthetic_first32": text.data[:32].tolist(),
        "batch_step3_b8_s32_rank1_world2_x": x.tolist(),
        "batch_step3_b8_s32_rank1_world2_y_sha256": sha(y),
        "gpt_small_seed0_sha256": sha(w),
        "gpt_small_seed0_first8": w[:8].tolist(),
        "gpt_small_numel": w.numel(),
    }
    with open(os.path.join(HERE, "data.json"), "w") as f:
        json.dump(out, f, indent=0)


CFG = Config(seq=32, layers=2, heads=2, dim=32)
STEPS, BATCH = 6, 12


def train_rank(g, strategy, bucket_bytes):
    torch.manual_seed(0)
    text = synthetic(20_000)
    model = GPT(CFG)
    losses = []
    if strategy == "ddp":
        z = DDP(model, g, bucket_bytes=bucket_bytes)
        opt = torch.optim.AdamW(model.parameters(), lr=3e-3, weight_decay=0.1, foreach=False)
    else:
        sopt = ShardedAdamW(lr=3e-3, weight_decay=0.1)
        stage = int(strategy[-1])
        z = ZeRO(model, g, stage, sopt, bucket_bytes) if stage < 3 else FSDP(model, g, sopt)
    for step in range(STEPS):
        x, y = text.batch(step, BATCH, CFG.seq, rank=g.rank, world=g.size)
        loss = z(x, y)
        loss.backward()
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
        extra = {}
    return {"losses": losses, "sha256": sha(w), "first8": w[:8].tolist(), "last8": w[-8:].tolist(), **extra}


def write_train():
    for world in (2, 3, 4):
        out = {"cfg": {"seq": 32, "layers": 2, "heads": 2, "dim": 32}, "steps": STEPS, "batch": BATCH,
               "lr": 3e-3, "weight_decay": 0.1, "bucket_bytes": 4 << 10, "torch": torch.__version__}
        for strategy in ("ddp", "zero1", "zero2", "zero3"):
            out[strategy] = launch(train_rank, world, strategy, 4 << 10, slot_bytes=1024)
        with open(os.path.join(HERE, f"train_w{world}.json"), "w") as f:
            json.dump(out, f, indent=0)


def train_rank_typed(g, strategy, bucket_bytes, dtype_name):
    """The same run with the model in another floating type: the reference's wrappers, engine and optimizer take any."""
    torch.manual_seed(0)
    text = synthetic(20_000)
    model = GPT(CFG).to(getattr(torch, dtype_name))
    losses = []
    if strategy == "ddp":
        z = DDP(model, g, bucket_bytes=bucket_bytes)
        opt = torch.optim.AdamW(model.parameters(), lr=3e-3, weight_decay=0.1, foreach=False)
    else:
        sopt = ShardedAdamW(lr=3e-3, weight_decay=0.1)
        stage = int(strategy[-1])
        z = ZeRO(model, g, stage, sopt, bucket_bytes) if stage < 3 else FSDP(model, g, sopt)
    for step in range(4):
        x, y = text.batch(step, BATCH, CFG.seq, rank=g.rank, world=g.size)
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
    raw = w.view(torch.int16) if w.element_size() == 2 else w
    return {"losses": losses, "sha256": sha(raw), "first8": w[:8].double().tolist(), "last8": w[-8:].double().tolist()}


def train_rank_accumulating(g, strategy, bucket_bytes, micro_batches, zero_every=1):
    """Several backward passes before each step: the reference's ZeRO and FSDP keep adding into their gradient
    (shard) until zero_grad() (tandem/zero.py:139-153,165-170,306-317), its DDP skips the all-reduce under no_sync()."""
    torch.manual_seed(0)
    text = synthetic(20_000)
    model = GPT(CFG)
    losses = []
    if strategy == "ddp":
        z = DDP(model, g, bucket_bytes=bucket_bytes)
        opt = torch.optim.AdamW(model.parameters(), lr=3e-3, weight_decay=0.1, foreach=False)
    else:
        sopt = ShardedAdamW(lr=3e-3, weight_decay=0.1)
        stage = int(strategy[-1])
        z = ZeRO(model, g, stage, sopt, bucket_bytes) if stage < 3 else FSDP(model, g, sopt)
    for step in range(3):
        for micro in range(micro_batches):
            x, y = text.batch(step * micro_batches + micro, BATCH, CFG.seq, rank=g.rank, world=g.size)
            if strategy == "ddp" and micro < micro_batches - 1:
                with z.no_sync():
                    loss = z(x, y)
                    (loss / micro_batches).backward()
            else:
                loss = z(x, y)
                (loss / micro_batches).backward()
            losses.append(loss.item())
        last = (step + 1) % zero_every == 0  # zero_every=2: every other step keeps its gradients for the next one
        if strategy == "ddp":
            opt.step()
            if last:
                opt.zero_grad()
        else:
            z.step()
            if last:
                z.zero_grad()
    w = z.full_parameters() if strategy == "zero3" else torch.cat([p.detach().reshape(-1) for p in model.parameters()])
    return {"losses": losses, "sha256": sha(w), "first8": w[:8].tolist(), "last8": w[-8:].tolist()}


def fsdp_rank_without_prefetch(g):
    torch.manual_seed(0)
    text = synthetic(20_000)
    z = FSDP(GPT(CFG), g, ShardedAdamW(lr=3e-3, weight_decay=0.1), prefetch=False)
    losses = []
    for step in range(3):
        x, y = text.batch(step, BATCH, CFG.seq, rank=g.rank, world=g.size)
        loss = z(x, y)
        loss.backward()
        losses.append(loss.item())
        z.step()
        z.zero_grad()
    return {"losses": losses, "sha256": sha(z.full_parameters()), "max_live": z.max_live, "live": z.live}


def write_train_accumulating():
    out = {"steps": 3, "batch": BATCH, "micro_batches": 2, "bucket_bytes": 4 << 10, "torch": torch.__version__}
    for world in (2, 3):
        out[str(world)] = {strategy: launch(train_rank_accumulating, world, strategy, 4 << 10, 2, slot_bytes=1024)
                           for strategy in ("ddp", "zero1", "zero2", "zero3")}
    # a step that is not followed by zero_grad(): the next backward adds to what is there (zero_grad after every second step)
    out["zero_grad_every_second_step"] = {str(world): {strategy: launch(train_rank_accumulating, world, strategy, 4 << 10, 1, 2, slot_bytes=1024)
                                                       for strategy in ("ddp", "zero1", "zero2", "zero3")} for world in (2, 3)}
    out["fsdp_without_prefetch"] = {str(world): launch(fsdp_rank_without_prefetch, world, slot_bytes=1024) for world in (2, 3)}
    with open(os.path.join(HERE, "train_accumulating.json"), "w") as f:
        json.dump(out, f, indent=0)


def write_train_dtypes():
    out = {"cfg": {"seq": 32, "layers": 2, "heads": 2, "dim": 32}, "steps": 4, "batch": BATCH, "lr": 3e-3, "weight_decay": 0.1,
           "bucket_bytes": 4 << 10, "torch": torch.__version__}
    for dtype_name in ("bfloat16", "float64"):
        out[dtype_name] = {}
        for world in (2, 3):
            out[dtype_name][str(world)] = {strategy: launch(train_rank_typed, world, strategy, 4 << 10, dtype_name, slot_bytes=1024)
                                           for strategy in ("ddp", "zero1", "zero2", "zero3")}
    with open(os.path.join(HERE, "train_dtypes.json"), "w") as f:
        json.dump(out, f, indent=0)


if __name__ == "__main__":
    writers = {"ring": write_ring, "adamw": write_adamw, "adamw_dtypes": write_adamw_dtypes, "plans": write_plans,
               "data": write_data, "train": write_train, "train_dtypes": write_train_dtypes,
               "train_accumulating": write_train_accumulating}
    only = sys.argv[2:] or list(writers)
    for name in only:
        writers[name]()
    print("golden fixtures", only, "written to", HERE)
