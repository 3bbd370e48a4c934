"""Group(backend="hip"): ranks are processes sharing the one GPU through HIP IPC
memory and event handles. Mirrors the reference's tests/test_engine_cuda.py and
tests/test_comm.py, but every comparison is bit-exact against the CPU oracle
(and the reference engine's fixtures), at every world size. Run with -m gpu."""

import os

import numpy as np
import pytest
import torch

from helpers import bits, golden_npz, npz_json, seeded

pytestmark = pytest.mark.gpu

KINDS = {torch.float32: "f32", torch.float64: "f64", torch.float16: "f16", torch.bfloat16: "bf16", torch.int64: "i64",
         torch.int32: "i32", torch.int16: "i16", torch.int8: "i8", torch.uint8: "u8"}
TIMEOUT = 60.0


def to_np(t):
    t = t.detach().cpu()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def values(rank, n, dtype):
    g = torch.Generator().manual_seed(1234 + rank)
    if dtype.is_floating_point:
        return torch.randn(n, generator=g).to(dtype)
    if dtype == torch.int64:
        return torch.randint(-1000, 1000, (n,), generator=g)
    info = torch.iinfo(dtype)  # the narrower integers over their whole range: most sums wrap around
    return torch.randint(info.min, info.max + 1, (n,), generator=g).to(dtype)


def collectives(g, dtype, n):
    dev, w, r = g.device, g.size, g.rank
    out = {}
    x = values(r, n, dtype).to(dev)
    t = x.clone(); g.all_reduce(t); out["ar_sum"] = t.cpu()
    if dtype.is_floating_point:
        t = x.clone()
        work = g.all_reduce(t, op="avg", async_op=True)
        busy = torch.randn(256, 256, device=dev)
        for _ in range(4):
            busy = busy @ busy.T / 256  # the GPU works on something else meanwhile
        work.wait()
        out["ar_avg"] = t.cpu()
    sizes = [n // w + (1 if q < n % w else 0) for q in range(w)]
    sizes = sizes[1:] + sizes[:1]
    lo = sum(sizes[:r])
    for op in (("sum", "avg") if dtype.is_floating_point else ("sum",)):
        t = x.clone()
        mine = g.reduce_scatter(t, sizes, op=op)
        assert mine.data_ptr() == t.data_ptr() + lo * t.element_size() and mine.numel() == sizes[r]
        out[f"rs_{op}"] = t.cpu()
        t = x.clone()
        mine = g.reduce_scatter(t, sizes, op=op, partial_sums=False)  # the rest of t stays as it was
        assert mine.data_ptr() == t.data_ptr() + lo * t.element_size() and mine.numel() == sizes[r]
        out[f"rso_{op}"] = t.cpu()
    t = torch.zeros(n, dtype=dtype, device=dev)
    t[lo:lo + sizes[r]] = x[lo:lo + sizes[r]]
    g.all_gather(t, sizes)
    out["ag"] = t.cpu()
    t = x.clone(); g.broadcast(t, root=w - 1); out["bcast"] = t.cpu()
    if w == 2:
        got = torch.empty(n, dtype=dtype, device=dev)
        g.sendrecv(x, 1 - r, got, 1 - r)
        out["sendrecv"] = got.cpu()
    codes = torch.zeros(n, dtype=torch.complex64, device=dev)  # a dtype the kernels do not know: gathered as bytes
    codes[lo:lo + sizes[r]] = complex(r + 1, -r)
    g.all_gather(codes, sizes)
    out["bytes_ag_ok"] = bool(torch.equal(codes.cpu(), torch.cat([torch.full((sizes[q],), complex(q + 1, -q), dtype=torch.complex64) for q in range(w)])))
    flags = torch.arange(n, device=dev) % 2 == 0  # bool: copied as bytes
    if r != 0:
        flags = torch.zeros_like(flags)
    g.broadcast(flags, root=0)
    out["bool_bcast_ok"] = bool(torch.equal(flags.cpu(), torch.arange(n) % 2 == 0))
    torch.cuda.synchronize()
    return out


def collectives_of(g, dtypes, n):
    """One group, every dtype in turn (starting a group costs more than the collectives)."""
    return {str(d): collectives(g, d, n) for d in dtypes}


def test_a_group_of_one():
    """World 1 (tests/test_comm.py:55 in the reference runs its collectives at world 1 too):
    every collective leaves the tensor as it is, averaging included."""
    from tandem_amd import launch

    n = 1000
    (out,) = launch(collectives, 1, torch.float32, n, gpus=[0], timeout=TIMEOUT)
    x = values(0, n, torch.float32)
    for key in ("ar_sum", "ar_avg", "rs_sum", "rs_avg", "rso_sum", "rso_avg", "ag", "bcast"):
        assert torch.equal(out[key], x), key
    assert out["bool_bcast_ok"] and out["bytes_ag_ok"]


@pytest.mark.parametrize("world", [8, 9])
def test_eight_and_nine_ranks(world):
    """Eight ranks are the most the single-launch folds take (the staged forms); a group
    of nine goes through the slots' ring for everything. The ring's order for every
    chunk, whichever way it was summed."""
    from oracle import ring
    from tandem_amd import launch

    n, dtype = 10_007, torch.float32
    res = launch(collectives_of, world, [dtype], n, slot_bytes=4096, gpus=[0] * world, timeout=TIMEOUT)
    xs = [to_np(values(q, n, dtype)) for q in range(world)]
    sizes = [n // world + (1 if q < n % world else 0) for q in range(world)]
    sizes = sizes[1:] + sizes[:1]
    for r, per_dtype in enumerate(res):
        out = per_dtype[str(dtype)]
        assert np.array_equal(bits(to_np(out["ar_sum"])), bits(ring.expected_all_reduce(xs, False, "f32"))), r
        assert np.array_equal(bits(to_np(out["ar_avg"])), bits(ring.expected_all_reduce(xs, True, "f32"))), r
        assert np.array_equal(bits(to_np(out["rs_avg"])), bits(ring.expected_reduce_scatter(xs, sizes, True, "f32")[r])), r
        lo = sum(sizes[:r])
        own = ring.expected_reduce_scatter(xs, sizes, True, "f32")[r][lo:lo + sizes[r]]
        assert np.array_equal(bits(to_np(out["rso_avg"])[lo:lo + sizes[r]]), bits(own)), r
        assert np.array_equal(bits(to_np(out["ag"])), bits(ring.expected_all_gather(xs, sizes))), r
        assert np.array_equal(bits(to_np(out["bcast"])), bits(xs[world - 1])), r
        assert out["bool_bcast_ok"] and out["bytes_ag_ok"]


def choose(monkeypatch, algo):
    """The engine's ways through all_reduce / all_gather: staged through memory the
    peers map (default: tensors up to 32 MiB with one handshake; "two": the two-handshake
    passes also for small tensors; "small": 4 KiB halves, so n = 10,007 takes several
    passes and both halves are reused), or the reference's ring through the slots."""
    monkeypatch.setenv("TANDEM_HIP_ALGO", "ring" if algo == "ring" else "staged")
    if algo == "small":
        monkeypatch.setenv("TANDEM_HIP_STAGING_BYTES", "4096")
    else:
        monkeypatch.delenv("TANDEM_HIP_STAGING_BYTES", raising=False)
    if algo == "two":  # no one-handshake form for small tensors: the two-handshake passes at every size
        monkeypatch.setenv("TANDEM_HIP_SMALL_BYTES", "0")
    else:
        monkeypatch.delenv("TANDEM_HIP_SMALL_BYTES", raising=False)


@pytest.mark.parametrize("algo", ["staged", "two", "small", "ring"])
@pytest.mark.parametrize("world", [2, 3, 4])
def test_collectives_bit_exact(world, algo, monkeypatch):
    """4 KiB slots and n = 10,007: every collective runs through several pieces,
    reuses each slot, and ends on a short piece (tests/test_engine_cuda.py:84-96 in
    the reference, which only asks for a tolerance at world 3). Every dtype at world 2;
    at world 3 the narrower selection except in the several-pass cases; fp16 and fp64
    not again at world 4."""
    from oracle import ring
    from tandem_amd import launch

    dtypes = [torch.float32, torch.bfloat16, torch.float16, torch.int64, torch.float64, torch.int32, torch.int16, torch.int8, torch.uint8]
    if world == 4:
        dtypes = [torch.float32, torch.bfloat16, torch.int64, torch.int16, torch.uint8]
    elif world == 3 and algo not in ("small", "staged"):
        dtypes = [torch.float32, torch.bfloat16, torch.int8]
    choose(monkeypatch, algo)
    n = 10_007
    res = launch(collectives_of, world, dtypes, n, slot_bytes=4096, gpus=[0] * world, timeout=TIMEOUT)
    sizes = [n // world + (1 if q < n % world else 0) for q in range(world)]
    sizes = sizes[1:] + sizes[:1]
    for dtype in dtypes:
        kind = KINDS[dtype]
        xs = [to_np(values(q, n, dtype)) for q in range(world)]
        for r, per_dtype in enumerate(res):
            out = per_dtype[str(dtype)]
            assert np.array_equal(bits(to_np(out["ar_sum"])), bits(ring.expected_all_reduce(xs, False, kind))), (dtype, r, "ar_sum")
            if dtype.is_floating_point:
                assert np.array_equal(bits(to_np(out["ar_avg"])), bits(ring.expected_all_reduce(xs, True, kind))), (dtype, r, "ar_avg")
                assert np.array_equal(bits(to_np(out["rs_avg"])), bits(ring.expected_reduce_scatter(xs, sizes, True, kind)[r])), (dtype, r, "rs_avg")
            assert np.array_equal(bits(to_np(out["rs_sum"])), bits(ring.expected_reduce_scatter(xs, sizes, False, kind)[r])), (dtype, r, "rs_sum")
            lo = sum(sizes[:r])
            for op in (("sum", "avg") if dtype.is_floating_point else ("sum",)):
                got = to_np(out[f"rso_{op}"])
                own = ring.expected_reduce_scatter(xs, sizes, op == "avg", kind)[r][lo:lo + sizes[r]]
                assert np.array_equal(bits(got[lo:lo + sizes[r]]), bits(own)), (dtype, r, op, "owner's chunk")
                if algo != "ring":  # (the ring leaves its partial sums there in any case)
                    rest = np.ones(n, bool)
                    rest[lo:lo + sizes[r]] = False
                    assert np.array_equal(bits(got[rest]), bits(xs[r][rest])), (dtype, r, op, "rest untouched")
            assert np.array_equal(bits(to_np(out["ag"])), bits(ring.expected_all_gather(xs, sizes))), (dtype, r, "ag")
            assert np.array_equal(bits(to_np(out["bcast"])), bits(xs[world - 1])), (dtype, r, "bcast")
            if world == 2:
                assert np.array_equal(bits(to_np(out["sendrecv"])), bits(xs[1 - r])), dtype
            assert out["bool_bcast_ok"] and out["bytes_ag_ok"]


def tiny_slots(g, sizes_list):
    """The reference's tests/test_comm.py shape: integer-valued data, 64-byte slots,
    so that every message travels in many pieces and every slot is reused."""
    r, w = g.rank, g.size
    ok = True
    for dtype in (torch.float32, torch.int64, torch.bfloat16):
        hi = 30 if dtype == torch.bfloat16 else 100
        for n in sizes_list:
            def data(q, seed=0):
                gen = torch.Generator().manual_seed(seed * 1000 + q)
                return torch.randint(-hi, hi, (n,), generator=gen).to(dtype)
            want = sum(data(q).double() for q in range(w)) if n else torch.zeros(0, dtype=torch.float64)
            x = data(r).to(g.device)
            g.all_reduce(x)
            ok &= torch.equal(x.cpu().double(), want)
            sizes = [n // w] * w
            sizes[-1] += n - sum(sizes)
            sizes = sizes[1:] + sizes[:1]  # uneven chunks, one of them empty when n < w
            x = data(r).to(g.device)
            mine = g.reduce_scatter(x, sizes)
            lo = sum(sizes[:r])
            ok &= torch.equal(mine.cpu().double(), want[lo:lo + sizes[r]])
            full = want.to(dtype)
            x = torch.full((n,), -7, dtype=dtype)
            x[lo:lo + sizes[r]] = full[lo:lo + sizes[r]]
            x = x.to(g.device)
            g.all_gather(x, sizes)
            ok &= torch.equal(x.cpu(), full)
            x = data(r, seed=1).to(g.device)
            g.broadcast(x, root=w - 1)
            ok &= torch.equal(x.cpu(), data(w - 1, seed=1))
    x = torch.arange(37, dtype=torch.float32, device=g.device) * (r + 1)
    g.all_reduce(x, op="avg")
    want = sum(torch.arange(37, dtype=torch.float64) * (q + 1) for q in range(w)) / w
    ok &= torch.allclose(x.cpu().double(), want, rtol=0, atol=1e-5)
    torch.cuda.synchronize()
    return bool(ok)


@pytest.mark.parametrize("world", [2, 3])
def test_many_pieces_through_64_byte_slots(world):
    from tandem_amd import launch

    assert launch(tiny_slots, world, [0, 1, 5, 64, 1000], slot_bytes=64, gpus=[0] * world, timeout=TIMEOUT) == [True] * world


def replay_fixture(g, inputs, cases):
    x = torch.from_numpy(inputs[g.rank].copy()).to(g.device)
    out = {}
    t = x.clone(); g.all_reduce(t, op="avg"); out["ar_avg"] = t.cpu().numpy()
    t = x.clone(); g.reduce_scatter(t, None, op="avg"); out["rs_avg_even"] = t.cpu().numpy()
    for name, sizes in cases.items():
        t = x.clone(); g.reduce_scatter(t, sizes, op="avg"); out[f"rs_avg_{name}"] = t.cpu().numpy()
        t = x.clone(); g.all_gather(t, sizes); out[f"ag_{name}"] = t.cpu().numpy()
    return out


@pytest.mark.parametrize("algo", ["staged", "two", "small", "ring"])
@pytest.mark.parametrize("world", [2, 3, 4])
def test_reference_fixtures(world, algo, monkeypatch):
    """The same inputs and slot size as the reference engine's run."""
    from tandem_amd import launch

    choose(monkeypatch, algo)
    d = golden_npz(f"ring_w{world}.npz")
    inputs = [d[f"r{r}_in"] for r in range(world)]
    res = launch(replay_fixture, world, inputs, npz_json(d, "sizes_json"), slot_bytes=256, gpus=[0] * world, timeout=TIMEOUT)
    for r in range(world):
        for key, got in res[r].items():
            assert np.array_equal(bits(got), bits(d[f"r{r}_{key}"])), (world, r, key)


def direct_gather(g, numel):
    """Shards in the shared arena, read directly by the peers; fences around every rewrite."""
    w, r = g.size, g.rank
    sizes = [numel // w + (1 if q < numel % w else 0) for q in range(w)]
    pad = lambda n: (n + 3) // 4 * 4
    arena = g.shared_empty(2 * max(pad(s) for s in sizes) + 8)
    offs = [0] * w                               # unit 0 sits at the start of every arena
    offs2 = [pad(s) * 4 for s in sizes]          # unit 1 right behind it (bytes)
    mine, mine2 = arena[:sizes[r]], arena[pad(sizes[r]):pad(sizes[r]) + sizes[r]]
    out = []
    for round_ in range(3):
        g.fence()
        mine.copy_(values(r + 10 * round_, sizes[r], torch.float32).to(g.device))
        mine2.copy_(values(r + 10 * round_ + 5, sizes[r], torch.float32).to(g.device))
        g.fence()
        full = torch.full((numel,), -7.0, device=g.device)
        full2 = torch.full((numel,), -7.0, device=g.device)
        wk = g.gather_unit(full, mine, sizes, async_op=True, peer_offsets=offs)
        g.gather_unit(full2, mine2, sizes, peer_offsets=offs2)
        wk.wait()
        out.append((full.cpu(), full2.cpu()))
    assert g.arena_offset(mine2) == pad(sizes[r]) * 4 and g.arena_offset(torch.zeros(4, device=g.device)) is None
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("where", ["caller", "stream", "stream-words", "stream-events"])
@pytest.mark.parametrize("world", [2, 3])
def test_direct_gather_from_shared_arenas(world, where, monkeypatch):
    """The copies run on the caller's own stream (default) or on a side stream of the engine, ordered against the
    caller's stream by an event from a ring and a value word, by value words alone, or by fresh events."""
    from tandem_amd import launch

    monkeypatch.setenv("TANDEM_HIP_GATHER", where)

    numel = 100_003
    sizes = [numel // world + (1 if q < numel % world else 0) for q in range(world)]
    res = launch(direct_gather, world, numel, gpus=[0] * world, timeout=TIMEOUT)
    for out in res:
        for round_, (full, full2) in enumerate(out):
            want = torch.cat([values(q + 10 * round_, sizes[q], torch.float32) for q in range(world)])
            want2 = torch.cat([values(q + 10 * round_ + 5, sizes[q], torch.float32) for q in range(world)])
            assert torch.equal(full, want) and torch.equal(full2, want2), round_


def direct_collectives(g, dtype, ns):
    """Tensors in the shared arenas. Every rank first takes a different amount of
    the arena, so the tensors sit at different offsets on different ranks."""
    from tandem_amd import CommError

    dev, w, r = g.device, g.size, g.rank
    es = torch.empty(0, dtype=dtype).element_size()
    g.share_arena(32 << 20)
    used = [0] * w  # every rank tracks every rank's arena use, as a symmetric program can
    for q in range(w):
        used[q] = 256 * (q + 1)
    g.shared_empty(256 * (r + 1), torch.uint8)

    def alloc(n):
        at = [-(-u // 256) * 256 for u in used]
        for q in range(w):
            used[q] = at[q] + n * es
        t = g.shared_empty(n, dtype)
        assert n == 0 or g.arena_offset(t) == at[r]
        return t, at

    out = {}
    for n in ns:
        x = values(r, n, dtype).to(dev)
        sizes = [n // w + (1 if q < n % w else 0) for q in range(w)]
        sizes = sizes[1:] + sizes[:1]
        lo = sum(sizes[:r])
        for op in (("sum", "avg") if dtype.is_floating_point else ("sum",)):
            t, at = alloc(n)
            t.copy_(x)
            work = g.all_reduce(t, op=op, async_op=True, direct=at)
            assert work.wait() is t
            out[f"ar_{op}_{n}"] = t.cpu()
            t, at = alloc(n)
            t.copy_(x)
            mine = g.reduce_scatter(t, sizes, op=op, direct=at)
            assert mine.numel() == sizes[r] and (sizes[r] == 0 or mine.data_ptr() == t.data_ptr() + lo * es)
            out[f"rs_{op}_{n}"] = t.cpu()
        t, at = alloc(n)
        t.zero_()
        t[lo:lo + sizes[r]] = x[lo:lo + sizes[r]]
        g.all_gather(t, sizes, direct=at)
        out[f"ag_{n}"] = t.cpu()
    # the same offset on every rank: direct=True
    pad = max(used) - used[r]
    if pad:
        g.shared_empty(pad, torch.uint8)
    t = g.shared_empty(1000, dtype)
    t.copy_(values(r, 1000, dtype).to(dev))
    g.all_reduce(t, direct=True)
    out["ar_same"] = t.cpu()
    with pytest.raises(CommError, match="shared_empty"):
        g.all_reduce(torch.zeros(8, dtype=dtype, device=dev), direct=True)
    with pytest.raises(CommError, match="do not fit"):
        g.shared_empty(64 << 20, torch.uint8)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int64, torch.float64])
@pytest.mark.parametrize("world", [2, 3, 4])
def test_direct_collectives_bit_exact(dtype, world):
    """The arena-to-arena forms give the ring's bits: all_reduce and all_gather whole,
    reduce_scatter on the owner's chunk (the rest of the tensor stays as it was)."""
    from oracle import ring
    from tandem_amd import launch

    kind = KINDS[dtype]
    ns = (0, 1, 5, 1000, 10_007, 65_536 + 3)
    res = launch(direct_collectives, world, dtype, ns, gpus=[0] * world, timeout=TIMEOUT)
    for n in ns:
        xs = [to_np(values(q, n, dtype)) for q in range(world)]
        sizes = [n // world + (1 if q < n % world else 0) for q in range(world)]
        sizes = sizes[1:] + sizes[:1]
        for r, out in enumerate(res):
            lo = sum(sizes[:r])
            for op in (("sum", "avg") if dtype.is_floating_point else ("sum",)):
                want = ring.expected_all_reduce(xs, op == "avg", kind)
                assert np.array_equal(bits(to_np(out[f"ar_{op}_{n}"])), bits(want)), (n, r, op)
                ring_rs = ring.expected_reduce_scatter(xs, sizes, op == "avg", kind)[r]
                want = xs[r].copy()
                want[lo:lo + sizes[r]] = ring_rs[lo:lo + sizes[r]]
                assert np.array_equal(bits(to_np(out[f"rs_{op}_{n}"])), bits(want)), (n, r, op)
            assert np.array_equal(bits(to_np(out[f"ag_{n}"])), bits(ring.expected_all_gather(xs, sizes))), (n, r)
    xs = [to_np(values(q, 1000, dtype)) for q in range(world)]
    for out in res:
        assert np.array_equal(bits(to_np(out["ar_same"])), bits(ring.expected_all_reduce(xs, False, kind)))


def zero2_steps(g, ns, steps):
    """Group.zero2_step on flat buffers in the arenas: gradients differ per rank and step,
    parameters start equal; returns this rank's parameter buffer and optimizer state."""
    from tandem_amd import CommError, ShardedAdamW
    from tandem_amd.optim import step_scalars

    dev, w, r = g.device, g.size, g.rank
    g.share_arena(8 << 20)
    out = {}
    for n in ns:
        sizes = [n // w + (1 if q < n % w else 0) for q in range(w)]
        lo = sum(sizes[:r])
        params, grads = g.shared_empty(n), g.shared_empty(n)
        params.copy_(seeded(3, 0, n) * 0.02)
        opt = ShardedAdamW(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
        for step in range(steps):
            grads.copy_(seeded(100 + step, r, n) * 1e-3)
            scalars, m, v, order = opt.begin_step("flat", params[lo:lo + sizes[r]])
            got = g.zero2_step(params, grads, sizes, m, v, scalars, order)
            assert got is params
        out[n] = (params.cpu(), m.cpu(), v.cpu())
    # what it refuses
    n = 1000
    sizes = [n // w + (1 if q < n % w else 0) for q in range(w)]
    arena, plain = g.shared_empty(n), torch.zeros(n, device=dev)
    state = torch.zeros(sizes[r], device=dev)
    s = step_scalars(1.0, 3e-4, (0.9, 0.95), 1e-8, 0.1)
    refused = 0
    for p_, g_, m_, sz in ((plain, arena, state, sizes), (arena, plain, state, sizes), (arena, arena, torch.zeros(sizes[r] + 1, device=dev), sizes),
                           (arena, arena, state, sizes[:-1]), (arena.double(), arena, state, sizes)):
        try:
            g.zero2_step(p_, g_, sz, m_, m_.clone(), s, 0)
        except CommError:
            refused += 1
    out["refused"] = refused
    return out


@pytest.mark.parametrize("world", [2, 3, 4])
def test_zero2_step_in_one_launch_per_rank(world):
    """Every rank's parameters after the fused step equal the oracle's reduce-scatter,
    `0 + mine`, AdamW per shard and all-gather; each rank's state equals its shard's."""
    from oracle import ring
    from oracle.adamw import AdamW
    from tandem_amd import launch

    ns, steps = (0, 3, 1001, 40_007), 3
    res = launch(zero2_steps, world, ns, steps, gpus=[0] * world, timeout=TIMEOUT)
    for n in ns:
        sizes = [n // world + (1 if q < n % world else 0) for q in range(world)]
        want = (seeded(3, 0, n) * 0.02).numpy()
        opts = [AdamW(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1) for _ in range(world)]
        for step in range(steps):
            xs = [(seeded(100 + step, q, n) * 1e-3).numpy() for q in range(world)]
            outs = ring.expected_reduce_scatter(xs, sizes, True)
            for q in range(world):
                lo = sum(sizes[:q])
                opts[q].update("flat", want[lo:lo + sizes[q]], np.float32(0.0) + outs[q][lo:lo + sizes[q]])
        for r, out in enumerate(res):
            p, m, v = out[n]
            assert np.array_equal(bits(p.numpy()), bits(want)), (world, n, r)
            if sizes[r]:
                assert np.array_equal(bits(m.numpy()), bits(opts[r].state["flat"][1])), (world, n, r)
                assert np.array_equal(bits(v.numpy()), bits(opts[r].state["flat"][2])), (world, n, r)
    assert all(out["refused"] == 5 for out in res)


def zero2_steps_typed(g, name, ns, steps):
    """zero2_steps over buffers of another shard type: begin_step hands out the constants as doubles."""
    from tandem_amd import CommError, ShardedAdamW
    from tandem_amd._lib import AdamwHyper
    from tandem_amd.optim import step_scalars

    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f64": torch.float64}[name]
    w, r = g.size, g.rank
    g.share_arena(8 << 20)
    out = {}
    for n in ns:
        sizes = [n // w + (1 if q < n % w else 0) for q in range(w)]
        lo = sum(sizes[:r])
        params, grads = g.shared_empty(n, dtype), g.shared_empty(n, dtype)
        params.copy_((seeded(3, 0, n).double() * 0.02).to(dtype))
        opt = ShardedAdamW(lr=1e-3, betas=(0.9, 0.95), eps=1e-6, weight_decay=0.1)
        for step in range(steps):
            grads.copy_((seeded(100 + step, r, n).double() * (2e-2 if name == "f16" else 1e-3)).to(dtype))
            constants, m, v, order = opt.begin_step("flat", params[lo:lo + sizes[r]])
            assert isinstance(constants, AdamwHyper) and m.dtype == dtype
            assert g.zero2_step(params, grads, sizes, m, v, constants, order) is params
        view = (lambda t: t.cpu().view(torch.int16).numpy().view(np.uint16).copy()) if name != "f64" else (lambda t: t.cpu().numpy().copy())
        out[n] = (view(params), view(m), view(v))
    refused = 0
    n = 1000
    sizes = [n // w + (1 if q < n % w else 0) for q in range(w)]
    arena, state = g.shared_empty(n, dtype), torch.zeros(sizes[r], device=g.device, dtype=dtype)
    for constants, order in ((step_scalars(1.0, 3e-4, (0.9, 0.95), 1e-8, 0.1), 0), (opt.begin_step("other", arena[:sizes[r]])[0], 1)):
        try:  # fp32 constants with another dtype; the device order on another dtype
            g.zero2_step(arena, g.shared_empty(n, dtype), sizes, state, state.clone(), constants, order)
        except (CommError, ValueError):
            refused += 1
    out["refused"] = refused
    return out


@pytest.mark.parametrize("name", ["bf16", "f16", "f64"])
@pytest.mark.parametrize("world", [2, 3, 4])
def test_zero2_step_in_one_launch_per_rank_on_other_shard_types(world, name):
    """The same fused step between process ranks over bfloat16, float16 and float64 buffers
    (tdm_direct_zero2_step_typed): the ring's fold in the type's own rounding, 0 + mine, the typed AdamW,
    the new parameters in every rank's buffer; bit for bit with the oracle, state included, at worlds 2 to 4."""
    from oracle import ring
    from oracle.adamw import AdamW
    from tandem_amd import launch

    ns, steps = (0, 5, 1001, 40_007), 3
    dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f64": torch.float64}[name]
    raw = (lambda t: t.view(torch.int16).numpy().view(np.uint16).copy()) if name != "f64" else (lambda t: t.numpy().copy())
    res = launch(zero2_steps_typed, world, name, ns, steps, gpus=[0] * world, timeout=TIMEOUT)
    for n in ns:
        sizes = [n // world + (1 if q < n % world else 0) for q in range(world)]
        want = raw((seeded(3, 0, n).double() * 0.02).to(dtype))
        opts = [AdamW(lr=1e-3, betas=(0.9, 0.95), eps=1e-6, weight_decay=0.1, kind=name if name != "f64" else None) for _ in range(world)]
        for step in range(steps):
            xs = [raw((seeded(100 + step, q, n).double() * (2e-2 if name == "f16" else 1e-3)).to(dtype)) for q in range(world)]
            outs = ring.expected_reduce_scatter(xs, sizes, True, name)
            for q in range(world):
                lo = sum(sizes[:q])
                mine = outs[q][lo:lo + sizes[q]].copy()
                if name != "f64":
                    mine[mine == 0x8000] = 0  # 0 + (-0) = +0
                else:
                    mine = 0.0 + mine
                opts[q].update("flat", want[lo:lo + sizes[q]], mine)
        for r, out in enumerate(res):
            p, m, v = out[n]
            assert np.array_equal(bits(p), bits(want)), (world, n, r)
            if sizes[r]:
                assert np.array_equal(bits(m), bits(opts[r].state["flat"][1])), (world, n, r)
                assert np.array_equal(bits(v), bits(opts[r].state["flat"][2])), (world, n, r)
    assert all(out["refused"] == 2 for out in res)


def async_order(g):
    # several collectives in flight complete in submission order with the right values
    xs = [torch.full((3000 + k,), float(g.rank + k), device=g.device) for k in range(5)]
    works = [g.all_reduce(x, async_op=True) for x in xs]
    g.tracing = True
    big = torch.ones(1 << 22, device=g.device)
    w2 = g.all_reduce(big, op="avg", async_op=True)
    for k, (x, wk) in enumerate(zip(xs, works)):
        assert wk.wait() is x
        want = float(sum(q + k for q in range(g.size)))
        assert torch.equal(x.cpu(), torch.full((3000 + k,), want))
    w2.wait()
    torch.cuda.synchronize()
    assert w2.is_completed() and float(big.sum()) == float(1 << 22)
    assert len(g.trace) == 6 and g.trace[-1][0] == "all_reduce" and g.trace[-1][3] == 4 << 22
    assert all(t1 >= t0 for _, t0, t1, _ in g.trace)
    return True


def test_async_and_large_message_default_slots():
    from tandem_amd import launch

    assert launch(async_order, 3, gpus=[0, 0, 0], timeout=TIMEOUT) == [True, True, True]


def traced(g, mib, gemms):
    """The reference's protocol for a collective's own time (bench/engine_one_gpu.py
    there: the span from Group.trace while the default stream is idle, then while
    it runs matmuls the collective does not depend on)."""
    import time

    from tandem_amd.profile import summarize

    n = mib * (1 << 20) // 4
    x = torch.ones(n, device=g.device)
    a = torch.randn(2048, 2048, device=g.device)
    g.all_reduce(x)
    a @ a
    torch.cuda.synchronize()
    # Whatever the algorithm, a rank reads W chunks and writes one to fold its own, and
    # reads and writes the W-1 others: that much traffic at HBM peak bounds the span.
    chunk = 4 * n / g.size
    floor = ((g.size + 1) + 2 * (g.size - 1)) * chunk / 8e12
    out = {}
    for mode in ("idle", "busy", "host"):
        os.environ["TANDEM_HIP_TRACE"] = "host" if mode == "host" else "device"
        g.barrier()
        x.fill_(1.0)
        torch.cuda.synchronize()
        g.trace.clear()
        g.waits.clear()
        g.tracing = True
        t = time.perf_counter()
        w = g.all_reduce(x, async_op=True)
        for _ in range(gemms if mode == "busy" else 0):
            a @ a
        w.wait()
        waited = time.perf_counter()
        torch.cuda.synchronize()
        end = time.perf_counter()
        g.tracing = False
        assert len(g.trace) == 1
        name, s, e, nbytes = g.trace[-1]
        assert name == "all_reduce" and nbytes == 4 * n
        assert torch.equal(x, torch.full_like(x, float(g.size)))
        if mode == "host":  # the progress thread's own clock readings
            assert t <= s <= e <= end
        else:  # the GPU's span, on the host's clock: inside the bracket, no shorter than the traffic allows
            assert t - 1e-3 <= s <= e <= end + 1e-3, (mode, s - t, e - t, end - t)
            assert e - s >= floor, (mode, e - s, floor)
        summary = summarize([], g.trace, list(g.waits), end - t)
        assert summary["comm_bytes"] == 4 * n and abs(summary["comm_s"] - (e - s)) < 1e-12
        assert summary["exposed_comm_s"] <= summary["comm_s"] + 1e-12 and 0.0 <= summary["overlap"] <= 1.0
        out[mode] = {"span_ms": (e - s) * 1e3, "wait_returned_ms": (waited - t) * 1e3, "total_ms": (end - t) * 1e3}
    os.environ.pop("TANDEM_HIP_TRACE", None)
    return out


def test_trace_holds_the_gpu_span_of_a_collective():
    from tandem_amd import launch

    res = launch(traced, 2, 64, 40, gpus=[0, 0], timeout=TIMEOUT)
    print("\ntrace of a 64 MiB all_reduce, 2 ranks:", res[0])
    for r in res:
        # behind 40 matmuls the collective still finishes long before they do
        assert r["busy"]["span_ms"] < r["busy"]["total_ms"]


def errors(g):
    from tandem_amd import CommError

    seen = []
    for bad in (lambda: g.all_reduce(torch.zeros(4)),  # a CPU tensor
                lambda: g.all_reduce(torch.zeros(8, device=g.device)[::2]),  # not contiguous
                lambda: g.all_reduce(torch.zeros(4, device=g.device), op="max"),
                lambda: g.reduce_scatter(torch.zeros(10, device=g.device), [5, 6]),
                lambda: g.all_reduce(torch.zeros(4, device=g.device, dtype=torch.int64), op="avg"),
                lambda: g.all_reduce(torch.zeros(4, device=g.device, dtype=torch.bool))):
        try:
            bad()
            seen.append(False)
        except CommError:
            seen.append(True)
    # Sums of dtypes outside the nine the kernels know are refused by name, where the reference's engine
    # falls back to add_ (tandem/csrc/collectives.cpp:254-256 there); copying them works, as bytes.
    texts = []
    for dtype in (torch.bool, torch.complex64, torch.uint16):
        for call in (g.all_reduce, g.reduce_scatter):
            try:
                call(torch.zeros(8, device=g.device, dtype=dtype))
                texts.append("accepted")
            except CommError as e:
                texts.append(str(e))
        t = torch.full((8,), g.rank + 1).to(dtype).to(g.device)
        g.broadcast(t, root=1)
        texts.append(bool(torch.equal(t.cpu().view(torch.uint8), torch.full((8,), 2).to(dtype).view(torch.uint8))))
    g.barrier()
    return seen, texts


def test_errors_surface_as_commerror():
    from tandem_amd import launch

    for seen, texts in launch(errors, 2, gpus=[0, 0], timeout=TIMEOUT):
        assert seen == [True] * 6
        for k, dtype in enumerate(("torch.bool", "torch.complex64", "torch.uint16")):
            assert texts[3 * k] == texts[3 * k + 1] == f"the hip backend cannot reduce {dtype}", texts[3 * k]
            assert texts[3 * k + 2] is True


def failing(g):
    if g.rank == 1:
        raise ValueError("boom")
    return True


def test_error_propagates_from_a_rank():
    from tandem_amd import launch

    import glob

    before = set(glob.glob("/dev/shm/tandem-*"))
    with pytest.raises(Exception, match="boom"):
        launch(failing, 2, gpus=[0, 0], timeout=10.0)
    # the rank that was killed because its peer failed never unlinked its shared-memory region: launch() did
    assert set(glob.glob("/dev/shm/tandem-*")) <= before
    assert launch(failing, 1, gpus=[0], timeout=10.0) == [True]
    assert set(glob.glob("/dev/shm/tandem-*")) <= before


def out_of_step(g):
    from tandem_amd import CommError

    x = torch.ones(1000, device=g.device)
    if g.rank == 0:
        try:
            g.all_reduce(x)  # rank 1 never joins: the wait for its piece must time out, on the host
        except CommError as e:
            return "timed out" in str(e.__cause__)
        return False
    return True


def test_a_missing_peer_times_out_on_the_host():
    """Forced from the host: every kernel that was launched still finishes; the
    progress thread gives up waiting for a message after the group's timeout."""
    from tandem_amd import launch

    with pytest.raises(Exception, match="timed out|barrier|drained"):
        launch(out_of_step, 2, gpus=[0, 0], timeout=3.0)


def mixed_sequence(g, seed, count):
    """The same seeded sequence of collectives on every rank, sizes and kinds mixed, some
    waited for at once and some later, in submission order."""
    import random

    rng = random.Random(seed)
    w, r, dev = g.size, g.rank, g.device
    results, pending = [], []
    for k in range(count):
        kind = rng.choice(["ar_sum", "ar_avg", "ag", "rs", "rso", "bcast", "barrier"])
        n = rng.choice([0, 1, 7, 300, 1023, 4096, 10_007, 40_000])
        cut = sorted(rng.randint(0, n) for _ in range(w - 1))
        sizes = [b - a for a, b in zip([0] + cut, cut + [n])]
        later = rng.random() < 0.5
        x = (torch.randn(n, generator=torch.Generator().manual_seed(seed * 7919 + k * 31 + r)) * 0.5).to(dev)
        if kind == "barrier":
            g.barrier()
            continue
        if kind.startswith("ar"):
            work = g.all_reduce(x, op=kind[3:], async_op=True)
        elif kind == "ag":
            work = g.all_gather(x, sizes, async_op=True)
        elif kind == "bcast":
            work = g.broadcast(x, root=k % w, async_op=True)
        else:
            work = g.reduce_scatter(x, sizes, op="avg", async_op=True, partial_sums=kind == "rs")
        pending.append((k, kind, sizes, x, work))
        if not later:
            while pending:  # waits happen in submission order
                k2, kind2, sizes2, x2, w2 = pending.pop(0)
                w2.wait()
                results.append((k2, kind2, sizes2, x2.cpu().numpy()))
    for k2, kind2, sizes2, x2, w2 in pending:
        w2.wait()
        results.append((k2, kind2, sizes2, x2.cpu().numpy()))
    torch.cuda.synchronize()
    return results


@pytest.mark.parametrize("algo", ["staged", "small", "stream"])
@pytest.mark.parametrize("world", [2, 3])
def test_a_long_mixed_sequence_stays_bit_exact(world, algo, monkeypatch):
    """Forty collectives of mixed kinds and sizes in flight behind one another: the
    staging halves, slots and handshakes are reused in every order the mix produces."""
    from oracle import ring
    from tandem_amd import launch

    choose(monkeypatch, "staged" if algo == "stream" else algo)
    if algo == "stream":  # wait() parks the caller's stream on a word instead of blocking the host
        monkeypatch.setenv("TANDEM_HIP_WAIT", "stream")
    seed, count = 11 + world, 40
    res = launch(mixed_sequence, world, seed, count, slot_bytes=4096, gpus=[0] * world, timeout=TIMEOUT)
    for r, results in enumerate(res):
        for k, kind, sizes, got in results:
            n = sum(sizes)
            xs = [(torch.randn(n, generator=torch.Generator().manual_seed(seed * 7919 + k * 31 + q)) * 0.5).numpy() for q in range(world)]
            lo = sum(sizes[:r])
            if kind.startswith("ar"):
                want = ring.expected_all_reduce(xs, kind == "ar_avg")
            elif kind == "ag":
                want = ring.expected_all_gather(xs, sizes)
            elif kind == "bcast":
                want = xs[k % world]
            elif kind == "rs":
                want = ring.expected_reduce_scatter(xs, sizes, True)[r]
            else:  # only the owner's chunk is specified
                want = ring.expected_reduce_scatter(xs, sizes, True)[r][lo:lo + sizes[r]]
                got = got[lo:lo + sizes[r]]
            assert np.array_equal(bits(got), bits(want)), (world, algo, r, k, kind, sizes)


def disagree(g, what):
    """Ranks that call different collectives, or the same one on tensors of different
    sizes: found out at the first handshake, on every rank, not by reading stale bytes."""
    from tandem_amd import CommError

    x = torch.ones(1000 + (g.rank if what == "size" else 0), device=g.device)
    try:
        if what == "kind" and g.rank == 1:
            g.all_gather(x)
        else:
            g.all_reduce(x)
    except CommError as e:
        g.abandon()
        return "out of step" in str(e.__cause__)
    return False


@pytest.mark.parametrize("algo", ["staged", "ring"])
@pytest.mark.parametrize("what", ["size", "kind"])
def test_ranks_that_disagree_are_found_out(what, algo, monkeypatch):
    """Staged: the fence's tag. Slot ring: every piece's message says what its sender is doing (the reference's
    protocol says nothing: there the all_gather of one rank takes the other's reduce-scatter pieces for its own)."""
    from tandem_amd import launch

    monkeypatch.delenv("TANDEM_HIP_WAIT", raising=False)  # with waits that only park the stream the NEXT call reports it (tested below)
    monkeypatch.setenv("TANDEM_HIP_ALGO", algo)
    assert launch(disagree, 2, what, gpus=[0, 0], timeout=TIMEOUT) == [True, True]


def late_failure(g):
    """With stream-ordered waiting a collective's wait() can return before the collective
    has run; when it then fails (here: the peer never joins), the caller's stream is let
    go, and the next call on the group reports the failure."""
    import time

    from tandem_amd import CommError

    x = torch.ones(1000, device=g.device)
    if g.rank == 1:
        time.sleep(5.0)  # never joins; leaves after rank 0 has given up
        g.abandon()
        return True
    g.all_reduce(x)  # returns at once: the stream is parked behind the collective
    torch.cuda.synchronize()  # ... and released when the collective gives up
    try:
        g.all_reduce(x)
    except CommError as e:
        g.abandon()
        return "an earlier collective failed" in str(e) and "timed out" in str(e)
    return False


def test_stream_ordered_wait_reports_a_failure_at_the_next_call(monkeypatch):
    from tandem_amd import launch

    monkeypatch.setenv("TANDEM_HIP_WAIT", "stream")
    monkeypatch.delenv("GPU_MAX_HW_QUEUES", raising=False)  # with a single hardware queue nothing is parked: the wait itself reports it
    assert launch(late_failure, 2, gpus=[0, 0], timeout=2.0) == [True, True]


def parked_too_long(g):
    """A stream parked on a collective whose end does not come within the park limit lets itself go (the wait is a
    kernel of the library's own with a time limit), and the next call on the group says so. The collective itself still
    runs when the late peer arrives, which must not be left waiting for this rank."""
    import time

    from tandem_amd import CommError

    x = torch.full((1000,), float(g.rank + 1), device=g.device)
    if g.rank == 1:
        time.sleep(1.5)
        g.all_reduce(x)
        torch.cuda.synchronize()
        ok = float(x[0]) == 3.0
        g.abandon()
        return ok
    t0 = time.perf_counter()
    g.all_reduce(x, async_op=True).wait(stream_ordered=True)  # returns at once: the peer has not even called yet
    torch.cuda.synchronize()  # ... and the stream is let go by its own limit, long before the peer comes
    took = time.perf_counter() - t0
    try:
        g.all_reduce(x)
    except CommError as e:
        time.sleep(2.0)  # the first collective still runs when the peer arrives
        g.abandon()
        return 0.15 < took < 1.2 and "gave up" in str(e)
    return False


def test_a_parked_stream_gives_up_by_itself(monkeypatch):
    from tandem_amd import launch

    monkeypatch.setenv("TANDEM_HIP_PARK_LIMIT_S", "0.2")
    monkeypatch.delenv("GPU_MAX_HW_QUEUES", raising=False)
    assert launch(parked_too_long, 2, gpus=[0, 0], timeout=5.0) == [True, True]


def test_unknown_backend_and_cpu_device_are_refused():
    from tandem_amd import CommError, Group, launch

    with pytest.raises(CommError, match="unknown backend"):
        launch(failing, 2, backend="python")
    with pytest.raises(CommError, match="no CPU path"):
        Group(0, 1, "cpu", None, backend="hip", job="x")


def stream_ordered_waits(g):
    """Work.wait(stream_ordered=True): the call may return before the collective has run; whatever the caller's
    stream does next must still see the reduced tensor. The stream is kept busy first, so that most waits find their
    collective still queued."""
    dev, w = g.device, g.size
    n = 300_001
    busy = torch.randn(1024, 1024, device=dev)
    ok, parked = True, 0
    for k in range(40):
        x = torch.full((n,), float(g.rank + 1 + k), device=dev)
        for _ in range(3):
            busy = (busy @ busy) * 1e-3  # the all-reduce's inputs are ready only after these
        x += busy[0, 0] * 0  # (a dependency on the busy work)
        work = g.all_reduce(x, async_op=True)
        parked += 0 if work.is_completed() else 1
        out = work.wait(stream_ordered=True)
        y = out * 2  # queued right behind the wait
        want = 2.0 * sum(q + 1 + k for q in range(w))
        ok = ok and bool((y == want).all())
    g.barrier()
    torch.cuda.synchronize()
    return ok, parked


@pytest.mark.parametrize("world", [2, 3])
def test_waits_that_only_order_the_stream(world):
    from tandem_amd import launch

    for ok, parked in launch(stream_ordered_waits, world, gpus=[0] * world, timeout=TIMEOUT):
        assert ok
        assert parked > 0, "every collective had run before its wait: the test did not exercise the parked path"


def more_works_than_words(g):
    """Every Work in flight owns one of the engine's 1024 done words; those beyond wait on an event as before."""
    dev, w = g.device, g.size
    count, n = 1100, 257
    rows = torch.arange(count, device=dev, dtype=torch.float32).unsqueeze(1).expand(count, n)
    x = (rows + float(g.rank)).contiguous()
    works = [g.all_reduce(x[k], async_op=True) for k in range(count)]
    done_before = sum(wk.is_completed() for wk in works)
    for wk in works:
        wk.wait()
    y = x * 1  # on the caller's stream, behind every wait
    ok = bool((y == rows * w + float(sum(range(w)))).all()) and all(wk.is_completed() for wk in works[:8])
    torch.cuda.synchronize()
    ok = ok and all(wk.is_completed() for wk in works)
    del works
    z = torch.ones(5, device=dev)
    g.all_reduce(z)  # the words are free again
    return ok and bool((z == w).all()), done_before


def test_more_collectives_in_flight_than_done_words():
    from tandem_amd import launch

    for ok, _ in launch(more_works_than_words, 2, gpus=[0, 0], timeout=TIMEOUT):
        assert ok


def several_arenas(g):
    """Every rank shares three arenas; rank q's tensors lie in arena (q + k) % 3, so every collective reaches into
    different arenas of different peers. Offsets are named as arena index * 2^31 + byte offset."""
    dev, w, r = g.device, g.size, g.rank
    arenas = []
    for _ in range(3):
        g.share_arena(1 << 20)
        arenas.append(g._arena)
    assert g.arena_count == 3

    def place(q, k, n):  # (arena, byte offset) of rank q's k-th tensor of n floats: the same rule on every rank
        return (q + k) % 3, 256 * (1 + q + 3 * k) + 4096 * k

    out = {}
    n = 10_007
    sizes = [n // w + (1 if q < n % w else 0) for q in range(w)]
    lo = sum(sizes[:r])
    for k, what in enumerate(("all_reduce", "reduce_scatter", "all_gather", "gather_unit")):
        a, off = place(r, k, n)
        t = arenas[a][off:off + 4 * n].view(torch.float32)
        offs = [(place(q, k, n)[0] << 31) + place(q, k, n)[1] for q in range(w)]
        assert g.arena_offset(t) == offs[r]
        x = values(r + 7 * k, n, torch.float32).to(dev)
        if what == "all_reduce":
            t.copy_(x)
            g.all_reduce(t, op="avg", direct=offs)
        elif what == "reduce_scatter":
            t.copy_(x)
            g.reduce_scatter(t, sizes, direct=offs)
        elif what == "all_gather":
            t.zero_()
            t[lo:lo + sizes[r]] = x[lo:lo + sizes[r]]
            g.all_gather(t, sizes, direct=offs)
        else:  # the shard in the arena, the full buffer anywhere
            shard = t[:sizes[r]]
            shard.copy_(x[lo:lo + sizes[r]])
            full = torch.zeros(n, device=dev)
            g.fence()
            g.gather_unit(full, shard, sizes, peer_offsets=offs)
            g.fence()
            t = full
        out[what] = t.cpu().clone()
    assert g.arena_offset(torch.zeros(4, device=dev)) is None
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("world", [2, 3])
def test_tensors_in_several_arenas(world):
    from oracle import ring
    from tandem_amd import launch

    n = 10_007
    sizes = [n // world + (1 if q < n % world else 0) for q in range(world)]
    res = launch(several_arenas, world, gpus=[0] * world, timeout=TIMEOUT)
    for r, out in enumerate(res):
        lo = sum(sizes[:r])
        xs = [to_np(values(q, n, torch.float32)) for q in range(world)]
        assert np.array_equal(bits(to_np(out["all_reduce"])), bits(ring.expected_all_reduce(xs, True, "f32")))
        xs = [to_np(values(q + 7, n, torch.float32)) for q in range(world)]
        want = xs[r].copy()
        want[lo:lo + sizes[r]] = ring.expected_reduce_scatter(xs, sizes, False, "f32")[r][lo:lo + sizes[r]]
        assert np.array_equal(bits(to_np(out["reduce_scatter"])), bits(want))
        for k, what in ((2, "all_gather"), (3, "gather_unit")):
            xs = [to_np(values(q + 7 * k, n, torch.float32)) for q in range(world)]
            assert np.array_equal(bits(to_np(out[what])), bits(ring.expected_all_gather(xs, sizes))), what


def two_groups(g):
    """A second group of the same ranks in the same processes (its own engine, thread, streams, slots and region): collectives
    of the two are in flight at once and waited for in the opposite order."""
    from tandem_amd import Group

    dev, w, r = g.device, g.size, g.rank
    other = Group(r, w, dev, g._barrier, slot_bytes=g.slot_bytes, slots=g.slots, timeout=g.timeout, job="second" + str(os.getppid()))
    ok = True
    try:
        for k in range(12):
            n = (1, 1000, 70_001)[k % 3]
            a = torch.full((n,), float(r + k), device=dev)
            b = torch.full((n,), float(2 * r + k), device=dev)
            wa = g.all_reduce(a, async_op=True)
            wb = other.all_reduce(b, op="avg", async_op=True)
            wb.wait(stream_ordered=bool(k % 2))
            wa.wait()
            ok = ok and bool((a == sum(q + k for q in range(w))).all()) and bool((b == sum(2 * q + k for q in range(w)) / w).all())
        x = other.shared_empty(64)
        x.fill_(float(r))
        other.all_reduce(x, direct=True)
        ok = ok and bool((x == sum(range(w))).all()) and g.arena_count == 0 and other.arena_count == 1
        torch.cuda.synchronize()
    finally:
        other.close()
    g.barrier()
    return ok


def test_two_groups_in_the_same_processes():
    from tandem_amd import launch

    assert launch(two_groups, 2, gpus=[0, 0], timeout=TIMEOUT) == [True, True]


def on_a_stream_of_the_callers(g):
    """Everything on a stream the caller made: the collective starts behind what that stream holds at the call, and both kinds
    of wait order that stream (not the default one) behind the collective."""
    from tandem_amd import LocalWorld

    dev, w = g.device, g.size
    s = torch.cuda.Stream()
    busy = torch.randn(1024, 1024, device=dev)
    torch.cuda.synchronize()
    ok = True
    with torch.cuda.stream(s):
        for k in range(20):
            for _ in range(3):
                busy = (busy @ busy) * 1e-3
            x = torch.full((100_003,), float(g.rank + 1 + k), device=dev) + busy[0, 0] * 0
            work = g.all_reduce(x, async_op=True)
            y = work.wait(stream_ordered=bool(k % 2)) * 2
            ok = ok and bool((y == 2.0 * sum(q + 1 + k for q in range(w))).all())
        # ranks that are buffers of this process, on the same stream
        bufs = [torch.full((50_001,), float(q + 1), device=dev) + busy[0, 0] * 0 for q in range(3)]
        LocalWorld(3).all_reduce(bufs)
        ok = ok and all(bool((b == 6.0).all()) for b in bufs)
    s.synchronize()
    g.barrier()
    return ok


def test_collectives_on_a_stream_of_the_callers():
    from tandem_amd import launch

    assert launch(on_a_stream_of_the_callers, 2, gpus=[0, 0], timeout=TIMEOUT) == [True, True]


def dropped_without_a_wait(g):
    """A Work that is dropped before anybody waited for it: its tensors stay alive until the collective has run (nothing
    orders the caller's stream behind it, so the allocator must not hand their memory out again)."""
    dev, w = g.device, g.size
    busy = torch.randn(2048, 2048, device=dev)
    for _ in range(10):
        busy = (busy @ busy) * 1e-4  # the collectives' inputs are ready only behind these
    where = []
    for k in range(8):
        x = torch.full((200_003,), float(g.rank + k), device=dev) + busy[0, 0] * 0
        where.append(x.data_ptr())
        g.all_reduce(x, async_op=True)  # the Work goes at once
        del x
    held = len(g._orphans)
    fresh = [torch.zeros(200_003, device=dev) for _ in range(8)]
    aliased = sum(f.data_ptr() in where for f in fresh)
    y = torch.full((1000,), float(g.rank), device=dev)
    g.all_reduce(y)  # in order behind the dropped ones
    g.barrier()
    torch.cuda.synchronize()
    g._reap()
    return held, aliased, len(g._orphans), bool((y == sum(range(w))).all())


def test_a_work_dropped_without_a_wait_keeps_its_tensors():
    from tandem_amd import launch

    for held, aliased, left, ok in launch(dropped_without_a_wait, 2, gpus=[0, 0], timeout=TIMEOUT):
        assert held >= 1, "every collective had finished before its Work was dropped: nothing was exercised"
        assert aliased == 0 or held < 8
        assert left == 0 and ok
