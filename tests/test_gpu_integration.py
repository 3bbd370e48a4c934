"""tandem_amd/hip_engine.py, the binding offered to a tandem maintainer, driven on
the GPU the way the reference's own Group drives its native engine (tandem/comm.py:149-170:
create, the launcher's barrier, connect, barrier; tandem/comm.py:326-452: every collective
returns a handle that is waited for), by two processes that share the GPU. Results against
the fixtures the reference's Python engine wrote (tests/golden/ring_w2.npz). tandem_amd's own
Group is not involved. Run with -m gpu."""

import json
import os
import tempfile
import time
import uuid

import numpy as np
import pytest
import torch
import torch.multiprocessing as mp

from helpers import GOLDEN, bits

pytestmark = pytest.mark.gpu


def rank_main(rank, size, job, barrier, outdir):
    from tandem_amd import hip_engine

    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    assert hip_engine.cuda is True
    d = np.load(os.path.join(GOLDEN, "ring_w2.npz"))
    cases = json.loads(bytes(d["sizes_json"]).decode())
    # tandem/comm.py:149-160: engine, every rank has created its links, connect, barrier
    engine = hip_engine.Engine(job, rank, size, 2, 4096, 60.0, 0)
    barrier.wait(timeout=60)
    engine.connect()
    engine.barrier().wait()
    x = torch.from_numpy(d[f"r{rank}_in"].copy()).to(dev)
    out = {}

    def run(name, t, start):
        before = time.perf_counter()
        handle = start(t)
        handle.wait()           # the current stream now waits for the collective
        torch.cuda.synchronize()
        after = time.perf_counter()
        assert handle.done()
        assert before <= handle.started <= handle.finished <= after, (name, before, handle.started, handle.finished, after)
        out[name] = t.cpu().numpy()

    run("ar_avg", x.clone(), lambda t: engine.all_reduce(t, True))
    run("ar_sum", x.clone(), lambda t: engine.all_reduce(t, False))
    run("rs_avg_even", x.clone(), lambda t: engine.reduce_scatter(t, [], True))
    for name, sizes in cases.items():
        run(f"rs_avg_{name}", x.clone(), lambda t: engine.reduce_scatter(t, sizes, True))
        run(f"rs_sum_{name}", x.clone(), lambda t: engine.reduce_scatter(t, sizes, False))
        run(f"ag_{name}", x.clone(), lambda t: engine.all_gather(t, sizes))
    run("tiny_ar_avg", torch.from_numpy(d[f"r{rank}_tiny_in"].copy()).to(dev), lambda t: engine.all_reduce(t, True))
    # broadcast, send/recv, a dtype that only travels as bytes, a 2-d tensor
    t = (x.clone() if rank == 1 else torch.zeros_like(x)).view(-1, 11)
    engine.broadcast(t, 1).wait()
    out["bcast_from_1"] = t.cpu().numpy().reshape(-1)
    flags = (torch.arange(1000, device=dev) % 3 == 0) if rank == 0 else torch.zeros(1000, dtype=torch.bool, device=dev)
    engine.broadcast(flags, 0).wait()
    out["bool_ok"] = np.array(bool(torch.equal(flags.cpu(), torch.arange(1000) % 3 == 0)))
    got = torch.empty_like(x)
    engine.sendrecv(x, 1 - rank, got, 1 - rank).wait()
    out["sendrecv"] = got.cpu().numpy()
    if rank == 0:
        engine.send(x[:100].contiguous(), 1).wait()
    else:
        part = torch.empty(100, device=dev)
        engine.recv(part, 0).wait()
        out["recv_100"] = part.cpu().numpy()
    # what it refuses, as the reference's binding does (ValueError for bad arguments)
    for bad, call in (("bool", lambda: engine.all_reduce(torch.zeros(8, dtype=torch.bool, device=dev), False)),
                      ("cpu", lambda: engine.all_reduce(torch.zeros(8), False)),
                      ("strided", lambda: engine.all_reduce(torch.zeros(8, 8, device=dev).t(), False)),
                      ("sizes", lambda: engine.reduce_scatter(x.clone(), [1, 2], False))):
        try:
            call()
        except ValueError:
            out[f"refused_{bad}"] = np.array(True)
    # a handle dropped before anybody waited for it: its tensor must outlive the collective (the reference's engine
    # holds it until the job has run, tandem/csrc/collectives.cpp:314-324). Rank 1 arrives late, so on rank 0 the
    # collective has certainly not run when the handle goes; memory allocated right afterwards must not be the tensor's.
    big = torch.full((1 << 20,), float(rank + 1), device=dev)
    address = big.data_ptr()
    torch.cuda.synchronize()
    if rank == 1:
        time.sleep(0.3)
    handle = engine.all_reduce(big, False)
    del handle, big
    decoys = [torch.full((1 << 20,), -5.0, device=dev) for _ in range(3)]
    out["dropped_parked"] = np.array(rank == 1 or len(engine._orphans) == 1)
    out["dropped_not_reused"] = np.array(all(t.data_ptr() != address for t in decoys) or rank == 1)
    engine.barrier().wait()
    torch.cuda.synchronize()
    out["decoys_intact"] = np.array(all(bool((t == -5.0).all()) for t in decoys))
    engine.barrier().wait()  # the next call lets go of what has finished
    out["dropped_reaped"] = np.array(len(engine._orphans) == 0)
    torch.cuda.synchronize()
    engine.barrier().wait()
    engine.close()
    np.savez(os.path.join(outdir, f"rank{rank}.npz"), **out)


def test_the_documented_binding_runs_the_reference_fixtures():
    job = uuid.uuid4().hex[:12]
    ctx = mp.get_context("spawn")
    barrier = ctx.Barrier(2)
    d = np.load(os.path.join(GOLDEN, "ring_w2.npz"))
    with tempfile.TemporaryDirectory(prefix="tandem-binding-") as outdir:
        mp.spawn(rank_main, args=(2, job, barrier, outdir), nprocs=2, join=True)
        res = [dict(np.load(os.path.join(outdir, f"rank{r}.npz"))) for r in range(2)]
    fixture_keys = [k[3:] for k in d.keys() if k.startswith("r0_") and not k.endswith("_in")]
    assert len(fixture_keys) >= 16
    for r in range(2):
        for key in fixture_keys:
            assert np.array_equal(bits(res[r][key]), bits(d[f"r{r}_{key}"])), (r, key)
        assert np.array_equal(bits(res[r]["bcast_from_1"]), bits(d["r1_in"]))
        assert np.array_equal(bits(res[r]["sendrecv"]), bits(d[f"r{1 - r}_in"]))
        assert bool(res[r]["bool_ok"])
        for bad in ("bool", "cpu", "strided", "sizes"):
            assert bool(res[r].get(f"refused_{bad}", False)), (r, bad)
        for what in ("dropped_parked", "dropped_not_reused", "decoys_intact", "dropped_reaped"):
            assert bool(res[r][what]), (r, what)
    assert np.array_equal(bits(res[1]["recv_100"]), bits(d["r0_in"][:100]))
