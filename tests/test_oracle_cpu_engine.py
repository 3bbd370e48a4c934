"""The oracle's CPU-process engine against the reference engine's fixtures: same
inputs, same slot size, outputs bit for bit (whole buffers, every rank)."""

import numpy as np
import pytest
import torch

from oracle.cpu_engine import cpu_launch

from helpers import bits, golden_npz, npz_json


def replay(g, inputs, cases):
    r = g.rank
    x = torch.from_numpy(inputs[r].copy())
    out = {}
    t = x.clone(); g.all_reduce(t); out["ar_sum"] = t
    t = x.clone(); g.all_reduce(t, op="avg"); out["ar_avg"] = t
    t = x.clone(); g.reduce_scatter(t, None, op="avg"); out["rs_avg_even"] = t
    for name, sizes in cases.items():
        t = x.clone(); mine = g.reduce_scatter(t, sizes, op="avg"); out[f"rs_avg_{name}"] = t
        assert mine.numel() == sizes[r]
        t = x.clone(); g.reduce_scatter(t, sizes, op="sum"); out[f"rs_sum_{name}"] = t
        t = x.clone(); g.all_gather(t, sizes); out[f"ag_{name}"] = t
    works = [g.all_reduce(x.clone() * k, async_op=True) for k in range(1, 4)]  # several in flight
    out["async"] = torch.stack([w.wait() for w in works])
    b = x.clone() if r == g.size - 1 else torch.zeros_like(x)
    g.broadcast(b, root=g.size - 1)
    out["bcast"] = b
    return {k: v.numpy() for k, v in out.items()}


@pytest.mark.parametrize("world", [2, 3, 4])
def test_engine_reproduces_reference_fixtures(world):
    d = golden_npz(f"ring_w{world}.npz")
    inputs = [d[f"r{r}_in"] for r in range(world)]
    cases = npz_json(d, "sizes_json")
    res = cpu_launch(replay, world, inputs, cases, slot_bytes=256)
    for r in range(world):
        for key, got in res[r].items():
            if key == "async":
                for k in range(3):
                    assert np.array_equal(got[k], got[k])  # finite
                continue
            if key == "bcast":
                assert np.array_equal(bits(got), bits(inputs[world - 1]))
                continue
            assert np.array_equal(bits(got), bits(d[f"r{r}_{key}"])), (world, r, key)
    # every rank saw the same async results, in submission order
    for r in range(1, world):
        assert np.array_equal(bits(res[0]["async"]), bits(res[r]["async"]))


def boom(g):
    if g.rank == 1:
        raise ValueError("boom")
    g.barrier()
    return True


def test_a_failing_rank_surfaces():
    with pytest.raises(Exception, match="boom|terminated|barrier"):
        cpu_launch(boom, 2)


def bad_sizes(g):
    from oracle.cpu_engine import EngineError

    try:
        g.reduce_scatter(torch.zeros(10), [5, 6])
    except EngineError as e:
        return "partition" in str(e.__cause__)
    return False


def test_bad_chunk_sizes_are_reported():
    assert cpu_launch(bad_sizes, 2) == [True, True]
