"""Host-side planning (bucket packing, shard sizes, fold segments) against the
plans the reference itself produced (tests/golden/plans.json), and on random
inputs against element-by-element brute force."""

import math

from hypothesis import given, settings, strategies as st

from helpers import golden_json
from tandem_amd.buckets import FlatLayout, fold_segments, pack, zero_buckets
from tandem_amd.local import chunk_bounds, split_sizes


def numels_of(params):
    return [math.prod(s) for _, s in params]


def test_ddp_packing_matches_reference():
    plan = golden_json("plans.json")
    for params_key, key, limit in (("medium_params", "medium_ddp_25MiB", 25 << 20),
                                   ("small_params", "small_ddp_64KiB", 64 << 10),
                                   ("small_params", "small_ddp_4KiB", 4 << 10)):
        names = [n for n, _ in plan[params_key]]
        numels = numels_of(plan[params_key])
        order = list(range(len(numels)))[::-1]
        groups = pack([numels[i] * 4 for i in order], limit)
        assert [[names[order[k]] for k in g] for g in groups] == plan[key]
    assert sum(numels_of(plan["medium_params"])) == 85_842_432
    assert len(plan["medium_ddp_25MiB"]) == 16


def test_zero_buckets_and_bucket_sizes_match_reference():
    plan = golden_json("plans.json")
    for params_key, key, limit, world in (("medium_params", "medium_zero_25MiB_w4", 25 << 20, 4),
                                          ("small_params", "small_zero_4KiB_w3", 4 << 10, 3)):
        numels = numels_of(plan[params_key])
        want = plan[key]
        zb = zero_buckets(numels, 4, limit)
        assert [[a, b] for a, b, _ in zb] == want["ranges"]
        assert [len(ps) for _, _, ps in zb] == want["counts"]
        fl = FlatLayout(numels, world, 1)
        assert fl.sizes == want["shard_sizes"]
        assert [fl.bucket_sizes(a, b) for a, b, _ in zb] == want["bucket_sizes"]
        for a, b, _ in zb:
            assert sum(fl.bucket_sizes(a, b)) == b - a
        assert (fl.lo, fl.hi) == (want["shard_sizes"][0], want["shard_sizes"][0] + want["shard_sizes"][1])


def test_split_sizes_match_reference():
    for key, want in golden_json("plans.json")["split_sizes"].items():
        n, w = map(int, key.split("/"))
        assert split_sizes(n, w) == want
        assert [hi - lo for lo, hi in chunk_bounds(n, w)] == want


def test_unit_sizes():
    plan = golden_json("plans.json")
    assert plan["medium_units"][0] == 589_824 and plan["medium_units"][-1] == 198_144
    assert set(plan["medium_units"][1:-1]) == {7_087_872} and len(plan["medium_units"]) == 14


def test_fold_segments_cover_the_bucket_once():
    for numels, world in (([5, 1, 0, 9, 3], 4), ([1], 3), ([100, 100], 2), ([7, 7, 7], 8)):
        segs = fold_segments(numels, world)
        bounds = chunk_bounds(sum(numels), world)
        seen = [0] * len(numels)
        pos = 0
        for i, off, count, chunk in segs:
            assert count > 0 and off == seen[i]
            seen[i] += count
            lo, hi = bounds[chunk]
            assert lo <= pos and pos + count <= hi  # inside one ring chunk
            pos += count
        assert seen == numels and pos == sum(numels)


# ---- properties on random inputs, checked against element-by-element brute force

@settings(max_examples=150, deadline=None)
@given(st.integers(0, 300), st.integers(1, 9))
def test_split_sizes_are_tensor_splits(n, world):
    import torch

    want = [c.numel() for c in torch.tensor_split(torch.empty(n), world)]
    assert split_sizes(n, world) == want
    bounds = chunk_bounds(n, world)
    assert [hi - lo for lo, hi in bounds] == want and (not bounds or bounds[0][0] == 0)


@settings(max_examples=150, deadline=None)
@given(st.lists(st.integers(0, 40), min_size=1, max_size=12), st.integers(1, 6), st.data())
def test_bucket_sizes_count_the_elements_of_each_shard(numels, world, data):
    lay = [FlatLayout(numels, world, r) for r in range(world)]
    n = lay[0].numel
    owner = [r for r in range(world) for _ in range(lay[r].hi - lay[r].lo)]
    assert len(owner) == n and all(l.lo == sum(lay[0].sizes[:r]) for r, l in enumerate(lay))
    a = data.draw(st.integers(0, n))
    b = data.draw(st.integers(a, n))
    assert lay[0].bucket_sizes(a, b) == [sum(1 for i in range(a, b) if owner[i] == r) for r in range(world)]


@settings(max_examples=150, deadline=None)
@given(st.lists(st.integers(0, 50), min_size=0, max_size=20), st.integers(1, 120))
def test_packing_rule(sizes, cap):
    groups = pack(sizes, cap)
    assert [i for g in groups for i in g] == list(range(len(sizes)))  # order kept, nothing lost
    for k, g in enumerate(groups):
        assert g and (sum(sizes[i] for i in g) <= cap or len(g) == 1)  # only a lone oversize tensor exceeds the limit
        if k + 1 < len(groups):  # greedy: the next tensor did not fit
            assert sum(sizes[i] for i in g) + sizes[groups[k + 1][0]] > cap


@settings(max_examples=150, deadline=None)
@given(st.lists(st.integers(0, 30), min_size=1, max_size=10), st.integers(1, 8))
def test_fold_segments_tag_every_element_with_its_ring_chunk(numels, world):
    total = sum(numels)
    chunk_of = [c for c, (lo, hi) in enumerate(chunk_bounds(total, world)) for _ in range(hi - lo)]
    seen = []
    starts = [sum(numels[:i]) for i in range(len(numels))]
    for i, off, count, c in fold_segments(numels, world):
        assert count > 0 and off + count <= numels[i]
        for e in range(starts[i] + off, starts[i] + off + count):
            assert chunk_of[e] == c
            seen.append(e)
    assert seen == list(range(total))  # flat order, each element once
