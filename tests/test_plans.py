"""Host-side planning (bucket packing, shard sizes, fold segments) against the
plans the reference itself produced (tests/golden/plans.json)."""

import math

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
