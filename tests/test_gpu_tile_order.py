"""Which tile a workgroup takes (tdm_set_xcd_group) is a launch-geometry choice: every
kernel family must give the same bits for every group shift, on sizes whose tile count
leaves whole groups, a ragged remainder and a partial last tile. The comparison is
against the plain order (shift 0), which the other GPU tests pin to the oracle. Run
with -m gpu."""

import pytest
import torch

from helpers import seeded

pytestmark = pytest.mark.gpu
SHIFTS = (1, 3, 5)
KINDS = dict(reduce=0, copy=1, fold=2, fold_table=3, adamw=4, step=5)


@pytest.fixture
def order():
    from tandem_amd._lib import lib

    L = lib()

    def set_(kind, shift):
        assert L.tdm_set_xcd_group(KINDS[kind], shift) == 0

    yield set_
    assert L.tdm_set_xcd_group(-1, -1) == 0  # back to the built-in defaults


def tiles_to_elems(tiles, extra):
    from tandem_amd._lib import lib

    return tiles * (lib().tdm_table_tile_bytes() // 4) + extra


@pytest.mark.parametrize("world", [2, 4])
def test_ring_and_fold_collectives(order, world):
    from tandem_amd import LocalWorld

    dev = torch.device("cuda", 0)
    lw = LocalWorld(world)
    n = world * tiles_to_elems(83, 0) + 4 * 37 + 3  # per chunk: 83 whole tiles and a bit; ragged chunk sizes
    xs = [seeded(3, r, n, 1e-2) for r in range(world)]

    def run(algorithm):
        bufs = [x.to(dev) for x in xs]
        lw.all_reduce(bufs, "avg", algorithm=algorithm)
        torch.cuda.synchronize()
        return [b.cpu() for b in bufs]

    for kinds, algorithm in ((("reduce", "copy"), "ring"), (("fold",), "fold")):
        for k in kinds:
            order(k, 0)
        want = run(algorithm)
        for s in SHIFTS:
            for k in kinds:
                order(k, s)
            got = run(algorithm)
            for a, b in zip(want, got):
                assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (algorithm, s)


def test_bucket_fold_table(order):
    from tandem_amd import LocalWorld
    from tandem_amd.buckets import pack

    dev = torch.device("cuda", 0)
    numels = [tiles_to_elems(40, 5), 7, tiles_to_elems(3, 0), tiles_to_elems(150, 1), 1024, tiles_to_elems(29, 12)]
    idx = list(range(len(numels)))[::-1]
    buckets = [[idx[k] for k in g] for g in pack([numels[i] * 4 for i in idx], 1 << 20)]
    for world in (2, 4):
        grads0 = [[seeded(5 + i, r, m, 1e-3) for i, m in enumerate(numels)] for r in range(world)]

        def run():
            grads = [[t.to(dev) for t in row] for row in grads0]
            LocalWorld(world).bucket_table(grads, buckets).run(True)
            torch.cuda.synchronize()
            return [t.cpu() for row in grads for t in row]

        order("fold_table", 0)
        want = run()
        for s in SHIFTS:
            order("fold_table", s)
            for a, b in zip(want, run()):
                assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (world, s)


@pytest.mark.parametrize("form", ["one_launch", "fold_then_adamw_gather"])
def test_zero2_step_forms(order, form):
    from tandem_amd.local import LocalZeRO2

    dev = torch.device("cuda", 0)
    world = 4
    numels = [tiles_to_elems(61, 3), 11, tiles_to_elems(200, 0), 513, tiles_to_elems(97, 2)]
    n = sum(numels)
    p0 = seeded(1, 0, n, 0.02)
    grads = [[seeded(20 + step, r, n, 1e-3) for r in range(world)] for step in range(2)]

    def run():
        z = LocalZeRO2(world, numels, dev, bucket_bytes=1 << 20, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
        for b in z.bufs:
            b.copy_(p0)
        for gs in grads:
            for r in range(world):
                z.staging[r].copy_(gs[r])
            if form == "one_launch":
                z.reduce_and_step()
            else:
                z.reduce_grads("fold")
                z.step(fused_gather=True)
            z.zero_grad()
        torch.cuda.synchronize()
        out = [b.cpu() for b in z.bufs]
        out += [t.cpu() for o in z.opts for t in o.state["flat"][1:]]
        return out

    kinds = ("step",) if form == "one_launch" else ("fold_table", "adamw")
    for k in kinds:
        order(k, 0)
    want = run()
    for s in SHIFTS:
        for k in kinds:
            order(k, s)
        for a, b in zip(want, run()):
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), (form, s)


def test_setter_refuses_nonsense(order):
    from tandem_amd._lib import lib

    L = lib()
    assert L.tdm_set_xcd_group(6, 0) == 1 and b"family" in L.tdm_last_error()
    assert L.tdm_set_xcd_group(0, 13) == 1 and b"shift" in L.tdm_last_error()
    assert L.tdm_set_xcd_group(-2, 0) == 1
