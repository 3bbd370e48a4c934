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


def test_occupancy_pad_changes_no_result():
    """The unused LDS that caps how many workgroups share a compute unit is geometry too:
    the one-launch step, AdamW with copies and the by-value fold give the same bits with no
    pad, the defaults and the largest pad."""
    from tandem_amd import LocalWorld
    from tandem_amd._lib import lib
    from tandem_amd.local import LocalZeRO2

    L = lib()
    dev = torch.device("cuda", 0)
    world = 4
    numels = [tiles_to_elems(61, 3), 11, tiles_to_elems(200, 0), 513]
    n = sum(numels)
    p0 = seeded(1, 0, n, 0.02)
    grads = [seeded(20, r, n, 1e-3) for r in range(world)]

    def run():
        z = LocalZeRO2(world, numels, dev, bucket_bytes=1 << 20, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
        for b in z.bufs:
            b.copy_(p0)
        for r in range(world):
            z.staging[r].copy_(grads[r])
        z.reduce_and_step()
        z.reduce_grads("fold")
        z.step(fused_gather=True)
        bufs = [g.to(dev) for g in grads]
        LocalWorld(world).all_reduce(bufs, "avg", algorithm="fold")
        torch.cuda.synchronize()
        return [b.cpu() for b in z.bufs] + [t.cpu() for o in z.opts for t in o.state["flat"][1:]] + [b.cpu() for b in bufs]

    try:
        assert L.tdm_set_occupancy_pad(-1, 0) == 0
        want = run()
        for pad in (-1, 65536, 4096):
            assert L.tdm_set_occupancy_pad(-1, pad) == 0
            for a, b in zip(want, run()):
                assert torch.equal(a.view(torch.int32), b.view(torch.int32)), pad
        assert L.tdm_set_occupancy_pad(0, 65537) == 1 and b"pad" in L.tdm_last_error()
        assert L.tdm_set_occupancy_pad(6, 0) == 1 and b"family" in L.tdm_last_error()
    finally:
        assert L.tdm_set_occupancy_pad(-1, -1) == 0


def test_stream_mix_probe_moves_what_it_says():
    """The measurement kernel: every written stream receives the same function of the read
    streams (their lane-wise 32-bit sum plus a pattern), whatever the geometry; bad arguments
    are refused."""
    import ctypes

    from tandem_amd._lib import stream_ptr
    from tandem_amd._probe import lib  # libtandem_probe.so, a library of its own beside the plug-in

    L = lib()
    dev = torch.device("cuda", 0)
    n = tiles_to_elems(37, 0) + 8
    src = [torch.randint(-2**31, 2**31 - 1, (n,), dtype=torch.int32, device=dev) for _ in range(3)]
    outs = {}
    for per_lane, shift, pad in ((1, 0, 0), (2, 3, 16384), (1, 6, 65536)):
        dst = [torch.zeros(n, dtype=torch.int32, device=dev) for _ in range(2)]
        rd = (ctypes.c_void_p * 8)(*[t.data_ptr() for t in src])
        wr = (ctypes.c_void_p * 8)(*[t.data_ptr() for t in dst])
        assert L.tdm_probe_stream_mix(rd, 3, wr, 2, n * 4, per_lane, shift, pad, stream_ptr(dev)) == 0
        torch.cuda.synchronize()
        assert torch.equal(dst[0], dst[1])
        outs[(per_lane, shift, pad)] = dst[0].cpu()
    first = outs[(1, 0, 0)]
    total = (src[0].cpu().to(torch.int64) + src[1].cpu() + src[2].cpu())
    lane = torch.arange(n) % 4
    # lanes 1..3 of every vector carry sum + 1, 2, 3; lane 0 carries sum + the vector's index within the launch
    want = ((total + lane) & 0xffffffff).to(torch.int64)
    got = first.to(torch.int64) & 0xffffffff
    assert torch.equal(got[lane != 0], want[lane != 0])
    assert torch.equal(outs[(1, 6, 65536)][lane != 0], first[lane != 0])
    assert torch.equal(outs[(2, 3, 16384)][lane != 0], first[lane != 0])
    rd = (ctypes.c_void_p * 8)(src[0].data_ptr())
    assert L.tdm_probe_stream_mix(rd, 1, None, 0, n * 4, 1, 0, 0, stream_ptr(dev)) == 0  # read-only
    assert L.tdm_probe_stream_mix(rd, 0, None, 0, n * 4, 1, 0, 0, stream_ptr(dev)) == 1 and b"streams" in L.tdm_probe_last_error()
    assert L.tdm_probe_stream_mix(rd, 1, None, 0, n * 4 + 4, 1, 0, 0, stream_ptr(dev)) == 1
    assert L.tdm_probe_stream_mix(rd, 1, None, 0, n * 4, 3, 0, 0, stream_ptr(dev)) == 1
    assert L.tdm_probe_stream_mix(rd, 9, None, 0, n * 4, 1, 0, 0, stream_ptr(dev)) == 1
    torch.cuda.synchronize()
