"""tdm_k2_bucket_fold_static, the bucket fold that allocates nothing: through the C ABI,
against tdm_k2_table_build + tdm_k2_bucket_fold on the same segments, bit for bit, on two
calls in a row (the second smaller, so that it finds the first call's records in the
shared table), then its refusal of a call beyond the fixed table, and calls that follow
each other on different streams and from different host threads without a wait between
them (the library orders their use of the shared table)."""

import ctypes

import numpy as np
import pytest
import torch

from helpers import bits

pytestmark = pytest.mark.gpu


def _segments(world, numels, seed, dev, dtype=torch.float32, out_of_place=True):
    """Per-rank gradients and outputs, and the bucket fold's segments over them."""
    from tandem_amd import _lib
    from tandem_amd.buckets import fold_segments

    gen = torch.Generator().manual_seed(seed)
    grads = [[(torch.randn(m, generator=gen) * 1e-3).to(dtype).to(dev) for m in numels] for _ in range(world)]
    outs = [[torch.full((m,), 7.0, dtype=dtype, device=dev) for m in numels] for _ in range(world)] if out_of_place else grads
    es = grads[0][0].element_size()
    rows = [(i, off, count, chunk) for i, off, count, chunk in fold_segments(list(numels), world)]
    segs = (_lib.FoldSeg * max(1, len(rows)))()
    for k, (i, off, count, chunk) in enumerate(rows):
        for r in range(world):
            segs[k].src[r] = grads[r][i].data_ptr() + off * es
            segs[k].dst[r] = outs[r][i].data_ptr() + off * es
        segs[k].count, segs[k].chunk = count, chunk
    return grads, outs, segs, len(rows)


def _with_table(segs, nseg, world, code, dev, average, accumulate):
    """The existing entry points: table image built on the host, copied to the device, folded."""
    from tandem_amd._lib import check, lib, stream_ptr

    nbytes = lib().tdm_k2_table_bytes(segs, nseg, code)
    ntiles = lib().tdm_k2_table_tiles(segs, nseg, code)
    image = torch.empty(max(16, nbytes), dtype=torch.uint8)
    check(lib().tdm_k2_table_build(segs, nseg, world, code, ctypes.c_void_p(image.data_ptr())))
    table = image.to(dev)
    check(lib().tdm_k2_bucket_fold(ctypes.c_void_p(table.data_ptr()), ntiles, code, world, average, accumulate, stream_ptr(dev)))
    torch.cuda.synchronize()
    return ntiles


def _static(segs, nseg, world, code, dev, average, accumulate):
    from tandem_amd._lib import check, lib, stream_ptr

    check(lib().tdm_k2_bucket_fold_static(segs, nseg, world, code, average, accumulate, stream_ptr(dev)))
    torch.cuda.synchronize()


def _same(a, b, what):
    for r, (xs, ys) in enumerate(zip(a, b)):
        for i, (x, y) in enumerate(zip(xs, ys)):
            assert np.array_equal(bits(x.float().cpu().numpy() if x.dtype == torch.bfloat16 else x.cpu().numpy()),
                                  bits(y.float().cpu().numpy() if y.dtype == torch.bfloat16 else y.cpu().numpy())), \
                f"{what}: rank {r}, tensor {i} differs"


CASES = [
    # (world, first call's tensors, second call's tensors (smaller), dtype, accumulate)
    (4, [300_001, 5, 70_000, 1_048_576, 4099, 1, 64] * 5, [4099, 64, 1000], torch.float32, 0),
    (2, [1_500_000, 3, 250_000], [1_000, 7], torch.float32, 1),
    (3, [40_000, 123_457] * 12, [513], torch.bfloat16, 0),
]


@pytest.mark.parametrize("world,first,second,dtype,accumulate", CASES)
def test_two_calls_in_a_row_match_the_table_entry_point(world, first, second, dtype, accumulate):
    from tandem_amd._lib import dtype_code

    dev = torch.device("cuda", 0)
    code = dtype_code(dtype)
    free_before = None
    for call, numels in enumerate((first, second)):
        print(f"static fold: world {world}, call {call}, {len(numels)} tensors, {sum(numels)} elements, {dtype}", flush=True)
        want_g, want_o, segs_a, nseg = _segments(world, numels, 11 + call, dev, dtype)
        got_g, got_o, segs_b, nseg_b = _segments(world, numels, 11 + call, dev, dtype)
        assert nseg == nseg_b
        ntiles = _with_table(segs_a, nseg, world, code, dev, 1, accumulate)
        if len(numels) > 16:
            assert nseg > 16, "this call should need more than one launch of the table's fill kernel"
        torch.cuda.synchronize()
        if call == 1:
            free_before = torch.cuda.mem_get_info(dev)[0]
        _static(segs_b, nseg, world, code, dev, 1, accumulate)
        if call == 1:
            assert torch.cuda.mem_get_info(dev)[0] == free_before, "the call changed the device's free memory"
        _same(want_o, got_o, f"call {call} ({ntiles} tiles) outputs")
        _same(want_g, got_g, f"call {call} inputs")


def test_in_place_and_integer_sum():
    from tandem_amd._lib import dtype_code

    dev = torch.device("cuda", 0)
    world, numels = 4, [70_001, 9, 2048]
    a = _segments(world, numels, 3, dev, torch.float32, out_of_place=False)
    b = _segments(world, numels, 3, dev, torch.float32, out_of_place=False)
    _with_table(a[2], a[3], world, dtype_code(torch.float32), dev, 1, 0)
    _static(b[2], b[3], world, dtype_code(torch.float32), dev, 1, 0)
    _same(a[0], b[0], "in place")
    a = _segments(world, numels, 4, dev, torch.float32)
    ia = [[(t * 1e6).to(torch.int32) for t in g] for g in a[0]]
    # integer tensors: rebuild the segments over them
    from tandem_amd import _lib
    from tandem_amd.buckets import fold_segments

    def segs_over(src, dst):
        rows = list(fold_segments(numels, world))
        segs = (_lib.FoldSeg * len(rows))()
        for k, (i, off, count, chunk) in enumerate(rows):
            for r in range(world):
                segs[k].src[r] = src[r][i].data_ptr() + off * 4
                segs[k].dst[r] = dst[r][i].data_ptr() + off * 4
            segs[k].count, segs[k].chunk = count, chunk
        return segs, len(rows)

    out1 = [[torch.zeros_like(t) for t in g] for g in ia]
    out2 = [[torch.zeros_like(t) for t in g] for g in ia]
    s1, n1 = segs_over(ia, out1)
    s2, n2 = segs_over(ia, out2)
    _with_table(s1, n1, world, dtype_code(torch.int32), dev, 0, 0)
    _static(s2, n2, world, dtype_code(torch.int32), dev, 0, 0)
    _same(out1, out2, "int32 sum")
    want = sum(t.cpu() for t in (ia[r][0] for r in range(world)))
    assert torch.equal(out2[2][0].cpu(), want)


def test_refuses_more_than_the_fixed_table_and_bad_segments():
    from tandem_amd import _lib
    from tandem_amd._lib import lib, stream_ptr

    dev = torch.device("cuda", 0)
    limit = lib().tdm_k2_static_max_tiles()
    tile_elems = lib().tdm_table_tile_bytes() // 4
    assert limit * 144 <= 4 << 20, "the fixed table is meant to stay modest"
    n = limit * tile_elems + 1  # one record too many
    x = [torch.zeros(n, device=dev) for _ in range(2)]
    before = [t.clone() for t in x]
    segs = (_lib.FoldSeg * 1)()
    for r in range(2):
        segs[0].src[r] = x[r].data_ptr()
        segs[0].dst[r] = x[r].data_ptr()
    segs[0].count, segs[0].chunk = n, 0
    status = lib().tdm_k2_bucket_fold_static(segs, 1, 2, 0, 1, 0, stream_ptr(dev))
    assert status == 1
    msg = lib().tdm_last_error().decode()
    assert "more than" in msg and str(limit) in msg and "split the call" in msg
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(x, before))
    segs[0].count = limit * tile_elems  # exactly the limit is accepted
    x[0].fill_(2.0)
    x[1].fill_(4.0)
    assert lib().tdm_k2_bucket_fold_static(segs, 1, 2, 0, 1, 0, stream_ptr(dev)) == 0
    torch.cuda.synchronize()
    assert bool((x[0][:limit * tile_elems] == 3.0).all()) and bool((x[1][:limit * tile_elems] == 3.0).all())
    assert float(x[0][-1]) == 2.0
    segs[0].chunk = 5
    assert lib().tdm_k2_bucket_fold_static(segs, 1, 2, 0, 1, 0, stream_ptr(dev)) == 1
    assert "chunk outside" in lib().tdm_last_error().decode()
    assert lib().tdm_k2_bucket_fold_static(segs, 0, 2, 0, 1, 0, stream_ptr(dev)) == 0  # nothing to do


def test_replayed_from_a_hip_graph():
    """The reason the entry point exists: a caller under HIP graph capture cannot allocate. Captured once (after one
    eager call, which looks the fixed table's address up), replayed three times over new gradients with eager work
    and a host wait between the replays: every replay's bits are those of the table entry point run eagerly."""
    from tandem_amd import LocalWorld

    dev = torch.device("cuda", 0)
    world = 4
    numels = [70_001, 9, 2048, 4099, 33, 1, 300_000] * 3  # 21 tensors: two launches of the fill kernel, then the fold
    buckets = [list(range(k, min(k + 4, len(numels)))) for k in range(0, len(numels), 4)]
    gen = torch.Generator().manual_seed(5)
    ins = [[[torch.randn(m, generator=gen) * 1e-3 for m in numels] for _ in range(world)] for _ in range(4)]
    grads = [[torch.empty(m, device=dev) for m in numels] for _ in range(world)]
    other = [[torch.empty(m, device=dev) for m in numels] for _ in range(world)]
    lw = LocalWorld(world)
    static, eager = lw.bucket_table(grads, buckets), lw.bucket_table(other, buckets)

    def load(k):
        for r in range(world):
            for i in range(len(numels)):
                grads[r][i].copy_(ins[k][r][i])
                other[r][i].copy_(ins[k][r][i])

    load(0)
    static.run_static(average=True)  # outside the capture
    torch.cuda.synchronize(dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static.run_static(average=True)
    for k in range(1, 4):
        load(k)
        graph.replay()
        eager.run(average=True)  # behind the replay on the same stream
        torch.cuda.synchronize(dev)
        for r in range(world):
            for i in range(len(numels)):
                assert np.array_equal(bits(grads[r][i].cpu().numpy()), bits(other[r][i].cpu().numpy())), (k, r, i)
        assert not torch.equal(grads[0][0].cpu(), ins[k][0][0])  # (the fold did run)


def test_calls_on_two_streams_and_from_two_threads_do_not_overlap():
    """All calls on a GPU share one table. A large call on one stream (its fold runs for a while) is followed at
    once, with no wait on the host, by a small call on another stream whose fill kernel overwrites the first
    records: the library makes the second stream wait for the first call's fold. Six such pairs alternating the
    streams, then the same from two host threads with a stream each; every call's result equals the table
    entry point's."""
    import threading

    from tandem_amd._lib import check, dtype_code, lib

    dev = torch.device("cuda", 0)
    world, code = 4, dtype_code(torch.float32)
    big, small = [1_048_576] * 12 + [300_001, 5, 4099], [4099, 64, 1000]
    streams = [torch.cuda.Stream(dev), torch.cuda.Stream(dev)]
    expected = {}
    for name, numels, seed in (("big", big, 21), ("small", small, 22)):
        g, o, segs, nseg = _segments(world, numels, seed, dev)
        _with_table(segs, nseg, world, code, dev, 1, 0)
        expected[name] = o

    def fresh(name, numels, seed):
        g, o, segs, nseg = _segments(world, numels, seed, dev)
        return dict(name=name, grads=g, outs=o, segs=segs, nseg=nseg)

    def enqueue(job, stream):
        check(lib().tdm_k2_bucket_fold_static(job["segs"], job["nseg"], world, code, 1, 0, ctypes.c_void_p(stream.cuda_stream)))

    for pair in range(6):
        a, b = fresh("big", big, 21), fresh("small", small, 22)
        torch.cuda.synchronize(dev)
        print(f"static fold on two streams: pair {pair}", flush=True)
        enqueue(a, streams[pair % 2])
        enqueue(b, streams[1 - pair % 2])  # nothing on the host between the two
        torch.cuda.synchronize(dev)
        _same(expected["big"], a["outs"], f"pair {pair}, the large call")
        _same(expected["small"], b["outs"], f"pair {pair}, the small call")

    jobs = [[fresh("big", big, 21), fresh("small", small, 22), fresh("big", big, 21)],
            [fresh("small", small, 22), fresh("big", big, 21), fresh("small", small, 22)]]
    torch.cuda.synchronize(dev)
    errors = []

    def worker(k):
        try:
            torch.cuda.set_device(dev)
            for job in jobs[k]:
                enqueue(job, streams[k])
        except Exception as e:  # surfaces in the main thread
            errors.append(e)

    print("static fold from two host threads", flush=True)
    threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize(dev)
    assert not errors, errors
    for k in range(2):
        for job in jobs[k]:
            _same(expected[job["name"]], job["outs"], f"thread {k}, a {job['name']} call")
