"""The host half of K2 and K2+K3: tdm_k2_table_* and tdm_k23_table_* cut segments into
tiles (tdm_table_tile_bytes() of every stream) and write the records the kernels walk. They build an image in
host memory and launch nothing, so they are checked here without a GPU: tile counts,
every record's pointers, counts, owner and alignment flag, and what they refuse."""

import ctypes

import numpy as np
import pytest

from tandem_amd import _lib
from tandem_amd._lib import lib

W = _lib.TDM_MAX_WORLD
F32, F64, F16, BF16, EINVAL = 0, 1, 2, 3, 1  # enum tdm_dtype and TDM_EINVAL of include/tandem_hip.h
FOLD_REC = np.dtype([("src", np.uint64, W), ("dst", np.uint64, W), ("count", np.int64), ("chunk", np.int32), ("vec_ok", np.int32)])
STEP_REC = np.dtype([("g", np.uint64, W), ("p", np.uint64, W), ("m", np.uint64), ("v", np.uint64), ("count", np.int64),
                     ("chunk", np.int32), ("vec_ok", np.int32)])
TILE_BYTES = lib().tdm_table_tile_bytes()


def fold_segs(world, es, rows):
    """rows: (count, chunk, byte offset added to every pointer[, extra bytes on the last rank's source])."""
    segs = (_lib.FoldSeg * len(rows))()
    for k, (count, chunk, off, *skew) in enumerate(rows):
        for r in range(world):
            segs[k].src[r] = (1 << 32) * (r + 1) + (k << 24) + off + (skew[0] if skew and r == world - 1 else 0)
            segs[k].dst[r] = (1 << 40) * (r + 1) + (k << 24) + off if r != 1 or world == 1 else 0  # rank 1 receives nothing
        segs[k].count, segs[k].chunk = count, chunk
    return segs


def walk(count, off, es, tile, skew=0):
    """How a segment is walked: (vectorised, head elements peeled, body elements, tiles). Pointers that all lie
    `off` bytes past a 16-byte boundary lose (16 - off) / es head elements and run vectorised from there; a segment
    no longer than its head, or one whose pointers disagree within 16 bytes, goes element by element."""
    if count == 0:
        return False, 0, 0, 0
    head = ((16 - off % 16) % 16) // es
    if skew % 16 or head >= count:
        return False, 0, count, -(-count // tile)
    return True, head, count - head, -(-(count - head) // tile)


@pytest.mark.parametrize("dtype,es", [(F32, 4), (F64, 8), (BF16, 2)])
@pytest.mark.parametrize("world", [1, 2, 3, 8])
def test_fold_table_records(world, dtype, es):
    tile = TILE_BYTES // es
    # aligned; off the grid by one element on every pointer (same phase: head peeled); a whole tile + 1 that ends up
    # exactly one tile after the peel; empty; 16 bytes in; a segment shorter than its head; pointers that disagree
    rows = [(1, 0, 0), (tile, world - 1, 0), (tile + 1, world // 2, es), (tile + 16 // es - 1, 0, es), (0, 0, 0), (5 * tile - 3, 0, 16),
            (17, world - 1, 32 + es), (1, 0, 16 - es), (3 * tile + 5, 0, es, es if world > 1 else 0)]
    segs = fold_segs(world, es, rows)
    plans = [walk(c, off, es, tile, *skew) for c, _, off, *skew in rows]
    assert any(p[0] and p[1] for p in plans) and any(not p[0] and p[2] for p in plans)
    ntiles = lib().tdm_k2_table_tiles(segs, len(rows), dtype)
    assert ntiles == sum(p[3] for p in plans)
    nbytes = lib().tdm_k2_table_bytes(segs, len(rows), dtype)
    assert nbytes == ntiles * FOLD_REC.itemsize
    image = np.full(nbytes, 0xAB, np.uint8)
    assert lib().tdm_k2_table_build(segs, len(rows), world, dtype, ctypes.c_void_p(image.ctypes.data)) == 0
    recs = image.view(FOLD_REC)
    at = 0
    for k, ((count, chunk, off, *skew), (vec, head, body, tiles)) in enumerate(zip(rows, plans)):
        done = 0
        while done < body:
            rec = recs[at]
            assert rec["count"] == min(tile, body - done) and rec["chunk"] == chunk
            # 0: element by element; 1: vectors; 1 + h on a segment's first record: h peeled elements lie before its pointers
            assert rec["vec_ok"] == (0 if not vec else 1 + head if done == 0 else 1), (k, done)
            for r in range(world):
                assert rec["src"][r] == segs[k].src[r] + (head + done) * es
                assert rec["dst"][r] == (segs[k].dst[r] + (head + done) * es if segs[k].dst[r] else 0)
                if vec:
                    assert rec["src"][r] % 16 == 0 and rec["dst"][r] % 16 == 0
            assert not rec["src"][world:].any() and not rec["dst"][world:].any()  # unused ranks stay zero
            done += int(rec["count"])
            at += 1
    assert at == ntiles


def step_segs(world, rows, dtype=F32):
    segs = (_lib.StepSeg * len(rows))()
    for k, (count, chunk, off) in enumerate(rows):
        segs[k].dtype = dtype
        for r in range(world):
            segs[k].grad[r] = (1 << 32) * (r + 1) + (k << 24) + off
            segs[k].param[r] = (1 << 40) * (r + 1) + (k << 24) + off
        segs[k].exp_avg, segs[k].exp_avg_sq = (1 << 50) + (k << 24) + off, (1 << 51) + (k << 24) + off
        segs[k].count, segs[k].chunk = count, chunk
    return segs


@pytest.mark.parametrize("dtype,es", [(F32, 4), (F64, 8), (BF16, 2), (F16, 2)])
@pytest.mark.parametrize("world", [1, 2, 4, 7])
def test_step_table_records(world, dtype, es):
    """A step segment names its element type (0 = fp32, what a caller that knows nothing of the field leaves there): a record
    covers tdm_table_tile_bytes() of every stream whatever the type, heads are peeled in elements of that type."""
    tile = TILE_BYTES // es
    rows = [(3, 0, 0), (2 * tile, world - 1, 0), (0, 0, 0), (tile + 9, world // 2, es), (4 * tile - 1, 0, 48), (tile + 2, 0, 8), (1, 0, 16 - es)]
    segs = step_segs(world, rows, dtype)
    plans = [walk(c, off, es, tile) for c, _, off in rows]
    assert any(p[0] and p[1] for p in plans)
    ntiles = lib().tdm_k23_table_tiles(segs, len(rows))
    assert ntiles == sum(p[3] for p in plans)
    nbytes = lib().tdm_k23_table_bytes(segs, len(rows))
    assert nbytes == ntiles * STEP_REC.itemsize
    image = np.full(nbytes, 0xCD, np.uint8)
    assert lib().tdm_k23_table_build(segs, len(rows), world, ctypes.c_void_p(image.ctypes.data)) == 0
    recs = image.view(STEP_REC)
    at = 0
    for k, ((count, chunk, off), (vec, head, body, tiles)) in enumerate(zip(rows, plans)):
        done = 0
        while done < body:
            rec = recs[at]
            assert rec["count"] == min(tile, body - done) and rec["chunk"] == chunk
            assert rec["vec_ok"] == (0 if not vec else 1 + head if done == 0 else 1), (k, done)
            for r in range(world):
                assert rec["g"][r] == segs[k].grad[r] + (head + done) * es and rec["p"][r] == segs[k].param[r] + (head + done) * es
            assert rec["m"] == segs[k].exp_avg + (head + done) * es and rec["v"] == segs[k].exp_avg_sq + (head + done) * es
            assert not rec["g"][world:].any() and not rec["p"][world:].any()
            done += int(rec["count"])
            at += 1
    assert at == ntiles


def test_step_tables_refuse_mixed_and_unknown_dtypes():
    L = lib()
    image = np.zeros(1 << 16, np.uint8)
    ptr = ctypes.c_void_p(image.ctypes.data)
    segs = step_segs(2, [(100, 0, 0), (100, 1, 0)], BF16)
    assert L.tdm_k23_table_build(segs, 2, 2, ptr) == 0
    segs[1].dtype = F64
    assert L.tdm_k23_table_build(segs, 2, 2, ptr) == EINVAL and "share one dtype" in L.tdm_last_error().decode()
    segs[0].dtype = segs[1].dtype = 5  # TDM_I32: not a shard type
    assert L.tdm_k23_table_tiles(segs, 2) == -1
    assert L.tdm_k23_table_build(segs, 2, 2, ptr) == EINVAL and "dtype" in L.tdm_last_error().decode()
    segs[0].dtype = segs[1].dtype = F64
    segs[0].grad[0] += 4  # a double 4 bytes off its grid
    assert L.tdm_k23_table_build(segs, 2, 2, ptr) == EINVAL and "element size" in L.tdm_last_error().decode()
    # the typed launch and the typed update check their arguments before they touch the GPU
    hyper = _lib.AdamwHyper()
    assert L.tdm_k23_zero2_step_typed(ptr, 1, 2, 1, 5, ctypes.byref(hyper), 0, None) == EINVAL and "dtype" in L.tdm_last_error().decode()
    assert L.tdm_k23_zero2_step_typed(ptr, 1, 2, 1, F64, ctypes.byref(hyper), 1, None) == EINVAL and "fp32 shards only" in L.tdm_last_error().decode()
    assert L.tdm_k23_zero2_step_typed(ptr, 1, 9, 1, F64, ctypes.byref(hyper), 0, None) == EINVAL and "world" in L.tdm_last_error().decode()
    assert L.tdm_k3_adamw_typed(ptr, ptr, ptr, ptr, 4, 5, ctypes.byref(hyper), 0, None, 0, None) == EINVAL and "dtype" in L.tdm_last_error().decode()
    assert L.tdm_k3_adamw_typed(ptr, ptr, ptr, ptr, 4, BF16, ctypes.byref(hyper), 1, None, 0, None) == EINVAL and "fp32 shards only" in L.tdm_last_error().decode()
    assert L.tdm_k3_adamw_typed(ptr, ptr, ptr, ptr, 0, BF16, ctypes.byref(hyper), 0, None, 0, None) == 0  # nothing to do
    # so does the step over one segment passed in the launch
    one = step_segs(2, [(100, 1, 0)], F64)
    scalars = _lib.AdamwScalars()
    assert L.tdm_k23_zero2_step_segment(one, 2, 1, ctypes.byref(scalars), 0, None) == EINVAL and "fp32 shards" in L.tdm_last_error().decode()
    assert L.tdm_k23_zero2_step_segment_typed(one, 2, 1, ctypes.byref(hyper), 1, None) == EINVAL and "fp32 shards only" in L.tdm_last_error().decode()
    assert L.tdm_k23_zero2_step_segment_typed(one, 9, 1, ctypes.byref(hyper), 0, None) == EINVAL and "world" in L.tdm_last_error().decode()
    assert L.tdm_k23_zero2_step_segment_typed(one, 1, 1, ctypes.byref(hyper), 0, None) == EINVAL and "chunk" in L.tdm_last_error().decode()
    assert L.tdm_k23_zero2_step_segment_typed(one, 2, 1, None, 0, None) == EINVAL and L.tdm_k23_zero2_step_segment_typed(None, 2, 1, ctypes.byref(hyper), 0, None) == EINVAL
    one[0].grad[1] += 4
    assert L.tdm_k23_zero2_step_segment_typed(one, 2, 1, ctypes.byref(hyper), 0, None) == EINVAL and "element size" in L.tdm_last_error().decode()
    one[0].dtype = 7  # TDM_I16
    assert L.tdm_k23_zero2_step_segment_typed(one, 2, 1, ctypes.byref(hyper), 0, None) == EINVAL and "dtype" in L.tdm_last_error().decode()
    one[0].dtype, one[0].count = BF16, 0
    assert L.tdm_k23_zero2_step_segment_typed(one, 2, 1, ctypes.byref(hyper), 0, None) == 0  # nothing to do


@pytest.mark.parametrize("dtype_name", ["float32", "float64", "bfloat16", "float16"])
def test_state_and_gradient_shards_follow_the_parameter_shards_phase(dtype_name):
    """optim.zeros_at_phase_of and the layout LocalZeRO2 makes with it (on CPU tensors: nothing is launched): world 3
    over a flat buffer of odd length puts the shards at three different distances from a cache line, and every shard's
    gradient and both moments start at the same distance; with one_allocation every buffer lies inside the one pool
    and none overlap; the step table counts the tiles of the element type."""
    import torch

    from tandem_amd.local import LocalZeRO2
    from tandem_amd.optim import zeros_at_phase_of

    dtype = getattr(torch, dtype_name)
    es = torch.empty(0, dtype=dtype).element_size()
    flat = torch.zeros(4096, dtype=dtype)
    for lo in (0, 1, 3, 128 // es - 1, 128 // es + 5):
        like = flat[lo:lo + 100]
        z = zeros_at_phase_of(like)
        assert z.numel() == 100 and z.dtype == dtype and z.data_ptr() % 128 == like.data_ptr() % 128 and not z.any()
        assert zeros_at_phase_of(like, 7).numel() == 7
    numels = [4099, 10_007, 33, 5001, 1, 12_288, 782]
    for one in ([False, True] if dtype == torch.float32 else [False]):
        z = LocalZeRO2(3, numels, "cpu", bucket_bytes=16 << 10, dtype=dtype, one_allocation=one)
        phases = set()
        for r, l in enumerate(z.layouts):
            phase = z.bufs[r][l.lo:l.hi].data_ptr() % 128
            phases.add(phase)
            assert z.grad_shards[r].data_ptr() % 128 == phase
            assert z.opts[r].state["flat"][1].data_ptr() % 128 == z.opts[r].state["flat"][2].data_ptr() % 128 == phase
            assert z.grad_shards[r].dtype == z.opts[r].state["flat"][1].dtype == dtype
        assert len(phases) == 3
        parts = z.bufs + z.staging + z.grad_shards + [t for o in z.opts for t in o.state["flat"][1:]]
        spans = sorted((t.data_ptr(), t.data_ptr() + es * t.numel()) for t in parts)
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
        if one:
            assert spans[0][0] >= z._pool.data_ptr() and spans[-1][1] <= z._pool.data_ptr() + 4 * z._pool.numel()
        image, ntiles = z._step_table
        assert ntiles >= sum(numels) * es // TILE_BYTES and image.numel() == ntiles * STEP_REC.itemsize


def test_empty_tables_and_refusals():
    L = lib()
    none = (_lib.FoldSeg * 1)()
    assert L.tdm_k2_table_tiles(none, 0, F32) == 0 and L.tdm_k2_table_bytes(none, 0, F32) == 16
    assert L.tdm_k2_table_tiles(none, -1, F32) == -1 and L.tdm_k2_table_tiles(none, 1, 99) == -1
    assert L.tdm_k2_table_tiles(None, 1, F32) == -1
    image = np.zeros(1 << 16, np.uint8)
    ptr = ctypes.c_void_p(image.ctypes.data)

    def refused(call, needle):
        assert call() == EINVAL
        assert needle in L.tdm_last_error().decode(), L.tdm_last_error().decode()

    good = fold_segs(2, 4, [(10, 1, 0)])
    assert L.tdm_k2_table_build(good, 1, 2, F32, ptr) == 0
    refused(lambda: L.tdm_k2_table_build(good, 1, 0, F32, ptr), "world")
    refused(lambda: L.tdm_k2_table_build(good, 1, 9, F32, ptr), "world")
    refused(lambda: L.tdm_k2_table_build(good, 1, 2, 99, ptr), "dtype")
    refused(lambda: L.tdm_k2_table_build(good, 1, 2, F32, None), "bad table arguments")
    refused(lambda: L.tdm_k2_table_build(good, 1, 1, F32, ptr), "chunk")  # chunk 1 of a world of one
    bad = fold_segs(2, 4, [(10, 0, 0)])
    bad[0].count = -1
    refused(lambda: L.tdm_k2_table_build(bad, 1, 2, F32, ptr), "negative count")
    bad = fold_segs(2, 4, [(10, 0, 2)])
    refused(lambda: L.tdm_k2_table_build(bad, 1, 2, F32, ptr), "aligned")
    bad = fold_segs(2, 4, [(10, 0, 0)])
    bad[0].src[1] = 0
    refused(lambda: L.tdm_k2_table_build(bad, 1, 2, F32, ptr), "NULL source")

    step = step_segs(2, [(10, 1, 0)])
    assert L.tdm_k23_table_build(step, 1, 2, ptr) == 0
    assert L.tdm_k23_table_tiles(step, -1) == -1 and L.tdm_k23_table_bytes(None, 2) == -1
    refused(lambda: L.tdm_k23_table_build(step, 1, 9, ptr), "world")
    refused(lambda: L.tdm_k23_table_build(step, 1, 1, ptr), "chunk")
    refused(lambda: L.tdm_k23_table_build(step, 1, 2, None), "bad table arguments")
    for field, needle in (("exp_avg", "NULL optimizer state"), ("exp_avg_sq", "NULL optimizer state")):
        bad = step_segs(2, [(10, 0, 0)])
        setattr(bad[0], field, 0)
        refused(lambda: L.tdm_k23_table_build(bad, 1, 2, ptr), needle)
    bad = step_segs(2, [(10, 0, 0)])
    bad[0].param[1] = 0
    refused(lambda: L.tdm_k23_table_build(bad, 1, 2, ptr), "NULL gradient or parameter")
    bad = step_segs(2, [(10, 0, 2)])
    refused(lambda: L.tdm_k23_table_build(bad, 1, 2, ptr), "aligned")
    bad = step_segs(2, [(10, 0, 0)])
    bad[0].count = -5
    refused(lambda: L.tdm_k23_table_build(bad, 1, 2, ptr), "negative count")


def test_tile_order_is_a_permutation_that_keeps_runs_on_one_xcd():
    """Every workgroup index takes exactly one tile and every tile is taken (a tile left out
    would be data left unreduced); workgroups that go to the same XCD (index % 8) take
    runs of 1 << shift consecutive tiles; the ragged end past the last whole group keeps
    its own index; shift 0 is the plain order."""
    from tandem_amd._lib import lib

    L = lib()
    for shift in range(0, 6):
        span = 8 << shift
        for total in (1, 7, 8, span - 1, span, span + 1, 3 * span + 5, 5 * span, 1000):
            tiles = [L.tdm_tile_of(i, total, shift) for i in range(total)]
            assert sorted(tiles) == list(range(total)), (shift, total)
            whole = total - total % span
            assert tiles[whole:] == list(range(whole, total))
            if shift == 0:
                assert tiles == list(range(total))
            for i in range(0, whole - 8, 8):  # the same XCD's next workgroup
                same_run = (i % span) // 8 + 1 < (1 << shift)
                if same_run:
                    assert tiles[i + 8] == tiles[i] + 1, (shift, total, i)
    assert L.tdm_tile_of(5, 5, 0) == -1 and L.tdm_tile_of(-1, 5, 0) == -1 and L.tdm_tile_of(0, 5, 13) == -1
