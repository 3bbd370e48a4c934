"""A whole group on one GPU, in one process: rank r is a buffer in that GPU's HBM.

`LocalWorld(world)` runs tandem's ring collectives over a list of `world`
tensors (one per rank) with ONE kernel launch per ring step: the launch carries
every rank's (receive chunk, neighbour's chunk) pair, so a step that the
reference runs as `world` processes x pieces x (copy into a slot, add out of
it) is a single fused pass over HBM (an all-reduce can even be one launch). The results, including the partial sums a
bare reduce_scatter leaves in the other chunks, are bit for bit those of the
reference's Python engine (tandem/comm.py:301-385 there).

Everything is enqueued on torch's current stream; nothing synchronises.
"""

import ctypes

import torch

from . import _lib
from ._lib import Pair, check, dtype_code, lib, require_device_tensor, stream_ptr


def split_sizes(n, world):
    """Sizes of torch.tensor_split(flat, world): the first n % world chunks get
    one element more (tandem/comm.py:319-321, tandem/zero.py:29-30)."""
    base, extra = divmod(int(n), world)
    return [base + (1 if q < extra else 0) for q in range(world)]


def chunk_bounds(numel, world, sizes=None):
    """[lo, hi) per rank; explicit sizes must partition the tensor, as
    tandem/comm.py:322-324 demands."""
    if sizes is None:
        sizes = split_sizes(numel, world)
    sizes = [int(s) for s in sizes]
    if len(sizes) != world or sum(sizes) != numel or any(s < 0 for s in sizes):
        raise ValueError(f"chunk sizes {sizes} do not partition {numel} elements")
    out, lo = [], 0
    for s in sizes:
        out.append((lo, lo + s))
        lo += s
    return out


def _pairs(items):
    arr = (Pair * max(1, len(items)))()
    for i, (dst, src, count) in enumerate(items):
        arr[i].dst, arr[i].src, arr[i].count = dst, src, count
    return arr


class LocalWorld:
    def __init__(self, world):
        if world < 1:
            raise ValueError("world must be at least 1")
        if world > _lib.TDM_MAX_PAIRS:
            raise ValueError(f"LocalWorld handles up to {_lib.TDM_MAX_PAIRS} ranks per launch")
        self.world = world
        lib()  # fail now, not at the first collective, if the HIP library is missing

    # ---- checks
    def _ranks(self, bufs, what):
        """The rank buffers checked (one per rank, in GPU memory, contiguous, alike) and their
        addresses for the C ABI, with the count, dtype and device they share. No views are made:
        at small messages the host side of a call costs more than its launch."""
        if len(bufs) != self.world:
            raise ValueError(f"{what}: expected {self.world} rank buffers, got {len(bufs)}")
        t0 = bufs[0]
        require_device_tensor(t0, what)
        n, dtype, device = t0.numel(), t0.dtype, t0.device
        for t in bufs[1:]:
            require_device_tensor(t, what)
            if t.numel() != n or t.dtype != dtype or t.device != device:
                raise ValueError(f"{what}: rank buffers differ in size, dtype or device")
        return self._ptrs(bufs), n, dtype, device

    @staticmethod
    def _op(op):
        if op not in ("sum", "avg"):
            raise ValueError(f"unknown op {op}")
        return op == "avg"

    # ---- collectives over all ranks at once
    @staticmethod
    def _ptrs(flats):
        return (ctypes.c_void_p * len(flats))(*[f.data_ptr() for f in flats])

    @staticmethod
    def _sizes(bounds, given):
        if given is None:
            return (ctypes.c_int64 * 1)(), 0
        return (ctypes.c_int64 * len(bounds))(*[hi - lo for lo, hi in bounds]), len(bounds)

    def reduce_scatter(self, bufs, sizes=None, op="sum"):
        """In place on every rank's buffer; returns each rank's reduced chunk
        (a view), as Group.reduce_scatter does per rank (tandem/comm.py:349-369).
        One launch per ring step; the other chunks are left holding the same
        partial sums as in the reference."""
        average = self._op(op)
        ptrs, numel, dtype, device = self._ranks(bufs, "reduce_scatter")
        bounds = chunk_bounds(numel, self.world, sizes)
        arr, n = self._sizes(bounds, sizes)
        check(lib().tdm_local_reduce_scatter(ptrs, self.world, numel, dtype_code(dtype), arr, n, int(average), 1, stream_ptr(device)))
        return [bufs[r].reshape(-1)[bounds[r][0]:bounds[r][1]] for r in range(self.world)]

    def all_gather(self, bufs, sizes=None):
        """Rank r holds chunk r; afterwards every rank holds every chunk
        (tandem/comm.py:371-385). One launch per ring step."""
        ptrs, numel, dtype, device = self._ranks(bufs, "all_gather")
        bounds = chunk_bounds(numel, self.world, sizes)
        arr, n = self._sizes(bounds, sizes)
        check(lib().tdm_local_all_gather(ptrs, self.world, numel, dtype_code(dtype), arr, n, stream_ptr(device)))
        return bufs

    def all_reduce(self, bufs, op="sum", algorithm=None):
        """All-reduce in place (tandem/comm.py:326-347). algorithm="ring": the
        reduce-scatter then the all-gather, one launch per step. algorithm="fold"
        (the default up to 8 ranks): one launch that reads every rank's element,
        sums in the ring's order for the element's chunk and writes every rank;
        the same bits with about half the HBM traffic."""
        average = self._op(op)
        ptrs, numel, dtype, device = self._ranks(bufs, "all_reduce")
        if algorithm is None:
            algorithm = "fold" if self.world <= _lib.TDM_MAX_WORLD else "ring"
        if algorithm not in ("ring", "fold"):
            raise ValueError(f"unknown all-reduce algorithm {algorithm}")
        code = _lib.ALLREDUCE_FOLD if algorithm == "fold" else _lib.ALLREDUCE_RING
        check(lib().tdm_local_all_reduce(ptrs, self.world, numel, dtype_code(dtype), int(average), code, stream_ptr(device)))
        return bufs

    def unit_gather(self, fulls, shards, sizes):
        """ZeRO-3's gather of one unit for every rank (tandem/zero.py:238-245): every rank's shard
        is read once and stored into its place in all the fulls[r], in one launch (up to 8 ranks)."""
        if len(fulls) != self.world or len(shards) != self.world:
            raise ValueError("unit_gather: one full buffer and one shard per rank")
        bounds = chunk_bounds(fulls[0].numel(), self.world, sizes)
        for t in list(fulls) + list(shards):
            require_device_tensor(t, "unit_gather")
        for q, (lo, hi) in enumerate(bounds):
            if shards[q].numel() != hi - lo or shards[q].dtype != fulls[0].dtype:
                raise ValueError(f"unit_gather: shard {q} has {shards[q].numel()} elements, its chunk {hi - lo}")
        code = dtype_code(fulls[0].dtype)
        ptrs = (ctypes.c_void_p * self.world)(*[s.data_ptr() for s in shards])
        outs = (ctypes.c_void_p * self.world)(*[f.data_ptr() for f in fulls])
        szs = (ctypes.c_int64 * self.world)(*[hi - lo for lo, hi in bounds])
        check(lib().tdm_k4_unit_gather_all(outs, ptrs, szs, self.world, code, stream_ptr(fulls[0].device)))
        return fulls

    def bucket_table(self, tensors_per_rank, buckets, out_per_rank=None):
        """Prepares the K2 launch for DDP's bucket path with every rank on this
        GPU. tensors_per_rank[r][i] is rank r's gradient of parameter i;
        `buckets` lists the parameter positions of each bucket in packing order
        (tandem/ddp.py:56-68). The table is built and uploaded once; run() then
        averages every gradient across the ranks in one launch, writing the result
        to out_per_rank[r][i] (default: in place), bit for bit what flattening into
        the bucket, ring all_reduce(op="avg") and reading the views back gives."""
        return FoldTable(self, tensors_per_rank, buckets, out_per_rank)


class FoldTable:
    def __init__(self, lw, tensors_per_rank, buckets, out_per_rank=None):
        from .buckets import fold_segments

        world = lw.world
        if world > _lib.TDM_MAX_WORLD:
            raise ValueError(f"the bucket fold handles up to {_lib.TDM_MAX_WORLD} ranks")
        if len(tensors_per_rank) != world:
            raise ValueError("bucket_table: one list of gradients per rank")
        outs = tensors_per_rank if out_per_rank is None else out_per_rank
        first = tensors_per_rank[0]
        for r in range(world):
            if len(tensors_per_rank[r]) != len(first) or len(outs[r]) != len(first):
                raise ValueError("bucket_table: ranks differ in their number of tensors")
            for i, t in enumerate(tensors_per_rank[r]):
                require_device_tensor(t, "bucket_table")
                require_device_tensor(outs[r][i], "bucket_table")
                if t.numel() != first[i].numel() or t.dtype != first[0].dtype or outs[r][i].numel() != t.numel():
                    raise ValueError("bucket_table: ranks differ in a tensor's size or dtype")
        self.world, self.dtype, self.device = world, first[0].dtype, first[0].device
        self._keep = (tensors_per_rank, outs)  # the table holds raw addresses of these
        es = first[0].element_size()
        rows = []
        for members in buckets:
            for i, off, count, chunk in fold_segments([first[i].numel() for i in members], world):
                rows.append((members[i], off, count, chunk))
        segs = (_lib.FoldSeg * max(1, len(rows)))()
        for k, (i, off, count, chunk) in enumerate(rows):
            for r in range(world):
                segs[k].src[r] = tensors_per_rank[r][i].data_ptr() + off * es
                segs[k].dst[r] = outs[r][i].data_ptr() + off * es
            segs[k].count, segs[k].chunk = count, chunk
        self._upload(segs, len(rows))

    @classmethod
    def from_segments(cls, world, dtype, device, rows, keep=()):
        """rows: (src addresses per rank, dst addresses per rank (0 = none), count, chunk)."""
        self = cls.__new__(cls)
        self.world, self.dtype, self.device, self._keep = world, dtype, torch.device(device), keep
        segs = (_lib.FoldSeg * max(1, len(rows)))()
        for k, (srcs, dsts, count, chunk) in enumerate(rows):
            for r in range(world):
                segs[k].src[r] = srcs[r]
                segs[k].dst[r] = dsts[r] or None
            segs[k].count, segs[k].chunk = count, chunk
        self._upload(segs, len(rows))
        return self

    def _upload(self, segs, nseg):
        self.nseg = nseg
        self._segs = segs
        self.elements = sum(segs[k].count for k in range(nseg))
        nbytes = lib().tdm_k2_table_bytes(segs, self.nseg, dtype_code(self.dtype))
        self.ntiles = lib().tdm_k2_table_tiles(segs, self.nseg, dtype_code(self.dtype))
        if nbytes < 0:
            raise ValueError("bucket_table: bad segment table")
        image = torch.empty(max(16, nbytes), dtype=torch.uint8)
        check(lib().tdm_k2_table_build(segs, self.nseg, self.world, dtype_code(self.dtype), ctypes.c_void_p(image.data_ptr())))
        self.image = image.to(self.device)

    def run(self, average=True, accumulate=False):
        check(lib().tdm_k2_bucket_fold(ctypes.c_void_p(self.image.data_ptr()), self.ntiles, dtype_code(self.dtype),
                                       self.world, int(average), int(accumulate), stream_ptr(self.device)))


    def run_static(self, average=True, accumulate=False):
        """The same fold without the uploaded table: its records are written on the GPU
        into a fixed array inside the library, so the call allocates nothing and copies
        nothing from the host (for callers under HIP graph capture or in loops that must
        not allocate). At most lib().tdm_k2_static_max_tiles() tiles per call. The calls
        on one GPU share that array and the library orders them, across streams and host
        threads; only graph replays holding such a call are the caller's to order."""
        check(lib().tdm_k2_bucket_fold_static(self._segs, self.nseg, self.world, dtype_code(self.dtype), int(average),
                                              int(accumulate), stream_ptr(self.device)))


class LocalZeRO2:
    """ZeRO stage 2's communication and optimizer step for a whole group on one
    GPU: rank r owns bufs[r] (all parameters, flat), staging[r] (its gradients,
    flat, in registration order), grad_shards[r] and its own optimizer state.

    reduce_grads() is what ZeRO._on_grad/_after_backward do with the buckets
    (tandem/zero.py:119-156 in the reference): every bucket [a, b) is
    reduce-scattered (avg) with chunk sizes bucket_sizes(a, b) and each rank adds
    its chunk into its gradient shard. Buckets are independent, so ring step s of
    all of them travels in as few launches as the 16-pair limit allows.
    step() is ZeRO.step (tandem/zero.py:158-163): sharded AdamW on every rank's
    shard, then the all-gather of the flat parameter buffer."""

    def __init__(self, world, numels, device, bucket_bytes=25 << 20, order="host", one_allocation=False, dtype=torch.float32,
                 **adamw):
        """dtype: the element type of parameters, gradients and optimizer state: fp32, float64, bfloat16 or float16 (all but fp32 in
        host order; their gradients are reduced by the fold, which rounds every addition to the type as the ring does).
        one_allocation: every buffer (the ranks' parameters and gradients, the gradient shards, the optimizer
        state) is carved out of a single allocation, back to back at 128-byte boundaries, instead of being an
        allocation of its own. Where the streams of a launch lie relative to each other is worth a few per cent
        either way on this memory system; the default is what measured faster for the one-launch step."""
        from .buckets import FlatLayout, zero_buckets
        from .optim import LINE, ShardedAdamW, zeros_at_phase_of

        from .optim import SHARD_DTYPES

        if dtype not in SHARD_DTYPES:
            raise ValueError(f"LocalZeRO2 handles fp32, float64, bfloat16 and float16 (got {dtype})")
        es = torch.empty(0, dtype=dtype).element_size()
        self.dtype = dtype
        self.lw = LocalWorld(world)
        self.world = world
        self.layouts = [FlatLayout(numels, world, r) for r in range(world)]
        n = self.layouts[0].numel
        self.numel = n
        self.buckets = zero_buckets(list(numels), es, bucket_bytes)
        if one_allocation:
            if dtype != torch.float32:
                raise ValueError("one_allocation lays out fp32 buffers")
            per = LINE // 4
            room = lambda m: -(-m // per) * per + per  # a line of slack for the phase
            shard_room = sum(room(l.hi - l.lo) for l in self.layouts)
            pool = torch.zeros(2 * world * room(n) + 3 * shard_room, device=device)
            cursor = [(-pool.data_ptr() % LINE) // 4]

            def zeros_like_phase(like, numel=None):
                m = like.numel() if numel is None else numel
                lead = ((like.data_ptr() - (pool.data_ptr() + 4 * cursor[0])) % LINE) // 4
                out = pool[cursor[0] + lead:cursor[0] + lead + m]
                cursor[0] += room(m)
                return out

            self._pool = pool
            self.bufs = [zeros_like_phase(pool[cursor[0]:], n) for _ in range(world)]
            self.staging = [zeros_like_phase(self.bufs[0], n) for _ in range(world)]
        else:
            zeros_like_phase = zeros_at_phase_of
            self.bufs = [torch.zeros(n, device=device, dtype=dtype) for _ in range(world)]
            self.staging = [torch.zeros(n, device=device, dtype=dtype) for _ in range(world)]
        # every shard's gradient (and, below, its optimizer state) at the phase of the parameter shard it belongs to
        self.grad_shards = [zeros_like_phase(self.bufs[r][l.lo:l.hi]) for r, l in enumerate(self.layouts)]
        self.opts = [ShardedAdamW(order=order, **adamw) for _ in range(world)]
        self.device = torch.device(device)
        # ring step s of every bucket: (dst, src, count) pairs, and the final adds
        self._steps = [[] for _ in range(world - 1)]
        self._adds = []
        rows = []
        sb = [t.data_ptr() for t in self.staging]
        for a, b, _ in self.buckets:
            sizes = self.layouts[0].bucket_sizes(a, b)
            lo = a
            for c, m in enumerate(sizes):
                if m:
                    for s in range(world - 1):
                        r = (c + s + 2) % world  # the rank that receives chunk c on step s
                        self._steps[s].append((sb[r] + lo * es, sb[(r - 1) % world] + lo * es, m))
                    shard_at = lo - self.layouts[c].lo
                    self._adds.append((self.grad_shards[c].data_ptr() + shard_at * es, sb[c] + lo * es, m))
                    dsts = [0] * world
                    dsts[c] = self.grad_shards[c].data_ptr() + shard_at * es
                    rows.append(([p + lo * es for p in sb], dsts, m, c))
                lo += m
        self._fold = (FoldTable.from_segments(world, dtype, device, rows, keep=(self.staging, self.grad_shards))
                      if world <= _lib.TDM_MAX_WORLD else None)
        # The whole step as one launch (reduce_and_step): the optimizer state must exist, at fixed addresses.
        self._shards_zero = True
        self._step_table = None
        if world <= _lib.TDM_MAX_WORLD:
            for r in range(world):
                self.opts[r].state["flat"] = [0.0, zeros_like_phase(self.grad_shards[r]), zeros_like_phase(self.grad_shards[r])]
            segs = (_lib.StepSeg * max(1, len(rows)))()
            bb = [t.data_ptr() for t in self.bufs]
            for k, (srcs, _dsts, m, c) in enumerate(rows):
                lo = (srcs[0] - sb[0]) // es  # the segment's offset in the flat buffers
                at = lo - self.layouts[c].lo
                _, exp_avg, exp_avg_sq = self.opts[c].state["flat"]
                for r in range(world):
                    segs[k].grad[r] = srcs[r]
                    segs[k].param[r] = bb[r] + lo * es
                segs[k].exp_avg = exp_avg.data_ptr() + at * es
                segs[k].exp_avg_sq = exp_avg_sq.data_ptr() + at * es
                segs[k].count, segs[k].chunk, segs[k].dtype = m, c, dtype_code(dtype)
            ntiles = lib().tdm_k23_table_tiles(segs, len(rows))
            image = torch.empty(max(16, lib().tdm_k23_table_bytes(segs, len(rows))), dtype=torch.uint8)
            check(lib().tdm_k23_table_build(segs, len(rows), world, ctypes.c_void_p(image.data_ptr())))
            self._step_table = (image.to(device), ntiles)

    def _launch(self, items, scale_dst, scale_src, writeback):
        st = stream_ptr(self.device)
        for k in range(0, len(items), _lib.TDM_MAX_PAIRS):
            part = items[k:k + _lib.TDM_MAX_PAIRS]
            check(lib().tdm_k1_reduce_step(_pairs(part), len(part), dtype_code(self.dtype), self.world if scale_dst else 1,
                                           int(scale_dst), int(scale_src), int(writeback), st))

    def reduce_grads(self, algorithm="fold"):
        """algorithm="ring": the reduce-scatter's ring steps (all buckets of a step
        together), then grad_shard += mine. algorithm="fold" (default, up to 8
        ranks): one launch that reads every rank's gradient, sums in the ring's
        order for the chunk, and adds into the owner's gradient shard; the same bits
        (including -0.0 + 0.0 = +0.0 from the add) with half the HBM traffic. The
        staging buffers are left untouched by the fold."""
        self._shards_zero = False
        if algorithm == "fold" and self._fold is not None:
            self._fold.run(average=True, accumulate=True)
            return
        for s, items in enumerate(self._steps):
            self._launch(items, True, s == 0, s == 0)
        self._launch(self._adds, False, False, False)  # grad_shard += mine

    def reduce_and_step(self):
        """reduce_grads() and step() as ONE launch: for every element the ranks' gradients
        are folded in the ring's order, added to the (zero) gradient shard as
        grad_shard.add_(mine) would, the owner takes its AdamW step and the new
        parameter goes into every rank's buffer. The same bits as reduce_grads(); step()
        with 8W + 20 instead of 12W + 28 bytes of HBM traffic per element. Needs the
        gradient shards at zero (no accumulation since zero_grad()) and at most 8 ranks;
        the shards stay zero."""
        from .optim import step_hyper, step_scalars

        if self._step_table is None or not self._shards_zero:
            self.reduce_grads()
            self.step()
            return
        for opt in self.opts:
            opt.state["flat"][0] += 1.0
        o = self.opts[0]
        image, ntiles = self._step_table
        if self.dtype != torch.float32:
            hyper = step_hyper(o.state["flat"][0], o.lr, o.betas, o.eps, o.weight_decay)
            check(lib().tdm_k23_zero2_step_typed(ctypes.c_void_p(image.data_ptr()), ntiles, self.world, 1, dtype_code(self.dtype),
                                                 ctypes.byref(hyper), o.order, stream_ptr(self.device)))
            return
        scalars = step_scalars(o.state["flat"][0], o.lr, o.betas, o.eps, o.weight_decay)
        check(lib().tdm_k23_zero2_step(ctypes.c_void_p(image.data_ptr()), ntiles, self.world, 1, ctypes.byref(scalars),
                                       o.order, stream_ptr(self.device)))

    def step(self, fused_gather=True):
        """Every rank's AdamW step on its shard, then the all-gather of the flat
        parameter buffers (tandem/zero.py:157-164 in the reference). fused_gather (up
        to 8 ranks): the update writes the new parameters into all ranks' buffers in
        the same pass, 28 + 4(W-1) bytes per element instead of 28 + 8(W-1), the same
        values everywhere."""
        fused = fused_gather and self.world <= _lib.TDM_MAX_WORLD
        for r in range(self.world):
            l = self.layouts[r]
            copies = [self.bufs[q][l.lo:l.hi] for q in range(self.world) if q != r] if fused else ()
            self.opts[r].update("flat", self.bufs[r][l.lo:l.hi], self.grad_shards[r], copies)
        if not fused:
            self.lw.all_gather(self.bufs, self.layouts[0].sizes)

    def zero_grad(self):
        if not self._shards_zero:
            for g in self.grad_shards:
                g.zero_()
        self._shards_zero = True
