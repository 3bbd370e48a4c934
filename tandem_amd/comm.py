"""Collectives between processes that share one MI355X: tandem's `Group`,
`Work`, `CommError` and `launch` with one backend, "hip".

The class is a drop-in for the reference's plug-in point (tandem/comm.py:110-147
there: `Group(rank, size, device, sync, queues, slot_bytes, slots, timeout,
transport, priority, backend, job)`), so the DDP / ZeRO / FSDP wrappers and any
`fn(group, *args)` written for tandem run unchanged with `backend="hip"`. All
work happens in libtandem_hip.so: an engine per rank with its own progress
thread and HIP stream, slots shared through HIP IPC memory handles, ordered by
interprocess events. A collective returns a Work immediately; `wait()` makes the
caller's current stream wait for it without blocking the host on the GPU.

There is no CPU path and no Python engine here: any other backend, or a CPU
device, raises CommError.
"""

import ctypes
import os
import time

import torch
import torch.multiprocessing as mp

from . import _lib
from ._lib import AdamwHyper, check, dtype_code, lib

DEFAULT_SLOT_BYTES = 4 << 20
DEFAULT_SLOTS = 2
DEFAULT_TIMEOUT = float(os.environ.get("TANDEM_TIMEOUT", "600"))
DEFAULT_BACKEND = os.environ.get("TANDEM_BACKEND", "hip")


class CommError(RuntimeError):
    pass


class Work:
    """A collective in flight on the engine's thread and stream."""

    def __init__(self, name, group, handle, result, nbytes, keep):
        self.name, self._group, self._handle, self.result, self._nbytes = name, group, handle, result, nbytes
        self._keep = keep  # the tensors the engine reads and writes stay alive until waited for
        self._recorded = False
        self._waited = False

    def wait(self, stream_ordered=False):
        """Returns the collective's result once the caller's current stream is ordered behind it
        (tandem/comm.py:92-107 in the reference). stream_ordered=True: a collective that has not run yet is not
        waited for on the host; the stream is parked on it and the call returns at once, so the host can go on
        queueing work (an optimizer's launches, say) behind it. A failure of such a collective is raised by the
        next call on the group instead of by this one. The parked stream waits in a kernel with a time limit
        (the group's timeout and ten seconds; TANDEM_HIP_PARK_LIMIT_S): should the collective's end never reach
        it, the stream goes on and the next call on the group fails with "gave up". In a process limited to
        fewer than four hardware queues (GPU_MAX_HW_QUEUES) nothing is parked and this is the plain wait."""
        g = self._group
        if self._handle is None:
            return self.result
        t0 = time.perf_counter() if g.tracing and not self.is_completed() else None
        try:
            wait = lib().tdm_work_wait_stream if stream_ordered else lib().tdm_work_wait
            check(wait(self._handle, _lib.stream_ptr(g.device)))
        except Exception as e:
            raise CommError(f"{self.name} failed") from e
        if t0 is not None:
            g.waits.append((self.name, t0, time.perf_counter()))
        if g.tracing and not self._recorded:
            g._untimed.append(self)  # its span is read when Group.trace is next looked at
        self._recorded = True
        self._waited = True
        return self.result

    def is_completed(self):
        return self._handle is None or bool(lib().tdm_work_done(self._handle))

    def __del__(self):
        h, self._handle = getattr(self, "_handle", None), None
        if h is None:
            return
        try:
            g = self._group
            if not self._waited and self._keep and not g._closed:
                # Dropped without a wait: nothing orders the caller's stream behind the collective, so the tensors must
                # outlive it here (the reference's engine holds them until the job has run, tandem/csrc/collectives.cpp:314-317).
                g._orphans.append((h, self._keep))
                return
            lib().tdm_work_free(h)
        except Exception:
            pass


class Group:
    """One rank's view of the group."""

    stream_ordered_waits = True  # Work.wait(stream_ordered=True) exists (the wrappers ask before they use it)

    def __init__(self, rank, size, device, sync, queues=None, slot_bytes=DEFAULT_SLOT_BYTES, slots=DEFAULT_SLOTS,
                 timeout=DEFAULT_TIMEOUT, transport=None, priority=None, backend=None, job=None):
        self.rank, self.size = rank, size
        self.device = torch.device(device)
        self.slot_bytes, self.slots, self.timeout = slot_bytes, slots, timeout
        self.transport = transport or "device"
        self.priority = 0  # every stream here runs at the default priority
        self.backend = backend or DEFAULT_BACKEND
        self._trace, self._untimed, self.waits, self._tracing = [], [], [], False
        self._closed = False
        self._engine = None
        self._arena = None
        self.arena_count = 0  # arenas shared so far
        self._orphans = []  # (handle, tensors) of collectives whose Work was dropped before anybody waited for it
        if self.backend != "hip":
            raise CommError(f"unknown backend {self.backend} (tandem_amd provides \"hip\")")
        if self.transport != "device":
            raise CommError(f"unknown transport {self.transport} (ranks share one GPU's memory)")
        if self.device.type != "cuda":
            raise CommError("the hip backend needs device=\"cuda\": there is no CPU path")
        if job is None:
            raise CommError("the hip engine needs a job name (launch() makes one)")
        self._barrier = sync[2] if isinstance(sync, (tuple, list)) else sync
        index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self.device = torch.device("cuda", index)
        handle = ctypes.c_void_p()
        try:
            check(lib().tdm_engine_create(job.encode(), rank, size, slots, slot_bytes, float(timeout), index,
                                          ctypes.byref(handle)))
            self._engine = handle
            self._barrier.wait(timeout=timeout)  # every rank has published its slots and events
            check(lib().tdm_engine_connect(self._engine))
        except CommError:
            raise
        except Exception as e:
            raise CommError(f"could not start the hip engine: {e}") from e
        self.barrier()

    @staticmethod
    def make_sync(ctx, size, slots):
        """What a launcher creates once and every rank inherits, with the reference's signature and shape
        (tandem/comm.py:175-181 there): (full, free, barrier). The hip engine hands pieces over through its own
        shared-memory rings, so only the barrier is used; the two semaphore lists are there so that code written
        for the reference's launcher runs unchanged."""
        full = [ctx.Semaphore(0) for _ in range(size * size)]
        free = [ctx.Semaphore(slots) for _ in range(size * size)]
        return full, free, ctx.Barrier(size)

    # ---- tracing (tandem/comm.py:132-134 there: trace, waits, tracing)
    @property
    def tracing(self):
        return self._tracing

    @tracing.setter
    def tracing(self, on):
        """While on, every collective waited for leaves (name, start, end, bytes) in
        `trace` and the time its caller was blocked in `waits`, on time.perf_counter's
        clock. start and end are the GPU's: from the moment the inputs were ready on
        the engine's stream to the end of the collective's last kernel (device time
        stamps placed on the host clock), unless TANDEM_HIP_TRACE=host asks for the
        progress thread's own start and end as the reference's engine records them
        (tandem/csrc/collectives.cpp:203-223)."""
        self._tracing = bool(on)
        if self._engine is not None and os.environ.get("TANDEM_HIP_TRACE", "device") != "host":
            check(lib().tdm_engine_set_timing(self._engine, 1 if on else 0))

    @property
    def trace(self):
        # Reading a device time stamp waits for that collective's last kernel, so the
        # spans are filled in here, when somebody looks, and not inside wait().
        pending, self._untimed = self._untimed, []
        for w in pending:
            a, b = ctypes.c_double(0), ctypes.c_double(0)
            try:
                check(lib().tdm_work_times(w._handle, ctypes.byref(a), ctypes.byref(b)))
            except Exception as e:
                raise CommError(f"{w.name}: could not read its time stamps") from e
            self._trace.append((w.name, a.value, b.value, w._nbytes))  # steady clock == perf_counter's clock
        return self._trace

    @trace.setter
    def trace(self, spans):
        self._untimed = []
        self._trace = spans

    # ---- plumbing
    def _reap(self):
        """Lets go of the tensors of dropped collectives that have finished on the GPU."""
        still = []
        for h, keep in self._orphans:
            if lib().tdm_work_done(h):
                lib().tdm_work_free(h)
            else:
                still.append((h, keep))
        self._orphans = still

    def _start(self, name, call, result, nbytes, async_op, keep=()):
        if self._closed:
            raise CommError("group is closed")
        if self._orphans:
            self._reap()
        out = ctypes.c_void_p()
        try:
            check(call(ctypes.byref(out)))
        except (ValueError, RuntimeError, TimeoutError) as e:
            raise CommError(f"{name}: {e}") from e
        work = Work(name, self, out, result, nbytes, keep)
        return work if async_op else work.wait()

    def _flat(self, t, what):
        if not isinstance(t, torch.Tensor) or t.device != self.device:
            raise CommError(f"{what}: the tensor is not on {self.device}")
        if not t.is_contiguous():
            raise CommError("collectives need contiguous tensors")
        return t.reshape(-1)

    def _sizes(self, flat, sizes):
        if sizes is None:
            return None, (ctypes.c_int64 * 1)(), 0
        sizes = [int(s) for s in sizes]
        if len(sizes) != self.size or sum(sizes) != flat.numel() or any(s < 0 for s in sizes):
            raise CommError(f"chunk sizes {sizes} do not partition {flat.numel()} elements")
        return sizes, (ctypes.c_int64 * len(sizes))(*sizes), len(sizes)

    def _chunk_of_rank(self, flat, sizes):
        if sizes is None:
            return torch.tensor_split(flat, self.size)[self.rank]
        lo = sum(sizes[:self.rank])
        return flat[lo:lo + sizes[self.rank]]

    @staticmethod
    def _code(t, reduce):
        code = _lib.DTYPES.get(t.dtype)
        if code is None:
            if reduce:
                raise CommError(f"the hip backend cannot reduce {t.dtype}")
            return _lib.TDM_BYTES
        return code

    @staticmethod
    def _count(t, code):
        return t.numel() * t.element_size() if code == _lib.TDM_BYTES else t.numel()

    def _stream(self):
        return _lib.stream_ptr(self.device)

    # ---- collectives
    def _direct_offsets(self, flat, direct, what):
        """Arena offsets of every rank's tensor for a direct collective: `direct=True`
        says every rank holds it at the same place of its arenas (ranks that allocate
        the same things in the same order do), a list gives them (arena_offset())."""
        if flat.numel() == 0:  # nothing to read, but the ranks still meet
            return (ctypes.c_int64 * self.size)()
        mine = self.arena_offset(flat)
        if mine is None:
            raise CommError(f"{what}: direct collectives need a tensor from shared_empty()")
        offs = [mine] * self.size if direct is True else [int(o) for o in direct]
        if len(offs) != self.size or offs[self.rank] != mine:
            raise CommError(f"{what}: one arena offset per rank, this rank's own among them")
        return (ctypes.c_int64 * self.size)(*offs)

    def all_reduce(self, t, op="sum", async_op=False, direct=False):
        """Ring all-reduce in place: reduce-scatter, then all-gather. With `direct`
        (tensors in the ranks' shared arenas) each rank folds its own chunk straight
        out of its peers' tensors, in the ring's order, and writes the result into
        every rank's tensor: the same bits, without slots."""
        if op not in ("sum", "avg"):
            raise CommError(f"unknown op {op}")
        flat = self._flat(t, "all_reduce")
        code = self._code(flat, True)
        if direct:
            offs = self._direct_offsets(flat, direct, "all_reduce")
            return self._start("all_reduce", lambda out: lib().tdm_direct_all_reduce(
                self._engine, ctypes.c_void_p(flat.data_ptr()), flat.numel(), code, int(op == "avg"), offs, self.size,
                self._stream(), out), t, t.numel() * t.element_size(), async_op, keep=(flat,))
        return self._start("all_reduce", lambda out: lib().tdm_all_reduce(
            self._engine, ctypes.c_void_p(flat.data_ptr()), flat.numel(), code, int(op == "avg"), self._stream(), out),
            t, t.numel() * t.element_size(), async_op, keep=(flat,))

    partial_sums_optional = True  # reduce_scatter(partial_sums=False) exists: wrappers that drop the rest may ask for it

    def reduce_scatter(self, t, sizes=None, op="sum", async_op=False, direct=False, partial_sums=True):
        """Sums `t` across ranks, leaving rank r's chunk (chunk r of
        torch.tensor_split, or of `sizes`) reduced in place; returns that view.
        The other chunks hold the ring's partial sums afterwards, as in the
        reference (tandem/comm.py:350-352). A caller that only wants its chunk says
        `partial_sums=False`: the rest of `t` is then left as it was, and the engine
        needs one handshake per pass instead of two per piece. `direct` (tensors
        in the shared arenas) implies it."""
        if op not in ("sum", "avg"):
            raise CommError(f"unknown op {op}")
        flat = self._flat(t, "reduce_scatter")
        code = self._code(flat, True)
        sizes, arr, n = self._sizes(flat, sizes)
        mine = self._chunk_of_rank(flat, sizes)
        if direct:
            offs = self._direct_offsets(flat, direct, "reduce_scatter")
            return self._start("reduce_scatter", lambda out: lib().tdm_direct_reduce_scatter(
                self._engine, ctypes.c_void_p(flat.data_ptr()), flat.numel(), code, arr, n, int(op == "avg"), offs,
                self.size, self._stream(), out), mine, t.numel() * t.element_size(), async_op, keep=(flat,))
        call = lib().tdm_reduce_scatter if partial_sums else lib().tdm_reduce_scatter_owner
        return self._start("reduce_scatter", lambda out: call(
            self._engine, ctypes.c_void_p(flat.data_ptr()), flat.numel(), code, arr, n, int(op == "avg"), self._stream(), out),
            mine, t.numel() * t.element_size(), async_op, keep=(flat,))

    def all_gather(self, t, sizes=None, async_op=False, direct=False):
        """Each rank holds its own chunk of `t` (chunk r); fills in the rest (with
        `direct`, by copying every chunk straight from its owner's arena)."""
        flat = self._flat(t, "all_gather")
        code = self._code(flat, False)
        sizes, arr, n = self._sizes(flat, sizes)
        if direct:
            if code == _lib.TDM_BYTES:
                raise CommError(f"all_gather: direct gathers need one of {sorted(str(d) for d in _lib.DTYPES)}")
            offs = self._direct_offsets(flat, direct, "all_gather")
            return self._start("all_gather", lambda out: lib().tdm_direct_all_gather(
                self._engine, ctypes.c_void_p(flat.data_ptr()), flat.numel(), code, arr, n, offs, self.size,
                self._stream(), out), t, t.numel() * t.element_size(), async_op, keep=(flat,))
        if code == _lib.TDM_BYTES and n:
            arr = (ctypes.c_int64 * n)(*[s * flat.element_size() for s in sizes])
        return self._start("all_gather", lambda out: lib().tdm_all_gather(
            self._engine, ctypes.c_void_p(flat.data_ptr()), self._count(flat, code), code, arr, n, self._stream(), out),
            t, t.numel() * t.element_size(), async_op, keep=(flat,))

    def zero2_step(self, params, grads, sizes, exp_avg, exp_avg_sq, scalars, order, op="avg", async_op=False):
        """ZeRO stage 2's reduce_scatter, gradient add, AdamW and all_gather as one
        launch per rank (tandem/zero.py:141-163 in the reference, which makes a
        reduce_scatter per bucket, `grad_shard.add_`, seven elementwise passes and an
        all_gather of it). `params` and `grads` are the flat parameter and gradient
        buffers, from shared_empty() at the same arena offsets on every rank; `sizes`
        the shard sizes; `exp_avg`/`exp_avg_sq` this rank's state for its shard;
        `scalars` from optim.step_scalars (fp32 buffers) or optim.step_hyper (fp32, fp64,
        bf16 or fp16 buffers). The same bits as the separate calls when the gradient shard
        was zero before."""
        if op not in ("sum", "avg"):
            raise CommError(f"unknown op {op}")
        p, g = self._flat(params, "zero2_step"), self._flat(grads, "zero2_step")
        typed = isinstance(scalars, AdamwHyper)  # doubles: any of the shard types; fp32 constants: fp32 buffers
        kinds = (torch.float32, torch.float64, torch.bfloat16, torch.float16) if typed else (torch.float32,)
        if p.dtype not in kinds or g.dtype != p.dtype or p.numel() != g.numel():
            raise CommError("zero2_step: two buffers of one length and dtype (fp32; with constants from optim.step_hyper also fp64, bf16, fp16)")
        es = p.element_size()
        sizes, _, _ = self._sizes(p, sizes if sizes is not None else [c.numel() for c in torch.tensor_split(p, self.size)])
        lo, n = sum(sizes[:self.rank]), sizes[self.rank]
        for name, t in (("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq)):
            if t.device != self.device or t.dtype != p.dtype or t.numel() != n or not t.is_contiguous():
                raise CommError(f"zero2_step: {name} must be this rank's shard ({n} {p.dtype} elements on {self.device})")
        bases = []
        for t in (p, g):
            off = self.arena_offset(t) if t.numel() else 0  # empty buffers: nothing to read, but the ranks still meet
            if off is None:
                raise CommError("zero2_step: the buffers must come from shared_empty()")
            bases.append((ctypes.c_int64 * self.size)(*[off + lo * es] * self.size))
        mine_p, mine_g = p[lo:lo + n], g[lo:lo + n]
        head = (self._engine, ctypes.c_void_p(mine_p.data_ptr()), bases[0], ctypes.c_void_p(mine_g.data_ptr()), bases[1], self.size,
                ctypes.c_void_p(exp_avg.data_ptr()), ctypes.c_void_p(exp_avg_sq.data_ptr()), n, p.numel(), int(op == "avg"))
        if typed:
            call = lambda out: lib().tdm_direct_zero2_step_typed(*head, dtype_code(p.dtype), ctypes.byref(scalars), order, self._stream(), out)
        else:
            call = lambda out: lib().tdm_direct_zero2_step(*head, ctypes.byref(scalars), order, self._stream(), out)
        return self._start("zero2_step", call, params, (2 * self.size + 5) * es * n, async_op, keep=(p, g, exp_avg, exp_avg_sq, scalars))

    # ---- shared arenas: long-lived data that peers read (and the direct collectives write) in place
    ARENA_LIMIT = (1 << 31) - 4096  # an arena is one exported allocation, and those stay under 2 GiB

    def share_arena(self, nbytes):
        """Shares an arena: `nbytes` (under 2 GiB) of device memory owned by the engine
        (freed by close()) and exported once through HIP IPC, so that the other ranks can
        read and write it directly. A group may share up to 64; shared_empty() carves from
        the newest."""
        nbytes = max(16, int(nbytes))
        ptr = ctypes.c_void_p()
        try:
            check(lib().tdm_engine_share(self._engine, nbytes, ctypes.byref(ptr)))
        except (ValueError, RuntimeError) as e:
            raise CommError(f"share_arena: {e}") from e

        class _Raw:  # what torch needs to wrap foreign device memory
            __cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (ptr.value, False), "version": 3}

        self._arena = torch.as_tensor(_Raw(), device=self.device)
        self._arena_used = 0
        self.arena_count += 1

    def shared_empty(self, numel, dtype=torch.float32, grow=None):
        """A tensor of `numel` elements in this rank's newest shared arena, for
        gather_unit(..., peer_offsets=...) and the `direct` collectives (256-byte aligned,
        never given back). Without an arena, one of exactly this size is shared first. A
        tensor that does not fit into what is left is refused, unless `grow` says how many
        bytes a further arena should have (at least the tensor's): then one is shared and
        the tensor starts it. Every change of an arena tensor that peers read on their own
        (gather_unit) must sit between two fence() calls; the direct collectives fence by
        themselves."""
        es = torch.empty(0, dtype=dtype).element_size()
        need = numel * es
        if self._arena is None:
            self.share_arena(need if grow is None else max(need, min(int(grow), self.ARENA_LIMIT)))
        at = -(-self._arena_used // 256) * 256
        if at + need > self._arena.numel():
            if grow is None:
                raise CommError(f"shared_empty: {need} bytes do not fit in the arena "
                                f"({self._arena.numel() - at} of {self._arena.numel()} left)")
            self.share_arena(max(need, min(int(grow), self.ARENA_LIMIT)))
            at = 0
        self._arena_used = at + need
        return self._arena[at:at + need].view(dtype)

    def arena_offset(self, t):
        """Where tensor `t` lies in this rank's arenas, as the one number the peers name the place by (the
        arena's index times 2^31 plus the byte offset within it); None if it does not lie within one of them."""
        off = ctypes.c_int64(-1)
        check(lib().tdm_engine_arena_offset(self._engine, ctypes.c_void_p(t.data_ptr() if t.numel() else 0),
                                            t.numel() * t.element_size(), ctypes.byref(off)))
        return off.value if off.value >= 0 else None

    def fence(self):
        """A barrier ordered against the GPU: returns (on the caller's stream) once
        every rank's work queued before its fence() has finished on its GPU streams."""
        return self._start("fence", lambda out: lib().tdm_fence(self._engine, self._stream(), out), None, 0, False)

    def gather_unit(self, full, shard, sizes=None, async_op=False, peer_offsets=None):
        """ZeRO-3's gather of one unit: `shard` (this rank's chunk) is placed into
        `full` and the other ranks' chunks are gathered, all on the engine's
        stream. Same result as `full[lo:hi].copy_(shard); all_gather(full, sizes)`."""
        flat = self._flat(full, "gather_unit")
        sh = self._flat(shard, "gather_unit")
        if sh.dtype != flat.dtype:
            raise CommError("gather_unit: shard and full buffer differ in dtype")
        code = self._code(flat, False)
        sizes, arr, n = self._sizes(flat, sizes)
        if self._chunk_of_rank(flat, sizes).numel() != sh.numel():
            raise CommError(f"gather_unit: the shard has {sh.numel()} elements, this rank's chunk another count")
        if peer_offsets is not None:
            # every rank's chunk is read straight from that rank's arena: no staging, no handshake
            if len(peer_offsets) != self.size:
                raise CommError("gather_unit: one arena offset per rank")
            offs = (ctypes.c_int64 * self.size)(*[int(o) for o in peer_offsets])
            return self._start("gather_unit", lambda out: lib().tdm_unit_gather_direct(
                self._engine, ctypes.c_void_p(flat.data_ptr()), flat.numel(), code, ctypes.c_void_p(sh.data_ptr()), arr, n,
                offs, self.size, self._stream(), out), full, full.numel() * full.element_size(), async_op, keep=(flat, sh))
        if code == _lib.TDM_BYTES and n:
            arr = (ctypes.c_int64 * n)(*[s * flat.element_size() for s in sizes])
        return self._start("gather_unit", lambda out: lib().tdm_unit_gather(
            self._engine, ctypes.c_void_p(flat.data_ptr()), self._count(flat, code), code, ctypes.c_void_p(sh.data_ptr()),
            arr, n, self._stream(), out), full, full.numel() * full.element_size(), async_op, keep=(flat, sh))

    def pack(self, flat, pieces):
        """Bucket flatten as one gather: flat[offset : offset + t.numel()] = t for
        every (offset, t) in `pieces`, in launches of up to 16 streams each on the
        caller's current stream (the gradients were produced there). Replaces one
        `view.copy_(p.grad)` per parameter (tandem/ddp.py:92-94, tandem/zero.py:130,297
        in the reference)."""
        dst = self._flat(flat, "pack")
        code = self._code(dst, True)
        es = dst.element_size()
        items = []
        for off, t in pieces:
            src = self._flat(t, "pack")
            if src.dtype != dst.dtype:
                raise CommError("pack: a piece differs in dtype from the flat buffer")
            if off < 0 or off + src.numel() > dst.numel():
                raise CommError("pack: a piece does not fit the flat buffer")
            if src.numel():
                items.append((dst.data_ptr() + off * es, src.data_ptr(), src.numel()))
        for k in range(0, len(items), _lib.TDM_MAX_PAIRS):
            part = items[k:k + _lib.TDM_MAX_PAIRS]
            arr = (_lib.Pair * len(part))()
            for i, (d, s, n) in enumerate(part):
                arr[i].dst, arr[i].src, arr[i].count = d, s, n
            try:
                check(lib().tdm_k1_copy_step(arr, len(part), code, 0, self._stream()))
            except (ValueError, RuntimeError) as e:
                raise CommError(f"pack: {e}") from e
        return flat

    def broadcast(self, t, root=0, async_op=False):
        """Pipelined along the ring from root."""
        flat = self._flat(t, "broadcast")
        code = self._code(flat, False)
        return self._start("broadcast", lambda out: lib().tdm_broadcast(
            self._engine, ctypes.c_void_p(flat.data_ptr()), self._count(flat, code), code, root, self._stream(), out),
            t, t.numel() * t.element_size(), async_op, keep=(flat,))

    def send(self, t, dst, async_op=False):
        flat = self._flat(t, "send")
        code = self._code(flat, False)
        return self._start(f"send->{dst}", lambda out: lib().tdm_sendrecv(
            self._engine, ctypes.c_void_p(flat.data_ptr()), self._count(flat, code), dst, None, 0, -1, code, self._stream(), out),
            t, t.numel() * t.element_size(), async_op, keep=(flat,))

    def recv(self, t, src, async_op=False):
        flat = self._flat(t, "recv")
        code = self._code(flat, False)
        return self._start(f"recv<-{src}", lambda out: lib().tdm_sendrecv(
            self._engine, None, 0, -1, ctypes.c_void_p(flat.data_ptr()), self._count(flat, code), src, code, self._stream(), out),
            t, t.numel() * t.element_size(), async_op, keep=(flat,))

    def sendrecv(self, send, dst, recv, src, async_op=False):
        """Sends one tensor while receiving another, piece by piece in lockstep."""
        sf, rf = self._flat(send, "sendrecv"), self._flat(recv, "sendrecv")
        if sf.dtype != rf.dtype:
            raise CommError("sendrecv: the two tensors differ in dtype")
        code = self._code(sf, False)
        return self._start(f"sendrecv->{dst}<-{src}", lambda out: lib().tdm_sendrecv(
            self._engine, ctypes.c_void_p(sf.data_ptr()), self._count(sf, code), dst, ctypes.c_void_p(rf.data_ptr()),
            self._count(rf, code), src, code, self._stream(), out),
            recv, (send.numel() + recv.numel()) * send.element_size(), async_op, keep=(sf, rf))

    def barrier(self):
        return self._start("barrier", lambda out: lib().tdm_barrier(self._engine, out), None, 0, False)

    def close(self):
        if self._closed:
            return
        self.trace  # spans still owed are read while the engine is alive
        self.barrier()
        self._closed = True
        eng, self._engine = self._engine, None
        orphans, self._orphans = self._orphans, []  # tdm_engine_close runs what is queued and waits for the GPU
        self._arena = None  # the engine frees it; tensors carved from it must not be used after close()
        try:
            check(lib().tdm_engine_close(eng))
        except Exception as e:
            raise CommError(f"close: {e}") from e
        finally:
            for h, _ in orphans:
                lib().tdm_work_free(h)
            lib().tdm_engine_destroy(eng)

    def abandon(self):
        """After a failure on this rank: drop the engine without the closing
        handshake (the other ranks time out or fail on their own)."""
        self._closed = True
        self._untimed = []
        eng, self._engine = self._engine, None
        orphans, self._orphans = self._orphans, []
        if eng is not None:
            lib().tdm_engine_destroy(eng)
        for h, _ in orphans:
            lib().tdm_work_free(h)


def _worker(rank, size, fn, args, barrier, device, slot_bytes, slots, backend, job, gpus, timeout, results):
    if device != "cuda":
        raise CommError("tandem_amd.launch runs ranks on the GPU only (device=\"cuda\")")
    index = gpus[rank] if gpus else 0
    torch.cuda.set_device(index)
    g = Group(rank, size, torch.device("cuda", index), barrier, None, slot_bytes, slots, timeout=timeout, backend=backend,
              job=job)
    try:
        out = fn(g, *args)
        torch.cuda.synchronize(index)
        g.close()
    except BaseException:
        try:
            barrier.abort()  # ranks still starting up fail fast
        except Exception:
            pass
        g.abandon()
        raise
    if out is not None:
        torch.save(out, os.path.join(results, f"rank{rank}.pt"))


def launch(fn, size, *args, device="cuda", slot_bytes=DEFAULT_SLOT_BYTES, slots=DEFAULT_SLOTS, transport=None,
           priority=None, backend=None, gpus=None, timeout=DEFAULT_TIMEOUT):
    """Runs fn(group, *args) on `size` processes and returns each rank's return
    value, in rank order (tandem/comm.py:517-547 in the reference). The ranks
    share GPU 0 unless `gpus` names a device per rank; this build is measured with
    every rank on one GPU. Return values travel back through files, so keep them
    small (CPU tensors, numbers, lists)."""
    import tempfile
    import uuid

    backend = backend or DEFAULT_BACKEND
    if backend != "hip":
        raise CommError(f"unknown backend {backend} (tandem_amd provides \"hip\")")
    if transport not in (None, "device"):
        raise CommError(f"unknown transport {transport}")
    lib()  # load (and fail) here, not in every rank at once
    job = uuid.uuid4().hex[:12]
    ctx = mp.get_context("spawn")
    barrier = ctx.Barrier(size)
    with tempfile.TemporaryDirectory(prefix="tandem-") as results:
        try:
            mp.spawn(_worker, args=(size, fn, args, barrier, device, slot_bytes, slots, backend, job, gpus, timeout, results),
                     nprocs=size, join=True)
        finally:
            # A rank unlinks its shared-memory region when its engine goes; ranks that were killed because another
            # one failed never get there. The job's name is this call's own, so whatever is left is ours to remove.
            for r in range(size):
                try:
                    os.unlink(f"/dev/shm/tandem-{job}-{r}-hip")
                except OSError:
                    pass
        out = []
        for r in range(size):
            path = os.path.join(results, f"rank{r}.pt")
            out.append(torch.load(path, weights_only=False) if os.path.exists(path) else None)
    return out
