"""A CPU-process ring engine speaking the protocol of tandem's Python engine
(TEST INFRASTRUCTURE ONLY: the checker for host logic and the timed CPU baseline).

Written from the protocol description, not from the reference's code:
  * one process per rank, one torch thread per rank (tandem/comm.py:504);
  * for every ordered pair of ranks a mailbox of `slots` buffers of `slot_bytes`
    in shared memory, guarded by two counting semaphores, "pieces waiting" and
    "slots free" (tandem/comm.py:1-27,172-181);
  * a message larger than a slot travels as pieces of slot_bytes // itemsize
    elements; sender and receiver alternate put and take piece by piece
    (tandem/comm.py:256-298);
  * collectives run in submission order on one background thread per rank and
    hand back a Work (tandem/comm.py:211-242);
  * averaging divides the whole tensor first, then the ring reduce-scatter adds
    `into + received` in the ring's rank order (tandem/comm.py:301-311,336-343).

The arithmetic is torch's CPU div_ / add_ / copy_, the same library calls the
reference makes, so results are the reference's bit for bit (checked against the
fixtures in tests/golden/).
"""

import math
import os
import queue
import tempfile
import threading
import time

import torch
import torch.multiprocessing as mp

from .ring import split_sizes


class EngineError(RuntimeError):
    pass


class TorchCpuAdamW:
    """The optimizer of the CPU baseline: the update of tandem/optim.py:16-37 as the
    same sequence of torch CPU tensor operations (one pass over the shard each), which is what tandem's CPU-process backend runs. The bit-exact checker
    is oracle.adamw.AdamW; this class is timed, and checked against that one with
    torch's own sqrt substituted (tests/test_oracle_adamw.py)."""

    def __init__(self, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2):
        self.lr, self.betas, self.eps, self.weight_decay = lr, betas, eps, weight_decay
        self.state = {}

    def update(self, key, param, grad):
        entry = self.state.setdefault(key, {"t": 0.0, "m": torch.zeros_like(param), "v": torch.zeros_like(param)})
        entry["t"] += 1.0
        if param.numel() == 0:
            return
        t, m, v = entry["t"], entry["m"], entry["v"]
        b1, b2 = self.betas
        if self.weight_decay != 0:
            param.mul_(1 - self.lr * self.weight_decay)
        m.lerp_(grad, 1 - b1)
        v.mul_(b2).addcmul_(grad, grad, value=1 - b2)
        root = (1 - b2 ** t) ** 0.5
        spread = (v.sqrt() / root).add_(self.eps)  # two temporaries, as tandem/optim.py:36 makes
        param.addcdiv_(m, spread, value=-(self.lr / (1 - b1 ** t)))


class PendingWork:
    """Handle of a queued collective; wait() returns its result or re-raises."""

    def __init__(self, name, owner):
        self.name, self._owner = name, owner
        self._finished = threading.Event()
        self._failure = None
        self.result = None

    def wait(self):
        own = self._owner
        if own is not None and own.tracing and not self._finished.is_set():
            t0 = time.perf_counter()
            self._finished.wait()
            own.waits.append((self.name, t0, time.perf_counter()))
        self._finished.wait()
        if self._failure is not None:
            raise EngineError(f"{self.name} failed") from self._failure
        return self.result

    def is_completed(self):
        return self._finished.is_set()


class _Mailbox:
    """One direction of one pair: the sender writes slot seq % slots, the
    receiver reads it; the semaphores carry both the flow control and the
    memory ordering."""

    def __init__(self, store, pieces_waiting, slots_free, timeout):
        self.store, self.waiting, self.free, self.timeout = store, pieces_waiting, slots_free, timeout
        self.count = 0  # pieces this side has moved so far

    def _next_slot(self, nbytes):
        slot = self.store[self.count % self.store.shape[0], :nbytes]
        self.count += 1
        return slot

    def put(self, piece):
        if not self.free.acquire(timeout=self.timeout):
            raise EngineError("timed out waiting for a free slot")
        raw = piece.reshape(-1).view(torch.uint8)
        self._next_slot(raw.numel()).copy_(raw)
        self.waiting.release()

    def take(self, into, reduce):
        if not self.waiting.acquire(timeout=self.timeout):
            raise EngineError("timed out waiting for a piece")
        got = self._next_slot(into.numel() * into.element_size()).view(into.dtype)
        if reduce:
            into.add_(got)
        else:
            into.copy_(got)
        self.free.release()


class CpuGroup:
    def __init__(self, rank, size, plumbing, slot_bytes, slots, timeout=600.0):
        self.rank, self.size = rank, size
        self.device = torch.device("cpu")
        self.slot_bytes, self.slots, self.timeout = slot_bytes, slots, timeout
        self.backend = "oracle-cpu"
        self.tracing, self.trace, self.waits = False, [], []
        stores, waiting, free, self._barrier = plumbing
        pair = lambda a, b: a * size + b
        self._to = {q: _Mailbox(stores[pair(rank, q)], waiting[pair(rank, q)], free[pair(rank, q)], timeout)
                    for q in range(size) if q != rank}
        self._from = {q: _Mailbox(stores[pair(q, rank)], waiting[pair(q, rank)], free[pair(q, rank)], timeout)
                      for q in range(size) if q != rank}
        self._jobs = queue.Queue()
        self._closed = False
        self._worker = threading.Thread(target=self._serve, name=f"oracle-comm-{rank}", daemon=True)
        self._worker.start()
        self.barrier()

    # ---- background thread
    def _serve(self):
        while True:
            item = self._jobs.get()
            if item is None:
                return
            work, fn, nbytes = item
            t0 = time.perf_counter()
            try:
                work.result = fn()
                if self.tracing:
                    self.trace.append((work.name, t0, time.perf_counter(), nbytes))
            except BaseException as e:  # handed to whoever waits
                work._failure = e
            work._finished.set()

    def _enqueue(self, name, fn, nbytes, async_op):
        if self._closed:
            raise EngineError("group is closed")
        work = PendingWork(name, self)
        self._jobs.put((work, fn, nbytes))
        return work if async_op else work.wait()

    # ---- pieces
    def _swap(self, outgoing, dst, incoming, src, reduce):
        """Sends `outgoing` to dst and receives `incoming` from src in lockstep."""
        ref = outgoing if outgoing is not None else incoming
        per = max(1, self.slot_bytes // ref.element_size())
        n_out = math.ceil(outgoing.numel() / per) if outgoing is not None else 0
        n_in = math.ceil(incoming.numel() / per) if incoming is not None else 0
        for k in range(max(n_out, n_in)):
            if k < n_out:
                self._to[dst].put(outgoing[k * per:(k + 1) * per])
            if k < n_in:
                self._from[src].take(incoming[k * per:(k + 1) * per], reduce)

    def _cut(self, flat, sizes):
        if sizes is None:
            sizes = split_sizes(flat.numel(), self.size)
        elif len(sizes) != self.size or sum(sizes) != flat.numel():
            raise EngineError(f"chunk sizes {sizes} do not partition {flat.numel()} elements")
        return list(torch.split(flat, [int(s) for s in sizes]))

    def _scatter_phase(self, chunks):
        n, r = self.size, self.rank
        for s in range(n - 1):
            self._swap(chunks[(r - s - 1) % n], (r + 1) % n, chunks[(r - s - 2) % n], (r - 1) % n, True)

    def _gather_phase(self, chunks):
        n, r = self.size, self.rank
        for s in range(n - 1):
            self._swap(chunks[(r - s) % n], (r + 1) % n, chunks[(r - s - 1) % n], (r - 1) % n, False)

    @staticmethod
    def _flat(t):
        if not t.is_contiguous():
            raise EngineError("collectives need contiguous tensors")
        return t.reshape(-1)

    # ---- collectives
    def all_reduce(self, t, op="sum", async_op=False):
        if op not in ("sum", "avg"):
            raise EngineError(f"unknown op {op}")
        flat = self._flat(t)

        def job():
            if op == "avg":
                flat.div_(self.size)
            if self.size > 1:
                chunks = self._cut(flat, None)
                self._scatter_phase(chunks)
                self._gather_phase(chunks)
            return t

        return self._enqueue("all_reduce", job, t.numel() * t.element_size(), async_op)

    def reduce_scatter(self, t, sizes=None, op="sum", async_op=False):
        flat = self._flat(t)

        def job():
            if op == "avg":
                flat.div_(self.size)
            chunks = self._cut(flat, sizes)
            if self.size > 1:
                self._scatter_phase(chunks)
            return chunks[self.rank]

        return self._enqueue("reduce_scatter", job, t.numel() * t.element_size(), async_op)

    def all_gather(self, t, sizes=None, async_op=False):
        flat = self._flat(t)

        def job():
            if self.size > 1:
                self._gather_phase(self._cut(flat, sizes))
            return t

        return self._enqueue("all_gather", job, t.numel() * t.element_size(), async_op)

    # ---- the two helpers tandem_amd's wrappers ask of a group, with torch's CPU copy_
    def pack(self, flat, pieces):
        dst = self._flat(flat)
        for off, t in pieces:
            dst[off:off + t.numel()].copy_(t.reshape(-1))
        return flat

    def gather_unit(self, full, shard, sizes=None, async_op=False):
        flat = self._flat(full)
        self._cut(flat, sizes)[self.rank].copy_(shard.reshape(-1))
        return self.all_gather(full, sizes, async_op=async_op)

    def broadcast(self, t, root=0, async_op=False):
        flat = self._flat(t)

        def job():
            n = self.size
            hops = (self.rank - root) % n  # distance from the root along the ring
            per = max(1, self.slot_bytes // max(1, flat.element_size()))
            for k in range(0, flat.numel(), per):
                piece = flat[k:k + per]
                if hops > 0:
                    self._from[(self.rank - 1) % n].take(piece, False)
                if hops < n - 1:
                    self._to[(self.rank + 1) % n].put(piece)
            return t

        return self._enqueue("broadcast", job, t.numel() * t.element_size(), async_op)

    def barrier(self):
        def job():
            try:
                self._barrier.wait(timeout=self.timeout)
            except threading.BrokenBarrierError as e:
                raise EngineError("barrier broken: a rank failed or timed out") from e

        return self._enqueue("barrier", job, 0, False)

    def close(self):
        if self._closed:
            return
        self.barrier()
        self._closed = True
        self._jobs.put(None)
        self._worker.join()


def _rank_main(rank, size, fn, args, plumbing, slot_bytes, slots, threads, outdir):
    torch.set_num_threads(threads)
    g = CpuGroup(rank, size, plumbing, slot_bytes, slots)
    try:
        out = fn(g, *args)
        g.close()
    except BaseException:
        g._closed = True
        plumbing[3].abort()  # let the other ranks fail fast instead of waiting out the timeout
        raise
    if out is not None:
        torch.save(out, os.path.join(outdir, f"{rank}.pt"))


def cpu_launch(fn, size, *args, slot_bytes=4 << 20, slots=2, threads=1):
    """Runs fn(group, *args) on `size` CPU processes; returns each rank's return
    value (CPU tensors, numbers, lists), in rank order."""
    ctx = mp.get_context("spawn")
    stores = [torch.zeros(slots, slot_bytes, dtype=torch.uint8).share_memory_() if a != b else None
              for a in range(size) for b in range(size)]
    waiting = [ctx.Semaphore(0) for _ in range(size * size)]
    free = [ctx.Semaphore(slots) for _ in range(size * size)]
    plumbing = (stores, waiting, free, ctx.Barrier(size))
    with tempfile.TemporaryDirectory(prefix="oracle-cpu-") as outdir:
        mp.spawn(_rank_main, args=(size, fn, args, plumbing, slot_bytes, slots, threads, outdir), nprocs=size, join=True)
        out = []
        for r in range(size):
            path = os.path.join(outdir, f"{r}.pt")
            out.append(torch.load(path, weights_only=False) if os.path.exists(path) else None)
    return out
