"""Data parallelism over a tandem group: every rank holds the whole model,
trains on its rows of the batch, and the ranks average gradients before each
optimizer step.

Drop-in for the reference's wrapper (tandem/ddp.py:36-129 there): same
constructor, `no_sync()`, bucket packing, launch order and one-time rebuild, so
the averaged gradients are the reference's bit for bit at any world size (the
ring's summation order depends on where a gradient sits in its bucket).

What differs is how a bucket is filled. The reference copies each gradient into
its view of the bucket as it arrives, one small copy per parameter. Here a
bucket's gradients are gathered by `group.pack`, a single table-driven launch,
when the bucket's last gradient has arrived, immediately before its all-reduce
is queued; after that each `p.grad` is its view of the bucket, so the all-reduce
lands in place and nothing is copied back.

`group` is anything with tandem's Group interface plus `pack(flat, pieces)`;
tandem_amd.Group(backend="hip") is the one that ships.
"""

import contextlib

import torch
from torch.autograd import Variable


class Bucket:
    """Parameters that travel together: one flat buffer, one view per parameter."""

    def __init__(self, params, device, dtype, flat=None):
        self.params = list(params)
        numel = sum(p.numel() for p in self.params)
        self.flat = torch.zeros(numel, device=device, dtype=dtype) if flat is None else flat
        assert self.flat.numel() == numel and self.flat.dtype == dtype
        self.views, self.offsets = {}, {}
        at = 0
        for p in self.params:
            self.offsets[p] = at
            self.views[p] = self.flat[at:at + p.numel()].view_as(p)
            at += p.numel()
        self.arrived = 0
        self.loose = []  # parameters whose gradient still lives outside the bucket
        self.work = None


class DDP(torch.nn.Module):
    def __init__(self, module, group, bucket_bytes=25 << 20, overlap=True, rebuild=True, direct=False, stream_ordered=False):
        """stream_ordered=False (the default): at the end of backward the host waits for every bucket, as the
        reference's DDP does (tandem/ddp.py:111-115), so a bucket that fails raises from this backward, before any
        optimizer step can apply gradients that were never reduced.
        stream_ordered=True (opt-in): the training stream is only ORDERED behind the buckets' all-reduces
        (`Work.wait(stream_ordered=True)`) and the host goes on, so the optimizer's launches are queued while the
        last buckets are still in flight (2-3 ms of a 30 ms step with torch's per-tensor AdamW). The price: when a
        bucket then fails, the stream is let go, the optimizer that is already queued steps on unreduced gradients,
        and the failure is raised by the next collective; the weights of that step must be thrown away.
        direct: the buckets live in the group's shared arenas (the gradients' size plus
        padding, in arenas of 1 GiB where that is more) and every
        all-reduce runs arena to arena (`group.all_reduce(..., direct=True)`): same
        bits, 2 instead of 4.5 passes over a bucket per rank at two ranks, two
        handshakes per bucket instead of two per 4 MiB piece."""
        super().__init__()
        if not hasattr(group, "pack"):
            raise TypeError("tandem_amd.DDP needs a group that provides pack() (tandem_amd.Group does)")
        if direct and not hasattr(group, "shared_empty"):
            raise TypeError("DDP(direct=True) needs a group with a shared arena (tandem_amd.Group has one)")
        self.module, self.g = module, group
        self.direct, self._pools = bool(direct), {}
        self.stream_ordered = bool(stream_ordered) and getattr(group, "stream_ordered_waits", False)
        self.bucket_bytes, self.overlap = bucket_bytes, overlap
        self._rebuild_pending = rebuild
        self.params = [p for p in module.parameters() if p.requires_grad]
        with torch.no_grad():
            for p in self.params:  # every rank starts from rank 0's weights
                self.g.broadcast(p.data, root=0)
        # Before any backward has shown the real order, assume gradients arrive in
        # reverse registration order.
        self._build(self.params[::-1])
        self._reduce_now = True
        self._arrival = []
        self._callback_queued = False
        for p in self.params:
            p.register_post_accumulate_grad_hook(self._on_grad)

    # ---- buckets
    def _build(self, order):
        from .buckets import pack

        groups = pack([p.numel() * p.element_size() for p in order], self.bucket_bytes, [p.dtype for p in order])
        self.buckets, self.bucket_of = [], {}
        carved = {}  # per dtype: [slab, elements used of it]
        for members in groups:
            ps = [order[i] for i in members]
            flat = None
            if self.direct:
                # Carved from arena tensors ("slabs") per dtype, the same way on every rank (so a
                # bucket has the same arena offset everywhere), 256-byte aligned. A rebuild carves
                # the same slabs again.
                dtype, numel = ps[0].dtype, sum(p.numel() for p in ps)
                k, at = carved.get(dtype, (0, 0))
                if at + numel > self._slab(dtype, k, numel).numel():
                    k, at = k + 1, 0
                flat = self._slab(dtype, k, numel)[at:at + numel].zero_()
                carved[dtype] = (k, at + -(-numel // 64) * 64)
            b = Bucket(ps, ps[0].device, ps[0].dtype, flat)
            self.buckets.append(b)
            for p in ps:
                self.bucket_of[p] = b
        self._cursor = 0  # next bucket to launch: every rank launches in the same order

    SLAB_BYTES = 1 << 30  # an arena is one exported allocation and stays under 2 GiB: larger models take several

    def _slab(self, dtype, k, numel):
        """Slab `k` of this dtype's buckets: room for every gradient of the dtype plus padding when that stays
        under SLAB_BYTES, else slabs of that size (at least `numel` elements), each an arena of its own."""
        slabs = self._pools.setdefault(dtype, [])
        while len(slabs) <= k:
            es = torch.empty(0, dtype=dtype).element_size()
            mine = [p for p in self.params if p.dtype == dtype]
            whole = sum(p.numel() for p in mine) + 64 * len(mine)  # the padding of at most one bucket per parameter
            room = max(min(whole, self.SLAB_BYTES // es), numel)
            slabs.append(self.g.shared_empty(room, dtype, grow=room * es))
        return slabs[k]

    def _gather(self, bucket):
        """Moves the bucket's loose gradients into it with one gather, and points
        each p.grad at its view."""
        if bucket.loose:
            self.g.pack(bucket.flat, [(bucket.offsets[p], p.grad) for p in bucket.loose])
            for p in bucket.loose:
                p.grad = bucket.views[p]
            bucket.loose = []

    def forward(self, *args, **kwargs):
        return self.module(*args, **kwargs)

    @contextlib.contextmanager
    def no_sync(self):
        """Gradient accumulation: backward passes inside only accumulate
        locally; the next one outside reduces the sum."""
        before, self._reduce_now = self._reduce_now, False
        try:
            yield
        finally:
            self._reduce_now = before

    # ---- backward
    def _on_grad(self, p):
        b = self.bucket_of[p]
        if p.grad is not b.views[p]:  # first gradient since zero_grad
            b.loose.append(p)
        if not self._reduce_now:
            self._gather(b)  # accumulate inside the bucket from now on
            return
        if not self._callback_queued:
            self._callback_queued = True
            Variable._execution_engine.queue_callback(self._after_backward)
        if self._rebuild_pending:
            self._arrival.append(p)
        b.arrived += 1
        while self._cursor < len(self.buckets):
            nxt = self.buckets[self._cursor]
            if nxt.arrived != len(nxt.params):
                break
            self._gather(nxt)
            nxt.work = (self.g.all_reduce(nxt.flat, op="avg", async_op=True, direct=True) if self.direct
                        else self.g.all_reduce(nxt.flat, op="avg", async_op=True))
            if not self.overlap:
                nxt.work.wait()
            self._cursor += 1

    def _after_backward(self):
        self._callback_queued = False
        short = [b for b in self.buckets if b.arrived != len(b.params)]
        if short:
            unused = [tuple(p.shape) for b in short for p in b.params if p.grad is None]
            raise RuntimeError(f"tandem DDP: some parameters received no gradient ({unused[:3]}...); every parameter must be used")
        for b in self.buckets:
            b.work.wait(stream_ordered=True) if self.stream_ordered else b.work.wait()
            b.arrived, b.work = 0, None
        self._cursor = 0
        if self._rebuild_pending and len(self._arrival) == len(self.params):
            # Once: rebuild the buckets in the order gradients really arrived, so
            # the first bucket to fill is the first to be sent.
            order, self._arrival, self._rebuild_pending = self._arrival, [], False
            # (direct: the new buckets are carved from the memory the old ones lie in)
            old = {p: (p.grad.clone() if self.direct else p.grad) for p in self.params}
            self._build(order)
            for b in self.buckets:
                self.g.pack(b.flat, [(b.offsets[p], old[p]) for p in b.params])
                for p in b.params:
                    p.grad = b.views[p]
        else:
            self._arrival = []
