"""ZeRO stages 1, 2 and 3 over a tandem group (Rajbhandari et al., 2020): data
parallelism that shards what every rank would otherwise keep a full copy of.

  ZeRO(stage=1)  optimizer state sharded. Gradients are all-reduced bucket by
                 bucket as in DDP; each rank updates its shard of one flat
                 parameter buffer and the ranks all-gather the result.
  ZeRO(stage=2)  gradients sharded as well: each bucket is reduce-scattered from a
                 staging buffer, a rank keeps only the sums that fall in its
                 shard, the staging buffer is dropped.
  FSDP           stage 3, parameters sharded too, one unit of the model at a time
                 (model.units()): see fsdp.py.

Drop-ins for the reference's classes (tandem/zero.py:69-170 there): same
constructors, same `loss = z(x, y); loss.backward(); z.step(); z.zero_grad()`
protocol, same bucket ranges, shard boundaries and submission order, so every
collective sees the same chunks and the results are the reference's bit for bit.
Differences: gradients enter a bucket through one `group.pack` gather per bucket
instead of one copy per parameter; the optimizer is the fused ShardedAdamW kernel.

`group` is anything with tandem's Group interface plus pack().
"""

import torch
from torch.autograd import Variable

from .buckets import FlatLayout, zero_buckets
from .optim import ShardedAdamW, zeros_at_phase_of


def _need(group, *names):
    missing = [n for n in names if not hasattr(group, n)]
    if missing:
        raise TypeError(f"this wrapper needs a group that provides {missing} (tandem_amd.Group does)")


class _Range:
    """A bucket of ZeRO-1/2: the parameters whose flat offsets fill [a, b)."""

    def __init__(self, params, a, b):
        self.params, self.a, self.b = params, a, b
        self.arrived = 0
        self.loose = []
        self.work = None
        self.staging = None


class ZeRO(torch.nn.Module):
    """Stages 1 and 2."""

    def __init__(self, module, group, stage=1, optimizer=None, bucket_bytes=25 << 20, direct=False, fused_step=False,
                 stream_ordered=False):
        """stream_ordered (opt-in): step() only orders the training stream behind the all-gather of the new
        parameters instead of making the host wait for it; should that all-gather fail, the next forward reads
        parameters that never arrived and the failure is raised by the next collective. The default waits on the
        host, as the reference's step() does (tandem/zero.py:157-164), and raises from step().

        direct: the flat parameter buffer and the gradient buffer (stage 2: one
        staging buffer the size of the model, kept, instead of one per bucket that is
        dropped) live in the group's shared arenas (one of twice the model's size if the
        group has none; an arena each once that would reach 2 GiB, the size one arena
        stops at, so the model itself must stay under it), and every collective runs arena to arena
        (`direct=True` of tandem_amd.Group): same bits, fewer passes over memory, no
        slots.

        fused_step (stage 2 with direct): backward only packs the gradients; step()
        is then ONE launch per rank (`group.zero2_step`) that folds this rank's shard
        out of every rank's gradients in the ring's order, takes the AdamW step and
        writes the new parameters into every rank's buffer: the reduce_scatters,
        `grad_shard.add_`, the update and the all_gather in one pass, same bits.
        `grad_shard` is then only filled when a second backward comes before step()
        (accumulation) or after a step() without zero_grad() in between: that backward
        first reduces the gradients still packed in the pool the ordinary way, and the
        step after it is the ordinary one."""
        super().__init__()
        if stage not in (1, 2):
            raise ValueError("ZeRO handles stages 1 and 2; stage 3 is FSDP")
        _need(group, "pack")
        if direct:
            _need(group, "shared_empty", "share_arena")
        self.module, self.g, self.stage = module, group, stage
        self.direct = bool(direct)
        self.opt = optimizer if optimizer is not None else ShardedAdamW()
        self.fused_step = bool(fused_step)
        self.stream_ordered = bool(stream_ordered) and getattr(group, "stream_ordered_waits", False)
        if self.fused_step:
            if stage != 2 or not direct:
                raise ValueError("fused_step needs stage=2 and direct=True")
            _need(group, "zero2_step")
            if not hasattr(self.opt, "begin_step"):
                raise TypeError("fused_step needs an optimizer with begin_step() (tandem_amd.ShardedAdamW has it)")
        self._packed = False      # fused_step: a whole backward's gradients lie packed in the pool, not yet reduced
        self._applied = False     # fused_step: the pool's gradients went into a step but never into grad_shard
        self._shard_zero = True   # nothing has been added to grad_shard since zero_grad()
        params = [p for p in module.parameters() if p.requires_grad]
        self.params = params
        dev, dtype = params[0].device, params[0].dtype
        self.flat = FlatLayout([p.numel() for p in params], group.size, group.rank)
        self.offset = dict(zip(params, self.flat.offsets))
        if self.direct:
            nbytes = self.flat.numel * params[0].element_size()
            if getattr(group, "_arena", None) is None and 2 * (nbytes + 4096) < group.ARENA_LIMIT:
                group.share_arena(2 * (nbytes + 4096))  # both in one arena while that stays one allocation
            self.buf = group.shared_empty(self.flat.numel, dtype, grow=nbytes)
            self._pool = group.shared_empty(self.flat.numel, dtype, grow=nbytes).zero_()  # stage 1: gradients; stage 2: staging
        else:
            self.buf = torch.empty(self.flat.numel, device=dev, dtype=dtype)
        with torch.no_grad():
            self.g.pack(self.buf, [(self.offset[p], p.data) for p in params])
            self.g.broadcast(self.buf, root=0)  # every rank starts from rank 0's weights
            for p in params:
                o = self.offset[p]
                p.data = self.buf[o:o + p.numel()].view_as(p)
        if stage == 1:
            self.grad = self._pool if self.direct else torch.zeros_like(self.buf)
        else:
            # at the phase of this rank's parameter shard (tensor_split shards start anywhere): the update runs on vectors
            self.grad_shard = zeros_at_phase_of(self.buf[self.flat.lo:self.flat.hi])
        # Buckets are contiguous ranges of the flat buffer taken from its end: the
        # order backward produces gradients in.
        self.buckets, self.bucket_of = [], {}
        for a, b, members in zero_buckets(self.flat.numels, params[0].element_size(), bucket_bytes):
            rng = _Range([params[i] for i in members], a, b)
            self.buckets.append(rng)
            for p in rng.params:
                self.bucket_of[p] = rng
        self._cursor = 0
        self._callback_queued = False
        for p in params:
            p.register_post_accumulate_grad_hook(self._on_grad)

    def forward(self, *args, **kwargs):
        return self.module(*args, **kwargs)

    def _grad_view(self, p):
        o = self.offset[p]
        return self.grad[o:o + p.numel()].view_as(p)

    def _launch(self, rng):
        if self.stage == 1:
            if rng.loose:  # gradients that are not yet views of the flat gradient buffer
                self.g.pack(self.grad, [(self.offset[p], p.grad) for p in rng.loose])
                for p in rng.loose:
                    p.grad = self._grad_view(p)
                rng.loose = []
            rng.work = self.g.all_reduce(self.grad[rng.a:rng.b], op="avg", async_op=True, **self._how)
        else:
            if self._packed or self._applied:
                # the previous backward's gradients, before they are overwritten: accumulation over several
                # backward passes, or a step() that was not followed by zero_grad() (the reference's
                # grad_shard still holds that sum then, tandem/zero.py:150-170)
                self._reduce_packed()
            p0 = rng.params[0]
            rng.staging = (self._pool[rng.a:rng.b] if self.direct
                           else torch.empty(rng.b - rng.a, device=p0.device, dtype=p0.dtype))
            self.g.pack(rng.staging, [(self.offset[p] - rng.a, p.grad) for p in rng.params])
            for p in rng.params:
                p.grad = None  # the full-size gradient is not kept
            if self.fused_step and self._shard_zero:
                return  # step() reduces, updates and gathers in one launch
            rng.work = self.g.reduce_scatter(rng.staging, self.flat.bucket_sizes(rng.a, rng.b), op="avg", async_op=True,
                                             **self._how, **self._mine_only)

    def _on_grad(self, p):
        rng = self.bucket_of[p]
        if self.stage == 1 and p.grad.data_ptr() != self._grad_view(p).data_ptr():
            rng.loose.append(p)  # first gradient since zero_grad: still outside the flat gradient buffer
        if not self._callback_queued:
            self._callback_queued = True
            Variable._execution_engine.queue_callback(self._after_backward)
        rng.arrived += 1
        while self._cursor < len(self.buckets):
            nxt = self.buckets[self._cursor]
            if nxt.arrived != len(nxt.params):
                break
            self._launch(nxt)
            self._cursor += 1

    def _after_backward(self):
        self._callback_queued = False
        if any(r.arrived != len(r.params) for r in self.buckets):
            raise RuntimeError("tandem ZeRO: every parameter must receive a gradient")
        if self.fused_step and self._shard_zero:
            for rng in self.buckets:
                rng.arrived, rng.staging = 0, None
            self._cursor, self._packed = 0, True
            return
        for rng in self.buckets:
            mine = rng.work.wait()
            if self.stage == 2:
                self._add_mine(rng, mine)
                rng.staging = None
            rng.arrived, rng.work = 0, None
        self._cursor = 0

    def _add_mine(self, rng, mine):
        if mine.numel():
            at = max(rng.a, self.flat.lo) - self.flat.lo
            self.grad_shard[at:at + mine.numel()].add_(mine)
        self._shard_zero = False

    @torch.no_grad()
    def _reduce_packed(self):
        """fused_step: what backward would have done bucket by bucket, for gradients
        that were only packed."""
        works = [self.g.reduce_scatter(self._pool[r.a:r.b], self.flat.bucket_sizes(r.a, r.b), op="avg", async_op=True, direct=True)
                 for r in self.buckets]
        for rng, work in zip(self.buckets, works):
            self._add_mine(rng, work.wait())
        self._packed = self._applied = False

    @torch.no_grad()
    def step(self):
        lo, hi = self.flat.lo, self.flat.hi
        if self._packed:
            scalars, exp_avg, exp_avg_sq, order = self.opt.begin_step("flat", self.buf[lo:hi])
            self.g.zero2_step(self.buf, self._pool, self.flat.sizes, exp_avg, exp_avg_sq, scalars, order, op="avg")
            self._packed, self._applied = False, True
            return
        grad = self.grad[lo:hi] if self.stage == 1 else self.grad_shard
        self.opt.update("flat", self.buf[lo:hi], grad)
        if self.stream_ordered:
            # the next forward only has to come after the gather on the stream: the host does not wait for it
            self.g.all_gather(self.buf, self.flat.sizes, async_op=True, **self._how).wait(stream_ordered=True)
        else:
            self.g.all_gather(self.buf, self.flat.sizes, **self._how)

    @property
    def _how(self):
        return {"direct": True} if self.direct else {}

    @property
    def _mine_only(self):
        """Stage 2 keeps only `mine` of a bucket's reduce_scatter and drops the staging
        buffer: a group that can skip the other chunks' partial sums is told so."""
        return {"partial_sums": False} if getattr(self.g, "partial_sums_optional", False) and not self.direct else {}

    def zero_grad(self):
        if self.stage == 1:
            for p in self.params:
                p.grad = None
        else:
            self._packed = self._applied = False  # packed gradients not yet reduced are dropped with the rest
            if not self._shard_zero:
                self.grad_shard.zero_()
            self._shard_zero = True


from .fsdp import FSDP  # noqa: E402,F401  (stage 3 has a file of its own; importable from here as in the reference)
