"""ZeRO stages 1, 2 and 3 over a tandem group (Rajbhandari et al., 2020): data
parallelism that shards what every rank would otherwise keep a full copy of.

  ZeRO(stage=1)  optimizer state sharded. Gradients are all-reduced bucket by
                 bucket as in DDP; each rank updates its shard of one flat
                 parameter buffer and the ranks all-gather the result.
  ZeRO(stage=2)  gradients sharded as well: each bucket is reduce-scattered from a
                 staging buffer, a rank keeps only the sums that fall in its
                 shard, the staging buffer is dropped.
  FSDP           stage 3, parameters sharded too, one unit of the model at a time
                 (model.units()): a unit's full parameters exist only while it
                 runs; the next unit's gather is already under way on the engine's
                 stream while this one computes.

Drop-ins for the reference's classes (tandem/zero.py:69-336 there): same
constructors, same `loss = z(x, y); loss.backward(); z.step(); z.zero_grad()`
protocol, same bucket ranges, shard boundaries and submission order, so every
collective sees the same chunks and the results are the reference's bit for bit.
Differences: gradients enter a bucket through one `group.pack` gather per bucket
(per unit for FSDP) instead of one copy per parameter; FSDP's gather is
`group.gather_unit` (shard placement + all-gather on the engine's stream); the
optimizer is the fused ShardedAdamW kernel.

`group` is anything with tandem's Group interface plus pack() and gather_unit().
"""

import warnings

import torch
from torch.autograd import Variable

from .buckets import FlatLayout, zero_buckets
from .optim import ShardedAdamW


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

    def __init__(self, module, group, stage=1, optimizer=None, bucket_bytes=25 << 20, direct=False, fused_step=False):
        """direct: the flat parameter buffer and the gradient buffer (stage 2: one
        staging buffer the size of the model, kept, instead of one per bucket that is
        dropped) live in the group's shared arena (created here if the group has none:
        twice the model, under 2 GiB), and every collective runs arena to arena
        (`direct=True` of tandem_amd.Group): same bits, fewer passes over memory, no
        slots.

        fused_step (stage 2 with direct): backward only packs the gradients; step()
        is then ONE launch per rank (`group.zero2_step`) that folds this rank's shard
        out of every rank's gradients in the ring's order, takes the AdamW step and
        writes the new parameters into every rank's buffer: the reduce_scatters,
        `grad_shard.add_`, the update and the all_gather in one pass, same bits.
        `grad_shard` is then only filled when a second backward comes before step()
        (accumulation): that backward first reduces the packed gradients the ordinary
        way, and the step after it is the ordinary one."""
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
        if self.fused_step:
            if stage != 2 or not direct:
                raise ValueError("fused_step needs stage=2 and direct=True")
            _need(group, "zero2_step")
            if not hasattr(self.opt, "begin_step"):
                raise TypeError("fused_step needs an optimizer with begin_step() (tandem_amd.ShardedAdamW has it)")
        self._packed = False      # fused_step: a whole backward's gradients lie packed in the pool, not yet reduced
        self._shard_zero = True   # nothing has been added to grad_shard since zero_grad()
        params = [p for p in module.parameters() if p.requires_grad]
        self.params = params
        dev, dtype = params[0].device, params[0].dtype
        self.flat = FlatLayout([p.numel() for p in params], group.size, group.rank)
        self.offset = dict(zip(params, self.flat.offsets))
        if self.direct:
            if getattr(group, "_arena", None) is None:
                group.share_arena(2 * (self.flat.numel * params[0].element_size() + 4096))
            self.buf = group.shared_empty(self.flat.numel, dtype)
            self._pool = group.shared_empty(self.flat.numel, dtype).zero_()  # stage 1: gradients; stage 2: staging
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
            self.grad_shard = torch.zeros(self.flat.hi - self.flat.lo, device=dev, dtype=dtype)
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
            if self._packed:
                self._reduce_packed()  # accumulation: the previous backward's gradients, before they are overwritten
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
        self._packed = False

    @torch.no_grad()
    def step(self):
        lo, hi = self.flat.lo, self.flat.hi
        if self._packed:
            scalars, exp_avg, exp_avg_sq, order = self.opt.begin_step("flat", self.buf[lo:hi])
            self.g.zero2_step(self.buf, self._pool, self.flat.sizes, exp_avg, exp_avg_sq, scalars, order, op="avg")
            self._packed = False
            return
        grad = self.grad[lo:hi] if self.stage == 1 else self.grad_shard
        self.opt.update("flat", self.buf[lo:hi], grad)
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
            self._packed = False  # packed gradients not yet reduced are dropped with the rest
            if not self._shard_zero:
                self.grad_shard.zero_()
            self._shard_zero = True


def _pad(n):
    """Shards start on 16-byte boundaries inside the arena (fp32: multiples of 4 elements)."""
    return (n + 3) // 4 * 4


class _Unit:
    def __init__(self, index, module, params, world, rank, device, dtype):
        self.index, self.module, self.params = index, module, params
        self.flat = FlatLayout([p.numel() for p in params], world, rank)
        self.offset = dict(zip(params, self.flat.offsets))
        self.full = torch.empty(self.flat.numel, device=device, dtype=dtype)
        self.nbytes = self.full.untyped_storage().nbytes()
        self.shard = None
        self.grad_shard = torch.zeros(self.flat.hi - self.flat.lo, device=device, dtype=dtype)
        self.gathered = True
        self.pending = None  # gather in flight
        self.arrived = 0
        self.rs = None  # reduce-scatter in flight
        self.staging = None
        self.peer_offsets = None


class FSDP(torch.nn.Module):
    """ZeRO stage 3 over model.units()."""

    def __init__(self, model, group, optimizer=None, prefetch=True, direct=None):
        super().__init__()
        _need(group, "pack", "gather_unit")
        self.module, self.g = model, group
        self.opt = optimizer if optimizer is not None else ShardedAdamW()
        self.prefetch = prefetch
        # The first unit's input (token ids) needs no gradient; torch then fires the
        # unit's backward pre-hook on its outputs, which is the moment wanted here.
        warnings.filterwarnings("ignore", message="Full backward hook is firing when gradients are computed with respect to module outputs")
        self.live = 0  # units whose full parameters exist right now
        self.max_live = 0
        self.units, self.unit_of = [], {}
        claimed = set()
        # Where the group offers it, all shards live in one arena that the other ranks
        # map once and read directly: a gather is then copies only, with a fence()
        # around the optimizer step instead of a handshake per gather.
        self._direct = direct if direct is not None else hasattr(group, "shared_empty")
        arena, arena_at, self._peer_at = None, 0, [0] * group.size
        if self._direct:
            from .buckets import FlatLayout as _L

            mods = model.units()
            seen, total = set(), [0] * group.size
            for m in mods:
                ps = [p for p in m.parameters() if p.requires_grad and id(p) not in seen]
                seen.update(id(p) for p in ps)
                sizes = _L([p.numel() for p in ps], group.size, 0).sizes
                total = [t + _pad(s) for t, s in zip(total, sizes)]
            p0 = next(model.parameters())
            try:
                arena = group.shared_empty(max(total), p0.dtype)
            except Exception:
                self._direct, arena = False, None  # too large for one IPC allocation: stage through the slots
        for i, m in enumerate(model.units()):
            ps = [p for p in m.parameters() if p.requires_grad and id(p) not in claimed]
            claimed.update(id(p) for p in ps)
            u = _Unit(i, m, ps, group.size, group.rank, ps[0].device, ps[0].dtype)
            with torch.no_grad():
                self.g.pack(u.full, [(u.offset[p], p.data) for p in ps])
                self.g.broadcast(u.full, root=0)
                for p in ps:
                    o = u.offset[p]
                    p.data = u.full[o:o + p.numel()].view_as(p)
                if arena is not None:
                    es = u.full.element_size()
                    u.shard = arena[self._peer_at[group.rank]:self._peer_at[group.rank] + (u.flat.hi - u.flat.lo)]
                    u.shard.copy_(u.full[u.flat.lo:u.flat.hi])
                    u.peer_offsets = [at * es for at in self._peer_at]  # this unit's shard in every rank's arena, bytes
                    self._peer_at = [at + _pad(s) for at, s in zip(self._peer_at, u.flat.sizes)]
                else:
                    u.shard = u.full[u.flat.lo:u.flat.hi].clone()
            for p in ps:
                self.unit_of[p] = u
                p.register_post_accumulate_grad_hook(self._on_grad)
            m.register_forward_pre_hook(self._before_forward(u))
            m.register_forward_hook(self._after_forward(u))
            m.register_full_backward_pre_hook(self._before_backward(u))
            self.live += 1  # _Unit allocated it whole
            self._release(u)
            self.units.append(u)
        if len(claimed) != sum(1 for p in model.parameters() if p.requires_grad):
            raise ValueError("every parameter must belong to one of model.units()")
        self._callback_queued = False
        self.max_live = 0
        if self._direct:
            self.g.fence()  # every rank's shards are in place before anyone gathers

    def forward(self, *args, **kwargs):
        return self.module(*args, **kwargs)

    # ---- a unit's full parameters: start gathering, wait, release
    def _start(self, u):
        if u.gathered or u.pending is not None:
            return
        u.full.untyped_storage().resize_(u.nbytes)
        self.live += 1
        self.max_live = max(self.max_live, self.live)
        if self._direct:
            u.pending = self.g.gather_unit(u.full, u.shard, u.flat.sizes, async_op=True, peer_offsets=u.peer_offsets)
        else:
            u.pending = self.g.gather_unit(u.full, u.shard, u.flat.sizes, async_op=True)

    def _ensure(self, u):
        self._start(u)
        if u.pending is not None:
            u.pending.wait()
            u.pending = None
            u.gathered = True

    def _release(self, u):
        if u.pending is not None:
            u.pending.wait()
            u.pending = None
        if u.full.untyped_storage().nbytes():
            self.live -= 1
        u.full.untyped_storage().resize_(0)
        u.gathered = False

    # ---- hooks
    def _before_forward(self, u):
        def hook(mod, args):
            self._ensure(u)
            if self.prefetch and u.index + 1 < len(self.units):
                self._start(self.units[u.index + 1])

        return hook

    def _after_forward(self, u):
        def hook(mod, args, out):
            # The last unit's backward comes first: keep it.
            if torch.is_grad_enabled() and u.index == len(self.units) - 1:
                return
            self._release(u)

        return hook

    def _before_backward(self, u):
        def hook(mod, grad_out):
            if not self._callback_queued:
                self._callback_queued = True
                Variable._execution_engine.queue_callback(self._after_backward)
            self._ensure(u)
            if self.prefetch and u.index > 0:
                self._start(self.units[u.index - 1])

        return hook

    def _on_grad(self, p):
        u = self.unit_of[p]
        u.arrived += 1
        if u.arrived == len(u.params):
            # The unit's backward is done: gather its gradients into one staging
            # buffer with a single launch, drop its full parameters, and send the
            # gradients on their way.
            u.staging = torch.empty(u.flat.numel, device=p.device, dtype=p.dtype)
            self.g.pack(u.staging, [(u.offset[q], q.grad) for q in u.params])
            for q in u.params:
                q.grad = None
            self._release(u)
            # only `mine` is kept of the staging buffer: the other chunks' partial sums are not needed
            how = {"partial_sums": False} if getattr(self.g, "partial_sums_optional", False) else {}
            u.rs = self.g.reduce_scatter(u.staging, u.flat.sizes, op="avg", async_op=True, **how)

    def _after_backward(self):
        self._callback_queued = False
        for u in self.units:
            if u.arrived != len(u.params):
                raise RuntimeError("tandem FSDP: every parameter must receive a gradient")
            mine = u.rs.wait()
            if mine.numel():
                u.grad_shard.add_(mine)
            u.rs, u.staging, u.arrived = None, None, 0
            if u.gathered:
                self._release(u)

    @torch.no_grad()
    def step(self):
        if self._direct:
            self.g.fence()  # no rank still reads the shards this step rewrites
        for u in self.units:
            self.opt.update(u.index, u.shard, u.grad_shard)
        if self._direct:
            self.g.fence()  # the new shards are complete before any rank gathers them

    def zero_grad(self):
        for u in self.units:
            u.grad_shard.zero_()

    @torch.no_grad()
    def full_parameters(self):
        """All parameters, gathered (for checkpoints and tests)."""
        out = []
        for u in self.units:
            full = torch.empty(u.flat.numel, device=u.shard.device, dtype=u.shard.dtype)
            if self._direct:
                self.g.gather_unit(full, u.shard, u.flat.sizes, peer_offsets=u.peer_offsets)
            else:
                self.g.gather_unit(full, u.shard, u.flat.sizes)
            out.append(full)
        return torch.cat(out)
