"""ZeRO stage 3 over model.units(): parameters, gradients and optimizer state all
sharded, one unit of the model whole at a time.

Drop-in for the reference's FSDP (tandem/zero.py:188-336 there: same constructor,
same `loss = f(x, y); loss.backward(); f.step(); f.zero_grad()` protocol, same
shard boundaries, the same gathers and reduce-scatters in the same order, the
same `live` / `max_live` accounting), built from three pieces of this package's
own:

  ShardHome     where every unit's shard lives. With a group that exports device
                memory (tandem_amd.Group) all shards of a rank lie in ONE arena that
                the peers map once; a gather is then W-1 copy kernels out of the
                peers' arenas with no message at all, and two fences around the
                optimizer step are the only handshakes of a training step.
  Unit          a state machine per unit, released -> gathering -> whole -> released,
                that owns the unit's buffers and both of its collectives (the gather
                of its parameters, the reduce-scatter of its gradients).
  Walk          the order in which a step needs the units, worked out once from the
                number of units and the prefetch distance: which unit to wait for,
                which to start fetching, which to keep, per hook.

`group` is anything with tandem's Group interface plus pack() and gather_unit().
"""

import warnings

import torch
from torch.autograd import Variable

from .buckets import FlatLayout
from .comm import CommError
from .optim import ShardedAdamW

RELEASED, GATHERING, WHOLE = "released", "gathering", "whole"


class Residency:
    """How many units hold their full parameters right now, and the most that ever
    did at once since the last reset (tandem/zero.py:202-203,242-243,258-259)."""

    def __init__(self):
        self.live = 0
        self.max_live = 0

    def took(self):
        self.live += 1
        self.max_live = max(self.max_live, self.live)

    def gave(self):
        self.live -= 1


class ShardHome:
    """Lays every unit's shard out in the ranks' shared arenas. Units are put into slabs: a slab is
    one arena tensor of the same size on every rank (so it has the same arena offset everywhere),
    large enough for the rank whose shards of the slab's units are longest; within a slab a unit's
    shard starts at the same element offset on every rank only when all earlier shards had equal
    sizes, so the offsets are kept per rank. Shards start on 128-byte boundaries (cache lines). An arena is one
    exported allocation and stays under 2 GiB, so a slab ends before SLAB_BYTES."""

    ALIGN_BYTES = 128  # every shard starts on a cache line: the gather and the update then move whole lines
    SLAB_BYTES = 1 << 30

    def __init__(self, group, unit_sizes, dtype):
        """unit_sizes[k][q]: elements of unit k's shard on rank q."""
        self.rank = group.rank
        world = group.size
        self.es = torch.empty(0, dtype=dtype).element_size()
        cap = max(self.SLAB_BYTES // self.es, 1)
        self.slab_of, self.at = [], []  # per unit: its slab, and the element offset of the shard within it on every rank
        extents, ends = [], [0] * world
        for sizes in unit_sizes:
            per = max(self.ALIGN_BYTES // self.es, 1)
            padded = [-(-s // per) * per for s in sizes]
            if max(ends) > 0 and max(e + p for e, p in zip(ends, padded)) > cap:
                extents.append(max(ends))
                ends = [0] * world
            self.slab_of.append(len(extents))
            self.at.append(list(ends))
            ends = [e + p for e, p in zip(ends, padded)]
        extents.append(max(max(ends), 1))
        self.slabs = [group.shared_empty(n, dtype, grow=n * self.es) for n in extents]
        # the same on every rank: the slabs are the same allocations in the same order everywhere
        self.base = [group.arena_offset(slab) for slab in self.slabs]

    def shard(self, k, numel):
        lo = self.at[k][self.rank]
        return self.slabs[self.slab_of[k]][lo:lo + numel]

    def peer_offsets(self, k):
        """Arena offsets of unit k's shard on every rank."""
        return [self.base[self.slab_of[k]] + a * self.es for a in self.at[k]]


class Unit:
    """One unit of the model under stage 3."""

    def __init__(self, index, module, params, group, residency):
        self.index, self.module, self.params = index, module, params
        self.group, self.residency = group, residency
        self.layout = FlatLayout([p.numel() for p in params], group.size, group.rank)
        self.where = dict(zip(params, self.layout.offsets))
        first = params[0]
        self.full = torch.empty(self.layout.numel, device=first.device, dtype=first.dtype)
        self._whole_bytes = self.full.untyped_storage().nbytes()
        residency.took()
        self.state = WHOLE  # as allocated; adopt() ends with the unit released
        self.mine = slice(self.layout.lo, self.layout.hi)
        self.shard = None
        self.peer_offsets = None
        self.grad_shard = torch.zeros(self.layout.hi - self.layout.lo, device=first.device, dtype=first.dtype)
        self._fetch = None      # the gather in flight
        self._scatter = None    # the gradients' reduce-scatter in flight
        self._staging = None
        self._owed = len(params)  # gradients of this backward still to arrive

    # ---- set-up
    @torch.no_grad()
    def adopt(self, home):
        """Rank 0's weights become everybody's; the parameters turn into views of
        `full`; this rank keeps its slice as the shard (tandem/zero.py:211-219)."""
        g = self.group
        g.pack(self.full, [(self.where[p], p.data) for p in self.params])
        g.broadcast(self.full, root=0)
        for p in self.params:
            o = self.where[p]
            p.data = self.full[o:o + p.numel()].view_as(p)
        own = self.full[self.mine]
        if home is not None:
            self.shard = home.shard(self.index, own.numel())
            self.shard.copy_(own)
            self.peer_offsets = home.peer_offsets(self.index)
        else:
            self.shard = own.clone()
        self.release()

    # ---- released -> gathering -> whole -> released
    def fetch(self):
        """Starts the gather unless the parameters are here or on their way."""
        if self.state != RELEASED:
            return
        self.full.untyped_storage().resize_(self._whole_bytes)
        self.residency.took()
        extra = {"peer_offsets": self.peer_offsets} if self.peer_offsets is not None else {}
        self._fetch = self.group.gather_unit(self.full, self.shard, self.layout.sizes, async_op=True, **extra)
        self.state = GATHERING

    def need(self):
        """Returns with the parameters whole (on the caller's stream)."""
        self.fetch()
        self._land()

    def _land(self):
        if self.state == GATHERING:
            self._fetch.wait()
            self._fetch = None
            self.state = WHOLE

    def release(self):
        self._land()  # a gather still in flight writes into the storage about to go
        if self.state == WHOLE:
            self.residency.gave()
            self.full.untyped_storage().resize_(0)
            self.state = RELEASED

    # ---- gradients
    def grad_arrived(self):
        """Called once per parameter and backward. With the last one the unit's backward
        is over: its gradients go into one staging buffer (one launch), its parameters
        are released and the reduce-scatter starts (tandem/zero.py:292-304)."""
        self._owed -= 1
        if self._owed:
            return
        first = self.params[0]
        self._staging = torch.empty(self.layout.numel, device=first.device, dtype=first.dtype)
        self.group.pack(self._staging, [(self.where[p], p.grad) for p in self.params])
        for p in self.params:
            p.grad = None
        self.release()
        # only this rank's chunk of the sum is kept: a group that can skip the partial sums is told so
        how = {"partial_sums": False} if getattr(self.group, "partial_sums_optional", False) else {}
        self._scatter = self.group.reduce_scatter(self._staging, self.layout.sizes, op="avg", async_op=True, **how)

    def settle(self):
        """End of backward: this rank's chunk of the averaged gradient joins the
        gradient shard (tandem/zero.py:309-316)."""
        if self._owed:
            raise RuntimeError("tandem FSDP: every parameter must receive a gradient")
        mine = self._scatter.wait()
        if mine.numel():
            self.grad_shard.add_(mine)
        self._scatter = self._staging = None
        self._owed = len(self.params)
        self.release()

    @torch.no_grad()
    def gathered_copy(self):
        out = torch.empty(self.layout.numel, device=self.shard.device, dtype=self.shard.dtype)
        extra = {"peer_offsets": self.peer_offsets} if self.peer_offsets is not None else {}
        self.group.gather_unit(out, self.shard, self.layout.sizes, **extra)
        return out


class Walk:
    """Which units a hook touches. Forward visits the units in order and backward in
    reverse; with prefetch the unit one step further along that walk is fetched while
    the current one computes. The last unit of the forward is the first of the backward
    and stays whole in between (tandem/zero.py:264-290)."""

    def __init__(self, count, prefetch):
        ahead = 1 if prefetch else 0
        self.forward = [(k, k + ahead if ahead and k + ahead < count else None) for k in range(count)]
        self.backward = [(k, k - ahead if ahead and k - ahead >= 0 else None) for k in range(count)]
        self.kept = count - 1

    def keeps(self, k, training):
        return training and k == self.kept


class FSDP(torch.nn.Module):
    """ZeRO stage 3 over model.units()."""

    def __init__(self, model, group, optimizer=None, prefetch=True, direct=None):
        super().__init__()
        for name in ("pack", "gather_unit"):
            if not hasattr(group, name):
                raise TypeError(f"FSDP needs a group that provides {name}() (tandem_amd.Group does)")
        self.module, self.g = model, group
        self.opt = optimizer if optimizer is not None else ShardedAdamW()
        self.prefetch = prefetch
        # torch says so whenever a unit's inputs need no gradient (the first unit's token ids);
        # the hook firing on the outputs instead is exactly the moment wanted
        warnings.filterwarnings("ignore", message="Full backward hook is firing when gradients are computed with respect to module outputs")
        self._residency = Residency()
        owned, seen = [], set()
        for module in model.units():
            params = [p for p in module.parameters() if p.requires_grad and id(p) not in seen]
            seen.update(id(p) for p in params)
            owned.append((module, params))
        if len(seen) != sum(1 for p in model.parameters() if p.requires_grad):
            raise ValueError("every parameter must belong to one of model.units()")
        self._direct = hasattr(group, "shared_empty") if direct is None else bool(direct)
        home = None
        if self._direct:
            sizes = [FlatLayout([p.numel() for p in ps], group.size, 0).sizes for _, ps in owned]
            try:
                home = ShardHome(group, sizes, owned[0][1][0].dtype)
            except CommError:
                if direct:  # asked for by name: say why it cannot be had
                    raise
                self._direct = False  # does not fit one exported allocation: gathers go through the group's own path
        self.units, self._unit_of = [], {}
        for k, (module, params) in enumerate(owned):
            unit = Unit(k, module, params, group, self._residency)
            unit.adopt(home)
            for p in params:
                self._unit_of[p] = unit
                p.register_post_accumulate_grad_hook(self._grad_ready)
            module.register_forward_pre_hook(self._entering(unit, forward=True))
            module.register_forward_hook(self._left(unit))
            module.register_full_backward_pre_hook(self._entering(unit, forward=False))
            self.units.append(unit)
        self._walk = Walk(len(self.units), prefetch)
        self._closing_queued = False
        self._residency.max_live = 0
        if self._direct:
            group.fence()  # every rank's shards are in place before anyone gathers

    live = property(lambda self: self._residency.live)
    max_live = property(lambda self: self._residency.max_live)

    def forward(self, *args, **kwargs):
        return self.module(*args, **kwargs)

    # ---- hooks
    def _entering(self, unit, forward):
        def before_forward(module, args):
            self._visit(self._walk.forward[unit.index])

        def before_backward(module, grad_output):
            if not self._closing_queued:
                self._closing_queued = True
                Variable._execution_engine.queue_callback(self._backward_over)
            self._visit(self._walk.backward[unit.index])

        return before_forward if forward else before_backward

    def _visit(self, stop):
        now, ahead = stop
        self.units[now].need()
        if ahead is not None:
            self.units[ahead].fetch()

    def _left(self, unit):
        def after_forward(module, args, output):
            if not self._walk.keeps(unit.index, torch.is_grad_enabled()):
                unit.release()

        return after_forward

    def _grad_ready(self, p):
        self._unit_of[p].grad_arrived()

    def _backward_over(self):
        self._closing_queued = False
        for unit in self.units:
            unit.settle()

    # ---- the optimizer's side
    @torch.no_grad()
    def step(self):
        if self._direct:
            self.g.fence()  # no rank still reads the shards this step rewrites
        for unit in self.units:
            self.opt.update(unit.index, unit.shard, unit.grad_shard)
        if self._direct:
            self.g.fence()  # the new shards are complete before any rank gathers them

    def zero_grad(self):
        for unit in self.units:
            unit.grad_shard.zero_()

    @torch.no_grad()
    def full_parameters(self):
        """All parameters, gathered (for checkpoints and tests)."""
        return torch.cat([unit.gathered_copy() for unit in self.units])
