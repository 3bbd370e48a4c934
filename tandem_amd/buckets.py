"""Host-side planning for gradient buckets and flat shards: pure integer work.

pack()            DDP's and ZeRO's greedy packing rule (tandem/ddp.py:56-68,
                  tandem/zero.py:92-103 in the reference).
FlatLayout        parameters as ranges of one flat buffer cut into one shard per
                  rank (tandem/zero.py:33-54).
fold_segments()   a bucket as the K2 kernel wants it: per-parameter ranges cut at
                  the ring's chunk boundaries, each tagged with its chunk.
"""

from .local import chunk_bounds, split_sizes


def pack(sizes_bytes, bucket_bytes, dtypes=None):
    """Greedy, in the given order: a bucket is closed when the next tensor would
    take it past bucket_bytes (or has another dtype); a tensor larger than the
    limit gets a bucket of its own. Returns lists of positions."""
    buckets, cur, size = [], [], 0
    for i, nb in enumerate(sizes_bytes):
        other = dtypes is not None and cur and dtypes[i] != dtypes[cur[0]]
        if cur and (size + nb > bucket_bytes or other):
            buckets.append(cur)
            cur, size = [], 0
        cur.append(i)
        size += nb
    if cur:
        buckets.append(cur)
    return buckets


class FlatLayout:
    """`numels` in registration order -> offsets in one flat buffer, shard sizes
    as torch.tensor_split would cut it, and this rank's [lo, hi)."""

    def __init__(self, numels, world, rank):
        self.numels = [int(n) for n in numels]
        self.offsets, off = [], 0
        for n in self.numels:
            self.offsets.append(off)
            off += n
        self.numel = off
        self.sizes = split_sizes(self.numel, world)
        self.lo = sum(self.sizes[:rank])
        self.hi = self.lo + self.sizes[rank]

    def bucket_sizes(self, a, b):
        """How much of the flat range [a, b) falls in each rank's shard."""
        out, lo = [], 0
        for s in self.sizes:
            out.append(max(0, min(b, lo + s) - max(a, lo)))
            lo += s
        return out


def zero_buckets(numels, elem_size, bucket_bytes):
    """ZeRO's buckets: contiguous ranges [a, b) of the flat buffer, packed from
    its end (reverse registration order). Returns [(a, b, [param positions])]."""
    order = list(range(len(numels)))[::-1]
    offsets, off = [], 0
    for n in numels:
        offsets.append(off)
        off += n
    out = []
    for grp in pack([numels[i] * elem_size for i in order], bucket_bytes):
        ps = [order[k] for k in grp]
        a = min(offsets[i] for i in ps)
        b = max(offsets[i] + numels[i] for i in ps)
        out.append((a, b, ps))
    return out


def fold_segments(numels, world):
    """One bucket whose flat buffer holds tensors of `numels` elements back to
    back. The ring all-reduce cuts that buffer with tensor_split; the summation
    order of an element depends on the chunk it falls in. Returns
    [(tensor position, offset inside the tensor, count, chunk)], in flat order."""
    total = sum(numels)
    bounds = chunk_bounds(total, world)
    segs, off = [], 0
    for i, n in enumerate(numels):
        a, b = off, off + n
        for c, (lo, hi) in enumerate(bounds):
            s, e = max(a, lo), min(b, hi)
            if e > s:
                segs.append((i, s - a, e - s, c))
        off = b
    return segs
