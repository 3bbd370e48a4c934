"""Ring collectives on the CPU, two ways (TEST INFRASTRUCTURE ONLY).

`fold` / `expected_*` evaluate the closed form of what the reference's ring
leaves in every rank's buffer; `simulate` replays the ring message by message,
piece by piece, the way tandem/comm.py:287-311 does, and knows nothing of the
closed form. Tests require the two to agree with each other and with the
fixtures written by the reference's Python engine.

Arrays are numpy; 16-bit floats travel as uint16 bit patterns with kind
"bf16" or "f16". All arithmetic is per element in the tensor's own precision
(16-bit: widen to fp32, operate, round to nearest even once), as ATen does.
"""

import ctypes

import numpy as np

from . import lib

KINDS = {"f32": np.float32, "f64": np.float64, "bf16": np.uint16, "f16": np.uint16, "i64": np.int64,
         "i32": np.int32, "i16": np.int16, "i8": np.int8, "u8": np.uint8}
# integer sums narrower than 64 bits wrap around; the C side adds their bit patterns as unsigned numbers of the same width
_WRAPPING = {"i32": ("u32", np.uint32), "i16": ("u16", np.uint16), "i8": ("u8", np.uint8), "u8": ("u8", np.uint8)}


def split_sizes(n, world):
    """torch.tensor_split(flat, world) sizes: the first n % world chunks get one
    more element (tandem/comm.py:319-321, tandem/zero.py:29-30)."""
    base, extra = divmod(n, world)
    return [base + (1 if q < extra else 0) for q in range(world)]


def chunk_bounds(numel, world, sizes=None):
    """[lo, hi) of every rank's chunk; explicit sizes must partition the tensor
    (tandem/comm.py:322-324)."""
    if sizes is None:
        sizes = split_sizes(numel, world)
    sizes = [int(s) for s in sizes]
    if len(sizes) != world or sum(sizes) != numel or min(sizes, default=0) < 0:
        raise ValueError(f"chunk sizes {sizes} do not partition {numel} elements")
    out, lo = [], 0
    for s in sizes:
        out.append((lo, lo + s))
        lo += s
    return out


def _ptr_array(xs):
    arr = (ctypes.c_void_p * len(xs))()
    for i, x in enumerate(xs):
        arr[i] = x.ctypes.data
    return arr


def fold(xs, c, lo, hi, average, kind="f32", upto=None):
    """Chunk c's elements [lo, hi) after the ring has passed `upto` ranks
    (default: all of them): acc = y[c+1]; acc = y[c+k] + acc for k = 2..upto,
    with y = x / n when averaging."""
    n = len(xs)
    upto = n if upto is None else upto
    dt = KINDS[kind]
    xs = [np.ascontiguousarray(x, dtype=dt) for x in xs]
    if kind in _WRAPPING:
        if average:
            raise ValueError("integer tensors are not averaged")
        kind, as_unsigned = _WRAPPING[kind]
        xs = [x.view(as_unsigned) for x in xs]
    out = np.empty(hi - lo, dtype=xs[0].dtype if xs else dt)
    fn = getattr(lib(), f"orc_ring_fold_{kind}")
    fn(_ptr_array(xs), ctypes.c_int(n), ctypes.c_int(c), ctypes.c_int(upto), ctypes.c_int(int(average)),
       ctypes.c_int64(lo), ctypes.c_int64(hi), ctypes.c_void_p(out.ctypes.data))
    return out.view(dt)


def expected_all_reduce(xs, average, kind="f32"):
    """The buffer every rank holds after all_reduce (tandem/comm.py:326-347)."""
    n, numel = len(xs), xs[0].shape[0]
    if n == 1:
        return np.array(xs[0], copy=True)
    out = np.empty(numel, dtype=KINDS[kind])
    for c, (lo, hi) in enumerate(chunk_bounds(numel, n)):
        out[lo:hi] = fold(xs, c, lo, hi, average, kind)
    return out


def expected_reduce_scatter(xs, sizes, average, kind="f32"):
    """Every rank's whole buffer after a bare reduce_scatter: chunk c on rank
    (c+k) % n holds the partial sum of k terms; k = n on the owner
    (tandem/comm.py:349-369)."""
    n, numel = len(xs), xs[0].shape[0]
    outs = [np.empty(numel, dtype=KINDS[kind]) for _ in range(n)]
    for c, (lo, hi) in enumerate(chunk_bounds(numel, n, sizes)):
        for k in range(1, n + 1):
            outs[(c + k) % n][lo:hi] = fold(xs, c, lo, hi, average, kind, upto=k)
    return outs


def expected_all_gather(xs, sizes):
    """Chunk q of every rank becomes rank q's chunk q (tandem/comm.py:371-385)."""
    n, numel = len(xs), xs[0].shape[0]
    out = np.empty_like(xs[0])
    for q, (lo, hi) in enumerate(chunk_bounds(numel, n, sizes)):
        out[lo:hi] = xs[q][lo:hi]
    return out


# ---- the step-by-step simulator: mailboxes, pieces, lockstep exchange

def _widen(a, kind):
    if kind == "bf16":
        return (a.astype(np.uint32) << 16).view(np.float32)
    if kind == "f16":
        return a.view(np.float16).astype(np.float32)
    return a


def _narrow(a, kind):
    if kind == "bf16":
        out = np.empty(a.shape, np.uint16)
        a = np.ascontiguousarray(a, dtype=np.float32)
        lib().orc_f32_to_bf16(ctypes.c_void_p(a.ctypes.data), ctypes.c_void_p(out.ctypes.data), ctypes.c_int64(a.size))
        return out
    if kind == "f16":
        return a.astype(np.float16).view(np.uint16)
    return a


def _div(a, n, kind):
    w = _widen(a, kind)
    return _narrow(w / w.dtype.type(n), kind)


def _add(a, b, kind):
    return _narrow(_widen(a, kind) + _widen(b, kind), kind)


def simulate(xs, collective, sizes=None, average=False, kind="f32", piece_elems=64):
    """Replays the ring on n in-memory ranks: every step, each rank puts its
    outgoing chunk into the next rank's mailbox piece by piece and takes (adds or
    copies) the pieces its predecessor left (tandem/comm.py:287-311). Returns
    every rank's buffer."""
    n, numel = len(xs), xs[0].shape[0]
    bufs = [np.array(x, dtype=KINDS[kind], copy=True) for x in xs]
    if collective in ("all_reduce", "reduce_scatter") and average:
        bufs = [_div(b, n, kind) for b in bufs]  # the whole tensor, before any sum
    if n == 1:
        return bufs
    bounds = chunk_bounds(numel, n, None if collective == "all_reduce" else sizes)

    def exchange(send_chunk_of, recv_chunk_of, reduce):
        mailbox = {}
        for r in range(n):  # put: rank r -> r+1, in pieces
            lo, hi = bounds[send_chunk_of(r)]
            mailbox[(r + 1) % n] = [bufs[r][k:min(k + piece_elems, hi)].copy() for k in range(lo, hi, piece_elems)]
        for r in range(n):  # take: pieces from r-1, in order
            lo, hi = bounds[recv_chunk_of(r)]
            pieces = mailbox[r]
            want = len(range(lo, hi, piece_elems))
            assert len(pieces) == want, "ring out of step"
            for j, k in enumerate(range(lo, hi, piece_elems)):
                into = bufs[r][k:min(k + piece_elems, hi)]
                assert into.shape == pieces[j].shape
                into[...] = _add(into, pieces[j], kind) if reduce else pieces[j]

    if collective in ("all_reduce", "reduce_scatter"):
        for s in range(n - 1):
            exchange(lambda r: (r - s - 1) % n, lambda r: (r - s - 2) % n, True)
    if collective in ("all_reduce", "all_gather"):
        for s in range(n - 1):
            exchange(lambda r: (r - s) % n, lambda r: (r - s - 1) % n, False)
    return bufs
