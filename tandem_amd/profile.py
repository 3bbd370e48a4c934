"""Where a step's time goes on one rank: the reference's tandem/profile.py
interface (`Timeline`, `summarize`, `chrome_trace`; tandem/profile.py:13-93 there)
over this package's Group.

Compute spans are taken on the training thread between device synchronisations
(`Timeline.span`), communication spans come from `Group.trace`, which here holds
the GPU's own start and end of every collective (device time stamps placed on
time.perf_counter's clock), and `Group.waits` holds the time the training thread
was blocked in `Work.wait()`. On this backend `wait()` returns once the collective's
last kernel has been enqueued, which (hand-over between ranks being ordered on the
host) is about when that kernel starts on the GPU; what the GPU's default stream
then still waits for shows in the Chrome trace, where compute and communication
rows share one clock.
"""

import contextlib
import json
import time

import torch


class Timeline:
    """Named spans on the calling thread; with a GPU device each end of a span
    waits for the device first (tandem/profile.py:13-35)."""

    def __init__(self, enabled=True, device=None):
        self.enabled = enabled
        self.device = None if device is None else torch.device(device)
        self.spans = []  # (name, start, end), perf_counter seconds

    def _now(self):
        if self.device is not None and self.device.type == "cuda":
            torch.cuda.synchronize(self.device)
        return time.perf_counter()

    @contextlib.contextmanager
    def span(self, name):
        if not self.enabled:
            yield
            return
        start = self._now()
        try:
            yield
        finally:
            self.spans.append((name, start, self._now()))


def _covered(intervals):
    """Sorted, disjoint intervals covering the same points as `intervals`."""
    merged = []
    for lo, hi in sorted((float(a), float(b)) for a, b in intervals if b > a):
        if merged and lo <= merged[-1][1]:
            if hi > merged[-1][1]:
                merged[-1][1] = hi
        else:
            merged.append([lo, hi])
    return merged


def overlap_seconds(a, b):
    """Total length of the points that lie in some interval of `a` and some
    interval of `b`."""
    a, b = _covered(a), _covered(b)
    total, i, j = 0.0, 0, 0
    while i < len(a) and j < len(b):
        lo, hi = max(a[i][0], b[j][0]), min(a[i][1], b[j][1])
        if hi > lo:
            total += hi - lo
        if a[i][1] <= b[j][1]:
            i += 1
        else:
            j += 1
    return total


def summarize(compute_spans, comm_spans, waits, step_time):
    """The reference's summary (tandem/profile.py:61-76): communication time is
    the sum of the collectives' own spans; exposed is the part of the caller's
    waits during which a collective was actually running; overlap is the share
    of communication that was not exposed (None without communication)."""
    comm = sum(end - start for _, start, end, _ in comm_spans)
    exposed = overlap_seconds([(s, e) for _, s, e in waits], [(s, e) for _, s, e, _ in comm_spans])
    return {
        "step_s": step_time,
        "compute_s": sum(end - start for _, start, end in compute_spans),
        "comm_s": comm,
        "exposed_comm_s": exposed,
        "overlap": (max(0.0, 1 - exposed / comm) if comm > 0 else None),
        "comm_bytes": sum(nbytes for _, _, _, nbytes in comm_spans),
    }


def chrome_trace(per_rank, path):
    """Writes a chrome://tracing / Perfetto file: one process per rank with a
    "compute" and a "communication" row. per_rank: [(compute_spans, comm_spans)]
    on a shared clock (tandem/profile.py:79-93)."""
    starts = [s for comp, comm in per_rank for _, s, _ in comp] + [s for comp, comm in per_rank for _, s, _, _ in comm]
    origin = min(starts) if starts else 0.0
    events = []
    for rank, (comp, comm) in enumerate(per_rank):
        events.append({"ph": "M", "pid": rank, "name": "process_name", "args": {"name": f"rank {rank}"}})
        for row, label in enumerate(("compute", "communication")):
            events.append({"ph": "M", "pid": rank, "tid": row, "name": "thread_name", "args": {"name": label}})
        for name, s, e in comp:
            events.append({"ph": "X", "pid": rank, "tid": 0, "name": name, "ts": (s - origin) * 1e6, "dur": (e - s) * 1e6})
        for name, s, e, nbytes in comm:
            events.append({"ph": "X", "pid": rank, "tid": 1, "name": name, "ts": (s - origin) * 1e6, "dur": (e - s) * 1e6,
                           "args": {"bytes": nbytes}})
    with open(path, "w") as f:
        json.dump({"traceEvents": events}, f)
