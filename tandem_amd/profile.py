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

import json
import time

import torch


class _Span:
    """One `with timeline.span(name):` block."""

    def __init__(self, timeline, name):
        self.timeline, self.name = timeline, name

    def __enter__(self):
        self.begin = self.timeline.clock() if self.timeline.enabled else None
        return self

    def __exit__(self, *exc):
        if self.begin is not None:
            self.timeline.spans.append((self.name, self.begin, self.timeline.clock()))
        return False


class Timeline:
    """Named spans on the calling thread, (name, start, end) in time.perf_counter seconds; with a
    GPU device each end of a span waits for the device first (tandem/profile.py:13-35)."""

    def __init__(self, enabled=True, device=None):
        self.enabled = enabled
        self.device = None if device is None else torch.device(device)
        self.spans = []

    def clock(self):
        if self.device is not None and self.device.type == "cuda":
            torch.cuda.synchronize(self.device)
        return time.perf_counter()

    def span(self, name):
        return _Span(self, name)


def overlap_seconds(a, b):
    """Total length of the points that lie in some interval of `a` and in some interval of
    `b`: one sweep over all end points, counting how many intervals of each family are open."""
    marks = []
    for family, intervals in enumerate((a, b)):
        for lo, hi in intervals:
            if hi > lo:
                marks.append((float(lo), family, +1))
                marks.append((float(hi), family, -1))
    marks.sort(key=lambda m: m[0])
    open_now, total, last = [0, 0], 0.0, None
    for at, family, step in marks:
        if open_now[0] and open_now[1]:
            total += at - last
        open_now[family] += step
        last = at
    return total


def summarize(compute_spans, comm_spans, waits, step_time):
    """The reference's summary (tandem/profile.py:61-76): communication time is the sum of the
    collectives' own spans; exposed is the part of the caller's waits during which a collective
    was actually running; overlap is the share of communication that was not exposed (None
    without communication)."""
    busy = [(start, end) for _, start, end, _ in comm_spans]
    blocked = [(start, end) for _, start, end in waits]
    comm = sum(end - start for start, end in busy)
    exposed = overlap_seconds(blocked, busy)
    out = {"step_s": step_time, "compute_s": sum(end - start for _, start, end in compute_spans)}
    out["comm_s"], out["exposed_comm_s"] = comm, exposed
    out["overlap"] = None if comm <= 0 else max(0.0, 1 - exposed / comm)
    out["comm_bytes"] = sum(span[3] for span in comm_spans)
    return out


def _name_row(pid, tid, label):
    what = {"ph": "M", "pid": pid, "args": {"name": label}}
    what.update({"name": "process_name"} if tid is None else {"name": "thread_name", "tid": tid})
    return what


def _slice(pid, tid, origin, name, start, end, **args):
    event = {"ph": "X", "pid": pid, "tid": tid, "name": name, "ts": (start - origin) * 1e6, "dur": (end - start) * 1e6}
    if args:
        event["args"] = args
    return event


def chrome_trace(per_rank, path):
    """Writes a chrome://tracing / Perfetto file: one process per rank with a "compute" row
    (tid 0) and a "communication" row (tid 1). per_rank: [(compute_spans, comm_spans)] on a
    shared clock (tandem/profile.py:79-93)."""
    origin = min((span[1] for compute, comm in per_rank for span in list(compute) + list(comm)), default=0.0)
    events = []
    for rank, (compute, comm) in enumerate(per_rank):
        events += [_name_row(rank, None, f"rank {rank}"), _name_row(rank, 0, "compute"), _name_row(rank, 1, "communication")]
        events += [_slice(rank, 0, origin, name, start, end) for name, start, end in compute]
        events += [_slice(rank, 1, origin, name, start, end, bytes=nbytes) for name, start, end, nbytes in comm]
    with open(path, "w") as f:
        json.dump({"traceEvents": events}, f)
