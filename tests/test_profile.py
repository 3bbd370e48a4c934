"""tandem_amd.profile: the reference's Timeline / summarize / chrome_trace interface
(tandem/profile.py there). Host logic only: runs without a GPU."""

import json
import random
import time

import pytest

from tandem_amd.profile import Timeline, chrome_trace, overlap_seconds, summarize


def test_exposed_counts_only_running_communication():
    """The reference's own expectation (tests/test_comm.py:106-112 there): waits
    0-10 and 20-30, collectives 5-12 and 25-40."""
    s = summarize([], [("a", 5, 12, 0), ("b", 25, 40, 0)], [("a", 0, 10), ("b", 20, 30)], 40)
    assert s["comm_s"] == 22 and s["exposed_comm_s"] == 10
    assert abs(s["overlap"] - (1 - 10 / 22)) < 1e-12
    assert s["step_s"] == 40 and s["compute_s"] == 0 and s["comm_bytes"] == 0


def test_summary_fields_and_no_communication():
    s = summarize([("forward", 0.0, 1.5), ("backward", 2.0, 4.0)], [], [("x", 0, 1)], 5.0)
    assert s == {"step_s": 5.0, "compute_s": 3.5, "comm_s": 0, "exposed_comm_s": 0.0, "overlap": None, "comm_bytes": 0}
    s = summarize([], [("all_reduce", 1.0, 2.0, 64), ("all_gather", 1.5, 3.0, 36)], [("all_reduce", 0.0, 10.0)], 10.0)
    # overlapping collectives: their own time adds up (2.5 s), the exposed part is
    # the covered stretch (2.0 s)
    assert s["comm_s"] == 2.5 and s["exposed_comm_s"] == 2.0 and s["comm_bytes"] == 100
    assert abs(s["overlap"] - 0.2) < 1e-12
    # fully exposed, and waits that overlap each other are not counted twice
    s = summarize([], [("a", 0.0, 4.0, 1)], [("a", 0.0, 3.0), ("a", 1.0, 4.0)], 4.0)
    assert s["exposed_comm_s"] == 4.0 and s["overlap"] == 0.0


def test_overlap_against_a_grid():
    """Integer end points, so counting unit cells that lie in both unions is exact."""
    rng = random.Random(3)
    for _ in range(200):
        a = [(lo, lo + rng.randint(0, 9)) for lo in (rng.randint(0, 60) for _ in range(rng.randint(0, 6)))]
        b = [(lo, lo + rng.randint(0, 9)) for lo in (rng.randint(0, 60) for _ in range(rng.randint(0, 6)))]
        cells = sum(1 for c in range(80) if any(lo <= c < hi for lo, hi in a) and any(lo <= c < hi for lo, hi in b))
        assert overlap_seconds(a, b) == cells, (a, b)
        assert overlap_seconds(b, a) == cells


def test_timeline_spans_and_switch():
    tl = Timeline()
    t0 = time.perf_counter()
    with tl.span("forward"):
        time.sleep(0.01)
    with pytest.raises(KeyError):
        with tl.span("backward"):
            raise KeyError("x")
    t1 = time.perf_counter()
    assert [n for n, _, _ in tl.spans] == ["forward", "backward"]  # a span that raised is still recorded
    (_, a, b), (_, c, d) = tl.spans
    assert t0 <= a <= b <= c <= d <= t1 and b - a >= 0.01
    off = Timeline(enabled=False)
    with off.span("forward"):
        pass
    assert off.spans == []


def test_chrome_trace_file(tmp_path):
    per_rank = [([("forward", 10.0, 10.5)], [("all_reduce", 10.25, 10.75, 4096)]),
                ([("forward", 10.1, 10.4)], [])]
    path = tmp_path / "trace.json"
    chrome_trace(per_rank, path)
    events = json.loads(path.read_text())["traceEvents"]
    names = {(e["pid"], e["args"]["name"]) for e in events if e["ph"] == "M" and e["name"] == "process_name"}
    assert names == {(0, "rank 0"), (1, "rank 1")}
    rows = {(e["pid"], e["tid"], e["args"]["name"]) for e in events if e["ph"] == "M" and e["name"] == "thread_name"}
    assert rows == {(r, 0, "compute") for r in (0, 1)} | {(r, 1, "communication") for r in (0, 1)}
    spans = [e for e in events if e["ph"] == "X"]
    assert len(spans) == 3
    fwd0 = next(e for e in spans if e["pid"] == 0 and e["tid"] == 0)
    assert fwd0["ts"] == 0 and abs(fwd0["dur"] - 0.5e6) < 1e-3  # microseconds from the earliest start
    ar = next(e for e in spans if e["tid"] == 1)
    assert ar["name"] == "all_reduce" and abs(ar["ts"] - 0.25e6) < 1e-3 and ar["args"] == {"bytes": 4096}
    chrome_trace([], path)
    assert json.loads(path.read_text()) == {"traceEvents": []}
