"""Benchmark of the data-parallel reduction hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--mib 256] [--no-sweep] [--no-cpu]

A step is one ring reduce-scatter (avg) + all-gather over four rank buffers of
`--mib` MiB fp32 each, all resident in one GPU's HBM (world size 4 on one GPU,
4 MiB ring slots as the sweep unit of the kernel's grid). Prints ONE JSON line:
whole-job algorithmic HBM throughput of the step, the roofline of the dominant
kernel (the fused ring-step reduce) measured with HIP events inside the timed
region, a size sweep, the ZeRO-2 step time at 85.8M parameters, and the CPU
baseline (the oracle's CPU-process engine on this box's host cores).
"""

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X, published
WORLD = 4


def seeded_grads(world, n, dev, scale):
    import torch

    out = []
    for r in range(world):
        g = torch.Generator(device=dev).manual_seed(r)
        out.append(torch.randn(n, device=dev, generator=g) * scale)
    return out


def ring_pass(lw, bufs, events=None):
    """One step: reduce-scatter (avg) then all-gather, the two halves bracketed by
    events on the launch stream when asked."""
    import torch

    from tandem_amd._lib import check, lib, stream_ptr

    flats = [b.reshape(-1) for b in bufs]
    ptrs, n, st = lw._ptrs(flats), flats[0].numel(), stream_ptr(flats[0].device)
    none = lw._sizes(None, None)[0]
    if events is not None:
        e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        e[0].record()
    check(lib().tdm_local_reduce_scatter(ptrs, lw.world, n, 0, none, 0, 1, 0, st))
    if events is not None:
        e[1].record()
    check(lib().tdm_local_all_gather(ptrs, lw.world, n, 0, none, 0, st))
    if events is not None:
        e[2].record()
        events.append(e)


def time_ring(lw, bufs, steps, warmup):
    import torch

    for _ in range(warmup):
        ring_pass(lw, bufs)
    events = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        ring_pass(lw, bufs, events)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    rs_ms = sum(e[0].elapsed_time(e[1]) for e in events)
    ag_ms = sum(e[1].elapsed_time(e[2]) for e in events)
    return wall / steps, rs_ms / steps, ag_ms / steps


def sweep(lw, dev, steps):
    """Per-rank message sizes 64 KiB ... 256 MiB; algorithmic bytes 15*B per pass."""
    import torch

    rows = []
    for kib in (64, 1024, 4096, 16384, 65536, 262144):
        n = kib * 1024 // 4
        bufs = seeded_grads(WORLD, n, dev, 1e-2)
        reps = max(steps, 20 if kib <= 16384 else steps)
        per, rs, ag = time_ring(lw, bufs, reps, 3)
        b = n * 4
        rows.append({"MiB": kib / 1024, "ms": round(per * 1e3, 4), "GBps": round(15 * b / per / 1e9, 1),
                     "algbw_GBps": round(b / per / 1e9, 1), "k1_frac_of_hbm": round(12 * n * (WORLD - 1) / (rs * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)})
        del bufs
        torch.cuda.empty_cache()
    return rows


def cpu_baseline(n_elems):
    """The oracle's closed-form ring fold in plain C on one host core, over a
    bounded sample of the same workload (world 4, N(0, 1e-2))."""
    import numpy as np

    from oracle import ring

    rng = np.random.default_rng(0)
    xs = [(rng.standard_normal(n_elems) * 1e-2).astype(np.float32) for _ in range(WORLD)]
    ring.expected_all_reduce([x[:1024] for x in xs], True)  # load the library
    t0 = time.perf_counter()
    ring.expected_all_reduce(xs, True)
    dt = time.perf_counter() - t0
    return {"value": round(15 * n_elems * 4 / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"world 4 ring all-reduce (avg) of {n_elems * 4 >> 20} MiB fp32 per rank, closed-form fold in C, one pass, {dt:.2f} s",
            "host_cores": os.cpu_count()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--mib", type=int, default=256)
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every rank of the group is a buffer in that GPU's HBM; run with --gpus 1")

    import torch

    from tandem_amd import LocalWorld, _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py needs the MI355X (no CPU path exists)")
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    lw = LocalWorld(WORLD)
    n = args.mib * (1 << 20) // 4
    bufs = seeded_grads(WORLD, n, dev, 1e-2)
    per, rs_ms, ag_ms = time_ring(lw, bufs, args.steps, args.warmup)
    b = n * 4
    k1_launch_s = rs_ms * 1e-3 / (WORLD - 1)
    k1_bytes = 12 * n  # one launch: W chunks of n/W elements, two loads and one store each
    achieved = k1_bytes / k1_launch_s / 1e9
    line = {
        "metric": "fused-reduce GB/s (ring reduce-scatter+all-gather, world 4 on one GPU)",
        "value": round(15 * b / per / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(per * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"ring reduce-scatter(avg)+all-gather, world 4 simulated on one MI355X, {args.mib} MiB fp32 per rank, N(0,1e-2) seeded per rank",
                   "algorithmic_bytes_per_step": 15 * b, "algbw_GBps": round(b / per / 1e9, 1),
                   "frac_of_hbm_peak": round(15 * b / per / 1e9 / HBM_PEAK_GBPS, 4)},
        "roofline": {"bound": "hbm", "kernel": "k1_reduce_kernel<float>", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "bytes_per_launch": k1_bytes, "launch_us": round(k1_launch_s * 1e6, 2),
                     "copy_step_GBps": round(8 * n / (ag_ms * 1e-3 / (WORLD - 1)) / 1e9, 1)},
    }
    del bufs
    torch.cuda.empty_cache()
    if not args.no_sweep:
        line["sweep"] = sweep(lw, dev, max(5, args.steps // 2))
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(16 << 20)
    name = ctypes_device_name(_lib)
    line["device"] = name
    print(json.dumps(line), flush=True)


def ctypes_device_name(_lib):
    import ctypes

    buf = ctypes.create_string_buffer(128)
    cus, mem = ctypes.c_int(0), ctypes.c_int64(0)
    _lib.check(_lib.lib().tdm_device_info(0, buf, 128, ctypes.byref(cus), ctypes.byref(mem)))
    return f"{buf.value.decode()} ({cus.value} CUs, {mem.value >> 30} GiB)"


if __name__ == "__main__":
    main()
