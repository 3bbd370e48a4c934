"""Benchmark of tandem's data-parallel reduction hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--mib 256] [--quick] [--no-cpu] [--no-fsdp]

A step is one ring reduce-scatter (avg) + all-gather over four rank buffers of
`--mib` MiB fp32 each, all resident in one GPU's HBM before the timed region
starts (world size 4 on one GPU). Prints ONE JSON line:

  value       algorithmic HBM bytes of the step (15 x message bytes) / step time
  roofline    the dominant kernel, the fused ring-step reduce (K1): 12 bytes per
              element per launch / the launch's duration, taken from HIP events
              recorded around the three back-to-back K1 launches of every step of
              a repeat of the timed steps (the timed steps carry no events: a record
              between two kernels holds the second one back), against the 8 TB/s
              HBM peak; `traffic` is the HBM traffic per
              launch measured with rocprofv3 counters
  sweep       message sizes 64 KiB .. 256 MiB, ring and single-launch fold
  bucket_path DDP's bucket flatten+average+unflatten (K2), 85.8M params, world 2
  zero2_step  reduce-scatter + AdamW + all-gather, 85.8M params, world 4
  fsdp_gather two processes sharing the GPU through HIP IPC: ZeRO-3 unit gathers
              of the 85.8M GPT, prefetched on the engine's stream
  ipc_allreduce_2_processes  Group(backend="hip") all_reduce between two processes
              sharing the GPU, the reference's one-GPU engine protocol and sizes
  cpu_baseline  the oracle's CPU-process engine (tandem's Python-engine protocol:
              one process per rank, 1 torch thread each, 2 x 4 MiB shared-memory
              slots per pair) on this box's host cores, same formula for GB/s
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
# HBM bytes per K1 launch at the default workload (4 chunk pairs of 64 MiB), from
# rocprofv3 FETCH_SIZE / WRITE_SIZE runs: kept in a tracked file next to the profile
# summary it comes from, together with the launch geometry of the build it was measured on.
K1_TRAFFIC_FILE = os.path.join(ROOT, "profiles", "k1_traffic.json")


def k1_traffic(mib, _lib):
    """Counter-derived HBM bytes per K1 launch, or None when the record does not describe
    this workload or this build (another tile size or workgroup size)."""
    import ctypes

    try:
        with open(K1_TRAFFIC_FILE) as f:
            rec = json.load(f)
        a, b, c = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
        _lib.check(_lib.lib().tdm_build_geometry(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)))
        if rec["mib_per_rank"] != mib or rec["world"] != WORLD:
            return None
        if rec["k1_tile_bytes"] != a.value or rec["workgroup_lanes"] != b.value:
            return None
        return int(rec["hbm_bytes_per_launch"])
    except (OSError, KeyError, ValueError):
        return None


def seeded_grads(world, n, dev, scale):
    import torch

    out = []
    for r in range(world):
        g = torch.Generator(device=dev).manual_seed(r)
        out.append(torch.randn(n, device=dev, generator=g) * scale)
    return out


def timed(fn, reps, warm=3):
    """Mean seconds per call, by HIP events on the launch stream."""
    import torch

    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / reps


def ring_pass(lw, flats, events=None, prepared=None):
    """One step: reduce-scatter (avg) then all-gather; the two halves bracketed by
    events on the launch stream when asked. `prepared`: the arguments of ring_args(), built once."""
    import torch

    from tandem_amd._lib import check

    rs, ag, ptrs, world, n, none, st = prepared or ring_args(lw, flats)
    if events is not None:
        e = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        e[0].record()
    check(rs(ptrs, world, n, 0, none, 0, 1, 0, st))
    if events is not None:
        e[1].record()
    check(ag(ptrs, world, n, 0, none, 0, st))
    if events is not None:
        e[2].record()
        events.append(e)


def ring_args(lw, flats):
    """The two C entry points and their arguments for ring_pass, on torch's current stream."""
    from tandem_amd._lib import lib, stream_ptr

    return (lib().tdm_local_reduce_scatter, lib().tdm_local_all_gather, lw._ptrs(flats), lw.world, flats[0].numel(),
            lw._sizes(None, None)[0], stream_ptr(flats[0].device))


def fold_call(lw, flats):
    """The all-reduce as a single launch, as a closure over arguments prepared once: what a
    compiled host calling the C ABI pays per call (the Python wrapper's checks and views cost
    more than the launch at small sizes)."""
    from tandem_amd import _lib

    ptrs, n, st = lw._ptrs(flats), flats[0].numel(), _lib.stream_ptr(flats[0].device)
    fn, world = _lib.lib().tdm_local_all_reduce, lw.world
    _lib.check(fn(ptrs, world, n, 0, 1, _lib.ALLREDUCE_FOLD, st))
    return lambda: fn(ptrs, world, n, 0, 1, _lib.ALLREDUCE_FOLD, st)


def time_ring(lw, bufs, steps, warmup):
    """Seconds per pass over exactly `steps` passes, bracketed by device synchronisations and
    nothing between the launches; then the same `steps` passes once more with HIP events
    around the reduce-scatter's and the all-gather's launches, for the kernels' own durations
    (an event record between two kernels holds the second one back: three per pass cost a
    256 MiB pass about 3 %, so the throughput is not taken from the instrumented passes)."""
    import torch

    flats = [b.reshape(-1) for b in bufs]
    prepared = ring_args(lw, flats)
    for _ in range(warmup):
        ring_pass(lw, flats, None, prepared)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        ring_pass(lw, flats, None, prepared)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    events = []
    for _ in range(steps):
        ring_pass(lw, flats, events, prepared)
    torch.cuda.synchronize()
    rs_ms = sum(e[0].elapsed_time(e[1]) for e in events)
    ag_ms = sum(e[1].elapsed_time(e[2]) for e in events)
    return wall / steps, rs_ms / steps, ag_ms / steps


def sweep(lw, dev, steps):
    """Per-rank message sizes 64 KiB ... 256 MiB, reduce-scatter (avg) + all-gather three ways.
    ring_*: the ring's steps, one launch each (K1 and the copy step), 15 B algorithmic bytes per
    pass of a per-rank message of B bytes. one_launch_*: the reduce-scatter as one launch and the
    all-gather as one launch, 11 B (what the library picks at this world size; the same bits in
    memory). fold_*: the all-reduce as a single launch, 8 B... 2 W B."""
    import torch

    from tandem_amd._lib import check, lib

    rows = []
    for kib in (64, 1024, 4096, 16384, 65536, 262144):
        n = kib * 1024 // 4
        bufs = seeded_grads(WORLD, n, dev, 1e-2)
        reps = steps if kib >= 65536 else max(steps, 30)
        check(lib().tdm_set_ring_form(1))  # reduce-scatter and all-gather as one launch each
        one, _, _ = time_ring(lw, bufs, reps, 3)
        check(lib().tdm_set_ring_form(0))  # the ring's steps, one launch each: K1 and the copy step
        per, rs, ag = time_ring(lw, bufs, reps, 3)
        flats = [x.reshape(-1) for x in bufs]
        fold = timed(fold_call(lw, flats), reps)
        b = n * 4
        graph_ms = fold_graph_ms = one_graph_ms = None
        if kib <= 65536:  # sizes where the gaps between the six launches still count: the same ring pass replayed from a HIP graph
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                ring_pass(lw, flats)
            graph_ms = round(timed(graph.replay, reps) * 1e3, 4)
            del graph
            check(lib().tdm_set_ring_form(1))
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                ring_pass(lw, flats)
            one_graph_ms = round(timed(graph.replay, reps) * 1e3, 4)
            del graph
            check(lib().tdm_set_ring_form(0))
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                lw.all_reduce(bufs, "avg", algorithm="fold")
            fold_graph_ms = round(timed(graph.replay, reps) * 1e3, 4)
            del graph
        rows.append({"MiB": kib / 1024, "ring_ms": round(per * 1e3, 4), "ring_GBps": round(15 * b / per / 1e9, 1),
                     "ring_algbw_GBps": round(b / per / 1e9, 1),
                     "k1_frac_of_hbm": round(12 * n * (WORLD - 1) / (rs * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                     "fold_ms": round(fold * 1e3, 4), "fold_GBps": round(2 * WORLD * b / fold / 1e9, 1),  # every rank's b bytes read once, written once
                     "fold_algbw_GBps": round(b / fold / 1e9, 1)})
        # one launch each: W reads + (W-1) writes per element, then every chunk read once and written W-1 times = (3W - 1) B per pass
        one_bytes = (3 * WORLD - 1) * b
        default_one = True  # at world 4 the library takes the one-launch forms at every size
        rows[-1].update({"one_launch_ms": round(one * 1e3, 4), "one_launch_GBps": round(one_bytes / one / 1e9, 1),
                         "one_launch_frac_of_hbm": round(one_bytes / one / 1e9 / HBM_PEAK_GBPS, 4),
                         "steps_ms_over_one_launch_ms": round(per / one, 3),
                         "default_form": "one_launch" if default_one else "steps"})
        if graph_ms is not None:
            rows[-1]["ring_hip_graph_ms"] = graph_ms
            rows[-1]["one_launch_hip_graph_ms"] = one_graph_ms
            rows[-1]["fold_hip_graph_ms"] = fold_graph_ms
        del bufs
        torch.cuda.empty_cache()
    check(lib().tdm_set_ring_form(-1))
    return rows


# (streams read, streams written) of each kernel at its benchmark workload
MIXES = {"k1_reduce": (2, 1), "ring_copy": (1, 1), "bucket_fold_w2": (2, 2), "zero2_fold_w4": (5, 1), "adamw": (4, 3),
         "adamw_gather_w4": (4, 6), "fold_all_reduce_w4": (4, 4), "zero2_step_one_launch_w4": (7, 6)}


def stream_mix(dev, reps):
    """What the memory system gives a kernel that only streams: for every kernel's mix of
    read and written streams, the probe library's kernel (no table, no arithmetic, the kernels'
    own launch geometry) over cold buffers of 85,842,432 fp32 each, best of a few launch
    geometries. The fused kernels are reported against these figures as well as against
    the 8 TB/s peak: a stream mix with many written streams does not reach the peak
    whatever the kernel."""
    import ctypes

    import torch

    from tandem_amd._lib import stream_ptr
    from tandem_amd._probe import check, lib  # libtandem_probe.so: a library of its own, not part of the plug-in

    n = 85_842_432
    whole = torch.empty(13 * n, device=dev).normal_()  # one allocation: the streams lie back to back
    bufs = [whole[k * n:(k + 1) * n] for k in range(13)]
    st = stream_ptr(dev)
    out = {"workload": "tdm_probe_stream_mix, 85,842,432 fp32 per stream, all streams cold (footprint 0.7-4.5 GB), "
                       "best of tile order shift 0/6 x occupancy pad 0/16/24 KiB, one 16-byte vector per lane and stream"}
    for name, (r, w) in MIXES.items():
        rd = (ctypes.c_void_p * 8)(*[b.data_ptr() for b in bufs[:r]])
        wr = (ctypes.c_void_p * 8)(*[b.data_ptr() for b in bufs[r:r + w]])
        best = None
        for shift in (0, 6):
            for pad in (0, 16384, 24576):
                t = timed(lambda: check(lib().tdm_probe_stream_mix(rd, r, wr, w, n * 4, 1, shift, pad, st)), reps, warm=2)
                rate = (r + w) * n * 4 / t / 1e9
                if best is None or rate > best[0]:
                    best = (rate, shift, pad)
        out[name] = {"reads": r, "writes": w, "GBps": round(best[0], 1), "frac_of_hbm_peak": round(best[0] / HBM_PEAK_GBPS, 4),
                     "xcd_shift": best[1], "occupancy_pad": best[2]}
    return out


def gpt_numels():
    import torch

    from tandem_amd.model import GPT, Config

    with torch.device("meta"):
        m = GPT(Config.preset("medium"))
    return [p.numel() for p in m.parameters()]


def bucket_path(dev, reps):
    """DDP's bucket path with both ranks on the GPU: 149 gradients per rank, 16
    buckets of up to 25 MiB in reverse registration order, averaged in place."""
    import torch

    from tandem_amd import LocalWorld
    from tandem_amd.buckets import pack

    numels = gpt_numels()
    n = sum(numels)
    order = list(range(len(numels)))[::-1]
    buckets = [[order[k] for k in g] for g in pack([numels[i] * 4 for i in order], 25 << 20)]
    world = 2
    grads = []
    for r in range(world):
        gen = torch.Generator(device=dev).manual_seed(100 + r)
        grads.append([torch.randn(m, device=dev, generator=gen) * 1e-3 for m in numels])
    table = LocalWorld(world).bucket_table(grads, buckets)
    t = timed(lambda: table.run(True), reps)
    nbytes = 8 * world * n
    return {"workload": "149 grads x 2 ranks, 85,842,432 fp32 params, 16 buckets of <= 25 MiB, one launch", "ms": round(t * 1e3, 4),
            "algorithmic_bytes": nbytes, "GBps": round(nbytes / t / 1e9, 1), "frac_of_hbm_peak": round(nbytes / t / 1e9 / HBM_PEAK_GBPS, 4),
            "segments": table.nseg}


def unit_gather(dev, reps):
    """K4 on its own: ZeRO-3's gather of one block unit of the 85.8M GPT (7,087,872 fp32) for both ranks of a
    world of two, the ranks being buffers of this process. Twelve units are gathered in turn, as a forward
    pass does, so no gather finds its shards in the caches. One launch serves both ranks: every shard is read
    once and stored into both ranks' full buffers, 4 (W + 1) bytes per element of the unit, which is what the
    throughput is counted on. (A rank gathering on its own moves 8 bytes per element; that figure over the same
    time is given beside it and is not a rate of this launch.)"""
    import torch

    from tandem_amd import LocalWorld

    world, unit, units = 2, 7_087_872, 12
    sizes = [unit // world] * world
    lw = LocalWorld(world)
    shards = [[torch.randn(sizes[r], device=dev) for r in range(world)] for _ in range(units)]
    fulls = [[torch.empty(unit, device=dev) for _ in range(world)] for _ in range(units)]

    def forward():
        for k in range(units):
            lw.unit_gather(fulls[k], shards[k], sizes)

    t = timed(forward, reps) / units
    nbytes = 4 * (world + 1) * unit
    out = {"workload": "ZeRO-3 unit gather, 7,087,872 fp32 per unit, 2 buffer ranks, 12 units in turn, one launch for both ranks",
           "us_per_unit": round(t * 1e6, 2), "algorithmic_bytes": nbytes, "GBps": round(nbytes / t / 1e9, 1),
           "frac_of_hbm_peak": round(nbytes / t / 1e9 / HBM_PEAK_GBPS, 4),
           "roofline_floor_us": round(nbytes / (HBM_PEAK_GBPS * 1e9) * 1e6, 2),
           "two_separate_gathers_equivalent_GBps": round(8 * unit * world / t / 1e9, 1)}
    # What a launch this SHORT can reach at all: the stream-mix probe (no table, no arithmetic) reading one stream of the unit's
    # size and writing two, over the same twelve sets of buffers in turn. A launch of 85 MB lasts about as long as it takes the
    # grid to fill the machine and drain again, so the yardstick for it is this and not the rate of a long stream.
    try:
        import ctypes

        from tandem_amd._lib import stream_ptr
        from tandem_amd._probe import check, lib

        sources = [torch.randn(unit, device=dev) for _ in range(units)]
        st = stream_ptr(dev)
        best = None
        for shift in (0, 3):
            def probes():
                for k in range(units):
                    rd = (ctypes.c_void_p * 8)(sources[k].data_ptr())
                    wr = (ctypes.c_void_p * 8)(fulls[k][0].data_ptr(), fulls[k][1].data_ptr())
                    check(lib().tdm_probe_stream_mix(rd, 1, wr, 2, unit * 4, 1, shift, 0, st))
            tp = timed(probes, reps) / units
            best = tp if best is None or tp < best else best
        out["same_size_probe_1r_2w_us"] = round(best * 1e6, 2)
        out["frac_of_mix_ceiling_at_this_size"] = round(best / t, 4)
    except Exception as e:  # the probe library is optional
        out["same_size_probe_error"] = repr(e)[:200]
    return out


def zero2_step(dev, reps):
    """ZeRO-2's reduce-scatter + AdamW + all-gather for the 85.8M GPT, world 4 on
    one GPU, all four shards stepped."""
    import torch

    from tandem_amd._lib import check, lib
    from tandem_amd.local import LocalZeRO2

    numels = gpt_numels()
    n = sum(numels)
    z = LocalZeRO2(WORLD, numels, dev, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    gen = torch.Generator(device=dev).manual_seed(7)
    p0 = torch.randn(n, device=dev, generator=gen) * 0.02
    grads = [torch.randn(n, device=dev, generator=gen) * 1e-3 for _ in range(WORLD)]
    for b in z.bufs:
        b.copy_(p0)

    def refill():
        for r in range(WORLD):
            z.staging[r].copy_(grads[r])
        z.zero_grad()

    # the refill (fresh gradients, zeroed shards) is outside the timed region: timed alone and subtracted
    t_refill = timed(refill, reps)
    out = {"workload": "85,842,432 fp32 params, world 4 on one GPU, 16 buckets of <= 25 MiB, AdamW(3e-4, (0.9, 0.95), 1e-8, 0.1) on all 4 shards"}
    shard = z.layouts[0].hi - z.layouts[0].lo
    opt = timed(lambda: [z.opts[r].update("bench", z.bufs[r][z.layouts[r].lo:z.layouts[r].hi], z.grad_shards[r]) for r in range(WORLD)], reps)
    # the same four updates on shards that start 4 bytes off a 128-byte boundary, as tensor_split shards may (p, g, m, v at one
    # phase), and on aligned shards cut from the very same allocations, so that only the phase differs between the two
    from tandem_amd.optim import ShardedAdamW

    stores = [[torch.zeros(shard + 64, device=dev).normal_(0.0, scale, generator=gen) for scale in (0.02, 1e-3)] for _ in range(WORLD)]
    for label, lead in (("on_grid", 0), ("off_grid", 1)):
        o = ShardedAdamW(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
        ps, gs = [st[0][lead:lead + shard] for st in stores], [st[1][lead:lead + shard] for st in stores]
        assert all(t.data_ptr() % 128 == 4 * lead for t in ps + gs)
        out[f"adamw_4_shards_{label}_ms"] = round(timed(lambda: [o.update(r, ps[r], gs[r]) for r in range(WORLD)], reps) * 1e3, 4)
        del o, ps, gs
    out["adamw_off_grid_over_on_grid"] = round(out["adamw_4_shards_off_grid_ms"] / out["adamw_4_shards_on_grid_ms"], 4)
    del stores
    # the all-gather of the flat parameter buffers in both of the library's forms, each on the bytes that form moves
    check(lib().tdm_set_ring_form(1))
    ag_one = timed(lambda: z.lw.all_gather(z.bufs, z.layouts[0].sizes), reps)
    check(lib().tdm_set_ring_form(0))
    ag_steps = timed(lambda: z.lw.all_gather(z.bufs, z.layouts[0].sizes), reps)
    check(lib().tdm_set_ring_form(-1))
    fused = timed(lambda: [z.opts[r].update("bench", z.bufs[r][z.layouts[r].lo:z.layouts[r].hi], z.grad_shards[r],
                                            [z.bufs[q][z.layouts[r].lo:z.layouts[r].hi] for q in range(WORLD) if q != r])
                           for r in range(WORLD)], reps)
    def refill_grads():
        for r in range(WORLD):
            z.staging[r].copy_(grads[r])

    t_refill_grads = timed(refill_grads, reps)
    one = timed(lambda: (refill_grads(), z.reduce_and_step()), reps) - t_refill_grads
    one_bytes = (8 * WORLD + 20) * n
    out.update({"one_launch_ms": round(one * 1e3, 4), "one_launch_algorithmic_bytes": one_bytes,
                "one_launch_GBps": round(one_bytes / one / 1e9, 1),
                "one_launch_roofline_floor_ms": round(one_bytes / (HBM_PEAK_GBPS * 1e9) * 1e3, 4)})
    # the same one-launch step with all 20 buffers carved out of ONE allocation instead of an allocation each
    z1 = LocalZeRO2(WORLD, numels, dev, one_allocation=True, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    for b in z1.bufs:
        b.copy_(p0)

    def refill_grads_1():
        for r in range(WORLD):
            z1.staging[r].copy_(grads[r])

    t1 = timed(refill_grads_1, reps)
    out["one_launch_one_allocation_ms"] = round((timed(lambda: (refill_grads_1(), z1.reduce_and_step()), reps) - t1) * 1e3, 4)
    del z1
    torch.cuda.empty_cache()
    for algorithm, rs_bytes in (("fold", (WORLD + 2) * 4 * n), ("ring", 12 * (WORLD - 1) * n + 12 * n)):
        # default: fold + the update that also writes the other ranks' copies; ring: three ring steps, update, and the
        # all-gather pinned to the ring's three copy steps (left alone the library takes its one-launch form at this world size)
        is_fold = algorithm == "fold"
        check(lib().tdm_set_ring_form(-1 if is_fold else 0))
        step = timed(lambda: (refill(), z.reduce_grads(algorithm), z.step(fused_gather=is_fold)), reps) - t_refill
        rs = timed(lambda: (refill(), z.reduce_grads(algorithm)), reps) - t_refill
        check(lib().tdm_set_ring_form(-1))
        nbytes = rs_bytes + ((28 + 4 * (WORLD - 1)) * n if is_fold else 28 * n + 8 * (WORLD - 1) * n)
        key = "" if algorithm == "fold" else "ring_"
        out.update({f"{key}ms": round(step * 1e3, 4), f"{key}reduce_scatter_ms": round(rs * 1e3, 4),
                    f"{key}algorithmic_bytes": nbytes, f"{key}GBps": round(nbytes / step / 1e9, 1),
                    f"{key}roofline_floor_ms": round(nbytes / (HBM_PEAK_GBPS * 1e9) * 1e3, 4)})
    # the same two kernels on the other shard types: AdamW over four shards (7 x the element size per element), and the whole
    # step as one launch ((2 W + 5) x the element size per element), in bfloat16, float16 and float64
    for dtype, tag in ((torch.bfloat16, "bf16"), (torch.float16, "f16"), (torch.float64, "f64")):
        es = torch.empty(0, dtype=dtype).element_size()
        zt = LocalZeRO2(WORLD, numels, dev, dtype=dtype, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
        for b in zt.bufs:
            b.copy_(p0)
        gt = [g.to(dtype) for g in grads]
        for r in range(WORLD):
            zt.grad_shards[r].copy_(gt[r][zt.layouts[r].lo:zt.layouts[r].hi])
        t_opt = timed(lambda: [zt.opts[r].update("bench", zt.bufs[r][zt.layouts[r].lo:zt.layouts[r].hi], zt.grad_shards[r])
                               for r in range(WORLD)], reps)
        zt.zero_grad()
        zt._shards_zero = True

        def refill_t():
            for r in range(WORLD):
                zt.staging[r].copy_(gt[r])

        t_fill = timed(refill_t, reps)
        t_one = timed(lambda: (refill_t(), zt.reduce_and_step()), reps) - t_fill
        k3_bytes, one_b = 7 * es * shard * WORLD, (2 * WORLD + 5) * es * n
        out.update({f"adamw_{tag}_4_shards_ms": round(t_opt * 1e3, 4), f"adamw_{tag}_GBps": round(k3_bytes / t_opt / 1e9, 1),
                    f"adamw_{tag}_frac_of_hbm_peak": round(k3_bytes / t_opt / 1e9 / HBM_PEAK_GBPS, 4),
                    f"one_launch_{tag}_ms": round(t_one * 1e3, 4), f"one_launch_{tag}_GBps": round(one_b / t_one / 1e9, 1),
                    f"one_launch_{tag}_frac_of_hbm_peak": round(one_b / t_one / 1e9 / HBM_PEAK_GBPS, 4)})
        del zt, gt
        torch.cuda.empty_cache()
    ag_one_bytes, ag_steps_bytes = 4 * WORLD * n, 8 * (WORLD - 1) * n
    out.update({"adamw_4_shards_ms": round(opt * 1e3, 4), "adamw_GBps": round(28 * shard * WORLD / opt / 1e9, 1),
                "adamw_frac_of_hbm_peak": round(28 * shard * WORLD / opt / 1e9 / HBM_PEAK_GBPS, 4),
                "all_gather_ms": round(ag_one * 1e3, 4), "all_gather_form": "one launch: every chunk read once, stored W-1 times",
                "all_gather_algorithmic_bytes": ag_one_bytes, "all_gather_GBps": round(ag_one_bytes / ag_one / 1e9, 1),
                "all_gather_ring_steps_ms": round(ag_steps * 1e3, 4), "all_gather_ring_steps_algorithmic_bytes": ag_steps_bytes,
                "all_gather_ring_steps_GBps": round(ag_steps_bytes / ag_steps / 1e9, 1),
                "adamw_gather_4_shards_ms": round(fused * 1e3, 4),
                "adamw_gather_GBps": round((28 + 4 * (WORLD - 1)) * shard * WORLD / fused / 1e9, 1),
                "note": "one_launch_ms: reduce-scatter, gradient add, AdamW and all-gather fused into one kernel (LocalZeRO2.reduce_and_step); "
                        "ms: gradients reduced by the single-launch ring-order fold, then AdamW writing the new parameters to all "
                        "four ranks' buffers in the same pass (default); ring_ms: the ring's three reduce steps, the add into the shards, "
                        "AdamW, the ring's three copy steps (tdm_set_ring_form(0)); all_gather_*: 4 W N bytes as one launch, "
                        "8 (W-1) N bytes as the ring's steps"})
    return out


# ---------------------------------------------------------------- two processes, HIP IPC
def fsdp_rank(g, steps, prefetch):
    import torch

    from tandem_amd import ShardedAdamW
    from tandem_amd.data import synthetic
    from tandem_amd.model import GPT, Config
    from tandem_amd.zero import FSDP

    cfg = Config.preset("medium")
    torch.manual_seed(0)
    text = synthetic(100_000)
    model = GPT(cfg).to(g.device)
    f = FSDP(model, g, ShardedAdamW(lr=3e-4, betas=(0.9, 0.95), weight_decay=0.1), prefetch=prefetch)
    times, waits = [], []
    for step in range(steps + 3):
        traced = step == steps + 2  # one more step with the group's trace on, for the counts; the timed steps carry no time-stamp events
        x, y = text.batch(step, 8, cfg.seq, rank=g.rank, world=g.size, device=g.device)
        g.barrier()
        torch.cuda.synchronize()
        g.tracing = traced
        g.waits.clear()
        g.trace.clear()
        t0 = time.perf_counter()
        loss = f(x, y)
        loss.backward()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        f.step()
        f.zero_grad()
        torch.cuda.synchronize()
        if 2 <= step < steps + 2:
            times.append(t1 - t0)
        if traced:
            waits.append(sum(b - a for name, a, b in g.waits if name == "gather_unit"))
            traced_ms = (t1 - t0) * 1e3
    n_gathers = sum(1 for name, *_ in g.trace if name == "gather_unit")
    return {"fwd_bwd_ms": statistics.median(times) * 1e3, "fwd_bwd_ms_min": min(times) * 1e3, "fwd_bwd_ms_max": max(times) * 1e3,
            "traced_step_fwd_bwd_ms": traced_ms, "traced_step_host_blocked_on_gathers_ms": statistics.median(waits) * 1e3,
            "gathers_per_step": n_gathers, "max_live": f.max_live, "live": f.live, "loss": float(loss.detach())}


class FileBarrier:
    """What Group asks of the launcher's barrier, for ranks that were started as separate commands (each under a
    profiler of its own): every rank leaves a file and waits until all of them are there."""

    def __init__(self, job, rank, size):
        self.paths = [f"/dev/shm/tandem-bench-{job}-{r}.ready" for r in range(size)]
        self.mine = self.paths[rank]

    def wait(self, timeout=None):
        open(self.mine, "w").close()
        end = time.monotonic() + (timeout or 60.0)
        while not all(os.path.exists(p) for p in self.paths):
            if time.monotonic() > end:
                raise TimeoutError("the other ranks did not start")
            time.sleep(0.01)

    def abort(self):
        pass


def fsdp_rank_alone(rank, world, job, steps):
    """One rank of fsdp_gather's workload as a process of its own: `bench.py --fsdp-rank R --fsdp-job NAME`, started
    once per rank (by hand, each under `rocprofv3 --kernel-trace`, say); TANDEM_HIP_GATHER picks where the gathers run."""
    import torch

    from tandem_amd import Group

    torch.cuda.set_device(0)
    barrier = FileBarrier(job, rank, world)
    g = Group(rank, world, torch.device("cuda", 0), barrier, None, timeout=120.0, backend="hip", job=job)
    try:
        out = fsdp_rank(g, steps, True)
        torch.cuda.synchronize()
        g.close()
    finally:
        try:
            os.unlink(barrier.mine)
        except OSError:
            pass
    out["gather"] = os.environ.get("TANDEM_HIP_GATHER", "caller")
    print(json.dumps({k: (round(v, 3) if isinstance(v, float) else v) for k, v in out.items()}), flush=True)


def fsdp_gather(steps):
    """ZeRO-3's unit gathers: copies launched in order on the training stream (the
    default), or on the engine's side stream: started behind an event from a ring and ended by
    a value word ("stream"), value words for both, or a fresh event for each; with and without prefetch."""
    from tandem_amd import launch

    out = {}
    before = os.environ.get("TANDEM_HIP_GATHER")
    try:
        for label, where, prefetch in (("in_order", "caller", True), ("side_stream_prefetch", "stream", True),
                                       ("side_stream_words_prefetch", "stream-words", True),
                                       ("side_stream_fresh_events_prefetch", "stream-events", True),
                                       ("side_stream_no_prefetch", "stream", False)):
            os.environ["TANDEM_HIP_GATHER"] = where
            res = launch(fsdp_rank, 2, steps, prefetch, gpus=[0, 0], timeout=120.0)
            out[label] = {k: (round(v, 3) if isinstance(v, float) else v) for k, v in res[0].items()}
    finally:
        if before is None:
            os.environ.pop("TANDEM_HIP_GATHER", None)
        else:
            os.environ["TANDEM_HIP_GATHER"] = before
    out["workload"] = ("2 processes sharing the GPU (HIP IPC memory handles), 85.8M GPT = 14 units (12 blocks of 7,087,872), "
                       "batch 8x512 split over 2 ranks, shards read directly from the peers' arenas")
    return out


def train_rank(g, strategy, steps):
    """One training step (forward, backward, optimizer) of the 85.8M GPT on this
    rank's rows of a batch of 8 x 512 tokens, as the reference's bench/run.py times
    its strategies; "alone" runs the same rows without any communication."""
    import torch

    from tandem_amd import ShardedAdamW
    from tandem_amd.data import synthetic
    from tandem_amd.ddp import DDP
    from tandem_amd.model import GPT, Config
    from tandem_amd.zero import FSDP, ZeRO

    cfg = Config.preset("medium")
    torch.manual_seed(0)
    text = synthetic(100_000)
    model = GPT(cfg).to(g.device)
    adamw = dict(lr=3e-4, betas=(0.9, 0.95), weight_decay=0.1)
    fused = "+fused" in strategy
    direct = "+direct" in strategy or fused
    streamwait = strategy.endswith("+streamwait")  # DDP/ZeRO that only order the training stream behind their collectives (opt-in)
    overlap = "+nooverlap" not in strategy  # DDP(overlap=False): every bucket's all-reduce starts when backward has ended
    kind = strategy.split("+")[0]
    opt = None
    if kind == "alone":
        z, opt = model, torch.optim.AdamW(model.parameters(), foreach=False, **adamw)
    elif kind == "ddp":
        z, opt = DDP(model, g, overlap=overlap, direct=direct, stream_ordered=streamwait), torch.optim.AdamW(model.parameters(), foreach=False, **adamw)
    elif kind in ("zero1", "zero2"):
        z = ZeRO(model, g, int(kind[-1]), ShardedAdamW(**adamw), direct=direct, fused_step=fused, stream_ordered=streamwait)
    else:
        z = FSDP(model, g, ShardedAdamW(**adamw))
    from tandem_amd.profile import Timeline, summarize

    times = []
    tl = Timeline(enabled=False, device=g.device)
    for step in range(steps + 3):
        x, y = text.batch(step, 8, cfg.seq, rank=g.rank, world=g.size, device=g.device)
        g.barrier()
        torch.cuda.synchronize()
        if step == steps + 2:  # one more step, profiled as the reference's bench/run.py profiles its last one
            g.trace.clear()
            g.waits.clear()
            g.tracing = tl.enabled = True
        t0 = time.perf_counter()
        with tl.span("forward"):
            loss = z(x, y)
        with tl.span("backward"):
            loss.backward()
        with tl.span("optimizer"):
            if opt is not None:
                opt.step()
                opt.zero_grad()
            else:
                z.step()
                z.zero_grad()
        torch.cuda.synchronize()
        if 2 <= step < steps + 2:
            times.append(time.perf_counter() - t0)
    g.tracing = False
    prof = summarize(tl.spans, [s for s in g.trace if s[0] != "barrier"], list(g.waits), time.perf_counter() - t0)
    prof.update({name + "_ms": round((e - s) * 1e3, 3) for name, s, e in tl.spans})
    return {"step_ms": statistics.median(times) * 1e3, "loss": loss.item(),
            "profile": {k: (round(v, 5) if isinstance(v, float) else v) for k, v in prof.items()}}


def train_steps(steps, world=2, strategies=("alone", "ddp", "ddp+nooverlap", "ddp+streamwait", "ddp+direct", "ddp+direct+streamwait", "zero1", "zero1+direct", "zero2", "zero2+streamwait", "zero2+direct", "zero2+fused", "zero3")):
    from tandem_amd import launch

    out = {"workload": f"{world} processes sharing the GPU, 85.8M GPT, batch 8x512 split over the ranks, fp32, full step "
                       "(forward, backward, optimizer); 'alone' = the same rows with no communication and torch AdamW; "
                       "'+direct' = buckets / flat buffers in the shared arenas, collectives arena to arena; '+fused' = that, and ZeRO-2's "
                       "reduce-scatters, AdamW and all-gather as one launch per rank; '+streamwait' = the training stream is only ordered "
                       "behind the collectives (stream_ordered=True, opt-in) where by default the host waits for them, as the reference's does; "
                       "'+nooverlap' = DDP(overlap=False), every all-reduce started after backward"}
    for s in strategies:
        res = launch(train_rank, world, s, steps, gpus=[0] * world, timeout=120.0)
        out[s] = {"step_ms": round(max(r["step_ms"] for r in res), 3), "loss": round(res[0]["loss"], 4),
                  "profile_rank0": res[0]["profile"]}
    return out


def ipc_rank(g, sizes_kib, reps, direct=False):
    """The reference's one-GPU engine benchmark (bench/engine_one_gpu.py there):
    barrier, then time all_reduce + device sync; median. direct: the tensor lives in
    the ranks' shared arenas and is reduced arena to arena, without slots."""
    import torch

    out = {}
    if direct:
        g.share_arena(max(sizes_kib) * 1024 + 4096)
        pool = g.shared_empty(max(sizes_kib) * 1024 // 4)
    for kib in sizes_kib:
        x = pool[:kib * 1024 // 4].fill_(1.0) if direct else torch.ones(kib * 1024 // 4, device=g.device)
        g.all_reduce(x, direct=direct)
        torch.cuda.synchronize()
        ts = []
        for _ in range(reps):
            g.barrier()
            torch.cuda.synchronize()
            t = time.perf_counter()
            g.all_reduce(x, direct=direct)
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t)
        out[kib] = statistics.median(ts)
    return out


def ipc_allreduce():
    from tandem_amd import launch

    sizes = [64, 256, 1024, 4096, 16384, 65536, 262144]  # KiB per rank; the reference's own sweep ends at 64 MiB
    out = {"workload": "all_reduce(sum) fp32 between 2 processes sharing the GPU through HIP IPC, barrier + all_reduce + device sync, median of 20",
           "reference_T4_cpp_engine_ms": {"64": 0.64, "256": 0.80, "1024": 0.83, "4096": 0.75, "16384": 1.72, "65536": 6.24}}

    def run(direct=False):
        res = launch(ipc_rank, 2, sizes, 20, direct, gpus=[0, 0], timeout=120.0)[0]
        return {str(k): round(v * 1e3, 3) for k, v in res.items()}

    out["staged_ms"] = run()  # the default: through peer-mapped staging memory
    out["direct_arena_ms"] = run(True)  # tensors in the shared arenas
    before = os.environ.get("TANDEM_HIP_ALGO")
    os.environ["TANDEM_HIP_ALGO"] = "ring"  # the reference's protocol: pieces through 2 x 4 MiB slots per pair
    try:
        out["slot_ring_2x4MiB_ms"] = run()
    finally:
        if before is None:
            del os.environ["TANDEM_HIP_ALGO"]
        else:
            os.environ["TANDEM_HIP_ALGO"] = before
    return out


# ---------------------------------------------------------------- CPU baseline
def cpu_rank(g, n, reps, numels):
    """Timed on the host: (i) the ring all-reduce(avg) of the GPU's main workload,
    (ii) the ZeRO-2 step (16 bucket reduce-scatters, shard add, AdamW, all-gather)."""
    import torch

    from oracle.cpu_engine import TorchCpuAdamW
    from tandem_amd.buckets import FlatLayout, zero_buckets

    x = torch.randn(n, generator=torch.Generator().manual_seed(g.rank)) * 1e-2
    g.all_reduce(x, op="avg")
    ts = []
    for _ in range(reps):
        g.barrier()
        t = time.perf_counter()
        g.all_reduce(x, op="avg")
        ts.append(time.perf_counter() - t)
    out = {"all_reduce_s": statistics.median(ts)}
    del x
    lay = FlatLayout(numels, g.size, g.rank)
    buckets = zero_buckets(numels, 4, 25 << 20)
    buf = torch.randn(lay.numel, generator=torch.Generator().manual_seed(5)) * 0.02
    grads = torch.randn(lay.numel, generator=torch.Generator().manual_seed(10 + g.rank)) * 1e-3
    staging = torch.empty_like(grads)
    shard = torch.zeros(lay.hi - lay.lo)
    opt = TorchCpuAdamW(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)  # torch ops, as tandem/optim.py:28-37
    ts = []
    for _ in range(3):
        staging.copy_(grads)
        shard.zero_()
        g.barrier()
        t = time.perf_counter()
        works = [g.reduce_scatter(staging[a:b], lay.bucket_sizes(a, b), op="avg", async_op=True) for a, b, _ in buckets]
        for (a, b, _), w in zip(buckets, works):
            mine = w.wait()
            if mine.numel():
                at = max(a, lay.lo) - lay.lo
                shard[at:at + mine.numel()].add_(mine)
        opt.update("flat", buf[lay.lo:lay.hi], shard)
        g.all_gather(buf, lay.sizes)
        ts.append(time.perf_counter() - t)
    out["zero2_step_s"] = statistics.median(ts)
    return out


def cpu_config1_rank(g, reps):
    """The reference's own CPU-runnable case: 2 ranks, 1,048,576 fp32 per rank, N(0,1)
    seeded by rank, all_reduce(avg); timed as its bench does (barrier, clock, all_reduce)."""
    import torch

    x = torch.randn(1 << 20, generator=torch.Generator().manual_seed(g.rank))
    g.all_reduce(x.clone(), op="avg")
    ts = []
    for _ in range(reps):
        y = x.clone()
        g.barrier()
        t = time.perf_counter()
        g.all_reduce(y, op="avg")
        ts.append(time.perf_counter() - t)
    return statistics.median(ts)


def cpu_two_rank_paths(g, numels):
    """The two-rank paths on the host. DDP's bucket path (tandem/ddp.py:89-119): 149 gradients copied into 16
    buckets of up to 25 MiB in reverse registration order, one all_reduce(avg) per bucket, copied back. ZeRO-3's
    unit gather (tandem/zero.py:238-252): the all_gather of one block unit of 7,087,872 fp32, twelve units in turn."""
    import torch

    from tandem_amd.buckets import pack

    gen = torch.Generator().manual_seed(100 + g.rank)
    grads = [torch.randn(m, generator=gen) * 1e-3 for m in numels]
    order = list(range(len(numels)))[::-1]
    buckets = [[order[k] for k in b] for b in pack([numels[i] * 4 for i in order], 25 << 20)]
    flats = [torch.empty(sum(numels[i] for i in b)) for b in buckets]
    ts = []
    for _ in range(3):
        g.barrier()
        t = time.perf_counter()
        works = []
        for b, flat in zip(buckets, flats):
            at = 0
            for i in b:
                flat[at:at + numels[i]].copy_(grads[i])
                at += numels[i]
            works.append(g.all_reduce(flat, op="avg", async_op=True))
        for b, flat, w in zip(buckets, flats, works):
            w.wait()
            at = 0
            for i in b:
                grads[i].copy_(flat[at:at + numels[i]])
                at += numels[i]
        ts.append(time.perf_counter() - t)
    out = {"bucket_path_s": statistics.median(ts)}
    del grads, flats
    unit, units = 7_087_872, 12
    sizes = [unit // g.size] * g.size
    lo = sum(sizes[:g.rank])
    fulls = [torch.zeros(unit) for _ in range(units)]
    for k, full in enumerate(fulls):
        full[lo:lo + sizes[g.rank]] = torch.randn(sizes[g.rank], generator=torch.Generator().manual_seed(7 * k + g.rank))
    g.all_gather(fulls[0], sizes)
    g.barrier()
    t = time.perf_counter()
    for full in fulls:
        g.all_gather(full, sizes)
    out["unit_gather_s"] = (time.perf_counter() - t) / units
    return out


def cpu_baseline(mib, reps):
    from oracle.cpu_engine import cpu_launch

    n = mib * (1 << 20) // 4
    t0 = time.perf_counter()
    res = cpu_launch(cpu_rank, WORLD, n, reps, gpt_numels())
    small = max(cpu_launch(cpu_config1_rank, 2, 20))
    two = cpu_launch(cpu_two_rank_paths, 2, gpt_numels())
    total = time.perf_counter() - t0
    t = max(r["all_reduce_s"] for r in res)
    z = max(r["zero2_step_s"] for r in res)
    return {"all_reduce_4MB_2_ranks_ms": round(small * 1e3, 3), "all_reduce_4MB_2_ranks_GBps": round((4 << 20) / small / 1e9, 3),"value": round(15 * n * 4 / t / 1e9, 3), "unit": "GB/s", "cores": WORLD, "kind": "port",
            "sample": f"oracle CPU-process engine (tandem's Python-engine protocol): ring all-reduce(avg), world 4 x 1 torch thread, "
                      f"{mib} MiB fp32 per rank (the GPU workload), 2 x 4 MiB shared-memory slots per pair, median of {reps}: "
                      f"{t * 1e3:.1f} ms per all-reduce; then 3 ZeRO-2 steps at 85,842,432 params (16 reduce-scatters, shard add, AdamW as torch ops, all-gather); {total:.1f} s in all, {total * WORLD:.0f} core-seconds",
            "algbw_GBps": round(n * 4 / t / 1e9, 3), "zero2_step_ms": round(z * 1e3, 1),
            "bucket_path_2_ranks_ms": round(max(r["bucket_path_s"] for r in two) * 1e3, 1),
            "unit_gather_2_ranks_ms": round(max(r["unit_gather_s"] for r in two) * 1e3, 2),
            "two_rank_sample": "2 ranks x 1 torch thread: DDP's bucket path for the 85.8M GPT (149 gradients into 16 buckets, all_reduce(avg) each, "
                               "copied back), median of 3; ZeRO-3's all_gather of a 7,087,872-element unit, mean of 12 units in turn",
            "host_cores": os.cpu_count()}


CONFIG_KEYS_KEPT = 24  # a record that keeps only the first keys of `config` must still hold the whole metric


def summarize(line):
    """The whole metric as plain numbers inside `config` and `roofline` (the sections keep the
    detail). `config` is written in order of importance and stays within CONFIG_KEYS_KEPT keys:
    first the ZeRO-2 step in ms and the other kernels of the path (AdamW, bucket path, unit
    gather), each with its fraction of the HBM peak, then the ring pass at 4, 16, 64 and 256 MiB
    per rank in the form the library takes by default. `roofline` gets K1's fraction at the same
    sizes and what a kernel that only streams reaches with each fused kernel's mix of streams."""
    cfg, roof = line["config"], line["roofline"]
    mix = line.get("stream_mix", {})

    def against(name, gbps):
        top = mix.get(name, {}).get("GBps")
        return round(gbps / top, 4) if top else None

    z = line.get("zero2_step")
    if z:
        cfg["zero2_step_one_launch_ms"] = z["one_launch_ms"]
        cfg["zero2_step_ms"] = z["ms"]
        cfg["zero2_step_one_launch_frac"] = round(z["one_launch_GBps"] / HBM_PEAK_GBPS, 4)
        cfg["adamw_ms"] = z["adamw_4_shards_ms"]
        cfg["adamw_frac"] = z["adamw_frac_of_hbm_peak"]
        if mix:
            z["one_launch_frac_of_mix_ceiling"] = against("zero2_step_one_launch_w4", z["one_launch_GBps"])
            z["adamw_frac_of_mix_ceiling"] = against("adamw", z["adamw_GBps"])
            z["adamw_gather_frac_of_mix_ceiling"] = against("adamw_gather_w4", z["adamw_gather_GBps"])
            roof["zero2_step_mix_ceiling_frac"] = mix["zero2_step_one_launch_w4"]["frac_of_hbm_peak"]
            roof["adamw_mix_ceiling_frac"] = mix["adamw"]["frac_of_hbm_peak"]
    b = line.get("bucket_path")
    if b:
        cfg["bucket_path_ms"] = b["ms"]
        cfg["bucket_path_frac"] = b["frac_of_hbm_peak"]
        if mix:
            b["frac_of_mix_ceiling"] = against("bucket_fold_w2", b["GBps"])
            roof["bucket_path_mix_ceiling_frac"] = mix["bucket_fold_w2"]["frac_of_hbm_peak"]
    u = line.get("unit_gather")
    if u:
        cfg["unit_gather_us"] = u["us_per_unit"]
        cfg["unit_gather_frac"] = u["frac_of_hbm_peak"]
    rows = {row["MiB"]: row for row in line.get("sweep", ())}
    for mib in (4.0, 16.0, 64.0, 256.0):
        row = rows.get(mib)
        if row is None:
            continue
        tag = f"{int(mib)}MiB"
        roof[f"k1_frac_{tag}"] = row["k1_frac_of_hbm"]
        # the pass as the library runs it by default at this size, on that form's own byte count
        one = row["default_form"] == "one_launch"
        cfg[f"pass_ms_{tag}"] = row["one_launch_ms"] if one else row["ring_ms"]
        cfg[f"pass_frac_{tag}"] = row["one_launch_frac_of_hbm"] if one else round(row["ring_GBps"] / HBM_PEAK_GBPS, 4)
    for mib in (64.0, 256.0):  # the ring's steps (K1 and the copy step), where the target is stated
        if mib in rows:
            cfg[f"pass_steps_frac_{int(mib)}MiB"] = round(rows[mib]["ring_GBps"] / HBM_PEAK_GBPS, 4)
    if 256.0 in rows:
        cfg["fold_pass_ms_256MiB"] = rows[256.0]["fold_ms"]
    if mix:
        roof["k1_mix_ceiling_frac"] = mix["k1_reduce"]["frac_of_hbm_peak"]
    assert len(cfg) <= CONFIG_KEYS_KEPT, f"config has {len(cfg)} keys: the last ones would be cut from a {CONFIG_KEYS_KEPT}-key record"


def accounting_offenders(node, path=""):
    """Every throughput above the HBM peak and every fraction of it above 1 in a bench line: a
    figure like that counts bytes its launch does not move. Keys are taken by name (`*GBps*`,
    `*frac*`); `peak` and the reference's numbers quoted for comparison are left out."""
    bad = []
    if isinstance(node, dict):
        for k, v in node.items():
            where = f"{path}.{k}" if path else k
            if isinstance(v, (dict, list)):
                bad += accounting_offenders(v, where)
            elif isinstance(v, (int, float)) and not isinstance(v, bool):
                if "GBps" in k and v > HBM_PEAK_GBPS:
                    bad.append((where, v))
                elif "frac" in k and "mix_ceiling" not in k and v > 1.0:
                    bad.append((where, v))
    elif isinstance(node, list):
        for i, v in enumerate(node):
            bad += accounting_offenders(v, f"{path}[{i}]")
    return bad


def device_name(_lib):
    import ctypes

    buf = ctypes.create_string_buffer(128)
    cus, mem = ctypes.c_int(0), ctypes.c_int64(0)
    _lib.check(_lib.lib().tdm_device_info(0, buf, 128, ctypes.byref(cus), ctypes.byref(mem)))
    return f"{buf.value.decode()} ({cus.value} CUs, {mem.value >> 30} GiB)"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--mib", type=int, default=256)
    ap.add_argument("--quick", action="store_true", help="only the main workload (for profiling runs)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-fsdp", action="store_true")
    ap.add_argument("--only", default="", help="comma list of single-process sections to run besides the main workload "
                                               "(sweep, bucket, gather, zero2, mix; fsdp: the two-process ZeRO-3 gather modes), for short profiling runs; "
                                               "implies --no-cpu and none of the other two-process sections")
    ap.add_argument("--fsdp-rank", type=int, default=-1, help="run ONE rank of the ZeRO-3 gather workload as this process "
                                                              "(with --fsdp-job; start every rank yourself, e.g. each under a profiler)")
    ap.add_argument("--fsdp-job", default="", help="a name the ranks started with --fsdp-rank share")
    ap.add_argument("--fsdp-world", type=int, default=2)
    args = ap.parse_args()
    if args.fsdp_rank >= 0:
        if not args.fsdp_job or args.fsdp_rank >= args.fsdp_world:
            sys.exit("--fsdp-rank needs --fsdp-job NAME and a rank below --fsdp-world")
        fsdp_rank_alone(args.fsdp_rank, args.fsdp_world, args.fsdp_job, args.steps)
        return
    only = {x for x in args.only.split(",") if x}
    if only - {"sweep", "bucket", "gather", "zero2", "mix", "fsdp"}:
        sys.exit("--only takes sweep, bucket, gather, zero2, mix and fsdp")
    if only:
        args.no_cpu = args.no_fsdp = True
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every rank of the group is a buffer in that GPU's HBM, or a process sharing it; "
                 "run with --gpus 1")

    # The two multi-process figures first, while this process has not touched the GPU.
    cpu = fsdp = None
    if not args.quick and not args.no_cpu:
        try:
            cpu = cpu_baseline(args.mib, 15)
        except Exception as e:  # reported, not measured by: the GPU figures must still come out
            cpu = {"error": repr(e)[:300]}
    ipc = train = train4 = None
    if "fsdp" in only:
        fsdp = fsdp_gather(8)
    if not args.quick and not args.no_fsdp:
        try:
            fsdp = fsdp_gather(8)
        except Exception as e:  # a secondary figure must not lose the line
            fsdp = {"error": repr(e)[:300]}
        try:
            ipc = ipc_allreduce()
        except Exception as e:
            ipc = {"error": repr(e)[:300]}
        try:
            train = train_steps(5)
        except Exception as e:
            train = {"error": repr(e)[:300]}
        try:
            train4 = train_steps(5, 4, ("alone", "ddp", "zero2", "zero2+direct", "zero2+fused", "zero3"))
        except Exception as e:
            train4 = {"error": repr(e)[:300]}
        os.environ["TANDEM_HIP_WAIT"] = "stream"  # every wait() parks the training stream instead of blocking the host
        try:
            train["stream_ordered_wait"] = {k: v["step_ms"] for k, v in train_steps(5, 2, ("ddp+direct", "zero2")).items()
                                            if k != "workload"}
        except Exception as e:
            train["stream_ordered_wait"] = {"error": repr(e)[:300]}
        finally:
            del os.environ["TANDEM_HIP_WAIT"]

    import torch

    from tandem_amd import LocalWorld, _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py needs the MI355X (tandem_amd has no CPU path)")
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    lw = LocalWorld(WORLD)
    n = args.mib * (1 << 20) // 4
    bufs = seeded_grads(WORLD, n, dev, 1e-2)
    _lib.check(_lib.lib().tdm_set_ring_form(0))  # the headline is the ring's steps (K1) at every --mib
    per, rs_ms, ag_ms = time_ring(lw, bufs, args.steps, args.warmup)
    _lib.check(_lib.lib().tdm_set_ring_form(-1))
    b = n * 4
    k1_launch_s = rs_ms * 1e-3 / (WORLD - 1)
    k1_bytes = 12 * n  # one launch: 4 chunk pairs of n/4 elements; two loads and one store of 4 bytes per element
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
        "config": {"workload": f"ring reduce-scatter(avg)+all-gather, world 4 simulated on one MI355X, {args.mib} MiB fp32 per rank, "
                               "N(0,1e-2) seeded per rank, inputs resident in HBM",
                   "algorithmic_bytes_per_step": 15 * b, "algbw_GBps": round(b / per / 1e9, 1),
                   "frac_of_hbm_peak": round(15 * b / per / 1e9 / HBM_PEAK_GBPS, 4)},
        "roofline": {"bound": "hbm", "kernel": "k1_reduce_kernel<float> (ring-step fused reduce)", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": k1_traffic(args.mib, _lib),
                     "bytes_per_launch": k1_bytes, "launch_us": round(k1_launch_s * 1e6, 2),
                     "launch_us_from": "HIP events on the launch stream around the three back-to-back K1 launches of each step, "
                                       "over a repeat of the timed steps (the timed steps themselves carry no events)",
                     "copy_step_GBps": round(8 * n / (ag_ms * 1e-3 / (WORLD - 1)) / 1e9, 1)},
    }
    del bufs
    torch.cuda.empty_cache()
    if not args.quick:
        if not only or "mix" in only:
            try:  # the probe is a library of its own; without it the line simply lacks the mix ceilings
                line["stream_mix"] = stream_mix(dev, 6)
            except Exception as e:
                line["stream_mix_error"] = repr(e)[:300]
            torch.cuda.empty_cache()
        def section(name, measure):
            """A section that fails is named in the line (and on stderr); the headline and the other sections still come out."""
            try:
                line[name] = measure()
            except Exception as e:
                line[name + "_error"] = repr(e)[:300]
                print(f"bench.py: section {name} failed: {e!r}", file=sys.stderr)
            torch.cuda.empty_cache()

        if not only or "sweep" in only:
            section("sweep", lambda: sweep(lw, dev, max(5, args.steps // 2)))
        if not only or "bucket" in only:
            section("bucket_path", lambda: bucket_path(dev, args.steps))
        if not only or "gather" in only:
            section("unit_gather", lambda: unit_gather(dev, args.steps))
        if not only or "zero2" in only:
            section("zero2_step", lambda: zero2_step(dev, max(5, args.steps // 2)))
        if fsdp is not None:
            line["fsdp_gather"] = fsdp
        if ipc is not None:
            line["ipc_allreduce_2_processes"] = ipc
        if train is not None:
            line["train_step_2_processes"] = train
        if train4 is not None:
            line["train_step_4_processes"] = train4
        if cpu is not None and "error" not in cpu:
            cpu["gpu_over_cpu"] = round(line["value"] / cpu["value"], 1)
            if "zero2_step" in line:
                cpu["zero2_step_gpu_over_cpu"] = round(cpu["zero2_step_ms"] / line["zero2_step"]["one_launch_ms"], 1)
            if "bucket_path" in line:
                cpu["bucket_path_gpu_over_cpu"] = round(cpu["bucket_path_2_ranks_ms"] / line["bucket_path"]["ms"], 1)
            if "unit_gather" in line:
                cpu["unit_gather_gpu_over_cpu"] = round(cpu["unit_gather_2_ranks_ms"] * 1e3 / line["unit_gather"]["us_per_unit"], 1)
        if cpu is not None:
            line["cpu_baseline"] = cpu
    summarize(line)
    line["device"] = device_name(_lib)
    bad = accounting_offenders(line)
    line["accounting"] = {"checked": "no *GBps* above the HBM peak, no *frac* above 1", "offenders": [f"{k}={v}" for k, v in bad]}
    print(json.dumps(line), flush=True)
    if bad:  # the line is out and names them; a figure above the roofline is a bug in this file's byte counts
        print(f"bench.py: figures above the roofline (bytes counted that the launch does not move?): {bad}", file=sys.stderr)


if __name__ == "__main__":
    main()
