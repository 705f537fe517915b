"""Benchmark of the EP dispatch + combine hot path on one MI355X.

A "step" is one MoE layer's dispatch followed by its combine (identity expert in between) on synthetic inputs that
are already resident in HBM.  The default workload is the prefill shape the headline metric is quoted on:
4096 tokens x 7168 bf16, 256 experts, top-8, Zipf(1.0) expert popularity ("C3").

Prints one JSON line: whole-step effective bandwidth (algorithmic bytes / time), per-layer latency, a roofline object
for the dominant kernel (timed with HIP events around that kernel on the stream it runs on) and the CPU oracle
timed on this box's host cores as a baseline.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
SCHEDULES = {
    "flags-serial": "tile flags published by dispatch and awaited by combine, one stream",
    "flags-overlapped": "tile flags published by dispatch and awaited by combine, combine on a second stream beside dispatch",
    "plain": "no tile flags, one stream",
}


def measured_traffic(workload, kernel):
    """HBM bytes per launch from the committed hardware-counter summary (profiles/hbm_traffic_<workload>.txt, lines
    `<kernel>_bytes_per_launch = N`), or None when no summary covers this workload."""
    path = os.path.join(ROOT, "profiles", f"hbm_traffic_{workload}.txt")
    if not os.path.exists(path):
        return None
    for line in open(path):
        parts = line.split("=")
        if len(parts) == 2 and parts[0].strip() == f"{kernel}_bytes_per_launch":
            return int(float(parts[1].strip()))
    return None


def trace_avg_us(path, section, kernel):
    """Average duration of a kernel from a committed rocprofv3 kernel-trace summary (profiles/*_kernel_stats.txt): the
    table row `<kernel template> calls avg_us ...` of the section whose header line `== [<section>] ...` names the
    configuration that was run, or None.  Event-bracketed times read a few microseconds above it (an event record
    holds the queue)."""
    path = os.path.join(ROOT, path)
    if not os.path.exists(path) or not kernel:
        return None
    inside = False
    for line in open(path):
        if line.startswith("=="):
            inside = f"[{section}]" in line
        elif inside and line.startswith(kernel):
            parts = line.rsplit(None, 5)
            try:
                return float(parts[-4])
            except (ValueError, IndexError):
                return None
    return None


def run_timed_passes(torch, ep, step, steps, comm, use_events, stride):
    """The timed region, twice over exactly `steps` steps each.  The first pass carries nothing but the steps: `value`
    comes from it.  The second records a (start, stop) pair of HIP events around the scatter and the reduce kernel on
    every `stride`-th step (the library records them on the stream the kernels are launched on); an event record between
    two kernels holds the queue for about 5 us on this GPU (about 22 us per bracketed step), which is why the pass that
    `value` is taken from has none.  Returns (seconds of pass 1, seconds of pass 2 or None, {step: event pairs})."""
    import time as _time
    torch.cuda.synchronize()
    t0 = _time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = _time.perf_counter() - t0
    if not use_events:
        return elapsed, None, {}
    sampled = [i for i in range(steps) if i % stride == 0]
    pairs = {i: [(ep.HipEvent(timing=True), ep.HipEvent(timing=True)) for _ in range(2)] for i in sampled}
    torch.cuda.synchronize()
    t0 = _time.perf_counter()
    for i in range(steps):
        if i in pairs:
            ep.set_kernel_timing_events(comm, ep.K_SCATTER, *pairs[i][0])
            ep.set_kernel_timing_events(comm, ep.K_REDUCE, *pairs[i][1])
            step()
            ep.set_kernel_timing_events(comm, ep.K_SCATTER, None, None)
            ep.set_kernel_timing_events(comm, ep.K_REDUCE, None, None)
        else:
            step()
    torch.cuda.synchronize()
    return elapsed, _time.perf_counter() - t0, pairs


def kernel_event_stats(pairs, byte_counts):
    """Per-kernel figures from the event pairs of run_timed_passes: {name: {...}} for (scatter, reduce)."""
    kernels = {}
    for which, (name, nbytes) in enumerate(byte_counts):
        times = sorted(p[which][0].elapsed_ms(p[which][1]) * 1e3 for p in pairs.values())
        avg = sum(times) / len(times)
        kernels[name] = {"avg_us": round(avg, 2), "min_us": round(times[0], 2), "p50_us": round(times[len(times) // 2], 2),
                         "max_us": round(times[-1], 2), "launches_timed": len(times), "algorithmic_bytes": nbytes,
                         "achieved_GBps": round(nbytes / (avg * 1e-6) / 1e9, 1)}
    return kernels


def roofline_of(kernels, dom, kernel_name, traffic, traffic_source, trace_us, trace_source):
    """The roofline object of the dominant kernel.  `achieved` / `frac` price the kernel by the committed rocprofv3
    kernel-trace summary when it holds a row for the very kernel template that was launched (no event records between
    kernels there); the figure from this run's HIP events stands beside it under `event_timed` and takes its place when
    no summary matches."""
    nbytes = kernels[dom]["algorithmic_bytes"]
    event = {"avg_launch_us": kernels[dom]["avg_us"], "launches_timed": kernels[dom]["launches_timed"],
             "achieved": kernels[dom]["achieved_GBps"], "frac": round(kernels[dom]["achieved_GBps"] / HBM_PEAK_GBPS, 4)}
    roofline = {"bound": "hbm", "kernel": kernel_name, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "algorithmic_bytes_per_launch": nbytes, "traffic": traffic, "traffic_source": traffic_source if traffic else None,
                "event_timed": event}
    if trace_us:
        achieved = nbytes / (trace_us * 1e-6) / 1e9
        roofline.update(achieved=round(achieved, 1), frac=round(achieved / HBM_PEAK_GBPS, 4), avg_launch_us=trace_us,
                        frac_source=f"rocprofv3 kernel trace, {trace_source}")
    else:
        roofline.update(achieved=event["achieved"], frac=event["frac"], avg_launch_us=event["avg_launch_us"],
                        frac_source="HIP events of this run (no committed kernel-trace row for this kernel template)")
    return roofline


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=100)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--workload", default="C3", choices=["C2", "C3", "C4", "C5", "M1"],
                   help="C2-C5: dispatch / combine by expert ids; M1: the plan-driven (MoonEP) stages at S=4096, K=8, "
                        "H=7168")
    p.add_argument("--moon-ranks", type=int, default=1,
                   help="M1: logical ranks of the world on this device (1 = one rank's share with every route local, "
                        "8 = the whole 8-rank world of the published shape)")
    p.add_argument("--moon-saved", action="store_true",
                   help="M1: dispatch with the saved duplicate plan instead of building it on every call")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-kernel-events", action="store_true",
                   help="do not record per-kernel HIP events inside the timed region")
    p.add_argument("--schedule", default="auto", choices=["auto", "flags-serial", "flags-overlapped", "plain"],
                   help="C2-C5: what a timed step is.  flags-serial: dispatch publishes tile readiness flags, combine "
                        "waits on them, both on one stream; flags-overlapped: the same with combine on a second "
                        "stream, reducing tiles while dispatch is still writing rows; plain: no flags; auto (default): "
                        "the faster of the two flag schedules, decided by a short calibration before the timed steps")
    p.add_argument("--overlap", action="store_true", help="same as --schedule flags-overlapped")
    p.add_argument("--tile-rows", type=int, default=64)
    p.add_argument("--no-overlap-leg", action="store_true",
                   help="skip the extra, separately timed runs of the schedules that are not the timed one (reported "
                        "under config.other_schedules)")
    p.add_argument("--no-graph-leg", action="store_true",
                   help="decode-sized workloads: skip the extra leg that replays a captured HIP graph of 16 layers "
                        "(reported under config.graph_replay)")
    p.add_argument("--no-stage-leg", action="store_true",
                   help="skip the extra leg with a slow expert-stage stand-in between dispatch and combine (reported under "
                        "config.expert_stage)")
    p.add_argument("--stage-workgroups", type=int, default=64,
                   help="expert-stage leg: workgroups of the producer (it must leave room for the waiting combine)")
    p.add_argument("--stage-tile-rows", type=int, default=16, help="expert-stage leg: rows per readiness tile")
    p.add_argument("--stage-tile-ns", type=int, default=40000,
                   help="expert-stage leg: time the producer spends on a tile at least, in nanoseconds")
    p.add_argument("--moon-cached-row-bytes", type=int, default=None,
                   help="M1: value for TileXRMoonEpSetCachedRowBytes (0 = always the scatter kernel that tolerates "
                        "token rows that come from HBM)")
    p.add_argument("--no-ceilings", action="store_true",
                   help="skip the memory-system yardsticks (probe kernels of the library) reported under `ceilings`")
    p.add_argument("--no-rotate-leg", action="store_true",
                   help="skip the extra leg that feeds every step a different input tensor (inputs not cache-resident)")
    p.add_argument("--event-stride", type=int, default=0,
                   help="record the per-kernel events on every N-th step of the second timed pass (0: steps // 16, at "
                        "least 1, so that even a short run brackets eight launches and more)")
    p.add_argument("--calibrate-copy", action="store_true",
                   help="also launch a plain 256 MiB read + 256 MiB write kernel before the warm-up, as the known-size "
                        "yardstick for hardware-counter runs")
    return p.parse_args()


def measured_ceilings(ep, torch, stream, dev, reps=10, narrow=None, far=False):
    """What this device's memory system delivers for plain access patterns, measured in this run with the library's
    own probe kernels (HIP events around `reps` launches each): pure read, pure write, copy, and the read : write
    mixes of the scatter (1 : 8) and the reduce (8 : 1).  GB/s of all bytes moved, reads plus writes.  The mixed
    patterns depend on how far apart their eight regions lie (5.6 to 6.6 TB/s for the 1 : 8 mix between 56 and 125 MiB),
    so they are run at three sizes and the best is kept: a ceiling, not an average."""
    patterns = {"read": ep.PROBE_READ, "write": ep.PROBE_WRITE, "copy": ep.PROBE_COPY, "fan_out_1r8w": ep.PROBE_FAN_OUT,
                "fan_in_8r1w": ep.PROBE_FAN_IN, "gather_rows_8r1w": ep.PROBE_GATHER_ROWS}
    sizes = (448, 472, 1000)       # MiB, each a multiple of eight rows of 14 KiB
    out = {"buffer_MiB": list(sizes), "launches": reps}
    for mib in sizes:
        nbytes = mib << 20
        src = torch.zeros((nbytes,), dtype=torch.uint8, device=dev)
        dst = torch.zeros((nbytes,), dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        moved = {"read": nbytes, "write": nbytes, "copy": 2 * nbytes, "fan_out_1r8w": nbytes + nbytes // 8,
                 "fan_in_8r1w": nbytes + nbytes // 8, "gather_rows_8r1w": nbytes + nbytes // 8}
        for name, pattern in patterns.items():
            if mib != sizes[0] and name in ("read", "write", "copy"):
                continue
            size = nbytes
            if name == "gather_rows_8r1w":      # whole groups of eight 14 KiB rows
                size = nbytes // (8 * 14336) * (8 * 14336)
                moved[name] = size + size // 8
            for _ in range(3):
                ep.check(ep.memory_probe(pattern, src, dst, size, stream), "memory probe")
            a, b = ep.HipEvent(timing=True), ep.HipEvent(timing=True)
            a.record(stream)
            for _ in range(reps):
                ep.check(ep.memory_probe(pattern, src, dst, size, stream), "memory probe")
            b.record(stream)
            stream.synchronize()
            us = a.elapsed_ms(b) * 1e3 / reps
            rate = round(moved[name] / (us * 1e-6) / 1e9, 1)
            out[name + "_GBps"] = max(rate, out.get(name + "_GBps", 0.0))
        if mib == sizes[0]:
            # the runtime's own device-to-device copy, as a yardstick that owes nothing to this library's kernels
            hip = ctypes.CDLL("libamdhip64.so")
            hip.hipMemcpyDtoDAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
            raw = ctypes.c_void_p(stream.cuda_stream)

            def runtime_copy():
                if hip.hipMemcpyDtoDAsync(dst.data_ptr(), src.data_ptr(), nbytes, raw) != 0:
                    raise RuntimeError("hipMemcpyDtoDAsync failed")

            for _ in range(3):
                runtime_copy()
            a, b = ep.HipEvent(timing=True), ep.HipEvent(timing=True)
            a.record(stream)
            for _ in range(reps):
                runtime_copy()
            b.record(stream)
            stream.synchronize()
            out["hipMemcpyDtoD_GBps"] = round(2 * nbytes / (a.elapsed_ms(b) * 1e-3 / reps) / 1e9, 1)
        del src, dst
    if far:
        # the two mixes once more over 2400 MiB: a source of 300 MiB that cannot stay in the 256 MiB memory-side cache
        # between launches and eight regions 300 MiB apart -- what a world of several ranks on one device looks like
        nbytes = 2400 << 20
        src = torch.zeros((nbytes,), dtype=torch.uint8, device=dev)
        dst = torch.zeros((nbytes,), dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        for name, pattern in (("fan_out_1r8w_far", ep.PROBE_FAN_OUT), ("fan_in_8r1w_far", ep.PROBE_FAN_IN)):
            for _ in range(3):
                ep.check(ep.memory_probe(pattern, src, dst, nbytes, stream), "memory probe")
            a, b = ep.HipEvent(timing=True), ep.HipEvent(timing=True)
            a.record(stream)
            for _ in range(reps):
                ep.check(ep.memory_probe(pattern, src, dst, nbytes, stream), "memory probe")
            b.record(stream)
            stream.synchronize()
            out[name + "_GBps"] = round((nbytes + nbytes // 8) / (a.elapsed_ms(b) * 1e-3 / reps) / 1e9, 1)
        del src, dst
    if narrow is not None:
        # the quantised reduce's mix with its addresses: rows of 2048 (4096) one-byte payloads, eight (six) per output
        # row of twice the width, at unrelated positions; the source sized like the workload's rows
        name, pattern, row_bytes, k = narrow
        # as many rows as the probe's row arithmetic allows (fewer than 2^17), so that the source exceeds the memory-side cache
        nbytes = min(600 << 20, ((1 << 17) - 1) * row_bytes) // (row_bytes * k) * (row_bytes * k)
        src = torch.zeros((nbytes,), dtype=torch.uint8, device=dev)
        dst = torch.zeros((nbytes * 2 // k,), dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        for _ in range(3):
            ep.check(ep.memory_probe(pattern, src, dst, nbytes, stream), "memory probe")
        a, b = ep.HipEvent(timing=True), ep.HipEvent(timing=True)
        a.record(stream)
        for _ in range(reps):
            ep.check(ep.memory_probe(pattern, src, dst, nbytes, stream), "memory probe")
        b.record(stream)
        stream.synchronize()
        out[name + "_GBps"] = round((nbytes + nbytes * 2 // k) / (a.elapsed_ms(b) * 1e-3 / reps) / 1e9, 1)
        del src, dst
    return out


def cpu_baseline(w, x, ids, weights, kept_rows):
    """The CPU oracle (a scalar C port of the reference path) on one host core, full layer, best of 3."""
    import numpy as np

    from oracle import ep as O
    from tilexr_amd import workloads

    xb = x.view(__import__("torch").int16).numpy().view(np.uint16)
    quant = {"none": O.Q_NONE, "int8": O.Q_TOKEN_INT8, "fp8_block128": O.Q_FP8_BLOCK128}[w.quant]
    case = O.Case(1, w.bs, w.h, w.top_k, w.experts, dtype=O.DT_BF16, quant_mode=quant, capacity=w.capacity)
    idn = ids.numpy()
    wn = weights.numpy()

    def layer():
        t0 = time.perf_counter()
        d = O.mem_dispatch(case, 0, xb[None], idn[None])
        t1 = time.perf_counter()
        O.mem_combine(O.Case(1, w.bs, w.h, w.top_k, w.experts, dtype=O.DT_BF16), 0, d["expand_x"][None]
                      if quant else d["expand_x"].view(np.uint16)[None], d["assist"][None], d["send_counts"][None],
                      expert_scales=wn, in_quant=quant if quant else 0,
                      in_scales=d["dyn_scales"] if quant else None)
        t2 = time.perf_counter()
        return (t2 - t0, t1 - t0, t2 - t1)

    best = min(layer() for _ in range(3))
    db, cb = workloads.algorithmic_bytes(w, kept_rows, inverse_index=True)
    # All cores: the port is scalar, so the host's cores are used the way a host would use them for this path -- one
    # independent layer per thread (the calls into the C library release the interpreter lock).
    from concurrent.futures import ThreadPoolExecutor
    threads = max(1, min(16, os.cpu_count() or 1))
    many = None
    with ThreadPoolExecutor(threads) as pool:
        for _ in range(2):
            t0 = time.perf_counter()
            list(pool.map(lambda _i: layer(), range(threads)))
            dt = time.perf_counter() - t0
            many = dt if many is None else min(many, dt)
    return {
        "value": round((db + cb) / best[0] / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
        "us_per_layer": round(best[0] * 1e6, 1), "dispatch_us": round(best[1] * 1e6, 1),
        "combine_us": round(best[2] * 1e6, 1), "host_cores_available": os.cpu_count(),
        "sample": f"full {w.name} layer ({w.bs} tokens), oracle C port, single thread, best of 3",
        "all_cores": {"value": round(threads * (db + cb) / many / 1e9, 3), "unit": "GB/s", "cores": threads,
                      "us_per_layer": round(many / threads * 1e6, 1),
                      "sample": f"{threads} independent {w.name} layers at once, one per thread, best of 2"},
    }


def moonep_cpu_baseline(world, s, k, h, experts):
    """The CPU oracle of the plan-driven stages on one host core, at a sample of the workload's tokens."""
    import numpy as np
    import torch

    from oracle import moonep as M
    from tilexr_amd import workloads

    sample = max(64, min(s, 4096 // world))
    g = torch.Generator().manual_seed(99)
    ids = torch.topk(torch.rand(world, sample, experts, generator=g), k, dim=2).indices.to(torch.int32)
    plan = workloads.moonep_home_plan(ids, experts)
    sh = M.Shape(world, sample, k, h, plan["nvs"])
    dst = plan["dst"].numpy()
    hidden = np.random.default_rng(1).integers(0, 0x4000, size=(world, sample, h), dtype=np.uint16)
    weights = np.ones((world, sample * k), np.float32)
    def layer():
        t0 = time.perf_counter()
        out, wout, _, dup = M.dispatch_world(sh, dst, hidden, weights, flags=M.FLAG_BUILD_DEDUP)
        t1 = time.perf_counter()
        M.combine_world(sh, M.build_dst_local(sh, dst), dup, out, wout)
        t2 = time.perf_counter()
        return (t2 - t0, t1 - t0, t2 - t1)

    best = min(layer() for _ in range(3))
    db, cb = workloads.moonep_algorithmic_bytes(sample, k, h)
    from concurrent.futures import ThreadPoolExecutor
    threads = max(1, min(16, os.cpu_count() or 1))
    many = None
    with ThreadPoolExecutor(threads) as pool:       # one independent layer per thread; the C calls release the lock
        for _ in range(2):
            t0 = time.perf_counter()
            list(pool.map(lambda _i: layer(), range(threads)))
            dt = time.perf_counter() - t0
            many = dt if many is None else min(many, dt)
    return {
        "all_cores": {"value": round(threads * world * (db + cb) / many / 1e9, 3), "unit": "GB/s", "cores": threads,
                      "us_per_layer": round(many / threads * 1e6, 1),
                      "sample": f"{threads} independent layers of the same sample at once, one per thread, best of 2"},
        "value": round(world * (db + cb) / best[0] / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
        "us_per_layer": round(best[0] * 1e6, 1), "dispatch_us": round(best[1] * 1e6, 1),
        "combine_us": round(best[2] * 1e6, 1), "host_cores_available": os.cpu_count(),
        "sample": f"{sample} of {s} tokens per rank, {world} rank(s), oracle C port, single thread, best of 3",
    }


def main_moonep(args):
    """Plan-driven stages: a step is one Dispatch (every rank of the world) followed by one Combine, identity expert."""
    import numpy as np
    import torch

    from tilexr_amd import ep, moonep as mp, workloads

    w = workloads.MOONEP_CONFIGS[args.workload]
    world = args.moon_ranks
    s, k, h = w.bs, w.top_k, w.h
    experts = w.experts if world > 1 else max(k, w.experts // w.ranks)    # one rank's share keeps its own experts
    g = torch.Generator().manual_seed(w.seed)
    ids = torch.topk(torch.rand(world, s, experts, generator=g), k, dim=2).indices.to(torch.int32)
    plan = workloads.moonep_home_plan(ids, experts)
    nvs = plan["nvs"]
    dst = plan["dst"]
    dst_local = workloads.moonep_dst_local(dst, nvs)
    torch.cuda.set_device(0)
    dev = "cuda:0"
    comms = [ep.Comm(world, r) for r in range(world)]
    streams = [torch.cuda.Stream() for _ in range(world)]
    ranks = []
    for r in range(world):
        t = dict(dst=dst[r].to(dev), dl=dst_local[r].to(dev),
                 groups=torch.zeros((nvs, 3), dtype=torch.int32, device=dev), loffs=torch.zeros(nvs, dtype=torch.int32, device=dev),
                 counts=torch.zeros(2, dtype=torch.int32, device=dev), status=torch.zeros(8, dtype=torch.int32, device=dev),
                 x=torch.randn(s, h, generator=g).to(torch.bfloat16).to(dev), wsk=torch.rand(s, k, generator=g).to(dev),
                 rows=torch.empty((nvs, h), dtype=torch.bfloat16, device=dev), wnv=torch.empty(nvs, dtype=torch.float32, device=dev),
                 y=torch.empty((s, h), dtype=torch.bfloat16, device=dev), wy=torch.empty((s, k), dtype=torch.float32, device=dev))
        t["plan"] = mp.plan(s * k, world, experts, 1, nvs, k, t["dst"], t["groups"], t["loffs"], t["counts"], t["status"])
        t["d_args"] = (mp.tensor(t["x"], mp.DT_BF16, (s, h)), mp.tensor(t["rows"], mp.DT_BF16, (nvs, h)))
        t["d_w"] = dict(weights_sk=mp.tensor(t["wsk"], mp.DT_FP32, (s, k)), weights_nvs=mp.tensor(t["wnv"], mp.DT_FP32, (nvs,)))
        t["c_args"] = (mp.tensor(t["rows"], mp.DT_BF16, (nvs, h)), mp.tensor(t["y"], mp.DT_BF16, (s, h)))
        t["c_w"] = dict(weights_nvs=mp.tensor(t["wnv"], mp.DT_FP32, (nvs,)), weights_sk=mp.tensor(t["wy"], mp.DT_FP32, (s, k)))
        ranks.append(t)

    def dispatch(flags):
        for r, t in enumerate(ranks):
            ep.check(mp.dispatch_v1(comms[r], t["plan"], *t["d_args"], streams[r], flags=flags, **t["d_w"]), "dispatch")

    def combine():
        for r, t in enumerate(ranks):
            ep.check(mp.combine_v1(comms[r], t["plan"], t["dl"], *t["c_args"], streams[r], **t["c_w"]), "combine")

    flags = 0 if args.moon_saved else mp.FLAG_BUILD_DEDUP
    if args.moon_cached_row_bytes is not None:
        mp.set_cached_row_bytes(args.moon_cached_row_bytes)

    def step():
        dispatch(flags)
        combine()

    if args.calibrate_copy:
        src = torch.zeros((64 << 20,), dtype=torch.int32, device=dev)
        dst_copy = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1, out=dst_copy)      # one elementwise kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst_copy
    torch.cuda.synchronize()
    dispatch(mp.FLAG_BUILD_DEDUP)       # the saved plan of a --moon-saved run
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    for t in ranks:
        assert int(t["status"][0].item()) == 0
    # identity expert: every token comes back as the sum of its routes, duplicate groups rounded first
    r0 = ranks[0]
    peer = torch.from_numpy(np.where(dst[0].numpy() >= 0, dst[0].numpy(), -dst[0].numpy().astype(np.int64) - 1) // nvs).reshape(s, k)
    per_rank = torch.zeros(s, world, dtype=torch.int64).scatter_add_(1, peer, torch.ones_like(peer)).to(dev)
    want = torch.zeros((s, h), dtype=torch.float32, device=dev)
    for q in range(world):
        want += (r0["x"].float() * per_rank[:, q:q + 1].float()).to(torch.bfloat16).float()
    if not torch.equal(want.to(torch.bfloat16).view(torch.int16), r0["y"].view(torch.int16)):
        print("combine(dispatch(x)) differs from the closed form", file=sys.stderr)
        sys.exit(1)

    dispatch_bytes, combine_bytes = workloads.moonep_algorithmic_bytes(s, k, h)
    use_events = not args.no_kernel_events
    stride = args.event_stride if args.event_stride > 0 else max(1, args.steps // 16)
    # the events are set on rank 0's communicator and bracket the launch for the whole world
    elapsed, event_pass_s, pairs = run_timed_passes(torch, ep, step, args.steps, comms[0], use_events, stride)
    names = {"scatter": ep.last_kernel_name(comms[0], ep.K_SCATTER), "reduce": ep.last_kernel_name(comms[0], ep.K_REDUCE)}

    ev = [ep.HipEvent(timing=True) for _ in range(3)]
    if world == 1:
        ev[0].record(streams[0])
        dispatch(flags)
        ev[1].record(streams[0])
        combine()
        ev[2].record(streams[0])
        torch.cuda.synchronize()
        split = (round(ev[0].elapsed_ms(ev[1]) * 1e3, 2), round(ev[1].elapsed_ms(ev[2]) * 1e3, 2))
    else:
        split = (None, None)

    # one rank once more with the token rows of every step in a different tensor, enough of them that none is still in
    # the 256 MiB memory-side cache when its turn comes again.  Not part of `value`.
    rotating = None
    if world == 1 and not args.no_rotate_leg:
        copies = max(2, -(-(384 << 20) // (s * h * 2)))
        xs = [r0["x"]] + [r0["x"].clone() for _ in range(copies - 1)]
        descs = [mp.tensor(x, mp.DT_BF16, (s, h)) for x in xs]
        rot_steps = max(copies, args.steps // 2)

        def rot_step(i):
            ep.check(mp.dispatch_v1(comms[0], r0["plan"], descs[i % copies], r0["d_args"][1], streams[0], flags=flags,
                                    **r0["d_w"]), "dispatch")
            combine()

        for i in range(copies):
            rot_step(i)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(rot_steps):
            rot_step(i)
        torch.cuda.synchronize()
        rot_us = (time.perf_counter() - t1) / rot_steps * 1e6
        rotating = {"input_tensors": copies, "steps": rot_steps, "us_per_layer": round(rot_us, 2),
                    "GBps": round((dispatch_bytes + combine_bytes) / (rot_us * 1e-6) / 1e9, 1)}
        del xs, descs

    ms_per_step = elapsed / args.steps * 1e3
    total_bytes = world * (dispatch_bytes + combine_bytes)
    gbps = total_bytes / (ms_per_step * 1e-3) / 1e9
    kernels, roofline = {}, None
    if use_events:
        # one launch of the scatter / reduce kernel covers every rank of the world
        kernels = kernel_event_stats(pairs, (("scatter", world * dispatch_bytes), ("reduce", world * combine_bytes)))
        dom = "scatter" if kernels["scatter"]["avg_us"] >= kernels["reduce"]["avg_us"] else "reduce"
        trace_file = f"profiles/moonep_dispatch_combine_{w.name}_kernel_stats.txt"
        section = f"ranks={world} {'saved' if args.moon_saved else 'built'} plan"
        roofline = roofline_of(kernels, dom, names[dom], measured_traffic(f"{w.name}_r{world}", dom),
                               f"profiles/hbm_traffic_{w.name}_r{world}.txt", trace_avg_us(trace_file, section, names[dom]),
                               trace_file)
        roofline["event_pass_us_per_layer"] = round(event_pass_s / args.steps * 1e6, 2)
    ceilings = None
    if not args.no_ceilings:
        ceilings = measured_ceilings(ep, torch, streams[0], dev, far=world > 1)
        if roofline is not None:
            suffix = "_far_GBps" if world > 1 else "_GBps"
            mix = ceilings["fan_out_1r8w" + suffix] if dom == "scatter" else ceilings["fan_in_8r1w" + suffix]
            roofline["frac_of_measured_mix"] = round(roofline["achieved"] / mix, 4)
            if dom == "reduce":
                roofline["frac_of_measured_row_gather"] = round(roofline["achieved"] / ceilings["gather_rows_8r1w_GBps"], 4)
    result = {
        "metric": "dispatch+combine effective HBM bandwidth per MoE layer (algorithmic bytes / time) on 1 MI355X",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "us_per_layer": round(ms_per_step * 1e3, 2),
        "us_per_layer_per_rank": round(ms_per_step * 1e3 / world, 2),
        "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{w.name}: plan-driven Dispatch + Combine, {world} logical rank(s) x {s} tokens x {h} bf16, "
                               f"top-{k} of {experts} experts, home plan, fp32 route weights",
                   "logical_ranks": world, "tokens_per_rank": s, "hidden": h, "top_k": k, "experts": experts, "nvs": nvs,
                   "duplicate_routes": int((dst < 0).sum()), "routes": int(dst.numel()), "rotating_inputs": rotating,
                   "dispatch": "saved duplicate plan" if args.moon_saved else "builds the duplicate plan",
                   "dispatch_bytes_per_rank": dispatch_bytes, "combine_bytes_per_rank": combine_bytes,
                   "dispatch_us": split[0], "combine_us": split[1], "seed": w.seed,
                   "dst_sha256": __import__("hashlib").sha256(dst.numpy().tobytes()).hexdigest()[:16]},
        "roofline": roofline, "kernels": kernels, "ceilings": ceilings,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = moonep_cpu_baseline(world, s, k, h, experts)
    torch.cuda.synchronize()
    for c in comms:
        c.destroy()
    print(json.dumps(result))


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one device's share of the dispatch/combine path: run it with --gpus 1 "
              "(no collective or second GPU is part of this build)", file=sys.stderr)
        sys.exit(2)
    if args.workload.startswith("M"):
        return main_moonep(args)

    import torch

    from tilexr_amd import ep, workloads

    w = workloads.CONFIGS[args.workload]
    x = workloads.make_x(w)
    ids, weights = workloads.make_routing(w)
    bs, h, K, E = w.bs, w.h, w.top_k, w.experts
    quant = {"none": ep.Q_NONE, "int8": ep.Q_TOKEN_INT8, "fp8_block128": ep.Q_FP8_BLOCK128}[w.quant]

    torch.cuda.set_device(0)
    dev = "cuda:0"
    stream = torch.cuda.Stream()
    comm = ep.Comm(1, 0)
    rows_max = bs * K
    row_bytes = h * 2 if quant == ep.Q_NONE else h
    d_x, d_ids, d_w = x.to(dev), ids.to(dev), weights.to(dev)
    expand_x = torch.empty((rows_max, row_bytes), dtype=torch.uint8, device=dev)
    assist = torch.empty((rows_max, 4), dtype=torch.int32, device=dev)
    token_nums = torch.empty((E,), dtype=torch.int64, device=dev)
    send_counts = torch.empty((E,), dtype=torch.int32, device=dev)
    row_map = torch.empty((bs, K), dtype=torch.int32, device=dev)
    y = torch.empty((bs, h), dtype=torch.bfloat16, device=dev)
    scales = None
    if quant == ep.Q_TOKEN_INT8:
        scales = torch.empty((rows_max,), dtype=torch.float32, device=dev)
    elif quant == ep.Q_FP8_BLOCK128:
        scales = torch.empty((rows_max, (h + 127) // 128), dtype=torch.float32, device=dev)

    side = torch.cuda.Stream()
    tiles = (rows_max + args.tile_rows - 1) // args.tile_rows
    flags = torch.zeros((tiles,), dtype=torch.int64, device=dev)
    status = torch.zeros((1,), dtype=torch.int32, device=dev)
    meta_ready, combined = ep.HipEvent(), ep.HipEvent()

    def step_plain(d_x=d_x, expand_x=expand_x, y=y):
        st, _ = ep.dispatch_memory_ex(d_x, d_ids, comm, bs, h, K, E, expand_x, assist, token_nums, send_counts,
                                      ep.DT_BF16, stream, quant_mode=quant, expert_capacity=w.capacity,
                                      dynamic_scales=scales, row_index_map=row_map)
        ep.check(st, "dispatch")
        ep.check(ep.combine_memory_ex(expand_x, assist, send_counts, comm, bs, h, K, E, y, ep.DT_BF16, stream,
                                      expert_out_quant_mode=quant, expert_out_scales=scales, expert_scales=d_w,
                                      row_index_map=row_map), "combine")

    def step_flags_serial(d_x=d_x, expand_x=expand_x, y=y):
        # dispatch publishes a readiness word per tile of rows, combine waits for the tiles of every row it reads;
        # one stream, so the waits find every tile published
        st, epoch = ep.dispatch_memory_ex(d_x, d_ids, comm, bs, h, K, E, expand_x, assist, token_nums, send_counts,
                                          ep.DT_BF16, stream, quant_mode=quant, expert_capacity=w.capacity,
                                          dynamic_scales=scales, row_index_map=row_map, tile_flags=flags,
                                          tile_rows=args.tile_rows)
        ep.check(st, "dispatch")
        ep.check(ep.combine_memory_ex(expand_x, assist, send_counts, comm, bs, h, K, E, y, ep.DT_BF16, stream,
                                      expert_out_quant_mode=quant, expert_out_scales=scales, expert_scales=d_w,
                                      row_index_map=row_map, tile_flags=flags, tile_rows=args.tile_rows,
                                      flag_epoch=epoch, device_status=status), "combine")

    def step_overlapped():
        # dispatch on `stream` publishes tiles; combine on `side` starts once the metadata is enqueued and reduces
        # tokens as their tiles land; the next dispatch waits until this combine has read the rows
        st, epoch = ep.dispatch_memory_ex(d_x, d_ids, comm, bs, h, K, E, expand_x, assist, token_nums, send_counts,
                                          ep.DT_BF16, stream, quant_mode=quant, expert_capacity=w.capacity,
                                          dynamic_scales=scales, row_index_map=row_map, tile_flags=flags,
                                          tile_rows=args.tile_rows, meta_ready_event=meta_ready.value)
        ep.check(st, "dispatch")
        meta_ready.wait_on(side)
        ep.check(ep.combine_memory_ex(expand_x, assist, send_counts, comm, bs, h, K, E, y, ep.DT_BF16, side,
                                      expert_out_quant_mode=quant, expert_out_scales=scales, expert_scales=d_w,
                                      row_index_map=row_map, tile_flags=flags, tile_rows=args.tile_rows,
                                      flag_epoch=epoch, device_status=status), "combine")
        combined.record(side)
        combined.wait_on(stream)

    steps_by_schedule = {"flags-serial": step_flags_serial, "flags-overlapped": step_overlapped, "plain": step_plain}
    schedule = "flags-overlapped" if args.overlap else args.schedule
    calibration = None
    # decode-sized calls (at most 2048 routes) take the library's single-launch dispatch: two launches per layer with or
    # without flags, and without them nothing waits for written-through rows before a workgroup may leave (16 against
    # 20 us per layer), which is what counts at this size
    small = bs * K <= 2048
    if schedule == "auto" and small:
        schedule = "plain"
    if schedule == "auto":
        # the faster of the two schedules that publish and consume flags, by a short calibration outside the timed region
        torch.cuda.synchronize()
        calibration = {}
        for name in ("flags-serial", "flags-overlapped"):
            for _ in range(5):
                steps_by_schedule[name]()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(20):
                steps_by_schedule[name]()
            torch.cuda.synchronize()
            calibration[name] = round((time.perf_counter() - t0) / 20 * 1e6, 2)
        schedule = min(calibration, key=calibration.get)
    step = steps_by_schedule[schedule]
    uses_flags = schedule != "plain"

    if args.calibrate_copy:
        src = torch.zeros((64 << 20,), dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1, out=dst)      # one elementwise kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    torch.cuda.synchronize()        # torch's fills ran on its default stream, the library runs on `stream`
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    kept_rows = int(send_counts[-1].item())
    dispatch_bytes, combine_bytes = workloads.algorithmic_bytes(w, kept_rows, inverse_index=True)

    use_events = not args.no_kernel_events
    stride = args.event_stride if args.event_stride > 0 else max(1, args.steps // 16)
    elapsed, event_pass_s, pairs = run_timed_passes(torch, ep, step, args.steps, comm, use_events, stride)
    kernel_names = {"scatter": ep.last_kernel_name(comm, ep.K_SCATTER), "reduce": ep.last_kernel_name(comm, ep.K_REDUCE)}

    if status.item() != 0:
        print("a tile-flag wait expired during the run", file=sys.stderr)
        sys.exit(1)
    # the identity expert makes the layer checkable on the device: every kept row is its token's row, so y is the
    # weighted sum of that row over the token's kept routes
    if quant == ep.Q_NONE:
        kept_w = torch.where(row_map >= 0, d_w, torch.zeros_like(d_w)).sum(1, keepdim=True)
        ref = d_x.float() * kept_w
        err = (y.float() - ref).abs().max().item()
        if not err <= 2e-2 * ref.abs().max().item():
            print(f"combine(dispatch(x)) is off by {err}", file=sys.stderr)
            sys.exit(1)
        del ref, kept_w

    # split of one step into its two calls, run back to back on one stream (outside the timed region), with the timed
    # schedule's flag settings: median of 20 event-bracketed layers (a single layer after an idle queue reads high)
    splits = []
    for _ in range(20):
        d_ev = [ep.HipEvent(timing=True) for _ in range(3)]
        d_ev[0].record(stream)
        st, epoch = ep.dispatch_memory_ex(d_x, d_ids, comm, bs, h, K, E, expand_x, assist, token_nums, send_counts, ep.DT_BF16,
                                          stream, quant_mode=quant, expert_capacity=w.capacity, dynamic_scales=scales,
                                          row_index_map=row_map, tile_flags=flags if uses_flags else None,
                                          tile_rows=args.tile_rows if uses_flags else 0)
        d_ev[1].record(stream)
        ep.combine_memory_ex(expand_x, assist, send_counts, comm, bs, h, K, E, y, ep.DT_BF16, stream,
                             expert_out_quant_mode=quant, expert_out_scales=scales, expert_scales=d_w, row_index_map=row_map,
                             tile_flags=flags if uses_flags else None, tile_rows=args.tile_rows if uses_flags else 0,
                             flag_epoch=epoch, device_status=status if uses_flags else None)
        d_ev[2].record(stream)
        splits.append(d_ev)
    torch.cuda.synchronize()
    dispatch_us = sorted(e[0].elapsed_ms(e[1]) * 1e3 for e in splits)[len(splits) // 2]
    combine_us = sorted(e[1].elapsed_ms(e[2]) * 1e3 for e in splits)[len(splits) // 2]

    # the schedules that were not timed, each on its own after the main region so that all three are on record; they
    # are not part of `value`
    other = None
    if not args.no_overlap_leg:
        other = []
        for name, other_step in steps_by_schedule.items():
            if name == schedule:
                continue
            other_steps = max(10, args.steps // 2)
            for _ in range(5):
                other_step()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(other_steps):
                other_step()
            torch.cuda.synchronize()
            other_us = (time.perf_counter() - t1) / other_steps * 1e6
            if status.item() != 0:
                print("a tile-flag wait expired during the run", file=sys.stderr)
                sys.exit(1)
            other.append({"schedule": SCHEDULES[name], "tile_rows": args.tile_rows if name != "plain" else None,
                          "steps": other_steps, "us_per_layer": round(other_us, 2),
                          "GBps": round((dispatch_bytes + combine_bytes) / (other_us * 1e-6) / 1e9, 1)})

    # decode-sized workloads: 16 layers captured once in a HIP graph and replayed, against the same layers launched one
    # call at a time.  Not part of `value`.
    graph_replay = None
    if small and not args.no_graph_leg:
        layers = 16
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(layers):
                step_plain()
        torch.cuda.synchronize()
        for _ in range(5):
            graph.replay()
        torch.cuda.synchronize()
        replays = max(10, args.steps // 4)
        t1 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        torch.cuda.synchronize()
        replay_us = (time.perf_counter() - t1) / replays / layers * 1e6
        t1 = time.perf_counter()
        for _ in range(replays * layers):
            step_plain()
        torch.cuda.synchronize()
        eager_us = (time.perf_counter() - t1) / (replays * layers) * 1e6
        graph_replay = {"layers_per_graph": layers, "replays": replays, "us_per_layer": round(replay_us, 2),
                        "eager_us_per_layer": round(eager_us, 2)}
        del graph

    # What the flags are for: an expert stage between dispatch and combine that is slower than memory and publishes
    # tiles as it finishes them.  A stand-in producer of the library (a few workgroups copy expandX to expertOut tile by
    # tile at a set pace) runs (a) followed by an ordinary combine on the same stream, (b) beside a combine on a second
    # stream that waits on the producer's flags and reduces every token as soon as its tiles are there.  Not part of
    # `value`.
    expert_stage = None
    if not args.no_stage_leg:
        expert_out = torch.empty_like(expand_x)
        stage_tile_rows = args.stage_tile_rows
        stage_flags = torch.zeros(((rows_max + stage_tile_rows - 1) // stage_tile_rows,), dtype=torch.int64, device=dev)
        stage_done, combine_done = ep.HipEvent(), ep.HipEvent()
        st, _ = ep.dispatch_memory_ex(d_x, d_ids, comm, bs, h, K, E, expand_x, assist, token_nums, send_counts, ep.DT_BF16,
                                      stream, quant_mode=quant, expert_capacity=w.capacity, dynamic_scales=scales,
                                      row_index_map=row_map)
        ep.check(st, "dispatch")
        torch.cuda.synchronize()
        epoch_counter = [1 << 20]

        stagger = [0]

        def producer():
            epoch_counter[0] += 1
            ep.check(ep.tile_producer_probe(expand_x, expert_out, kept_rows, row_bytes, stage_flags, stage_tile_rows,
                                            epoch_counter[0], args.stage_workgroups, args.stage_tile_ns, stream,
                                            stagger_ns=stagger[0]), "producer")
            return epoch_counter[0]

        def stage_alone():
            producer()

        def stage_then_combine():
            producer()
            ep.check(ep.combine_memory_ex(expert_out, assist, send_counts, comm, bs, h, K, E, y, ep.DT_BF16, stream,
                                          expert_out_quant_mode=quant, expert_out_scales=scales, expert_scales=d_w,
                                          row_index_map=row_map), "combine")

        def stage_beside_combine():
            # the producer is enqueued first; the next producer must not overwrite rows this combine still reads
            epoch = producer()
            ep.check(ep.combine_memory_ex(expert_out, assist, send_counts, comm, bs, h, K, E, y, ep.DT_BF16, side,
                                          expert_out_quant_mode=quant, expert_out_scales=scales, expert_scales=d_w,
                                          row_index_map=row_map, tile_flags=stage_flags, tile_rows=stage_tile_rows,
                                          flag_epoch=epoch, device_status=status), "combine")
            combine_done.record(side)
            combine_done.wait_on(stream)

        def timed(fn, n):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(n):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t1) / n * 1e6

        n_stage = max(10, args.steps // 4)

        def three_ways():
            alone = timed(stage_alone, n_stage)
            serial = timed(stage_then_combine, n_stage)
            y_serial = y.clone()
            beside = timed(stage_beside_combine, n_stage)
            if status.item() != 0:
                print("a tile-flag wait expired during the expert-stage leg", file=sys.stderr)
                sys.exit(1)
            if not torch.equal(y.view(torch.int16), y_serial.view(torch.int16)):
                print("combine beside the producer differs from combine after it", file=sys.stderr)
                sys.exit(1)
            return alone, serial, beside

        alone_us, serial_us, beside_us = three_ways()
        # the same producer with workgroups that do not move in step: tiles complete at a steady rate instead of
        # `workgroups` at a time, so the combine is not left with a last wave of tiles to follow
        stagger[0] = args.stage_tile_ns
        st_alone_us, st_serial_us, st_beside_us = three_ways()
        stagger[0] = 0
        expert_stage = {"producer": f"{args.stage_workgroups} workgroups copy expandX to expertOut tile by tile, at least "
                                    f"{args.stage_tile_ns} ns per tile, publish each tile (release at agent scope + flag word)",
                        "tile_rows": stage_tile_rows, "steps": n_stage, "producer_alone_us": round(alone_us, 2),
                        "combine_after_producer_us": round(serial_us, 2), "combine_beside_producer_us": round(beside_us, 2),
                        "saved_us": round(serial_us - beside_us, 2),
                        "staggered_workgroups": {"producer_alone_us": round(st_alone_us, 2),
                                                 "combine_after_producer_us": round(st_serial_us, 2),
                                                 "combine_beside_producer_us": round(st_beside_us, 2),
                                                 "saved_us": round(st_serial_us - st_beside_us, 2)},
                        "outputs_identical": True}
        del expert_out

    # the serial schedule once more with the token rows of every step in a different tensor, enough of them that none
    # is still in the 256 MiB memory-side cache when its turn comes again: what a caller sees whose x was produced long
    # before the dispatch.  Not part of `value`.
    rotating = None
    if not args.no_rotate_leg:
        copies = max(2, -(-(384 << 20) // (bs * h * 2)))
        xs = [d_x] + [d_x.clone() for _ in range(copies - 1)]
        rot_steps = max(copies, args.steps // 2)
        rot_step = step_plain if schedule == "plain" else step_flags_serial
        for i in range(copies):
            rot_step(xs[i])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(rot_steps):
            rot_step(xs[i % copies])
        torch.cuda.synchronize()
        rot_us = (time.perf_counter() - t1) / rot_steps * 1e6
        rotating = {"schedule": SCHEDULES["plain" if schedule == "plain" else "flags-serial"], "input_tensors": copies, "steps": rot_steps, "us_per_layer": round(rot_us, 2),
                    "GBps": round((dispatch_bytes + combine_bytes) / (rot_us * 1e-6) / 1e9, 1)}
        # and with the expanded rows and the output rotating too (sets of x, expandX, y of more than 1 GiB together): a
        # step that overwrites the rows the previous step has just read finds part of them in the memory-side cache,
        # a model whose layers have their own buffers, or whose expert stage runs between the two calls, does not
        set_bytes = bs * h * 2 * 2 + expand_x.numel() * expand_x.element_size()
        sets = max(2, -(-(1200 << 20) // set_bytes))
        bufs = [(xs[i % copies], torch.empty_like(expand_x), torch.empty_like(y)) for i in range(sets)]
        for b in bufs:
            rot_step(*b)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(rot_steps):
            rot_step(*bufs[i % sets])
        torch.cuda.synchronize()
        all_us = (time.perf_counter() - t1) / rot_steps * 1e6
        rotating["all_buffers"] = {"sets": sets, "MiB_per_set": set_bytes >> 20, "us_per_layer": round(all_us, 2),
                                   "GBps": round((dispatch_bytes + combine_bytes) / (all_us * 1e-6) / 1e9, 1)}
        del xs, bufs

    # the same layer through the reference's own entry points (TileXRMoeEpDispatchMemory / TileXRMoeEpCombineMemoryV2),
    # which carry no row map from dispatch to combine: combine rebuilds it from the assist tuples first.  Plain
    # payloads only (the quantised workloads need the extended calls).  Not part of `value`.
    reference_abi = None
    if quant == ep.Q_NONE and w.capacity == 0 and not args.no_rotate_leg:
        ref_steps = max(10, args.steps // 2)
        ref_x = expand_x.view(torch.bfloat16)

        def step_reference():
            ep.check(ep.dispatch_memory(d_x, d_ids, comm, bs, h, K, E, ref_x, token_nums, send_counts, assist, ep.DT_BF16,
                                        stream), "dispatch")
            ep.check(ep.combine_memory_v2(ref_x, assist, send_counts, comm, bs, h, K, E, y, ep.DT_BF16, stream,
                                          expert_scales=d_w), "combine")

        for _ in range(5):
            step_reference()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(ref_steps):
            step_reference()
        torch.cuda.synchronize()
        ref_us = (time.perf_counter() - t1) / ref_steps * 1e6
        reference_abi = {"entry_points": "TileXRMoeEpDispatchMemory + TileXRMoeEpCombineMemoryV2", "steps": ref_steps,
                         "us_per_layer": round(ref_us, 2),
                         "GBps": round((dispatch_bytes + combine_bytes + kept_rows * 16 - bs * K * 4) / (ref_us * 1e-6) / 1e9, 1)}

    ms_per_step = elapsed / args.steps * 1e3
    total_bytes = dispatch_bytes + combine_bytes
    gbps = total_bytes / (ms_per_step * 1e-3) / 1e9

    roofline = None
    kernels = {}
    if use_events:
        kernels = kernel_event_stats(pairs, (("scatter", dispatch_bytes), ("reduce", combine_bytes)))
        dom = "scatter" if kernels["scatter"]["avg_us"] >= kernels["reduce"]["avg_us"] else "reduce"
        trace_file = f"profiles/ep_dispatch_combine_{w.name}_kernel_stats.txt"
        roofline = roofline_of(kernels, dom, kernel_names[dom], measured_traffic(w.name, dom), f"profiles/hbm_traffic_{w.name}.txt",
                               trace_avg_us(trace_file, schedule, kernel_names[dom]), trace_file)
        # what the whole dispatch fetches and writes by the same counters: the scatter plus the routing launch, whose
        # extra workgroups read the token rows once so that the scatter finds them in the memory-side cache
        side_traffic = {k: measured_traffic(w.name, k) for k in ("scatter", "routing")}
        if all(side_traffic.values()):
            total = sum(side_traffic.values())
            roofline["dispatch_traffic"] = dict(side_traffic, total=total, over_algorithmic=round(total / dispatch_bytes, 4))
        roofline["event_pass_us_per_layer"] = round(event_pass_s / args.steps * 1e6, 2)

    ceilings = None
    if not args.no_ceilings:
        narrow = {("int8", 4096, 6): ("gather_rows_4k_6r_GBps"[:-5], ep.PROBE_GATHER_ROWS_4K_X6, 4096, 6),
                  ("fp8_block128", 2048, 8): ("gather_rows_2k_8r_GBps"[:-5], ep.PROBE_GATHER_ROWS_2K_X8, 2048, 8)}.get((w.quant, h, K))
        ceilings = measured_ceilings(ep, torch, stream, dev, narrow=narrow)
        if roofline is not None:
            mix = ceilings["fan_out_1r8w_GBps"] if dom == "scatter" else ceilings["fan_in_8r1w_GBps"]
            roofline["frac_of_measured_mix"] = round(roofline["achieved"] / mix, 4)
            if dom == "reduce":
                gather = ceilings[narrow[0] + "_GBps"] if narrow is not None else ceilings["gather_rows_8r1w_GBps"]
                roofline["frac_of_measured_row_gather"] = round(roofline["achieved"] / gather, 4)

    # decode-sized calls move so little that a kernel's time is its chain of dependent trips to memory, not its bytes:
    # how many loads must return, one after the other, before the kernel's stores can go out
    round_trips = None
    if small:
        round_trips = {
            "dispatch": {"kernel": kernel_names["scatter"],
                         "dependent_loads_before_store": {"ep_dispatch_small_route_kernel": 1, "ep_dispatch_small_kernel": 2}.get(kernel_names["scatter"]),
                         "chain": "expert ids and the token row are requested together; the row is stored when both are back"
                                  if kernel_names["scatter"] == "ep_dispatch_small_route_kernel" else
                                  "expert ids, then (per-expert counts known) the token rows, then the stores"},
            "combine": {"kernel": kernel_names["reduce"], "dependent_loads_before_store": 2,
                        "chain": "the token's row map entries, then all of its rows at once (eight in flight per lane), then the store"},
        }
    result = {
        "metric": "dispatch+combine effective HBM bandwidth per MoE layer (algorithmic bytes / time) on 1 MI355X",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "us_per_layer": round(ms_per_step * 1e3, 2),
        "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": dict(workloads.describe(w, ids), dependent_round_trips=round_trips, schedule=SCHEDULES[schedule], overlap=schedule == "flags-overlapped",
                       tile_rows=args.tile_rows if uses_flags else None, schedule_calibration_us=calibration,
                       other_schedules=other, expert_stage=expert_stage, graph_replay=graph_replay, rotating_inputs=rotating, reference_abi=reference_abi, kept_rows=kept_rows, dispatch_bytes=dispatch_bytes,
                       combine_bytes=combine_bytes, dispatch_us=round(dispatch_us, 2), combine_us=round(combine_us, 2)),
        "roofline": roofline, "kernels": kernels, "ceilings": ceilings,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, x, ids, weights, kept_rows)
    comm.destroy()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
