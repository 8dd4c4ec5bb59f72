#!/usr/bin/env python3
"""Benchmark of the MI355X MSCCL-IR executor.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c4] [--no-others] [--no-cpu]
    python bench.py --config c4 --sweep 1048576:536870912        (message-size sweep of one algorithm)

A step is one execution of the whole compiled algorithm (one launch of the executor kernel) over
buffers already resident in HBM.  The headline workload is the largest configuration, the two-level
AllReduce (4 x 8 = 32 virtual ranks, 2 instances, bf16, 128 MiB per rank); the other four
configurations are timed the same way and reported under "others".  One JSON line is printed.

Timing.  The all-reduce programs run in place, so a launch consumes its input: the send buffers are
restored from a pristine copy before every launch, outside the timed region, and every timed launch
reduces the same finite random data as the verified one.  Each of the K timed steps is bracketed by
a device synchronisation on both sides (wall clock) and by HIP events on the launch stream (kernel
time); ms_per_step and `value` are the mean of the K wall-clock intervals, `roofline` uses the mean
of the K event intervals.  The result of the LAST timed launch is verified as well as the first.
The all-gather and all-to-all programs do not consume their input; they are timed the same way.
"kernel_ms_queued" is the mean event interval of K more launches queued without host
synchronisation in between (restores in stream order): a launch on a stream that is kept busy,
which matters for the two latency-bound workloads (a launch on an idle GPU pays its dispatch).

metric/value: algbw in GB/s (nccl-tests convention, S / t).  "roofline": algorithmic bytes per launch
/ mean launch duration against the 8 TB/s HBM peak.  "cpu_baseline": the NumPy interpreter of the
same IR on this box's host cores (reported, not a target).  "host_us": what a caller pays on the host
for plan creation, configuration, binding and launching the first time, and what the executor cache
(msccl.executor.cache) makes of the same request when it comes again.  "roofline.streaming_reference": what torch's own
copy and add kernels reach on the same box over 1 GiB arrays (read + write bytes), a yardstick beside the peak.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "msccl-tools_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0
PMC_SUMMARY = os.path.join(ROOT, "profiles", "exec_kernel_hbm_traffic_pmc.txt")
ROOFLINE_NOTE = ("achieved = algorithmic bytes per launch / mean launch duration (HIP events); traffic = rocprofv3 FETCH_SIZE + "
                 "WRITE_SIZE per launch, counted between L2 and the fabric, so reads served by the memory-side cache are "
                 "included: the fraction is algorithmic bytes over the HBM peak, not proven DRAM traffic")


def measured_traffic():
    """HBM-side bytes per launch from the committed rocprofv3 --pmc summary (lines 'cN: traffic = B bytes per launch')."""
    out = {}
    try:
        text = open(PMC_SUMMARY).read()
    except OSError:
        return out
    for key, val in re.findall(r"^\s*(c\d) traffic = (\d+) bytes per launch", text, re.M):
        out[key] = int(val)
    return out


def streaming_reference():
    """What dependency-free streaming kernels reach on this box, read + write bytes over HIP-event time:
    torch's device copy and its bf16 add (2 reads : 1 write) over 1 GiB arrays, median of 7 after 3 warm-ups.
    A yardstick next to the 8 TB/s peak, not part of the executor."""
    import torch
    n = 1 << 30
    a = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda:0")
    b = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda:0")
    c = torch.empty_like(a)
    a16, b16, c16 = (t.view(torch.bfloat16) for t in (a, b, c))

    def median_us(fn):
        ts = []
        for it in range(10):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(); fn(); e1.record(); torch.cuda.synchronize()
            if it >= 3:
                ts.append(e0.elapsed_time(e1) * 1e3)
        return sorted(ts)[len(ts) // 2]
    copy_us = median_us(lambda: c.copy_(a))
    add_us = median_us(lambda: torch.add(a16, b16, out=c16))
    return {"copy_GBps": round(2 * n / copy_us / 1e3, 1), "add_GBps": round(3 * n / add_us / 1e3, 1), "bytes_per_array": n,
            "what": "torch copy_ and bf16 add on this box, read + write bytes / HIP-event time"}


def ensure_built():
    from msccl.executor import binding
    if not os.path.exists(binding.LIB_PATH):
        sys.path.insert(0, binding.CSRC_DIR)
        import build as csrc_build
        csrc_build.build(force=True, verbose=False)


def verify(w, x, res, orders):
    """Bit-exact check of the device result against the collective's closed form, on the device."""
    import torch
    n = w.ranks
    if w.coll == "allgather":
        want = torch.cat(x)
        return all(torch.equal(res[r], want) for r in range(n))
    if w.coll == "alltoall":
        blk = x[0].numel() // n
        return all(torch.equal(res[r], torch.cat([x[i][r * blk:(r + 1) * blk] for i in range(n)])) for r in range(n))
    E = x[0].numel() // w.nchunks
    itype = torch.int32 if x[0].element_size() == 4 else torch.int16

    def fold(order):
        if isinstance(order, int):
            return order
        acc = None
        for item in order:
            v = fold(item)
            v = x[v][c * E:(c + 1) * E] if isinstance(v, int) else v
            acc = v if acc is None else acc + v
        return acc
    for c in range(w.nchunks):
        want = fold(orders[c])
        for r in range(n):
            if not torch.equal(res[r][c * E:(c + 1) * E].view(itype), want.view(itype)):
                return False
    return True


def fold_orders(key):
    """Reduction order the IR of each all-reduce workload encodes (nested left folds over ranks)."""
    if key in ("c1", "c5"):
        n = 8 if key == "c1" else 64
        return [[(k + j) % n for j in range(n)] for k in range(n)]
    if key == "c5_chain":
        return [list(range(64))]
    if key == "c4":
        L, N = 8, 4
        one = []
        for q in range(L * N):
            b, j = q // N, q % N
            one.append([[node * L + (b + 1 + k) % L for k in range(L)] for node in [(j + 1 + m) % N for m in range(N)]])
        return one * 2
    return None


def run_workload(key, steps, warmup, device="cuda:0", bytes_per_rank=None, host_costs=False, knobs=None):
    import torch
    import gc
    from msccl.executor import Executor, cache, collective_buffers
    from msccl.executor.workloads import WORKLOADS, torch_input
    w = WORKLOADS[key] if bytes_per_rank is None else WORKLOADS[key].scaled(bytes_per_rank)
    xml = WORKLOADS[key].build()
    host = {}
    cache.clear()
    gc.collect()  # (a collection of the garbage the previous workload left would otherwise land in whichever step allocates next)
    t0 = time.perf_counter()
    tables = cache.tables_for(xml)
    host["parse_xml"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    ex = Executor(tables, device=device)
    host["plan_create"] = time.perf_counter() - t0
    info = ex.setup(w.chunk_bytes, w.dtype, **(knobs or {}))
    host["configure"] = ex.host_seconds["configure"]
    x = [torch_input(w, r, device) for r in range(w.ranks)]
    ins, outs, res = collective_buffers(ex.tables, w.chunk_bytes, w.dtype, device=device, inputs=x)
    consumes_input = w.coll == "allreduce"   # in place: a launch overwrites what it reads

    def restore():
        if consumes_input:
            for r in range(w.ranks):
                res[r][:x[r].numel()].copy_(x[r])

    torch.cuda.synchronize()
    ex.bind(ins, outs)
    host["bind_first"] = ex.host_seconds["bind"]
    ex.launch()  # first execution from pristine inputs
    ex.wait()
    torch.cuda.synchronize()
    ok = verify(w, x, res, fold_orders(key)) if bytes_per_rank is None else None  # the closed forms are written for the full size
    if host_costs:
        # a second set of buffers, then the first again: what a caller that passes fresh tensors pays per call
        ins2, outs2, _ = collective_buffers(ex.tables, w.chunk_bytes, w.dtype, device=device, inputs=None)
        torch.cuda.synchronize()
        ex.bind(ins2, outs2)
        host["bind_again"] = ex.host_seconds["bind"]
        ex.bind(ins, outs)
        host["bind_again"] = min(host["bind_again"], ex.host_seconds["bind"])
        del ins2, outs2
        # the executor cache: the first request for (document, chunk size, type, knobs) builds everything above once
        # more; the same request again is a lookup -- by the text's hash, or by the tables the caller kept
        gc.collect()
        t0 = time.perf_counter()
        kept = cache.executor_for(xml, w.chunk_bytes, w.dtype, device=device, **(knobs or {}))
        host["executor_for_first"] = time.perf_counter() - t0
        t0 = time.perf_counter()
        again = cache.executor_for(xml, w.chunk_bytes, w.dtype, device=device, **(knobs or {}))
        host["executor_for_again_from_text"] = time.perf_counter() - t0
        t0 = time.perf_counter()
        again2 = cache.executor_for(tables, w.chunk_bytes, w.dtype, device=device, **(knobs or {}))
        host["executor_for_again_from_tables"] = time.perf_counter() - t0
        assert again is kept and again2 is kept
        del kept, again, again2
        cache.clear()
    for _ in range(warmup):
        restore()
        ex.launch()
    ex.wait()
    torch.cuda.synchronize()
    wall, events, launch_host = [], [], []
    for _ in range(steps):
        restore()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)  # on the launch stream
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        ex.launch()
        t_l = time.perf_counter()
        e1.record()
        ex.wait()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        wall.append(t1 - t0)
        launch_host.append(t_l - t0)
        events.append(e0.elapsed_time(e1) * 1e-3)
    ok_last = verify(w, x, res, fold_orders(key)) if bytes_per_rank is None else None
    # the same K launches queued behind each other (restores in between, in stream order, no host
    # synchronisation until the end): what a caller sees whose stream is kept busy
    pairs = []
    for _ in range(steps):
        restore()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        ex.launch()
        e1.record()
        pairs.append((e0, e1))
    ex.wait()
    torch.cuda.synchronize()
    queued_s = sum(a.elapsed_time(b) for a, b in pairs) * 1e-3 / steps
    host["launch"] = sorted(launch_host)[len(launch_host) // 2]
    wall_s = sum(wall) / steps
    kernel_s = sum(events) / steps
    ab = ex.algorithmic_bytes()
    out = {"workload": w.description, "dtype": w.dtype, "ranks": w.ranks, "bytes_per_rank": w.bytes_per_rank,
           "ms_per_step": wall_s * 1e3, "kernel_ms": kernel_s * 1e3, "kernel_ms_min": min(events) * 1e3, "kernel_ms_max": max(events) * 1e3,
           "kernel_ms_queued": queued_s * 1e3,
           "algorithmic_bytes": ab,
           "verified": None if ok is None else bool(ok and ok_last), "inputs_restored_before_every_launch": consumes_input,
           "geometry": {k: v for k, v in info.as_dict().items() if k in ("workgroups", "threads", "slices", "piece_bytes", "fifo_depth", "passes")},
           "host_us": {k: round(v * 1e6, 1) for k, v in host.items()}}
    out.update({k: round(v, 4) for k, v in w.bandwidths(wall_s, ab).items()})
    out["roofline_frac_kernel"] = round(ab / kernel_s / 1e9 / HBM_PEAK_GBPS, 4)
    del x, ins, outs, res, ex
    torch.cuda.empty_cache()
    return out


# per-rank bytes of the CPU sample: bounded samples of the same algorithms (10 to 30 s of host work where the workload is large enough)
# Bytes per rank of the CPU baseline's run: the whole workload (the headline's 32 ranks x 128 MiB take the interpreter
# one to two seconds on the GPU box's host, ten times that on a small machine; a sample that fits the host's caches
# would run several times faster per byte than the workload does).
CPU_SAMPLE_BYTES = {"c1": 1 << 20, "c2": 32 << 20, "c3": 64 << 20, "c4": 128 << 20, "c5": 256 << 10, "c5_chain": 256 << 10}


def parse_knobs(text):
    knobs = {}
    for kv in filter(None, (text or "").split(",")):
        k, _, v = kv.partition("=")
        knobs[k] = v if k == "protocol" else int(v)
    return knobs


def time_program(path, chunk_sizes, steps, warmup, knobs):
    """Kernel time of one MSCCL-IR document at the given chunk sizes: HIP events around each of `steps` queued launches on the
    launch stream, median and mean.  Inputs are random; an all-reduce keeps reducing what the launch before left (finite for
    the few launches timed here)."""
    import gzip
    from msccl.executor import parse_algo_xml
    opener = gzip.open if path.endswith(".gz") else open
    with opener(path, "rt") as f:
        tables = parse_algo_xml(f.read())
    for row in time_tables(tables, os.path.basename(path), chunk_sizes, steps, warmup, knobs):
        print(json.dumps(row), flush=True)


def time_tables(tables, name, chunk_sizes, steps, warmup, knobs):
    """time_program's rows for tables that are already parsed."""
    import torch
    from msccl.executor import Executor
    from msccl.executor.binding import LOOP_NAMES
    from msccl.executor.workloads import HBM_PEAK_BYTES_PER_S
    rows = []
    for cb in chunk_sizes:
        ins = [torch.rand(int(tables.rank_chunks[r, 0]) * cb // 4, device="cuda:0") * 1e-3 if tables.rank_chunks[r, 0] else None for r in range(tables.ngpus)]
        outs = [torch.zeros(int(tables.rank_chunks[r, 1]) * cb // 4, device="cuda:0") if tables.rank_chunks[r, 1] else None for r in range(tables.ngpus)]
        ex = Executor(tables)
        info = ex.setup(cb, "float32", **knobs)
        ex.bind(ins, outs)
        for _ in range(max(1, warmup)):
            ex.launch()
        ex.wait()
        ts = sorted(ex.time(steps))
        ex.wait()
        med, mean = ts[len(ts) // 2] * 1e-3, sum(ts) / len(ts) * 1e-3
        ab = ex.algorithmic_bytes()
        rows.append({"program": name, "ranks": int(tables.ngpus), "collective": tables.coll, "chunk_bytes": cb,
                          "us_per_launch_median": round(med * 1e6, 2), "us_per_launch_mean": round(mean * 1e6, 2), "launches": steps,
                          "algorithmic_bytes": int(ab), "algorithmic_GBps": round(ab / med / 1e9, 1), "hbm_fraction": round(ab / med / HBM_PEAK_BYTES_PER_S, 4),
                          "step_loop": LOOP_NAMES.get(int(info.kernel_loop), str(int(info.kernel_loop))),
                          "geometry": {k: int(getattr(info, k)) for k in ("workgroups", "threads", "slices", "piece_bytes", "passes", "max_hosted", "protocol")},
                          "knobs": knobs})
        del ex, ins, outs
    return rows


def cpu_baseline(key):
    """NumPy interpreter (oracle/) on the same IR and input distribution, host cores of this box."""
    import numpy as np
    from msccl.executor.workloads import WORKLOADS, numpy_input
    from oracle import collectives as oc
    from oracle import ir_interp as oi
    full = WORKLOADS[key]
    w = full.scaled(CPU_SAMPLE_BYTES[key])
    algo = oi.parse_xml(full.build())
    esz = np.dtype(oi.DTYPES[w.dtype]).itemsize
    E = w.chunk_bytes // esz
    # one block of at most 16 MiB drawn as the benchmark definition says, laid end to end and shifted from rank to
    # rank: drawing ranks x sample fresh values would take several times longer than the run that is timed
    block = numpy_input(w, 0, nbytes=min(w.bytes_per_rank, 16 << 20))
    x = [np.resize(np.roll(block, 977 * r), w.bytes_per_rank // esz) for r in range(w.ranks)]
    runs = 2 if w.ranks * w.bytes_per_rank <= (1 << 30) else 1
    best = None
    for _ in range(runs):
        bufs = oc.place_inputs(algo, x, E, w.dtype)
        t0 = time.perf_counter()
        oi.Interpreter(algo).run(bufs, E, w.dtype)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
        del bufs
    ab = oi.algorithmic_bytes(algo, w.chunk_bytes)
    bw = w.bandwidths(best, ab)
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count()
    return {"value": round(bw["algbw_GBps"], 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{w.description.split(';')[0]}; {w.bytes_per_rank} of {full.bytes_per_rank} bytes per rank, best of {runs} run{'s' if runs > 1 else ''}, "
                      f"{best:.3f} s; single Python process (NumPy memcpy/ufuncs are single-threaded); host offers {cores} cores",
            "algorithmic_GBps": round(bw["algorithmic_GBps"], 4)}


def main():
    from msccl.executor.workloads import WORKLOADS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="c4", choices=sorted(WORKLOADS))
    ap.add_argument("--no-others", action="store_true", help="time only the headline workload")
    ap.add_argument("--knobs", default="", metavar="K=V,...", help="geometry of the headline workload instead of the automatic one, e.g. "
                    "threads=1024,workgroups=256,piece_bytes=131072 (for experiments; the line then carries them in config.knobs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the NumPy baseline")
    ap.add_argument("--sweep", metavar="LO:HI", help="instead of the benchmark line: time the chosen algorithm on LO, 2*LO, ... HI bytes per "
                    "rank (same inputs, same timing; results not verified) and print one JSON line holding the list")
    ap.add_argument("--xml", metavar="PATH", help="instead of the benchmark line: time the MSCCL-IR program in PATH (.xml or .xml.gz) on random "
                    "float32 inputs, automatic geometry unless --knobs says otherwise, one JSON line per chunk size (results not verified)")
    ap.add_argument("--chunk-bytes", default="4096", metavar="N[,N...]", help="with --xml: bytes of one IR chunk")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run five plain device copies of 1 GiB (known traffic: 1 GiB read + 1 GiB written each), "
                         "to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: every rank of the algorithm is a virtual rank on ONE GPU; run with --gpus 1 "
              "(a launch over several GPUs is not part of this build)", file=sys.stderr)
        sys.exit(2)
    ensure_built()
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the executor has no CPU path", file=sys.stderr)
        sys.exit(3)

    if args.xml:
        time_program(args.xml, [int(b) for b in args.chunk_bytes.split(",")], args.steps, args.warmup, parse_knobs(args.knobs))
        return

    if args.calibrate_copy:
        src = torch.randint(0, 255, (1 << 30,), dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "5 device copies of 1073741824 bytes"}))
        return
    if args.sweep:
        lo, hi = (int(v) for v in args.sweep.split(":"))
        rows = []
        size = lo
        while size <= hi:
            r = run_workload(args.config, args.steps, args.warmup, bytes_per_rank=size)
            rows.append({"bytes_per_rank": size, "kernel_us": round(r["kernel_ms"] * 1e3, 1), "algbw_GBps": round(r["algbw_GBps"], 2),
                         "busbw_GBps": round(r["busbw_GBps"], 2), "hbm_fraction": round(r["roofline_frac_kernel"], 4), **r["geometry"]})
            size *= 2
        print(json.dumps({"sweep": args.config, "workload": r["workload"].split(";")[0], "dtype": r["dtype"], "steps": args.steps, "rows": rows}))
        return
    traffic = measured_traffic()
    knobs = parse_knobs(args.knobs)
    head = run_workload(args.config, args.steps, args.warmup, host_costs=True, knobs=knobs)
    line = {
        "metric": "algbw_GBps", "value": head["algbw_GBps"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"int32": "i32", "uint8": "u8", "float32": "f32", "bfloat16": "bf16", "float16": "f16"}[head["dtype"]],
        "data": "synthetic", "config": {"workload": head["workload"], "virtual_ranks": head["ranks"], **head["geometry"], **({"knobs": knobs} if knobs else {})},
        "busbw_GBps": head["busbw_GBps"], "hbm_fraction": head["hbm_fraction"], "verified": head["verified"],
        "timing": "every timed launch starts from restored inputs (restore untimed) and is bracketed by a device synchronisation on both sides"
                  if head["inputs_restored_before_every_launch"] else "every timed launch is bracketed by a device synchronisation on both sides",
        "roofline": {"bound": "hbm", "achieved": round(head["algorithmic_bytes"] / (head["kernel_ms"] * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": head["roofline_frac_kernel"], "traffic": None if knobs else traffic.get(args.config),
                     "kernel": "exec_kernel", "algorithmic_bytes_per_launch": head["algorithmic_bytes"], "kernel_ms": round(head["kernel_ms"], 5),
                     "kernel_ms_min": round(head["kernel_ms_min"], 5), "kernel_ms_max": round(head["kernel_ms_max"], 5),
                     "kernel_ms_queued": round(head["kernel_ms_queued"], 5), "note": ROOFLINE_NOTE},
        "host_us": head["host_us"],
    }
    line["roofline"]["streaming_reference"] = streaming_reference()
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(args.config)
    if not args.no_others:
        line["others"] = {}
        for key in sorted(WORKLOADS):
            if key == args.config:
                continue
            r = run_workload(key, max(5, args.steps // 2), args.warmup, host_costs=key in ("c3", "c4", "c5"))
            line["others"][key] = {k: (round(v, 5) if isinstance(v, float) else v) for k, v in r.items() if k != "geometry"}
            line["others"][key].update(r["geometry"])
            line["others"][key]["traffic"] = traffic.get(key)
        # what msccl.init('mi355x', ...) hands out for an all-reduce below 16 MB per rank: the all-pairs program (msccl-tools'
        # msccl/programs/allreduce_allpairs.py), here on 8 ranks at 64 KiB and 4 MiB per rank (64 chunks of 1 KiB and of 64 KiB)
        from msccl.executor import parse_algo_xml
        from msccl.programs import catalog
        line["small_message_default"] = time_tables(parse_algo_xml(catalog.allpairs_allreduce(8, 1)), "allpairs_allreduce(8 ranks)", [1024, 65536],
                                                   max(5, args.steps // 2), args.warmup, {})
    print(json.dumps(line))


if __name__ == "__main__":
    main()
