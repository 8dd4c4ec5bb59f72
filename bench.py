#!/usr/bin/env python3
"""Benchmark of the MI355X MSCCL-IR executor.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2] [--no-others] [--no-cpu]
    python bench.py --config c4 --sweep 1048576:536870912        (message-size sweep of one algorithm)

A step is one execution of the whole compiled algorithm (one launch of the executor kernel) over
buffers already resident in HBM.  The headline workload is the ring AllGather configuration
(8 virtual ranks, 4 instances, int32, 32 MiB per rank); the other four configurations are timed
the same way and reported under "others".  One JSON line is printed.

metric/value: algbw in GB/s (nccl-tests convention, S / t) from the wall clock around exactly K
back-to-back launches.  "roofline": algorithmic bytes per launch / average launch duration taken
with HIP events on the launch stream over the same K launches, against the 8 TB/s HBM peak.
"cpu_baseline": the NumPy interpreter of the same IR on this box's host cores (reported, not a target).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "msccl-tools_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0
# HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/exec_kernel_c2_c3_c4_pmc.txt),
# each scaled by what the same counter reads for a plain device copy of 1 GiB (FETCH_SIZE x 2.0,
# WRITE_SIZE x 1.0).  Not measured for the two latency-bound workloads.
MEASURED_TRAFFIC_BYTES = {"c2": 3763694252, "c3": 3229607986, "c4": 20822006138}

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
    if key == "c4":
        L, N = 8, 4
        one = []
        for q in range(L * N):
            b, j = q // N, q % N
            one.append([[node * L + (b + 1 + k) % L for k in range(L)] for node in [(j + 1 + m) % N for m in range(N)]])
        return one * 2
    return None


def run_workload(key, steps, warmup, device="cuda:0", bytes_per_rank=None):
    import torch
    from msccl.executor import Executor, collective_buffers
    from msccl.executor.workloads import WORKLOADS, torch_input
    w = WORKLOADS[key] if bytes_per_rank is None else WORKLOADS[key].scaled(bytes_per_rank)
    xml = WORKLOADS[key].build()
    ex = Executor(xml, device=device)
    info = ex.setup(w.chunk_bytes, w.dtype)
    x = [torch_input(w, r, device) for r in range(w.ranks)]
    ins, outs, res = collective_buffers(ex.tables, w.chunk_bytes, w.dtype, device=device, inputs=x)
    ex.run(ins, outs)  # first execution from pristine inputs: the one that is verified
    torch.cuda.synchronize()
    ok = verify(w, x, res, fold_orders(key)) if bytes_per_rank is None else None  # the closed forms are written for the full size
    for _ in range(warmup):
        ex.launch()
    ex.wait()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)  # on the launch stream
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        ex.launch()
    e1.record()
    ex.wait()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall_s = (t1 - t0) / steps
    kernel_s = e0.elapsed_time(e1) * 1e-3 / steps
    ab = ex.algorithmic_bytes()
    out = {"workload": w.description, "dtype": w.dtype, "ranks": w.ranks, "bytes_per_rank": w.bytes_per_rank,
           "ms_per_step": wall_s * 1e3, "kernel_ms": kernel_s * 1e3, "algorithmic_bytes": ab, "verified": None if ok is None else bool(ok),
           "geometry": {k: v for k, v in info.as_dict().items() if k in ("workgroups", "threads", "slices", "piece_bytes", "fifo_depth", "passes")}}
    out.update({k: round(v, 4) for k, v in w.bandwidths(wall_s, ab).items()})
    out["roofline_frac_kernel"] = round(ab / kernel_s / 1e9 / HBM_PEAK_GBPS, 4)
    del x, ins, outs, res, ex
    torch.cuda.empty_cache()
    return out


# per-rank bytes of the CPU sample: the full headline workload, bounded samples of the heavier ones
CPU_SAMPLE_BYTES = {"c1": 1 << 20, "c2": 32 << 20, "c3": 16 << 20, "c4": 4 << 20, "c5": 256 << 10}


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
    x = [numpy_input(w, r) for r in range(w.ranks)]
    best = None
    for _ in range(2):
        bufs = oc.place_inputs(algo, x, E, w.dtype)
        t0 = time.perf_counter()
        oi.Interpreter(algo).run(bufs, E, w.dtype)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    ab = oi.algorithmic_bytes(algo, w.chunk_bytes)
    bw = w.bandwidths(best, ab)
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count()
    return {"value": round(bw["algbw_GBps"], 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{w.bytes_per_rank} of {full.bytes_per_rank} bytes per rank, best of 2 runs, {best:.3f} s; single Python "
                      f"process (NumPy memcpy/ufuncs are single-threaded); host offers {cores} cores",
            "algorithmic_GBps": round(bw["algorithmic_GBps"], 4)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c2", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--no-others", action="store_true", help="time only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the NumPy baseline")
    ap.add_argument("--sweep", metavar="LO:HI", help="instead of the benchmark line: time the chosen algorithm on LO, 2*LO, ... HI bytes per "
                    "rank (same inputs, same timing; results not verified) and print one JSON line holding the list")
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
    head = run_workload(args.config, args.steps, args.warmup)
    traffic = MEASURED_TRAFFIC_BYTES.get(args.config)
    line = {
        "metric": "algbw_GBps", "value": head["algbw_GBps"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"int32": "i32", "uint8": "u8", "float32": "f32", "bfloat16": "bf16", "float16": "f16"}[head["dtype"]],
        "data": "synthetic", "config": {"workload": head["workload"], "virtual_ranks": head["ranks"], **head["geometry"]},
        "busbw_GBps": head["busbw_GBps"], "hbm_fraction": head["hbm_fraction"], "verified": head["verified"],
        "roofline": {"bound": "hbm", "achieved": round(head["algorithmic_bytes"] / (head["kernel_ms"] * 1e-3) / 1e9, 2), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": head["roofline_frac_kernel"], "traffic": traffic,
                     "kernel": "exec_kernel", "algorithmic_bytes_per_launch": head["algorithmic_bytes"], "kernel_ms": round(head["kernel_ms"], 5)},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(args.config)
    if not args.no_others:
        line["others"] = {}
        for key in ("c1", "c2", "c3", "c4", "c5"):
            if key == args.config:
                continue
            r = run_workload(key, max(5, args.steps // 2), args.warmup)
            line["others"][key] = {k: (round(v, 5) if isinstance(v, float) else v) for k, v in r.items() if k != "geometry"}
            line["others"][key].update(r["geometry"])
            line["others"][key]["traffic"] = MEASURED_TRAFFIC_BYTES.get(key)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
