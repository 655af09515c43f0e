#!/usr/bin/env python3
"""Benchmark of the reduce-copy hot path on one MI355X.

A step is one pass of the hot path over one batch: one pccl_hip_reduce_copy launch of the
headline workload (bf16, 8 inputs -> 1 output, 256 MiB per buffer).  Inputs are resident in
HBM before the timed region.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBPS = 8000.0  # MI355X HBM3E, published

# HBM bytes per launch of the headline kernel come from a committed record of two rocprofv3 --pmc runs
# (FETCH_SIZE, WRITE_SIZE), each scaled by what the same counter reads for a plain copy of known size.
# `bench.py --traffic-record FETCH_DIR WRITE_DIR` writes the record from the two runs' output folders;
# a normal run reads it and says whether it still belongs to this kernel and this file.
HEADLINE_KERNEL = "pccl_dev::reduce_copy_lean_kernel<2, pccl_dev::OpSum, 8, 1, 2>"
CALIBRATION_KERNEL = "pccl_dev::reduce_copy_lean_kernel<2, pccl_dev::OpSum, 1, 1, 2>"
TRAFFIC_RECORD = os.path.join(ROOT, "profiles", "reduce_copy_bf16_8in_256MiB.traffic.txt")
PROFILE_COMMAND = "python3 bench.py --no-extras --no-cpu --steps 20 --warmup 5 --calibration-copy 10"


def bench_sha16():
    import hashlib
    with open(os.path.abspath(__file__), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def _counter_means(folder, counter):
    """Mean per-dispatch value of `counter` for the headline and the calibration kernel, from the
    *_counter_collection.csv files rocprofv3 left under `folder`."""
    import csv
    import glob
    vals = {HEADLINE_KERNEL: [], CALIBRATION_KERNEL: []}
    files = glob.glob(os.path.join(folder, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise SystemExit("no *_counter_collection.csv under %s" % folder)
    for path in files:
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                name = row["Kernel_Name"].replace("void ", "").split("(")[0].strip()
                if row["Counter_Name"] == counter and name in vals:
                    vals[name].append(float(row["Counter_Value"]))
    for k, v in vals.items():
        if not v:
            raise SystemExit("%s: no %s dispatches of %s" % (folder, counter, k))
    return {k: (sum(v) / len(v), len(v)) for k, v in vals.items()}


def write_traffic_record(fetch_dir, write_dir):
    import subprocess
    copy_kib = (1 << 28) / 1024.0   # the calibration copy reads and writes one 256 MiB buffer
    lines, total = [], 0.0
    for counter, folder in (("FETCH_SIZE", fetch_dir), ("WRITE_SIZE", write_dir)):
        m = _counter_means(folder, counter)
        (head, n_head), (cal, n_cal) = m[HEADLINE_KERNEL], m[CALIBRATION_KERNEL]
        factor = copy_kib / cal
        total += head * factor * 1024.0
        lines += ["%s_copy_kernel_per_dispatch: %.1f (%d dispatches; known %d KiB)" % (counter, cal, n_cal, copy_kib),
                  "%s_scale: %.6f" % (counter, factor),
                  "%s_headline_kernel_per_dispatch: %.1f (%d dispatches)" % (counter, head, n_head),
                  "%s_headline_kernel_scaled_KiB: %.0f" % (counter, head * factor)]
    commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    text = ["# HBM traffic per launch of the headline kernel (bf16 8 -> 1, 256 MiB per buffer), rocprofv3 --pmc",
            "kernel: %s" % HEADLINE_KERNEL,
            "calibration_kernel: %s (plain copy of one 256 MiB buffer)" % CALIBRATION_KERNEL,
            "command_fetch: rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir> -- %s" % PROFILE_COMMAND,
            "command_write: rocprofv3 --pmc WRITE_SIZE --output-format csv -d <dir> -- %s" % PROFILE_COMMAND,
            "git_commit: %s" % (commit or "unknown"),
            "bench_py_sha16: %s" % bench_sha16()] + lines + [
            "algorithmic_bytes: %d" % (9 << 28),
            "traffic_bytes: %d" % round(total)]
    with open(TRAFFIC_RECORD, "w") as f:
        f.write("\n".join(text) + "\n")
    print("\n".join(text))


def read_traffic_record():
    """(traffic bytes or None, where it comes from and whether it is stale)."""
    if not os.path.exists(TRAFFIC_RECORD):
        return None, {"file": None, "stale": True, "why": "no record committed"}
    rec = {}
    for line in open(TRAFFIC_RECORD):
        if ":" in line and not line.startswith("#"):
            k, v = line.split(":", 1)
            rec[k.strip()] = v.strip()
    why = []
    if rec.get("kernel") != HEADLINE_KERNEL:
        why.append("recorded for another kernel")
    if rec.get("bench_py_sha16") != bench_sha16():
        why.append("bench.py changed since the record was made")
    src = {"file": os.path.relpath(TRAFFIC_RECORD, ROOT), "kernel": rec.get("kernel"), "git_commit": rec.get("git_commit"),
           "bench_py_sha16": rec.get("bench_py_sha16"), "stale": bool(why)}
    if why:
        src["why"] = "; ".join(why)
    try:
        return int(rec["traffic_bytes"]), src
    except (KeyError, ValueError):
        return None, dict(src, stale=True, why="record has no traffic_bytes")


def through_the_drain(torch, hip, bound_ops, stream, steps=20):
    """The same graph through the persistent drain (PCCL_HIP_WIDE=0): what a graph whose entries wait for
    nothing cost before it ran as a wide launch, and what bounds the graphs that cannot run as one."""
    old = os.environ.get("PCCL_HIP_WIDE")
    os.environ["PCCL_HIP_WIDE"] = "0"
    try:
        g = hip.Graph(bound_ops)
    finally:
        if old is None:
            del os.environ["PCCL_HIP_WIDE"]
        else:
            os.environ["PCCL_HIP_WIDE"] = old
    t = event_times_us(torch, lambda: g.run(stream), steps, 3)
    info = g.info()
    g.destroy()
    return dict(stats(t), queue_entries=info["n_tiles"], workgroups=info["n_workgroups"])


def launch_kind(graph):
    return {"wide": "wide (one workgroup per entry)", "drain": "persistent drain", "launches": "plain launches",
            "chains": "wide (a few chains, one workgroup per 4 KiB of each)"}[graph.launch_kind()]


def queue_bytes_moved(hip, bound_ops, elem_bytes):
    """Bytes the queue executor moves for these ops (bound to addresses), which is less than their
    algorithmic bytes where ops chain: in a chain that runs in one pass an op does not read the
    value its predecessor hands it, and does not store an output that a later op of the chain
    writes again.  From the executor's own chain plan (pccl_hip_plan_chains, host only)."""
    plan = hip.plan_chains(bound_ops, [1] * len(bound_ops), elem_bytes)
    inside = {}
    for h, (nxt, length, forward, _) in enumerate(plan):
        if length > 1 and forward == 1:
            steps, u = [], h
            while u >= 0:
                steps.append(u)
                u = plan[u][0]
            for k, u in enumerate(steps):
                inside[u] = (k, steps)
    # (a chain that runs through memory: a copy of the previous op's output is stored by that op and never read back)
    folded = set(i for i, (_, _, forward, _) in enumerate(plan) if forward == 2 and i not in inside)
    total = 0
    for i, o in enumerate(bound_ops):
        if "ins" not in o:
            continue
        n_in, n_out = len(o["ins"]), len(o["outs"])
        if i in folded:
            n_in = 0
        if i in inside:
            k, steps = inside[i]
            if k > 0:
                n_in -= 1
            later = set(a for u in steps[k + 1:] for a in bound_ops[u]["outs"])
            n_out = sum(1 for a in o["outs"] if a not in later)
        total += (n_in + n_out) * o["count"] * elem_bytes
    return total


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-extras", action="store_true", help="headline workload only")
    ap.add_argument("--extras", default="all", metavar="LIST",
                    help="comma-separated secondary workloads to run: layout (the headline shape on torch tensors and through Engine::exeOp), nvls, accumulate, ring, plumbing, unaligned, footprint, "
                         "op64k, schedule (one persistent launch), schedule_launches (the same ops as 4096 launches), "
                         "or all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calibration-copy", type=int, default=0, metavar="N",
                    help="also launch N plain copies (1 input -> 1 output) of the same 256 MiB buffers: the "
                         "known-size kernel that rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by")
    ap.add_argument("--timeline", action="store_true",
                    help="instead of the benchmark: the queue executor's own per-entry timeline (pccl_hip_graph_trace) of one "
                         "rank's 14 ring steps of 32 MiB (copy steps reading buffers of their own) and of the all-reduces over "
                         "8 ranks x 32 MiB, as a JSON line: where the workgroups' time goes")
    ap.add_argument("--traffic-record", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="write %s from the output folders of the two rocprofv3 --pmc runs, then exit (no GPU needed)"
                         % os.path.relpath(TRAFFIC_RECORD, ROOT))
    return ap.parse_args()


def event_times_us(torch, fn, iters, warm):
    """Per-launch durations from HIP events recorded on the stream fn launches on."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return sorted(a.elapsed_time(b) * 1e3 for a, b in ev)


def stats(ts):
    return {"min_us": round(ts[0], 2), "median_us": round(ts[len(ts) // 2], 2), "mean_us": round(sum(ts) / len(ts), 2)}


def gbps(nbytes, us):
    return round(nbytes / us / 1e3, 1)


_GENERATORS = {}


def seeded(torch, seed):
    """The device generator of a workload: every configured workload draws from its own seed
    (plumbing 0, ring 1, multi-input reduce 2, unaligned 3, small-message schedule 4)."""
    if seed not in _GENERATORS:
        _GENERATORS[seed] = torch.Generator(device="cuda").manual_seed(seed)
    return _GENERATORS[seed]


def randn(torch, n, kind, sigma=1.0, seed=2):
    dt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[kind]
    # generated in slices to bound the fp32 temporary
    out = torch.empty(n, dtype=dt, device="cuda")
    step = 1 << 26
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        out[lo:hi] = (torch.randn(hi - lo, device="cuda", generator=seeded(torch, seed)) * sigma).to(dt)
    return out


def cpu_baseline(count_sample):
    """The CPU checker's reduce-copy (a port: the reference has no CPU reduce code) on a
    bounded sample of the headline workload, timed on this box's host cores."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import pccl_oracle as orc
    cores = min(16, os.cpu_count() or 1)
    t_begin = time.perf_counter()
    ins = [np.random.default_rng(k).integers(0x3c00, 0x4000, size=count_sample, dtype=np.uint16) for k in range(8)]
    out = np.empty(count_sample, dtype=np.uint16)
    nbytes = 9 * count_sample * 2
    best = {}
    for threads in (1, cores):
        ts = []
        reps = 2 if threads == 1 else 5
        for _ in range(reps):
            t0 = time.perf_counter()
            orc.reduce_copy("bf16", "sum", ins, [out], count_sample, nthreads=threads)
            ts.append(time.perf_counter() - t0)
        best[threads] = nbytes / min(ts) / 1e9
    # the two other shapes of the measurement plan, same code: f32 2 -> 1 at 4 MiB per buffer and one
    # ring reduce step (bf16 2 -> 2, 32 MiB per buffer)
    other = {}
    a32 = [np.random.default_rng(20 + k).random(1 << 20, dtype=np.float32) for k in range(2)]
    o32 = np.empty(1 << 20, dtype=np.float32)
    ring_in = [x[:1 << 24] if count_sample >= (1 << 24) else np.resize(x, 1 << 24) for x in ins[:2]]
    ring_out = [np.empty(1 << 24, dtype=np.uint16) for _ in range(2)]
    c3 = min(count_sample, 1 << 26)
    for name, dt, i_, o_, n_, nb in (("f32_2in_1out_4MiB", "f32", a32, [o32], 1 << 20, 3 * 4 << 20),
                                     ("bf16_2in_2out_32MiB_ring_step", "bf16", ring_in, ring_out, 1 << 24, 4 * 32 << 20),
                                     ("bf16_8in_1out_128MiB", "bf16", [x[:c3] for x in ins], [out[:c3]], c3, 9 * c3 * 2)):
        r = {}
        for threads in (1, cores):
            ts = []
            for _ in range(3):
                t0 = time.perf_counter()
                orc.reduce_copy(dt, "sum", i_, o_, n_, nthreads=threads)
                ts.append(time.perf_counter() - t0)
            r["GBps_%d_thread%s" % (threads, "" if threads == 1 else "s")] = round(nb / min(ts) / 1e9, 2)
        other[name] = r
    # one rank's 14 ring steps (7 reduce steps 2 -> 2, 7 copy steps) over 32 MiB chunks
    grad = np.resize(ins[0], 8 << 24)
    peers = [np.resize(ins[1 + s % 7], 1 << 24) for s in range(7)]
    result = np.empty(8 << 24, dtype=np.uint16)
    send = np.empty(1 << 24, dtype=np.uint16)
    ce = 1 << 24
    r = {}
    for threads in (1, cores):
        ts = []
        for _ in range(2):
            t0 = time.perf_counter()
            for s in range(7):
                c = (7 - s) % 8
                orc.reduce_copy("bf16", "sum", [peers[s], grad[c * ce:(c + 1) * ce]], [result[c * ce:(c + 1) * ce], send], ce, nthreads=threads)
            for s in range(7):
                c = (8 - s) % 8
                orc.reduce_copy("bf16", "sum", [peers[s]], [result[c * ce:(c + 1) * ce]], ce, nthreads=threads)
            ts.append(time.perf_counter() - t0)
        r["GBps_%d_thread%s" % (threads, "" if threads == 1 else "s")] = round((7 * 4 + 7 * 2) * ce * 2 / min(ts) / 1e9, 2)
        r["ms_%d_thread%s" % (threads, "" if threads == 1 else "s")] = round(min(ts) * 1e3, 1)
    other["bf16_ring_rank_share_14_steps_32MiB"] = r
    return {"value": round(best[cores], 2), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "bf16 8->1 sum, %d elements per buffer (%s), best of 5 (this leg took %.0f s); "
                      "single thread: %.2f GB/s" % (count_sample, "the whole headline step" if count_sample == 1 << 27 else
                                                    "1/%d of the headline buffers" % ((1 << 27) // count_sample),
                                                    time.perf_counter() - t_begin, best[1]),
            "other_shapes": other, "host_cpus_visible": os.cpu_count()}


def queue_timeline(torch, hip, graph, stream, runs=3):
    """Where the workgroups' time went in the last of `runs` traced runs of `graph`: shares of (workgroups x run
    time) spent inside parts, waiting for dependencies, between a part's end and the next claim, before the
    first claim and idle behind the last part; from the executor's per-entry records (claimed, ready, done)."""
    import numpy as np
    graph.trace(True)
    for _ in range(runs):
        graph.run(stream)
        torch.cuda.synchronize()
    tr = graph.read_trace(stream)
    graph.trace(False)
    tr = tr[tr[:, 1] > 0]
    t0 = int(tr[:, 1].min())
    wg = (tr[:, 0].astype(np.uint64) >> np.uint64(52)).astype(int)
    cl, rd, dn = ((tr[:, k].astype(np.int64) - t0) / 100.0 for k in (1, 2, 3))    # microseconds on the 100 MHz clock
    end, groups = float(dn.max()), sorted(set(wg.tolist()))
    gaps, tail, first, per_gap = 0.0, 0.0, 0.0, []
    for w in groups:
        m = wg == w
        order = np.argsort(cl[m])
        c, d = cl[m][order], dn[m][order]
        g = (c[1:] - d[:-1]).clip(min=0)
        per_gap += g.tolist()
        gaps += float(g.sum())
        tail += end - float(d[-1])
        first += float(c[0])
    total = end * len(groups)
    pct = lambda x: round(100.0 * x / total, 1)
    q = lambda a, p: round(float(np.percentile(a, p)), 2) if len(a) else None
    return {"traced_run_us": round(end, 1), "workgroups": len(groups), "entries": int(len(tr)),
            "pct_in_parts": pct(float((dn - rd).sum())), "pct_waiting_for_dependencies": pct(float((rd - cl).sum())),
            "pct_between_part_end_and_next_claim": pct(gaps), "pct_before_first_claim": pct(first), "pct_idle_at_the_end": pct(tail),
            "part_us_median": q(dn - rd, 50), "part_us_p95": q(dn - rd, 95), "gap_us_median": q(per_gap, 50), "gap_us_p95": q(per_gap, 95),
            "last_part_end_by_workgroup_us_p5_p50_p100": [q([float(dn[wg == w].max()) for w in groups], p) for p in (5, 50, 100)]}


def wide_timeline(torch, hip, graph, stream, runs=3):
    """A wide launch's entries in time (one short-lived workgroup per entry; first timestamp when the workgroup
    has its record, last when its stores are out): how long an entry lives, when the last one starts, and how
    many are running at tenths of the run."""
    import numpy as np
    graph.trace(True)
    for _ in range(runs):
        graph.run(stream)
        torch.cuda.synchronize()
    tr = graph.read_trace(stream)
    graph.trace(False)
    tr = tr[tr[:, 1] > 0]
    t0 = int(tr[:, 1].min())
    start, done = ((tr[:, k].astype(np.int64) - t0) / 100.0 for k in (1, 3))
    end = float(done.max())
    life = done - start
    return {"traced_run_us": round(end, 1), "entries": int(len(tr)),
            "entry_us_p5_p50_p95_max": [round(float(np.percentile(life, p)), 1) for p in (5, 50, 95, 100)],
            "last_entry_starts_at_us": round(float(start.max()), 1),
            "running_at_tenths_of_the_run": [int(((start <= x) & (done > x)).sum()) for x in np.linspace(0.0, end, 11)[1:-1]]}


def timeline_main():
    import torch
    from pccl_amd import hip, lang
    os.environ["PCCL_HIP_WIDE"] = "0"  # the persistent drain's own timeline, also for the graphs that would run as a wide launch
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream().cuda_stream
    out = {}
    W, ce = 8, 1 << 24
    grad = randn(torch, W * ce, "bf16", 1e-2, seed=1)
    peers = [randn(torch, ce, "bf16", 1e-2, seed=1) for _ in range(W - 1)]
    late = [randn(torch, ce, "bf16", 1e-2, seed=1) for _ in range(W - 1)]
    result = torch.empty(W * ce, dtype=torch.bfloat16, device="cuda")
    send = torch.empty(ce, dtype=torch.bfloat16, device="cuda")
    ops = []
    for s in range(W - 1):
        c = (W - 1 - s) % W
        ops.append(dict(dtype="bf16", compute="sum", ins=[peers[s], grad[c * ce:(c + 1) * ce]], outs=[result[c * ce:(c + 1) * ce], send],
                        count=ce, deps=[len(ops) - 1] if ops else []))
    for s in range(W - 1):
        c = (W - s) % W
        ops.append(dict(dtype="bf16", compute="sum", ins=[late[s]], outs=[result[c * ce:(c + 1) * ce]], count=ce, deps=[s - 1] if s else []))
    g = hip.Graph(ops)
    t = event_times_us(torch, lambda: g.run(stream), 20, 3)
    out["ring_rank_share_14_steps_32MiB_copy_steps_read_buffers_of_their_own"] = dict(queue_timeline(torch, hip, g, stream), untraced_events_median_us=round(t[len(t) // 2], 1))
    g.destroy()
    del grad, peers, late, result, send
    for kind, emit in (("ring_allreduce_8_ranks_x_32_MiB", lang.ring_allreduce), ("direct_allreduce_8_ranks_x_32_MiB", lang.direct_allreduce)):
        ir, per_rank = emit(8, (32 << 20) // 2 // 8, dtype="bf16")
        rb = {"in": [randn(torch, per_rank, "bf16", 1e-2, seed=1) for _ in range(8)],
              "out": [torch.zeros(per_rank, dtype=torch.bfloat16, device="cuda") for _ in range(8)]}
        g = hip.Graph(lang.bind(ir.lower(), lambda b, r, e: rb[b][r].data_ptr() + 2 * e))
        t = event_times_us(torch, lambda: g.run(stream), 20, 3)
        out[kind] = dict(queue_timeline(torch, hip, g, stream), untraced_events_median_us=round(t[len(t) // 2], 1))
        g.destroy()
        # ... and the same graph as the wide launch it runs as by default (a launch of chains), and as the
        # table-driven wide launch that it would be without that
        for key, env in (("as_the_launch_it_runs_as", {}), ("as_the_table_driven_wide_launch", {"PCCL_HIP_CHAIN_LAUNCH": "0"})):
            del os.environ["PCCL_HIP_WIDE"]
            os.environ.update(env)
            try:
                g = hip.Graph(lang.bind(ir.lower(), lambda b, r, e: rb[b][r].data_ptr() + 2 * e))
            finally:
                os.environ["PCCL_HIP_WIDE"] = "0"
                for k in env:
                    del os.environ[k]
            if g.launch_kind() in ("wide", "chains"):
                t = event_times_us(torch, lambda: g.run(stream), 20, 3)
                out[kind][key] = dict(wide_timeline(torch, hip, g, stream), launch=launch_kind(g), untraced_events_median_us=round(t[len(t) // 2], 1))
            g.destroy()
    print(json.dumps({"queue_timeline": out}))


def main():
    args = parse()
    if args.traffic_record:
        write_traffic_record(*args.traffic_record)
        return
    if args.timeline:
        timeline_main()
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (peers are HBM buffers on the "
              "same device); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from pccl_amd import hip
    from pccl_amd import lang
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    hip.lib()
    info = hip.device_info()
    stream = torch.cuda.current_stream().cuda_stream

    # ---- headline: bf16 8 -> 1, 256 MiB per buffer --------------------------------------
    count = 1 << 27
    ins = [randn(torch, count, "bf16") for _ in range(8)]
    out = torch.empty(count, dtype=torch.bfloat16, device="cuda")
    step_bytes = 9 * count * 2
    # The timed operands come from the device plugin's own allocator, as PCCL's operands do: nine
    # pccl_hip_alloc calls.  The same data in nine torch tensors is timed below.
    operands = [hip.alloc(count * 2) for _ in range(9)]
    for k in range(8):
        hip.reduce_copy("bf16", "sum", [ins[k]], [operands[k]], count, stream)
    torch.cuda.synchronize()

    def step():
        hip.reduce_copy("bf16", "sum", operands[:8], [operands[8]], count, stream)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    value = step_bytes * args.steps / wall / 1e9

    ts = event_times_us(torch, step, max(20, min(args.steps, 100)), 3)
    mean_us = sum(ts) / len(ts)
    achieved = step_bytes / mean_us / 1e3
    traffic, traffic_source = read_traffic_record()
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                "frac": round(achieved / PEAK_HBM_GBPS, 4), "traffic": traffic, "traffic_source": traffic_source,
                "kernel": HEADLINE_KERNEL, "algorithmic_bytes_per_launch": step_bytes,
                "launch_us": stats(ts)}

    # quick self-check of the timed buffers against torch's fp32 accumulate (same fold order)
    hip.reduce_copy("bf16", "sum", [operands[8]], [out], count, stream)
    torch.cuda.synchronize()
    ref = ins[0][:1 << 20].float()
    for k in range(1, 8):
        ref = ref + ins[k][:1 << 20].float()
    assert torch.equal(ref.to(torch.bfloat16), out[:1 << 20]), "headline output differs from fp32-accumulated fold"
    for _ in range(args.calibration_copy):
        hip.reduce_copy("bf16", "sum", [operands[0]], [operands[8]], count, stream)
    torch.cuda.synchronize()

    extras = {}
    chosen = set(args.extras.split(","))

    class secondary_leg:
        """A secondary workload that fails (an assertion, no memory left) is reported under its name and
        does not take the headline line with it."""
        def __init__(self, where, name):
            self.where, self.name = where, name

        def __enter__(self):
            return self

        def __exit__(self, kind, value, trace):
            if kind is None or not issubclass(kind, Exception):
                return False
            import traceback
            self.where.setdefault("failed_legs", {})[self.name] = "%s: %s (%s)" % (
                kind.__name__, value, traceback.format_tb(trace)[-1].strip().replace("\n", " "))
            print("bench.py: secondary workload '%s' failed: %s" % (self.name, self.where["failed_legs"][self.name]), file=sys.stderr)
            try:
                torch.cuda.synchronize()
            except Exception:
                pass
            return True

    def want(name):
        return "all" in chosen or name in chosen

    if not args.no_extras:
        # ---- the headline shape on nine separate allocations: the plugin's, and torch's ----------
        if want("layout"):
            with secondary_leg(extras, "layout"):
                full = out.clone()
                t = event_times_us(torch, lambda: hip.reduce_copy("bf16", "sum", ins, [out], count, stream), 30, 5)
                assert torch.equal(full, out), "torch-tensor run differs from the headline output"
                extras["headline_shape_foreign_allocations"] = dict(
                    stats(t), GBps_median=gbps(step_bytes, t[len(t) // 2]),
                    note="same kernel and data, operands in nine torch tensors instead of nine pccl_hip_alloc buffers")
                del full
                # the headline op as a one-op schedule through Engine::regOp / exeOp (input tensor = the eight
                # operands back to back, as exeOp's tensor layout has them)
                import tempfile
                from pccl_amd import engine as engine_mod
                with tempfile.TemporaryDirectory() as tmp:
                    path = os.path.join(tmp, "fold8.sched")
                    with open(path, "w") as f:
                        f.write("pccl-schedule 1\nname fold8\ndtype bf16\ncompute sum\ndevices 8\nelems_per_device %d\nops 1\n" % count)
                        f.write("op 0 REDUCE %d deps 0 src 8 %s dst 1 out 0 0\n" % (count, " ".join("in %d 0" % r for r in range(8))))
                    eng = engine_mod.Engine(0, 1)
                    eng.initEngine()
                    eng.regOp("fold8", path)
                    x = torch.cat(ins)
                    y = torch.zeros(8 * count, dtype=torch.bfloat16, device="cuda")
                    te = event_times_us(torch, lambda: eng.exeOp("fold8", x, y, stream), 20, 3)
                    eng.waitOp("fold8", stream)
                    assert torch.equal(y[:count], out), "engine result differs from the headline output"
                    extras["headline_op_via_engine_exeOp"] = dict(
                        stats(te), GBps_median=gbps(step_bytes, te[len(te) // 2]),
                        note="one-op schedule file -> Engine::regOp / exeOp; the executor runs a graph of one op as a plain launch; "
                             "operands are the eight 256 MiB regions of ONE input tensor")
                    eng.close()
                    del x, y

        # ---- 128 MiB variants: bf16 8->1 and fp16 8->2, operands from separate plugin allocations ----
        c3 = 1 << 26
        if want("nvls"):
            with secondary_leg(extras, "nvls"):
                sep = [hip.alloc(c3 * 2) for _ in range(10)]
                for k in range(8):
                    hip.reduce_copy("bf16", "sum", [ins[k][:c3]], [sep[k]], c3, stream)
                t = event_times_us(torch, lambda: hip.reduce_copy("bf16", "sum", sep[:8], [sep[8]], c3, stream), 30, 5)
                tf = event_times_us(torch, lambda: hip.reduce_copy("bf16", "sum", [x[:c3] for x in ins], [out[:c3]], c3, stream), 30, 5)
                hip.reduce_copy("bf16", "sum", [sep[8]], [operands[8]], c3, stream)   # (operands[8] is free to be overwritten here)
                check = torch.empty(c3, dtype=torch.bfloat16, device="cuda")
                hip.reduce_copy("bf16", "sum", [sep[8]], [check], c3, stream)
                torch.cuda.synchronize()
                assert torch.equal(check, out[:c3]), "128 MiB run on plugin allocations differs from the run on torch tensors"
                extras["nvls_bf16_8in_1out_128MiB"] = dict(
                    stats(t), GBps_median=gbps(9 * c3 * 2, t[len(t) // 2]),
                    foreign_allocations=dict(stats(tf), GBps_median=gbps(9 * c3 * 2, tf[len(tf) // 2])))
                ins16 = [randn(torch, c3, "f16") for _ in range(8)]
                for k in range(8):
                    hip.reduce_copy("f16", "sum", [ins16[k]], [sep[k]], c3, stream)
                t = event_times_us(torch, lambda: hip.reduce_copy("f16", "sum", sep[:8], sep[8:10], c3, stream), 30, 5)
                o16 = [torch.empty(c3, dtype=torch.float16, device="cuda") for _ in range(2)]
                tf = event_times_us(torch, lambda: hip.reduce_copy("f16", "sum", ins16, o16, c3, stream), 30, 5)
                hip.reduce_copy("f16", "sum", [sep[9]], [check.view(torch.float16)], c3, stream)
                torch.cuda.synchronize()
                assert torch.equal(o16[0], o16[1]) and torch.equal(o16[0], check.view(torch.float16))
                extras["nvls_f16_8in_2out_128MiB"] = dict(
                    stats(t), GBps_median=gbps(10 * c3 * 2, t[len(t) // 2]),
                    foreign_allocations=dict(stats(tf), GBps_median=gbps(10 * c3 * 2, tf[len(tf) // 2])))
                for p in sep:
                    hip.free(p)
                del ins16, o16, sep, check

        # ---- fold one 128 MiB input into 7 destinations (the multimem.red role) -------------
        if want("accumulate"):
            with secondary_leg(extras, "accumulate"):
                src = randn(torch, c3, "bf16")
                dsts = [randn(torch, c3, "bf16") for _ in range(7)]
                t = event_times_us(torch, lambda: hip.accumulate("bf16", "sum", src, dsts, c3, stream), 20, 3)
                extras["accumulate_bf16_1in_7dst_128MiB"] = dict(stats(t), GBps_median=gbps(15 * c3 * 2, t[len(t) // 2]))
                # what bounds it: the share of writes.  Two walks of the same width for comparison, a broadcast
                # copy 1 -> 7 (1 read stream, 7 write streams) and a fold 8 -> 7 (8 read streams, 7 write streams,
                # exactly the accumulate's traffic without its in-place destinations)
                more = [randn(torch, c3, "bf16") for _ in range(7)]
                t17 = event_times_us(torch, lambda: hip.reduce_copy("bf16", "sum", [src], dsts, c3, stream), 20, 3)
                t87 = event_times_us(torch, lambda: hip.reduce_copy("bf16", "sum", [src] + more, dsts, c3, stream), 20, 3)
                extras["accumulate_bf16_1in_7dst_128MiB"]["same_width_walks"] = {
                    "copy_1in_7out": dict(stats(t17), GBps_median=gbps(8 * c3 * 2, t17[len(t17) // 2])),
                    "fold_8in_7out": dict(stats(t87), GBps_median=gbps(15 * c3 * 2, t87[len(t87) // 2]))}
                del src, dsts, more

        # ---- ring all-reduce, one rank's share at world 8: 7 reduce-copy + 7 copy steps ----
        if want("ring"):
            with secondary_leg(extras, "ring"):
                W, ce = 8, 1 << 24  # 32 MiB chunks of a 256 MiB gradient
                grad = randn(torch, W * ce, "bf16", 1e-2, seed=1)
                peers = [randn(torch, ce, "bf16", 1e-2, seed=1) for _ in range(W - 1)]
                result = torch.empty(W * ce, dtype=torch.bfloat16, device="cuda")
                send = torch.empty(ce, dtype=torch.bfloat16, device="cuda")

                # The seven incoming buffers serve both phases (reduce step s and copy step s read the same
                # 32 MiB); `late` is a second set for the copy steps, so that no byte is read twice.
                late = [randn(torch, ce, "bf16", 1e-2, seed=1) for _ in range(W - 1)]

                def ring(gathered=None):
                    gathered = gathered or peers
                    for s in range(W - 1):  # local chunk + incoming -> output chunk + send buffer
                        c = (W - 1 - s) % W
                        hip.reduce_copy("bf16", "sum", [peers[s], grad[c * ce:(c + 1) * ce]],
                                        [result[c * ce:(c + 1) * ce], send], ce, stream)
                    for s in range(W - 1):  # incoming reduced chunk -> output chunk
                        c = (W - s) % W
                        hip.reduce_copy("bf16", "sum", [gathered[s]], [result[c * ce:(c + 1) * ce]], ce, stream)

                t = event_times_us(torch, ring, 20, 3)
                t_late = event_times_us(torch, lambda: ring(late), 20, 3)
                ring_bytes = 7 * 4 * ce * 2 + 7 * 2 * ce * 2
                tr = event_times_us(torch, lambda: hip.reduce_copy("bf16", "sum", [peers[0], grad[:ce]], [result[:ce], send], ce, stream), 50, 5)
                tc = event_times_us(torch, lambda: hip.reduce_copy("bf16", "sum", [peers[1]], [result[ce:2 * ce]], ce, stream), 50, 5)
                # the same 14 steps as ONE persistent launch of the queue executor: ordered only by the
                # hazards the buffers impose (every reduce step writes the one send buffer; copy step s
                # overwrites the output chunk that reduce step s - 1 wrote), and with each step
                # depending on the one before
                def ring_ops(chain, gathered=None):
                    gathered = gathered or peers
                    o = []
                    for s in range(W - 1):
                        c = (W - 1 - s) % W
                        o.append(dict(dtype="bf16", compute="sum", ins=[peers[s], grad[c * ce:(c + 1) * ce]],
                                      outs=[result[c * ce:(c + 1) * ce], send], count=ce, deps=[len(o) - 1] if o else []))
                    for s in range(W - 1):
                        c = (W - s) % W
                        deps = [len(o) - 1] if chain else ([s - 1] if s else [])
                        o.append(dict(dtype="bf16", compute="sum", ins=[gathered[s]], outs=[result[c * ce:(c + 1) * ce]], count=ce, deps=deps))
                    return o
                tq = {}
                ring()
                torch.cuda.synchronize()
                ref_result = result.clone()
                ring(late)
                torch.cuda.synchronize()
                ref_late = result.clone()
                for key, chain, gathered, expected in ((False, False, peers, ref_result), (True, True, peers, ref_result),
                                                       ("late", False, late, ref_late)):
                    g = hip.Graph(ring_ops(chain, gathered))
                    result.zero_()
                    tq[key] = event_times_us(torch, lambda: g.run(stream), 20, 3)
                    torch.cuda.synchronize()
                    assert torch.equal(result, expected), "ring walk through the queue differs from the 14 launches"
                    g.destroy()
                # ... and gated the way a rank really is: every step waits for the arrival of its incoming
                # chunk on a signal word (GET_NOTIFIED), and tells the next rank when its output is there
                # (NOTIFY).  The peers are not running here, so the host marks every chunk as arrived
                # before the launch; what orders the steps inside the launch is what would order them on
                # a rank: the one send buffer that all seven reduce steps write (a dependency from each
                # reduce step to the next, met part by part).
                sig = torch.zeros(64, dtype=torch.int32, device="cuda")

                def gated_ops(gathered):
                    gated = []
                    prev_reduce = None
                    for s in range(2 * (W - 1)):
                        reduce_phase = s < W - 1
                        g_i = len(gated)
                        gated.append(dict(primitive=hip.GET_NOTIFIED, signal=sig.data_ptr() + 4 * s, value=1, deps=[]))
                        if reduce_phase:
                            c = (W - 1 - s) % W
                            gated.append(dict(dtype="bf16", compute="sum", ins=[peers[s], grad[c * ce:(c + 1) * ce]],
                                              outs=[result[c * ce:(c + 1) * ce], send], count=ce,
                                              deps=[g_i] + ([prev_reduce] if prev_reduce is not None else [])))
                            prev_reduce = len(gated) - 1
                        else:
                            c = (W - (s - (W - 1))) % W
                            hazard = [3 * (s - W) + 1] if s > W - 1 else []   # the reduce step that wrote this output chunk
                            gated.append(dict(dtype="bf16", compute="sum", ins=[gathered[s - (W - 1)]], outs=[result[c * ce:(c + 1) * ce]],
                                              count=ce, deps=[g_i] + hazard))
                        gated.append(dict(primitive=hip.NOTIFY, signal=sig.data_ptr() + 4 * (32 + s), value=1, deps=[len(gated) - 1]))
                    return gated

                def run_gated(gathered, expected):
                    gated = gated_ops(gathered)
                    gg = hip.Graph(gated)
                    # arrival words far enough ahead of this run's signal base to satisfy every timed run
                    sig[:32] = ((gg.next_signal_base() + (200 << 16)) & 0x7fffffff)
                    torch.cuda.synchronize()
                    result.zero_()
                    times = event_times_us(torch, lambda: gg.run(stream), 20, 3)
                    done, total = gg.status(stream)
                    assert done == total == len(gated)
                    assert torch.equal(result, expected), "signal-gated ring walk differs from the 14 launches"
                    kinds = gg.dependency_kinds()
                    gg.destroy()
                    return times, kinds, len(gated)

                tg, gkinds, n_gated = run_gated(peers, ref_result)
                tg_late, _, _ = run_gated(late, ref_late)
                med = lambda ts: ts[len(ts) // 2]
                extras["ring_allreduce_rank_share"] = {
                    "all_14_steps_one_queue_launch_signal_gated": dict(
                        stats(tg), GBps_median=gbps(ring_bytes, med(tg)), ops=n_gated,
                        dependencies_part_by_part="%d of %d" % (sum(gkinds), len(gkinds))),
                    "all_14_steps": dict(stats(t), GBps_median=gbps(ring_bytes, med(t))),
                    "all_14_steps_one_queue_launch": dict(stats(tq[False]), GBps_median=gbps(ring_bytes, med(tq[False]))),
                    "all_14_steps_one_queue_launch_chained": dict(stats(tq[True]), GBps_median=gbps(ring_bytes, med(tq[True]))),
                    "copy_steps_read_buffers_of_their_own": {
                        "all_14_steps": dict(stats(t_late), GBps_median=gbps(ring_bytes, med(t_late))),
                        "all_14_steps_one_queue_launch": dict(stats(tq["late"]), GBps_median=gbps(ring_bytes, med(tq["late"]))),
                        "all_14_steps_one_queue_launch_signal_gated": dict(stats(tg_late), GBps_median=gbps(ring_bytes, med(tg_late))),
                        "note": "the workload as configured reads each of the seven incoming buffers twice (reduce step s "
                                "and copy step s); in one queue launch the two run side by side and share the L2, so less "
                                "than the algorithmic bytes comes from HBM.  Here the copy steps read seven further "
                                "buffers: every algorithmic byte is an HBM byte"},
                    "reduce_step_2in_2out_32MiB": dict(stats(tr), GBps_median=gbps(4 * ce * 2, med(tr))),
                    "copy_step_1in_1out_32MiB": dict(stats(tc), GBps_median=gbps(2 * ce * 2, med(tc))),
                    "note": "single steps re-touch 128/64 MiB and are helped by the 256 MB Infinity Cache; "
                            "the 14-step figures walk 1.1 GiB of distinct data (1.3 GiB where the copy steps read buffers of their own)"}
                # ... and the way the reference's host code would run the rank's share: the 14 steps as a schedule
                # file through Engine::regOp / exeOp (regions of one input and one output tensor; the executor
                # sends a graph of this shape to the queue: one launch)
                import tempfile
                from pccl_amd import engine as engine_mod
                share = {}
                for own_gather in (False, True):
                    irs, per_region = lang.ring_rank_share(W, ce, dtype="bf16", gather_buffers_of_their_own=own_gather)
                    with tempfile.TemporaryDirectory() as tmp:
                        path = os.path.join(tmp, "share.sched")
                        irs.save(path, per_region)
                        eng = engine_mod.Engine(0, 1)
                        eng.initEngine()
                        eng.regOp("share", path)
                        x = torch.cat([grad] + peers + [send] + ((late + [send]) if own_gather else []))
                        y = torch.zeros_like(x)
                        te = event_times_us(torch, lambda: eng.exeOp("share", x, y, stream), 20, 3)
                        eng.waitOp("share", stream)
                        assert torch.equal(y[:W * ce], ref_late if own_gather else ref_result), "engine result differs from the 14 launches"
                        share["copy_steps_read_buffers_of_their_own" if own_gather else "as_configured"] = dict(
                            stats(te), GBps_median=gbps(ring_bytes, med(te)))
                        eng.close()
                        del x, y
                extras["ring_allreduce_rank_share"]["via_engine_exeOp"] = share
                del late
                del grad, peers, result, send

                # the whole collective over 8 virtual ranks as ONE launch of the queue executor:
                # 112 ops (8 ranks x 14 steps), every dependency a read of what the step before wrote
                full = {}
                for per_rank_mib in (1, 8, 32):
                    ir, per_rank = lang.ring_allreduce(8, (per_rank_mib << 20) // 2 // 8, dtype="bf16")
                    low = ir.lower()
                    rb = {"in": [randn(torch, per_rank, "bf16", 1e-2, seed=1) for _ in range(8)],
                          "out": [torch.zeros(per_rank, dtype=torch.bfloat16, device="cuda") for _ in range(8)]}
                    ring_bound = lang.bind(low, lambda b, r, e: rb[b][r].data_ptr() + 2 * e)
                    g = hip.Graph(ring_bound)
                    tf = event_times_us(torch, lambda: g.run(stream), 20, 3)
                    done, total = g.status(stream)
                    assert done == total == len(low)
                    for r in range(1, 8):
                        assert torch.equal(rb["out"][r], rb["out"][0])
                    moved = sum((len(o["ins"]) + len(o["outs"])) * o["count"] * 2 for o in low)
                    really = queue_bytes_moved(hip, ring_bound, 2)
                    kinds = g.dependency_kinds()
                    full["8_ranks_x_%d_MiB" % per_rank_mib] = dict(stats(tf), GBps_median=gbps(moved, tf[len(tf) // 2]), ops=len(low),
                                                                  algorithmic_bytes=moved, bytes_moved=really,
                                                                  GBps_moved_median=gbps(really, tf[len(tf) // 2]),
                                                                  queue_entries=g.info()["n_tiles"], launch=launch_kind(g),
                                                                  dependencies_part_by_part="%d of %d" % (sum(kinds), len(kinds)))
                    g.destroy()
                    full["8_ranks_x_%d_MiB" % per_rank_mib]["through_the_persistent_drain"] = through_the_drain(torch, hip, ring_bound, stream)
                    # The same all-reduce written the way ranks on different devices write it: dependency
                    # edges inside a rank only, the hand-over between neighbours NOTIFY -> signal word ->
                    # GET_NOTIFIED (328 ops).  Nothing can stay in registers across such a hand-over.
                    if per_rank_mib <= 8:
                        irs, _ = lang.ring_allreduce_signalled(8, (per_rank_mib << 20) // 2 // 8, dtype="bf16")
                        lows = irs.lower()
                        words = torch.zeros(64, dtype=torch.int32, device="cuda")
                        first = rb["out"][0].clone()
                        for r in range(8):
                            rb["out"][r].zero_()
                        gs = hip.Graph(lang.bind(lows, lambda b, r, e: rb[b][r].data_ptr() + 2 * e, signals=words.data_ptr()))
                        ts = event_times_us(torch, lambda: gs.run(stream), 20, 3)
                        done, total = gs.status(stream)
                        assert done == total == len(lows)
                        for r in range(8):
                            assert torch.equal(rb["out"][r], first), "the ring linked by signal words differs from the ring linked by dependencies"
                        full["8_ranks_x_%d_MiB" % per_rank_mib]["linked_by_signal_words_only"] = dict(
                            stats(ts), ops=len(lows), queue_entries=gs.info()["n_tiles"])
                        gs.destroy()
                        # ... and with signals of a word per part of the chunk (schedule format version 2): a rank
                        # starts on part p of a step as soon as its neighbour has finished part p of the step before
                        K = 8 if per_rank_mib <= 1 else 32
                        irp, _ = lang.ring_allreduce_signalled(8, (per_rank_mib << 20) // 2 // 8, dtype="bf16", signal_parts=K)
                        lowp = irp.lower()
                        words = torch.zeros(256, dtype=torch.int32, device="cuda")
                        for r in range(8):
                            rb["out"][r].zero_()
                        gp = hip.Graph(lang.bind(lowp, lambda b, r, e: rb[b][r].data_ptr() + 2 * e, signals=words.data_ptr()))
                        tp = event_times_us(torch, lambda: gp.run(stream), 20, 3)
                        done, total = gp.status(stream)
                        assert done == total == len(lowp)
                        for r in range(8):
                            assert torch.equal(rb["out"][r], first), "the ring linked by per-part signals differs from the ring linked by dependencies"
                        full["8_ranks_x_%d_MiB" % per_rank_mib]["linked_by_signal_words_only"]["a_word_per_part"] = dict(
                            stats(tp), words_per_signal=K, ops=len(lowp), queue_entries=gp.info()["n_tiles"])
                        gp.destroy()
                        # What bounds these two: the schedule, not the signal words.  The same 112 data ops linked by
                        # DEPENDENCIES in the order the signalled form implies (an op behind its neighbour's op of the
                        # step before, part by part, and behind its own rank's op of the step before, as a whole),
                        # every op queueing its own entries; and without the in-rank order.
                        ordered = [dict(o) for o in low]
                        latest = {}
                        for i, o in enumerate(ordered):
                            rank = o["outs"][0][1]
                            if rank in latest and latest[rank] not in o["deps"]:
                                o["deps"] = list(o["deps"]) + [latest[rank]]
                            latest[rank] = i
                        by_deps = {}
                        os.environ["PCCL_HIP_CHAINS"] = "0"
                        try:
                            for key, ops_k in (("the_same_order_as_dependencies", ordered), ("neighbour_dependencies_only", low)):
                                for r in range(8):
                                    rb["out"][r].zero_()
                                gd = hip.Graph(lang.bind(ops_k, lambda b, r, e: rb[b][r].data_ptr() + 2 * e))
                                td = event_times_us(torch, lambda: gd.run(stream), 20, 3)
                                for r in range(8):
                                    assert torch.equal(rb["out"][r], first)
                                by_deps[key] = dict(stats(td), queue_entries=gd.info()["n_tiles"])
                                gd.destroy()
                        finally:
                            del os.environ["PCCL_HIP_CHAINS"]
                        full["8_ranks_x_%d_MiB" % per_rank_mib]["linked_by_signal_words_only"]["without_chains"] = by_deps
                    del rb
                full["note"] = ("GBps_median counts the algorithmic bytes of the 112 ops; the 14 ops of a chunk run as one chain that keeps "
                                "the value in registers and stores only what the chain does not overwrite itself: bytes_moved / GBps_moved_median.  "
                                "No entry of these graphs waits for another, so they run as a wide launch (a launch of chains: one short-lived "
                                "workgroup per 4 KiB of a chain); through_the_persistent_drain is the same graph with PCCL_HIP_WIDE=0")
                extras["ring_allreduce_one_launch"] = full

                # the same all-reduce as the one-exchange ("direct") schedule a fully connected node
                # prefers: rank d folds slice d of all 8 inputs in rank order (8 -> 1), then a copy
                # stores it into the 7 other ranks' outputs; 16 ops, one queue launch.  Beside it the
                # whole thing as ONE reduce-copy launch with 8 inputs and 8 outputs.
                direct = {}
                for per_rank_mib in (1, 8, 32):
                    ir, per_rank = lang.direct_allreduce(8, (per_rank_mib << 20) // 2 // 8, dtype="bf16")
                    low = ir.lower()
                    rb = {"in": [randn(torch, per_rank, "bf16", 1e-2, seed=1) for _ in range(8)],
                          "out": [torch.zeros(per_rank, dtype=torch.bfloat16, device="cuda") for _ in range(8)]}
                    g = hip.Graph(lang.bind(low, lambda b, r, e: rb[b][r].data_ptr() + 2 * e))
                    tf = event_times_us(torch, lambda: g.run(stream), 20, 3)
                    done, total = g.status(stream)
                    assert done == total == len(low)
                    want_sum = rb["in"][0].float()
                    for r in range(1, 8):
                        want_sum = want_sum + rb["in"][r].float()
                    want_sum = want_sum.to(torch.bfloat16)
                    for r in range(8):
                        assert torch.equal(rb["out"][r], want_sum), "direct all-reduce differs from the fp32 fold in rank order"
                        rb["out"][r].zero_()
                    moved = sum((len(o["ins"]) + len(o["outs"])) * o["count"] * 2 for o in low)
                    really = queue_bytes_moved(hip, lang.bind(low, lambda b, r, e: rb[b][r].data_ptr() + 2 * e), 2)
                    dkinds = g.dependency_kinds()
                    t1 = event_times_us(torch, lambda: hip.reduce_copy("bf16", "sum", rb["in"], rb["out"], per_rank, stream), 20, 3)
                    for r in range(8):
                        assert torch.equal(rb["out"][r], want_sum)
                    # ... and the way the reference's host code would run it: the schedule from its file through
                    # Engine::regOp / exeOp on one input and one output tensor.  The executor folds each copy into
                    # the fold that feeds it and joins the eight slices: one 8 -> 8 launch.
                    import tempfile
                    from pccl_amd import engine as engine_mod
                    with tempfile.TemporaryDirectory() as tmp:
                        path = os.path.join(tmp, "direct.sched")
                        ir.save(path, per_rank)
                        eng = engine_mod.Engine(0, 1)
                        eng.initEngine()
                        eng.regOp("direct", path)
                        x = torch.cat(rb["in"])
                        y = torch.zeros(8 * per_rank, dtype=torch.bfloat16, device="cuda")
                        te = event_times_us(torch, lambda: eng.exeOp("direct", x, y, stream), 20, 3)
                        eng.waitOp("direct", stream)
                        for r in range(8):
                            assert torch.equal(y[r * per_rank:(r + 1) * per_rank], want_sum), "engine result differs"
                        eng.close()
                        del x, y
                    direct["8_ranks_x_%d_MiB" % per_rank_mib] = dict(
                        stats(tf), GBps_median=gbps(moved, tf[len(tf) // 2]), ops=len(low), algorithmic_bytes=moved,
                        bytes_moved=really, GBps_moved_median=gbps(really, tf[len(tf) // 2]),
                        queue_entries=g.info()["n_tiles"], launch=launch_kind(g), dependencies_part_by_part="%d of %d" % (sum(dkinds), len(dkinds)),
                        as_one_launch_8in_8out=dict(stats(t1), GBps_median=gbps(16 * per_rank * 2, t1[len(t1) // 2])),
                        via_engine_exeOp=dict(stats(te), GBps_median=gbps(16 * per_rank * 2, te[len(te) // 2])))
                    g.destroy()
                    del rb, want_sum
                extras["direct_allreduce_one_launch"] = direct

        # ---- plumbing config: f32 2 -> 1, 4 MiB ---------------------------------------------
        if want("plumbing"):
            with secondary_leg(extras, "plumbing"):
                a, b = (torch.empty(1 << 20, dtype=torch.float32, device="cuda").uniform_(-1.0, 1.0, generator=seeded(torch, 0)) for _ in range(2))
                o = torch.empty_like(a)
                t = event_times_us(torch, lambda: hip.reduce_copy("f32", "sum", [a, b], [o], 1 << 20, stream), 100, 10)
                assert torch.equal(o, a + b)
                # where the time of one small launch goes: the host call (ctypes, argument checks, launch),
                # launches issued back to back (what the GPU front end sustains), and one launch between two
                # events (what `stats` reports; the kernel itself is 2.9 us by rocprofv3)
                torch.cuda.synchronize()
                n_calls = 2000
                t0 = time.perf_counter()
                for _ in range(n_calls):
                    hip.reduce_copy("f32", "sum", [a, b], [o], 1 << 20, stream)
                host_us = (time.perf_counter() - t0) / n_calls * 1e6
                torch.cuda.synchronize()
                pa, pb, po = a.data_ptr(), b.data_ptr(), o.data_ptr()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(n_calls):
                    hip.reduce_copy("f32", "sum", [pa, pb], [po], 1 << 20, stream)
                e1.record()
                torch.cuda.synchronize()
                extras["f32_2in_1out_4MiB"] = dict(
                    stats(t), host_call_us=round(host_us, 2), back_to_back_us_per_launch=round(e0.elapsed_time(e1) * 1e3 / n_calls, 2),
                    note="median_us = one launch between two events; host_call_us = Python ctypes call incl. the library's "
                         "argument checks and hipLaunchKernel, nothing waited for; back_to_back = 2000 launches between two events")

        # ---- unaligned operands: 4 -> 1, every buffer 4..60 bytes off a 64-byte boundary ----------
        # (the counts of 2^24 elements and more from the list that the parity tests run; the four
        # dtype / fold pairs at the longest prime count)
        if want("unaligned"):
            with secondary_leg(extras, "unaligned"):
                cmax = 1 << 28
                offs = [4, 12, 20, 60, 8]
                ipool = [torch.randint(-(1 << 20), (1 << 20) + 1, (cmax + 64,), dtype=torch.int32, device="cuda", generator=seeded(torch, 3)) for _ in range(4)]
                ou = torch.empty(cmax + 64, dtype=torch.int32, device="cuda")

                def unaligned_leg(dtype, compute, pool, cu):
                    ptr_in = [pool[k].data_ptr() + offs[k] for k in range(4)]
                    t = event_times_us(torch, lambda: hip.reduce_copy(dtype, compute, ptr_in, [ou.data_ptr() + offs[4]], cu, stream), 20, 5)
                    return dict(stats(t), GBps_median=gbps(5 * 4 * cu, t[len(t) // 2]))

                cu = (1 << 28) - 57
                extras["unaligned_i32_4in_1out_1GiB"] = dict(unaligned_leg("i32", "sum", ipool, cu), byte_offsets=offs)
                other = {}
                for c, label in (((1 << 24) - 3, "2^24-3"), (1 << 28, "2^28")):
                    other["i32_sum_count_" + label] = unaligned_leg("i32", "sum", ipool, c)
                other["i32_max_count_2^28-57"] = unaligned_leg("i32", "max", ipool, cu)
                del ipool
                fpool = [torch.empty(cmax + 64, dtype=torch.float32, device="cuda").uniform_(0.5, 2.0, generator=seeded(torch, 3)) for _ in range(4)]
                other["f32_min_count_2^28-57"] = unaligned_leg("f32", "min", fpool, cu)
                other["f32_prod_count_2^28-57"] = unaligned_leg("f32", "prod", fpool, cu)
                extras["unaligned_i32_4in_1out_1GiB"]["other_counts_and_folds"] = other
                del fpool, ou

        # ---- footprint: the same shapes at 256 MiB and at 1 GiB per operand, aligned ------------------
        # (4 -> 1 is the shape of the unaligned leg above; a copy and 2 -> 1 stand beside it as the simplest
        # walks over the same footprint; profiles/reduce_copy_4in_1GiB_counters.md holds the counters)
        if want("footprint"):
            with secondary_leg(extras, "footprint"):
                cmax = 1 << 28
                pool = [torch.randint(-(1 << 20), (1 << 20) + 1, (cmax,), dtype=torch.int32, device="cuda", generator=seeded(torch, 3)) for _ in range(4)]
                dst = torch.empty(cmax, dtype=torch.int32, device="cuda")
                foot = {}
                for label, c in (("256MiB", 1 << 26), ("1GiB", 1 << 28)):
                    for dtype, n_in in (("i32", 4), ("bf16", 4), ("i32", 2), ("i32", 1)):
                        cnt = c * (2 if dtype == "bf16" else 1)      # same bytes per operand
                        es = 2 if dtype == "bf16" else 4
                        srcs = [x[:c] for x in pool[:n_in]]
                        t = event_times_us(torch, lambda: hip.reduce_copy(dtype, "sum", srcs, [dst[:c]], cnt, stream), 12, 3)
                        foot["%s_%din_1out_%s" % (dtype, n_in, label)] = dict(stats(t), GBps_median=gbps((n_in + 1) * cnt * es, t[len(t) // 2]))
                chk = pool[0][:1 << 20] + pool[1][:1 << 20]
                hip.reduce_copy("i32", "sum", [x[:1 << 20] for x in pool[:2]], [dst[:1 << 20]], 1 << 20, stream)
                torch.cuda.synchronize()
                assert torch.equal(dst[:1 << 20], chk)
                extras["aligned_by_footprint"] = foot
                del pool, dst

        # ---- small ops: 64 KiB direct launch and through the queue --------------------------
        if want("op64k"):
            with secondary_leg(extras, "op64k"):
                n64 = 32768
                x, y = randn(torch, n64, "bf16", seed=4), randn(torch, n64, "bf16", seed=4)
                z = torch.empty_like(x)
                t = event_times_us(torch, lambda: hip.reduce_copy("bf16", "sum", [x, y], [z], n64, stream), 200, 20)
                extras["op_64KiB_direct_launch"] = stats(t)
                g1 = hip.Graph([dict(dtype="bf16", compute="sum", ins=[x, y], outs=[z], count=n64)])
                t = event_times_us(torch, lambda: g1.run(stream), 200, 20)
                extras["op_64KiB_via_queue"] = dict(stats(t), launch=launch_kind(g1),
                                                    through_the_persistent_drain=through_the_drain(
                                                        torch, hip, [dict(dtype="bf16", compute="sum", ins=[x, y], outs=[z], count=n64)], stream, 200))
                g1.destroy()

        # ---- the 4096-op small-message schedule: one persistent launch ----------------------
        if want("schedule"):
            with secondary_leg(extras, "schedule"):
                ir, per_rank = lang.small_message_allreduce()
                low = ir.lower()
                bufs = {"in": [randn(torch, per_rank, "bf16", seed=4) for _ in range(8)],
                        "out": [torch.zeros(per_rank, dtype=torch.bfloat16, device="cuda") for _ in range(8)]}
                bound = lang.bind(low, lambda b, r, e: bufs[b][r].data_ptr() + 2 * e)
                sched_bytes = sum((len(o["ins"]) + len(o["outs"])) * o["count"] * 2 for o in low)
                g = hip.Graph(bound)
                t = event_times_us(torch, lambda: g.run(stream), 30, 5)
                done, total = g.status(stream)
                assert done == total == len(low)
                for r in range(1, 8):  # all-reduce invariant on the ring part
                    assert torch.equal(bufs["out"][r][:per_rank // 2], bufs["out"][0][:per_rank // 2])
                ginfo = g.info()
                med = t[len(t) // 2]

                def individually():
                    for o in bound:
                        hip.reduce_copy("bf16", "sum", o["ins"], o["outs"], o["count"], stream)

                sched_moved = queue_bytes_moved(hip, bound, 2)
                # the same graph with every op queueing its own entries (no chains: nothing stays in registers,
                # every op reads and writes all its operands)
                os.environ["PCCL_HIP_CHAINS"] = "0"
                try:
                    g0 = hip.Graph(bound)
                finally:
                    del os.environ["PCCL_HIP_CHAINS"]
                for b in bufs["out"]:
                    b.zero_()
                t0 = event_times_us(torch, lambda: g0.run(stream), 30, 5)
                done, total = g0.status(stream)
                assert done == total == len(low)
                for r in range(1, 8):
                    assert torch.equal(bufs["out"][r][:per_rank // 2], bufs["out"][0][:per_rank // 2])
                unchained = dict(stats(t0), us_per_op=round(t0[len(t0) // 2] / len(low), 4), GBps_median=gbps(sched_bytes, t0[len(t0) // 2]),
                                 queue_entries=g0.info()["n_tiles"])
                g0.destroy()
                extras["schedule_4096_ops"] = {
                    "one_persistent_launch": dict(stats(t), us_per_op=round(med / len(low), 4), GBps_median=gbps(sched_bytes, med),
                                                  GBps_moved_median=gbps(sched_moved, med)),
                    "one_persistent_launch_without_chains": unchained,
                    "ops": len(low), "queue_entries": ginfo["n_tiles"], "workgroups": ginfo["n_workgroups"], "launch": launch_kind(g),
                    "algorithmic_bytes": sched_bytes, "bytes_moved": sched_moved,
                    "note": "GBps_median counts the algorithmic bytes of the 4096 ops; chains of 14 ops keep the value in registers "
                            "and skip stores they overwrite themselves (bytes_moved, GBps_moved_median).  one_persistent_launch is one "
                            "launch of whatever kind the library chooses: with chains no entry waits for another and it is a wide launch "
                            "(through_the_persistent_drain: the same graph with PCCL_HIP_WIDE=0); without chains it is the persistent drain"}
                extras["schedule_4096_ops"]["one_persistent_launch"]["through_the_persistent_drain"] = through_the_drain(torch, hip, bound, stream, 30)
                # the same schedule the way the reference's host code would drive it: written to a
                # schedule file, registered by name, executed on an input / output tensor pair
                # (Engine::regOp / exeOp; every exeOp binds the tensors and launches once)
                import tempfile
                from pccl_amd import engine
                with tempfile.TemporaryDirectory() as tmp:
                    path = os.path.join(tmp, "small_message.sched")
                    ir.save(path, per_rank)
                    eng = engine.Engine(0, 1)
                    eng.initEngine()
                    eng.regOp("small_message", path)
                    x = torch.cat(bufs["in"])
                    y = torch.zeros(8 * per_rank, dtype=torch.bfloat16, device="cuda")
                    te = event_times_us(torch, lambda: eng.exeOp("small_message", x, y, stream), 30, 5)
                    eng.waitOp("small_message", stream)
                    for r in range(8):
                        assert torch.equal(y[r * per_rank:(r + 1) * per_rank], bufs["out"][r]), "engine result differs from the bound graph's"
                    extras["schedule_4096_ops"]["via_engine_exeOp"] = dict(stats(te), us_per_op=round(te[len(te) // 2] / len(low), 4))
                    eng.close()
                    del x, y
                if want("schedule_launches"):  # the same ops as one launch each ("all" includes it)
                    t2 = event_times_us(torch, individually, 5, 1)
                    extras["schedule_4096_ops"]["as_4096_launches"] = dict(stats(t2), us_per_op=round(t2[len(t2) // 2] / len(low), 4))
                g.destroy()

    torch.cuda.synchronize()
    for p in operands:
        hip.free(p)

    result = {
        "metric": "reduce_copy_hbm_bandwidth", "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "bf16 sum of 8 inputs -> 1 output, 134217728 elements (256 MiB) per buffer, "
                               "N(0,1) from torch seed 2, fp32 accumulate, one launch per step, operands allocated by the "
                               "plugin's allocator (nine pccl_hip_alloc calls)",
                   "n_in": 8, "n_out": 1, "count": count, "bytes_per_step": step_bytes},
        "pct_of_peak_hbm": round(100.0 * value / PEAK_HBM_GBPS, 2),
        "roofline": roofline,
        "device": info,
    }
    if not args.no_cpu:
        try:
            result["cpu_baseline"] = cpu_baseline(1 << 27)
        except Exception as e:  # (the GPU figures above are not lost with it)
            print("bench.py: the CPU-baseline leg failed: %s: %s" % (type(e).__name__, e), file=sys.stderr)
            result["cpu_baseline"] = {"value": None, "unit": "GB/s", "cores": 0, "kind": "port", "sample": "failed: %s: %s" % (type(e).__name__, e)}
    if extras:
        result["extras"] = extras
    print(json.dumps(result))


if __name__ == "__main__":
    main()
