#!/usr/bin/env python3
"""Benchmark of the fused softmax -> top-k post-proc on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3]

A step is one call of the fused entry point (vkop_hip_softmax_topk, through the C
ABI) over one batch of synthetic logits already resident in HBM.  The default
workload is the one the metric is quoted on: [64,128256] float32, k = 50.  The
batches rotate over enough distinct device buffers (> 256 MB in total) that the
Infinity Cache cannot serve the reads; the figure with one buffer (cache
resident) is reported beside it.  Prints ONE JSON line.

How the K steps are timed.  Step i runs on lane i % L (L independent calls in
flight, each lane with its own stream, workspace and outputs); every lane's
share of the K steps is recorded once (a HIP graph) and the recordings are
replayed: W warm-up steps, then the K-step recordings once untimed (their first
launch uploads them), then timed: back to back until at least 400 steps are in
the timed region (one replay of 20 steps on 4 lanes is five calls a lane that
all start in the same phase: a pipeline filling, not running), lanes running
free.  The timed replays are enqueued behind a spin kernel on the launch
stream, so that all lanes are queued before the first of them starts and the
host's submission time is not inside the timed region; HIP events on that
stream bracket the region, with a device synchronize on both sides.  The host
wall clock of the same replays without the gate is reported as well
(`host_wall_ms_per_step`).

The CPU baseline leg times, on the host cores of the same machine, the CPU
oracle (test infrastructure, used here only as the thing being timed against)
and libtorch's CPU softmax + topk, which is what the reference's own tests
treat as truth.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Four calls in flight need four hardware queues of their own; with four queues
# per process (HIP's default, and what this pool exports) two of the streams end
# up sharing one.  --hw-queues sets GPU_MAX_HW_QUEUES for this process before the
# HIP runtime starts.  More than four calls in flight run slower on this part.
DEFAULT_HW_QUEUES = 8

HBM_PEAK_GBS = 8000.0   # MI355X published HBM3E bandwidth

WORKLOADS = {
    # name: (description, generator kwargs, k)
    "C1": ("[1,1000] f32 softmax+topk k=5", dict(kind="cls", rows=1, cols=1000), 5),
    "C2": ("[256,1000] f32 softmax+topk k=5", dict(kind="cls", rows=256, cols=1000), 5),
    "C3": ("[64,128256] f32 softmax+topk k=50", dict(kind="llm", rows=64, cols=128256), 50),
    "C4": ("[8,262144] f32 softmax+topk k=1024", dict(kind="grid", rows=8, cols=262144), 1024),
    # a variant of C3, not one of the reference's configurations: its logits truncated to bfloat16 precision
    # (what a bf16 LM head hands over); equal logits then straddle the k-th place in most rows
    "C3bf16": ("[64,128256] f32 softmax+topk k=50, bf16-valued logits", dict(kind="llm_bf16", rows=64, cols=128256), 50),
}

# kernels of a two-kernel streaming call, by the path the library takes (vkop_hip_measure_path)
PATH_KERNELS = {1: ("rows_chunk_kernel", "rows_merge_kernel"), 2: ("rows_scan_kernel", "rows_pick_kernel")}


def make_input(spec, seed):
    from vkop_amd import synth
    if spec["kind"] == "cls":
        return synth.classifier_logits(spec["rows"], spec["cols"], seed)
    if spec["kind"] == "llm":
        return synth.llm_logits(spec["rows"], spec["cols"], seed)
    if spec["kind"] == "llm_bf16":
        import numpy as np
        x = synth.llm_logits(spec["rows"], spec["cols"], seed)
        return np.ascontiguousarray((x.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32))
    return synth.grid_values(spec["rows"], spec["cols"], seed)


def traffic_from_profiles(workload, kernel):
    """HBM bytes per launch of `kernel`, from the committed rocprofv3 --pmc summary
    (FETCH_SIZE and WRITE_SIZE scaled by the same counters over a copy of known size);
    None if profiles/ holds no such line."""
    path = os.path.join(ROOT, "profiles", "softmax_topk_%s_hbm_traffic.txt" % workload)
    try:
        text = open(path).read()
    except OSError:
        return None
    m = re.search(r"^%s: read (\d+) B \+ written (\d+) B = (\d+) B of HBM traffic per launch" % re.escape(kernel), text, re.M)
    return int(m.group(3)) if m else None


def runtime_api_leg(runs=200):
    """The headline tensor through the operator interface a user of the reference has: the C++
    program's benchmark mode registers SOFTMAX + TOPK as post-processing of a [64,128256] output and
    calls Runtime::Run() in a loop, as benchmark/main.cpp:112-137 does, reporting the mean of the
    wall-clock milliseconds Run() returns.  Run as a child process, before this process touches the
    GPU."""
    import subprocess
    exe = os.path.join(ROOT, "vkop_amd", "host", "build", "test_ops")
    if not os.path.exists(exe):
        return {"error": "vkop_amd/host/build/test_ops is not built (make -C vkop_amd/host)"}
    try:
        r = subprocess.run([exe, "--bench-runtime", str(runs)], capture_output=True, text=True, timeout=300,
                           cwd=os.path.join(ROOT, "vkop_amd", "host"))
        legs = [json.loads(line) for line in r.stdout.splitlines() if line.startswith("{")]
        if r.returncode != 0 or not legs:
            return {"error": "test_ops --bench-runtime failed (%d): %s" % (r.returncode, (r.stderr or r.stdout)[-300:])}
        out = {"what": legs[0]["what"], "shape": legs[0]["shape"], "k": legs[0]["k"], "runs": legs[0]["runs"],
               "calls_in_flight": 1, "queues": "the runtime's own two (core/Runtime.hpp kInflight), one operator chain"}
        for leg in legs:
            out["fused" if leg["fused"] else "two_operators"] = {"mean_ms": leg["mean_ms"], "min_ms": leg["min_ms"],
                                                                 "operators": leg["operators"]}
        return out
    except Exception as exc:  # the figure is informative only
        return {"error": str(exc)}


def timeline_summary(rec, ms_per_step, nlanes, hw_queues):
    """What the timeline library's log of one timed pass says: records (tag, entry, exit) per logged workgroup,
    tag = kernel (bit 63: 0 scan, 1 pick) | workgroup << 40 | bits of the call's workspace address (= the lane);
    clocks in 10 ns.  The scan kernel logs every 16th workgroup and its last 48, the pick kernel all 64."""
    import numpy as np
    tag = rec[:, 0]
    t0 = rec[:, 1].astype(np.int64) * 10
    t1 = rec[:, 2].astype(np.int64) * 10
    kind = (tag >> np.uint64(63)).astype(np.int64)
    lane_id = (tag & np.uint64(0xFFFFFFFFFF)).astype(np.int64)
    order = np.argsort(t0, kind="stable")
    kind, lane_id, t0, t1 = kind[order], lane_id[order], t0[order], t1[order]
    # the timed replays follow the warm-up and the untimed replay after a pause (the gate): the last stretch without one
    cuts = np.nonzero(np.diff(t0) > 1_000_000)[0]
    first = int(cuts[-1]) + 1 if len(cuts) else 0
    kind, lane_id, t0, t1 = kind[first:], lane_id[first:], t0[first:], t1[first:]
    lanes = sorted(set(lane_id.tolist()))
    launches = []  # (start, end, lane, kernel)
    for li, w in enumerate(lanes):
        for kd in (0, 1):
            m = np.nonzero((lane_id == w) & (kind == kd))[0]
            if len(m) == 0:
                continue
            # a launch's workgroups enter within a few microseconds of each other; the lane's next launch of the
            # same kernel enters a whole call later
            groups = np.split(m, np.nonzero(np.diff(t0[m]) > 4000)[0] + 1)
            for g in groups:
                launches.append((int(t0[g].min()), int(t1[g].max()), li, kd))
    launches.sort()
    if len(launches) < 8 * nlanes:
        return {"error": "too few launches in the log", "records": int(len(rec))}
    # leave the pass's first and last calls out (lanes filling and draining)
    lo, hi = launches[2 * nlanes][0], launches[-2 * nlanes][0]
    mid = [l for l in launches if lo <= l[0] < hi]
    dur = {kd: [(e - s) / 1e3 for s, e, _, k2 in mid if k2 == kd] for kd in (0, 1)}
    gaps = {"scan_to_pick": [], "pick_to_scan": []}
    for li in range(len(lanes)):
        mine = [l for l in mid if l[2] == li]
        for a, b in zip(mine, mine[1:]):
            if a[3] != b[3]:
                gaps["scan_to_pick" if a[3] == 0 else "pick_to_scan"].append((b[0] - a[1]) / 1e3)
    # how many kernels are running, weighted by time
    ev = sorted([(s, 1) for s, e, _, _ in mid] + [(e, -1) for s, e, _, _ in mid])
    conc = {}
    cur, last = 0, ev[0][0]
    for t, d in ev:
        conc[cur] = conc.get(cur, 0) + (t - last)
        cur, last = cur + d, t
    total = float(sum(conc.values()))
    scans = [l for l in mid if l[3] == 0]
    span = (scans[-1][0] - scans[0][0]) / 1e3
    mean = lambda v: float(np.mean(v)) if len(v) else None
    return {
        "what": "device timestamps logged by the scan and pick kernels themselves (libvkop_hip_timeline.so), one timed pass, "
                "its first and last calls left out",
        "calls_in_flight": nlanes, "hw_queues": hw_queues, "lanes_seen": len(lanes),
        "calls": len(scans), "us_per_call_from_the_log": span / max(1, len(scans) - 1),
        "us_per_step_by_hip_events_same_run": ms_per_step * 1e3,
        "scan_kernel_us_first_entry_to_last_exit": {"mean": mean(dur[0]), "p10": float(np.percentile(dur[0], 10)), "p90": float(np.percentile(dur[0], 90))},
        "pick_kernel_us_first_entry_to_last_exit": {"mean": mean(dur[1]), "p10": float(np.percentile(dur[1], 10)), "p90": float(np.percentile(dur[1], 90))},
        "pick_workgroup_us_entry_to_exit_mean": float(np.mean((t1 - t0)[(kind == 1) & (t0 >= lo) & (t0 < hi)])) / 1e3,
        "gap_us_scan_exit_to_pick_entry_same_lane": mean(gaps["scan_to_pick"]),
        "gap_us_pick_exit_to_next_scan_entry_same_lane": mean(gaps["pick_to_scan"]),
        "share_of_time_with_n_kernels_running": {str(n): conc[n] / total for n in sorted(conc)},
        "mean_kernels_running": sum(n * v for n, v in conc.items()) / total,
    }


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(x, k, budget_s=14.0):
    """Times the CPU side on a bounded sample of the same workload."""
    import torch

    import oracle
    cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)
    rows = x.shape[0]
    # oracle, all rows spread over `cores` threads
    t0 = time.perf_counter()
    _, _, used = oracle.softmax_topk_mt(x, k, threads=cores)
    once = time.perf_counter() - t0
    reps = max(1, min(50, int(budget_s / 3 / max(once, 1e-6))))
    t0 = time.perf_counter()
    for _ in range(reps):
        oracle.softmax_topk_mt(x, k, threads=cores)
    t_oracle = (time.perf_counter() - t0) / reps
    # libtorch CPU: at::softmax + at::topk, the reference tests' expectation source,
    # on all host threads and on one
    xt = torch.from_numpy(x)

    def time_torch(threads, budget):
        torch.set_num_threads(threads)
        for _ in range(2):
            torch.topk(torch.softmax(xt, -1), k, -1, True, True)
        t0 = time.perf_counter()
        n = 0
        while time.perf_counter() - t0 < budget and n < 200:
            torch.topk(torch.softmax(xt, -1), k, -1, True, True)
            n += 1
        return (time.perf_counter() - t0) / max(n, 1), n, torch.get_num_threads()
    t_torch, n_torch, thr_torch = time_torch(cores, budget_s / 3)
    t_torch1, n_torch1, _ = time_torch(1, budget_s / 4)
    torch.set_num_threads(cores)
    # the reference's own CPU post-processing, restated: one row at a time, one thread (core/function.cpp:150-183)
    sample = min(rows, 8)
    t0 = time.perf_counter()
    for r in range(sample):
        oracle.get_top_k_predictions(x[r], k)
    t_post = (time.perf_counter() - t0) / sample
    what = ("torch.topk(torch.softmax(x,-1),k) on the host, as tests/SoftmaxTest.cpp:138 and tests/TopkTest.cpp:73 "
            "compute expectations")
    return {
        "value": rows / t_oracle, "unit": "rows/s", "cores": int(used), "kind": "port",
        "sample": "whole %dx%d batch, %d repeats of the C oracle (OpenMP over rows)" % (x.shape[0], x.shape[1], reps),
        "cpu_model": cpu_model(), "host_threads": cores,
        "libtorch_cpu": {"value": rows / t_torch, "unit": "rows/s", "threads": thr_torch, "version": torch.__version__,
                         "cpu_capability": torch.backends.cpu.get_cpu_capability(), "repeats": n_torch, "what": what},
        "libtorch_cpu_1_thread": {"value": rows / t_torch1, "unit": "rows/s", "threads": 1, "repeats": n_torch1},
        "reference_cpu_postproc": {"value": 1.0 / t_post, "unit": "rows/s", "cores": 1, "rows_timed": sample,
                                   "what": "Function::get_top_k_predictions restated (core/function.cpp:150-183): softmax of "
                                           "one row, full sort by probability, first k; the CPU code the GPU path replaces"},
    }


def copy_calibration(nbytes=256 << 20, launches=20):
    """A plain copy kernel of known size: reads nbytes and writes nbytes per launch."""
    import torch
    src = torch.empty(nbytes // 4, dtype=torch.float32, device="cuda").normal_()
    others = [torch.empty_like(src).normal_() for _ in range(2)]   # push src out of the Infinity Cache
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for i in range(launches):
        dst.copy_(src if i % 2 == 0 else others[0])
    torch.cuda.synchronize()
    print(json.dumps({"copy_bytes_read_per_launch": nbytes, "copy_bytes_written_per_launch": nbytes,
                      "launches": launches, "kernel": "__amd_rocclr_copyBuffer, the runtime's device copy kernel behind dst.copy_(src)"}))


def ulps(a, b):
    import numpy as np
    ia = a.view(np.int32).astype(np.int64)
    ib = b.view(np.int32).astype(np.int64)
    return np.abs(ia - ib)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="C3", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-host", action="store_true", help="skip the host-buffer (PCIe) round-trip leg")
    ap.add_argument("--no-runtime-api", action="store_true", help="skip the Runtime::Run() leg (the C++ program as a child process)")
    ap.add_argument("--headline-only", action="store_true",
                    help="time only the whole step with the given --hw-queues / --inflight and print a short JSON line (bench.py "
                         "runs itself this way, as a child process, for the figure with the environment's own number of "
                         "hardware queues)")
    ap.add_argument("--kernel-legs", action="store_true",
                    help="run only the legs that time each kernel of the step by itself and print them as one JSON line: "
                         "they need the benchmark build of the library (libvkop_hip_bench.so, whose measurement hook can "
                         "leave a kernel out of a call), so bench.py runs them in a child process of this form while its own "
                         "figures come from the library that ships")
    ap.add_argument("--hw-queues", type=int, default=DEFAULT_HW_QUEUES,
                    help="hardware queues this process may use (GPU_MAX_HW_QUEUES); 0 = leave the environment as it is")
    ap.add_argument("--inflight", type=int, default=0,
                    help="independent calls in flight (each on its own stream with its own workspace and outputs)")
    ap.add_argument("--rows-path", type=int, default=0, choices=(0, 1),
                    help="0 = the library's choice of streaming kernels, 1 = the chunk + merge kernels (vkop_hip_tune rows.path)")
    ap.add_argument("--no-gate", action="store_true", help="do not hold the timed replay behind a spin kernel")
    ap.add_argument("--eager", action="store_true",
                    help="launch every call from the host instead of replaying recordings (for counter runs under "
                         "rocprofv3 --pmc, which collects per dispatch; the timings of such a run are not the metric)")
    ap.add_argument("--timeline", action="store_true",
                    help="run the whole step with the given --hw-queues / --inflight on libvkop_hip_timeline.so (`make -C "
                         "vkop_amd/csrc timeline`), whose scan and pick kernels log device timestamps per workgroup, and print "
                         "what the log says about the lanes: each kernel's duration from its first workgroup's entry to its "
                         "last one's exit, the gaps between a lane's kernels, how many kernels run at the same time")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain device copy of known size (the yardstick for the FETCH_SIZE / "
                         "WRITE_SIZE counters) and print its size")
    args = ap.parse_args()
    env_as_started = dict(os.environ)
    if args.hw_queues > 0:
        os.environ["GPU_MAX_HW_QUEUES"] = str(min(args.hw_queues, 32))
    hw_queues = int(os.environ.get("GPU_MAX_HW_QUEUES", "4"))
    if args.inflight <= 0:
        args.inflight = 4 if hw_queues >= 6 else 3
    if args.copy_calibration:
        copy_calibration()
        return
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU; --gpus %d is not supported "
              "(rows are independent: shard the batch and run one process per GPU)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    # (child processes, before this one initialises the GPU)
    child = args.kernel_legs or args.headline_only or args.timeline
    runtime_api = None if (child or args.no_runtime_api or args.workload != "C3") else runtime_api_leg()
    kernel_legs = None
    default_queues = None
    if not child and not args.eager and args.hw_queues > 0:
        # the same step in the environment this process was started in (GPU_MAX_HW_QUEUES as it is: HIP's default
        # is 4, one of which the default stream takes): what a caller who changes nothing sees
        import subprocess
        legs = {}
        for name, inflight in (("same_calls_in_flight", max(1, args.inflight if args.inflight > 0 else 4)), ("calls_in_flight_3", 3)):
            cmd = [sys.executable, os.path.abspath(__file__), "--headline-only", "--hw-queues", "0", "--inflight", str(inflight),
                   "--steps", str(args.steps), "--warmup", str(args.warmup), "--workload", args.workload,
                   "--rows-path", str(args.rows_path)] + (["--no-gate"] if args.no_gate else [])
            try:
                r = subprocess.run(cmd, capture_output=True, text=True, timeout=600, env=env_as_started)
                lines = [line for line in r.stdout.splitlines() if line.startswith("{")]
                legs[name] = json.loads(lines[-1]) if r.returncode == 0 and lines else {"error": (r.stderr or r.stdout)[-300:]}
            except Exception as exc:
                legs[name] = {"error": str(exc)}
        default_queues = legs
    if not child and not args.eager:
        import subprocess
        cmd = [sys.executable, os.path.abspath(__file__), "--kernel-legs", "--steps", str(args.steps), "--warmup", str(args.warmup),
               "--workload", args.workload, "--hw-queues", str(args.hw_queues), "--inflight", str(args.inflight),
               "--rows-path", str(args.rows_path)] + (["--no-gate"] if args.no_gate else [])
        try:
            r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
            lines = [line for line in r.stdout.splitlines() if line.startswith("{")]
            kernel_legs = json.loads(lines[-1]) if r.returncode == 0 and lines else {"error": (r.stderr or r.stdout)[-300:]}
        except Exception as exc:
            kernel_legs = {"error": str(exc)}

    import numpy as np
    import torch

    import oracle
    from vkop_amd import capi, synth

    if args.kernel_legs:
        capi.use_bench_library()
    if args.timeline:
        capi.use_timeline_library()
    capi.lib()
    capi.init(0)
    capi.tune("rows.path", args.rows_path)
    desc, spec, k = WORKLOADS[args.workload]
    rows, cols = spec["rows"], spec["cols"]
    shape = (rows, cols)
    in_bytes = rows * cols * 4
    algo_bytes = in_bytes + rows * k * 8
    nbuf = min(64, max(2, -(-(288 << 20) // in_bytes)))
    seed0 = synth.SEEDS.get(args.workload[:2], 1)
    host_inputs = [make_input(spec, seed0 + 7919 * b) for b in range(min(nbuf, 3))]
    bufs = [torch.from_numpy(host_inputs[b % len(host_inputs)]).cuda() for b in range(nbuf)]
    # One "lane" per call in flight: its own stream, workspace and outputs, like the
    # reference's kInflight = 2 queues (core/runtime.cpp:408-446).  Step i runs on
    # lane i % L; steps on one lane are serialized, lanes overlap.
    ws_bytes = capi.softmax_topk_workspace_bytes(capi.F32, shape, -1, k)
    lanes = []
    for _ in range(max(1, args.inflight)):
        ws = torch.empty(ws_bytes + 256, dtype=torch.uint8, device="cuda")
        lanes.append({"vals": torch.empty((rows, k), dtype=torch.float32, device="cuda"),
                      "idx": torch.empty((rows, k), dtype=torch.int32, device="cuda"),
                      "ws": ws, "ws_ptr": ws.data_ptr() + (-ws.data_ptr()) % 256,
                      "stream": capi.stream_create(), "event": capi.event_create()})
    for ln in lanes:
        capi.workspace_init(ln["ws_ptr"], ws_bytes, ln["stream"])
        capi.stream_sync(ln["stream"])
    torch.cuda.synchronize()
    main_stream = lanes[0]["stream"]
    torch_main = torch.cuda.ExternalStream(main_stream)

    def call(buf, ln):
        capi.softmax_topk(buf.data_ptr(), 0, ln["vals"].data_ptr(), ln["idx"].data_ptr(), capi.F32, shape, -1, k, 1,
                          ln["ws_ptr"], ws_bytes, ln["stream"])

    # parity of what is about to be timed, on every lane: against the oracle (the bar)
    # and against libtorch's CPU result on the same tensor (reported)
    parity = {"indices_exact": True, "max_ulp_vs_oracle": 0}
    ov, oix = oracle.softmax_topk(host_inputs[0], k)
    for ln in lanes:
        call(bufs[0], ln)
        capi.stream_sync(ln["stream"])
        gi, gv = ln["idx"].cpu().numpy(), ln["vals"].cpu().numpy()
        parity["indices_exact"] = parity["indices_exact"] and bool(np.array_equal(gi, oix))
        parity["max_ulp_vs_oracle"] = max(parity["max_ulp_vs_oracle"], int(ulps(gv, ov).max()))
    if not parity["indices_exact"] or parity["max_ulp_vs_oracle"] > 2:
        print("bench.py: parity check failed: %s" % parity, file=sys.stderr)
        sys.exit(1)
    tv, ti = torch.topk(torch.softmax(torch.from_numpy(host_inputs[0]), -1), k, -1, True, True)
    same = ti.numpy().astype(np.int32) == gi
    d = ulps(gv, tv.numpy())[same]
    parity["vs_libtorch_cpu"] = {"indices_equal_fraction": float(same.mean()),
                                 "max_ulp": int(d.max()) if d.size else None, "mean_ulp": float(d.mean()) if d.size else None,
                                 "what": "values at the places where libtorch's index agrees; libtorch sums a long row in "
                                         "ISA-dependent float lanes and is itself several ulp from the exact sum"}

    def fork(nlanes):
        """The other lanes' streams start after everything already on the main stream."""
        if nlanes > 1:
            capi.event_record(lanes[0]["event"], main_stream)
            for ln in lanes[1:nlanes]:
                capi.stream_wait_event(ln["stream"], lanes[0]["event"])

    def join(nlanes):
        """The main stream continues after everything on the other lanes' streams."""
        for ln in lanes[1:nlanes]:
            capi.event_record(ln["event"], ln["stream"])
            capi.stream_wait_event(main_stream, ln["event"])

    # Each lane's calls are recorded once and the recordings are submitted side by
    # side, the way the reference records each operator into a command buffer and
    # Runtime::Run submits one batch per queue (core/runtime.cpp:404-458); a host
    # loop of ~10 us Python calls could not keep a ~10 us kernel fed.
    def record(count, first, nlanes, nb):
        """One recording per lane: the lane's share of steps first .. first+count-1, in order."""
        graphs = []
        for j in range(nlanes):
            mine = [i for i in range(first, first + count) if i % nlanes == j]
            if args.eager:
                graphs.append(mine)
                continue
            capi.graph_begin(lanes[j]["stream"])
            for i in mine:
                call(bufs[i % nb], lanes[j])
            graphs.append(capi.graph_end(lanes[j]["stream"]))
        return graphs

    def launch(graph, j, nb):
        if args.eager:
            for i in graph:
                call(bufs[i % nb], lanes[j])
        else:
            capi.graph_launch(graph, lanes[j]["stream"])

    def submit(graphs, nlanes, nb):
        fork(nlanes)
        for j in range(nlanes):
            launch(graphs[j], j, nb)
        join(nlanes)

    e0, e1 = capi.event_create(), capi.event_create()

    # spin kernel that holds the timed replay back until every lane is queued: sized
    # from a measurement of its own rate to about 2 ms (the host needs a few hundred
    # microseconds to queue the lanes from Python)
    gate_cycles, gate_ms = 0, 0.0
    if not args.no_gate and hasattr(torch.cuda, "_sleep"):
        probe = 1000000
        with torch.cuda.stream(torch_main):
            torch.cuda._sleep(probe)
            capi.event_record(e0, main_stream)
            torch.cuda._sleep(probe)
            capi.event_record(e1, main_stream)
        capi.event_sync(e1)
        per_cycle_ms = max(capi.event_elapsed_ms(e0, e1), 1e-6) / probe
        gate_ms = 4.0
        gate_cycles = int(gate_ms / per_cycle_ms)

    def gate():
        if gate_cycles:
            with torch.cuda.stream(torch_main):
                torch.cuda._sleep(gate_cycles)

    # The K-step recordings are replayed back to back until at least MIN_TIMED steps are
    # inside the timed region, lanes running free (no join between replays): with 20
    # steps and 4 lanes a single replay is five calls a lane, all lanes starting in the
    # same phase, which is the pipeline filling, not running.
    MIN_TIMED = 400
    replays = max(1, -(-MIN_TIMED // args.steps))

    def set_stages(stages):
        if args.kernel_legs:
            capi.measure_stages(stages)
        elif stages != 3:
            raise RuntimeError("one kernel by itself: only with --kernel-legs (the benchmark build of the library)")

    def timed(stages, nlanes, nb=nbuf, prime=False):
        """(device ms per step, host wall ms per step of ungated replays) after W warm-up steps."""
        set_stages(3)
        if prime:   # leave in every lane's workspace what a whole call on the (single) buffer leaves
            for ln in lanes[:nlanes]:
                call(bufs[0], ln)
                capi.stream_sync(ln["stream"])
        set_stages(stages)
        graphs = []
        if args.warmup > 0:
            gw = record(args.warmup, 0, nlanes, nb)
            graphs += gw
            submit(gw, nlanes, nb)
        gk = record(args.steps, args.warmup, nlanes, nb)
        graphs += gk

        def replay_all():
            fork(nlanes)
            for _ in range(replays):
                for j in range(nlanes):
                    launch(gk[j], j, nb)
            join(nlanes)
        # the recordings that are timed, once untimed: their first launch is not what is measured
        capi.stream_sync(main_stream)
        torch.cuda.synchronize()
        submit(gk, nlanes, nb)
        capi.stream_sync(main_stream)
        torch.cuda.synchronize()
        # host wall clock of the same replays without the gate (submission time included)
        t0 = time.perf_counter()
        replay_all()
        capi.stream_sync(main_stream)
        wall = (time.perf_counter() - t0) * 1e3
        torch.cuda.synchronize()
        # the timed replays: queued behind the gate, HIP events on the launch stream
        t0 = time.perf_counter()
        gate()
        capi.event_record(e0, main_stream)
        replay_all()
        capi.event_record(e1, main_stream)
        queued_ms = (time.perf_counter() - t0) * 1e3
        if gate_cycles and queued_ms > gate_ms:
            print("bench.py: queueing the lanes took %.2f ms, longer than the %.1f ms gate: the timed region "
                  "includes host submission time" % (queued_ms, gate_ms), file=sys.stderr)
        capi.event_sync(e1)
        torch.cuda.synchronize()
        if not args.eager:
            for g in graphs:
                capi.graph_destroy(g)
        set_stages(3)
        n = replays * args.steps
        return max(capi.event_elapsed_ms(e0, e1), 0.0) / n, wall / n

    # each kernel of the path by itself (same launches, same inputs, the other kernel
    # left out), then the whole step, which is the figure reported
    stage_ms = {}
    stage_overlapped = None
    plan = capi.rows_plan(capi.F32, shape, -1, k)
    path = capi.measure_path(capi.F32, shape, -1, k)
    names = PATH_KERNELS.get(path)
    two_kernels = names is not None and plan[2] > 1
    if args.kernel_legs:
        # one call in flight.  The second kernel by itself reads the workspace an earlier whole call
        # left; the pick kernel also reads the input again, so it is timed on one buffer with
        # that buffer's workspace (its few re-reads then come from the cache)
        if two_kernels:
            stage_ms[names[0]] = timed(1, 1)[0]
            stage_ms[names[1]] = timed(2, 1, 1, True)[0] if path == 2 else timed(2, 1)[0]
            if len(lanes) > 1:
                stage_overlapped = {names[0]: timed(1, len(lanes))[0] * 1e3,
                                    names[1]: (timed(2, len(lanes), 1, True)[0] if path == 2 else timed(2, len(lanes))[0]) * 1e3}
        print(json.dumps({"stage_ms": stage_ms, "stage_overlapped": stage_overlapped,
                          "library": os.path.basename(capi.LIB_PATH)}))
        return
    if args.timeline:
        capi.timeline_records()  # (the log starts here)
        ms, wall = timed(3, len(lanes))
        print(json.dumps(timeline_summary(capi.timeline_records(), ms, len(lanes), hw_queues)))
        return
    if args.headline_only:
        ms, wall = timed(3, len(lanes))
        print(json.dumps({"ms_per_step": ms, "rows_per_s": rows / (ms * 1e-3), "host_wall_ms_per_step": wall,
                          "calls_in_flight": len(lanes), "hw_queues": hw_queues,
                          "GPU_MAX_HW_QUEUES": os.environ.get("GPU_MAX_HW_QUEUES", "unset (HIP's default: 4)")}))
        return
    if kernel_legs is not None and "stage_ms" in kernel_legs:
        stage_ms = kernel_legs["stage_ms"]
        stage_overlapped = kernel_legs["stage_overlapped"]
    serial_ms = timed(3, 1)[0]
    ms_per_step, wall_per_step = timed(3, len(lanes))
    resident_ms = timed(3, len(lanes), 1)[0]
    # the kernel that moves the bytes (the first of the pair; the second reads a few kilobytes per row)
    dominant = names[0] if two_kernels else "the step's only kernel"
    dom_ms = stage_ms.get(dominant, serial_ms)

    achieved = algo_bytes / (dom_ms * 1e-3) / 1e9
    out = {
        "metric": "softmax+topk rows/s and % HBM roofline at [64,128256] fp32, k=50" if args.workload == "C3"
        else "softmax+topk rows/s, " + desc,
        "value": rows / (ms_per_step * 1e-3),
        "unit": "rows/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": desc, "k": k, "calls_in_flight": len(lanes), "hw_queues": hw_queues,
                   "kernels_per_call": 2 if two_kernels else 1, "kernels": list(names) if two_kernels else None,
                   "input_buffers_rotated": nbuf, "input_set_bytes": nbuf * in_bytes, "device": capi.device_info()[0],
                   "launch_shape": {"threads": plan[0], "loads_per_thread": plan[1], "chunks_per_row": plan[2]},
                   "timing": "HIP events on the launch stream around back-to-back replays of the recorded K steps (at least "
                             "400 steps in all, lanes running free), queued behind a spin kernel (%s); W warm-up steps and "
                             "one untimed replay of the same recordings before them"
                             % ("%.1f ms" % gate_ms if gate_cycles else "off")
                             if not args.eager else "EAGER host launches (a counter run): these timings are not the metric"},
        "steps_in_timed_region": replays * args.steps,
        "host_wall_ms_per_step": wall_per_step,
        "cache_resident_ms_per_step": resident_ms,
        "cache_resident_rows_per_s": rows / (resident_ms * 1e-3),
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic_from_profiles(args.workload, dominant),
                     "kernel": dominant,
                     "algorithmic_bytes_per_launch": algo_bytes,
                     "launch_us": dom_ms * 1e3,
                     "per_kernel_launch_us": {n: v * 1e3 for n, v in stage_ms.items()},
                     "per_kernel_us_with_calls_in_flight": stage_overlapped,
                     "whole_step_us": ms_per_step * 1e3,
                     "whole_step_frac": algo_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "whole_step_us_one_in_flight": serial_ms * 1e3,
                     "whole_step_frac_one_in_flight": algo_bytes / (serial_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "timing": "HIP events on the launch stream around %d back-to-back launches of that kernel alone, one "
                               "call in flight (recorded submissions); includes the gap between launches; measured in a child "
                               "process on libvkop_hip_bench.so, the library's build with the hook that leaves the other kernel "
                               "out (every other figure: libvkop_hip.so)" % (replays * args.steps),
                     "kernel_legs_error": (kernel_legs or {}).get("error")},
        "parity": parity,
    }
    # For a caller whose logits sit in host memory: upload over PCIe from pinned
    # memory, the fused call, results back to pinned memory, one call at a time on
    # one stream.  Reported beside the headline, never as it.
    try:
        if args.no_host:
            raise RuntimeError("skipped (--no-host)")
        ln = lanes[0]
        pin_in = torch.from_numpy(host_inputs[0]).pin_memory()
        pin_v = torch.empty((rows, k), dtype=torch.float32).pin_memory()
        pin_i = torch.empty((rows, k), dtype=torch.int32).pin_memory()
        reps = 20

        def host_round_trip():
            capi.memcpy_h2d(bufs[0].data_ptr(), pin_in.data_ptr(), in_bytes, ln["stream"])
            call(bufs[0], ln)
            capi.memcpy_d2h(pin_v.data_ptr(), ln["vals"].data_ptr(), rows * k * 4, ln["stream"])
            capi.memcpy_d2h(pin_i.data_ptr(), ln["idx"].data_ptr(), rows * k * 4, ln["stream"])
        host_round_trip()
        t0 = time.perf_counter()
        for _ in range(reps):
            host_round_trip()
        rt_ms = (time.perf_counter() - t0) * 1e3 / reps
        if not np.array_equal(pin_i.numpy(), oix):
            raise RuntimeError("host round trip returned other indices")
        out["host_buffers"] = {"ms_per_step": rt_ms, "rows_per_s": rows / (rt_ms * 1e-3),
                               "upload_GBps": in_bytes / (rt_ms * 1e-3) / 1e9,
                               "what": "pinned host logits -> device (PCIe) -> fused call -> top-k back to pinned host, "
                                       "blocking copies, one call at a time (host clock)"}
    except Exception as exc:  # the figure is informative only
        out["host_buffers"] = {"error": str(exc)}
    if default_queues is not None:
        out["with_the_environments_hw_queues"] = default_queues
    if runtime_api is not None:
        out["runtime_api"] = runtime_api
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(host_inputs[0], k)
    capi.event_destroy(e0)
    capi.event_destroy(e1)
    for ln in lanes:
        capi.event_destroy(ln["event"])
        capi.stream_destroy(ln["stream"])
    print(json.dumps(out))


if __name__ == "__main__":
    main()
