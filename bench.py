#!/usr/bin/env python3
"""Benchmark of the MI355X quantized FULLY_CONNECTED hot path (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-extras] [--skip-cpu]

A step is one pass of the headline workload: the hybrid dynamic-range FC of
14336 x 4096 (float32 activations quantized per row inside the op, int8 per-channel
weights) at decode batch sizes B = 1, 4 and 8, one op each. Every op is what the
delegate launches for the node: one kernel that quantizes the activation rows in its
prologue and streams the re-tiled int8 filter through the matrix cores. Inputs are resident in HBM before the timed region. Steps rotate over several
copies of the weights so that they are served from HBM rather than from the 256 MB
Infinity Cache ("cold"); the cache-hot rate is reported beside it.

Launches are replayed from HIP graphs, so the GPU runs kernels back to back and the
host's launch cost (which exceeds these kernels' few microseconds) stays out of the
measurement. Kernel durations for the roofline figures come from HIP events around
graph replays of that kernel alone.

The one JSON line printed at the end carries the headline value, the roofline of the
dominant kernel, the CPU baseline (the oracle port, one host core, bounded sample) and,
under "also", the other configurations of the benchmark contract.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "FC GEMV µs & HBM GB/s (% peak), int8 GEMM TOPS (% MFMA peak), 1 GPU"
HBM_PEAK_GBPS = 8000.0
INT8_MFMA_PEAK_TOPS = 5000.0
N_OUT, K_IN = 14336, 4096
BATCHES = (1, 4, 8)
WEIGHT_COPIES = 6  # 6 x 58.7 MB > 256 MB Infinity Cache


def hybrid_bytes(b, n=N_OUT, k=K_IN):
    """Algorithmic bytes of one hybrid FC op: W + per-channel scales + row sums + x + y."""
    return n * k + 4 * n + 4 * n + 4 * k * b + 4 * n * b


def int4_bytes(b, n, k, bs=32):
    return n * k // 2 + 2 * n * (k // bs) + 4 * k * b + 4 * n * b


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--skip-extras", action="store_true")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--traffic-probe-int4", action="store_true",
                    help="launch only what the int4 grouped kernel's counter runs need, then exit")
    ap.add_argument("--traffic-probe-int4-single", action="store_true",
                    help="launch only config 3's single-node int4 kernel (cold, 12 times) and the "
                         "64 MiB device copy (3 times), for a rocprofv3 counter or kernel-trace run")
    ap.add_argument("--gemm-probe", action="store_true",
                    help="launch only config 4's int8 GEMM: 10 times on the seeded operands, then 10 "
                         "times on constant operands (a second kernel name is not involved: the "
                         "two sets are told apart by launch order), for a rocprofv3 counter run")
    ap.add_argument("--sustain", type=float, default=0.0,
                    help="with --gemm-probe: afterwards keep launching the GEMM for this many seconds "
                         "on the seeded operands, then as long on the constant ones, printing a "
                         "time-stamped line at each switch; socket power (hwmon) and `rocm-smi --showclocks` are "
                         "sampled beside it by a child process and the medians per phase are printed")
    ap.add_argument("--roofline-probe", action="store_true",
                    help="only the cold B=1 launches of config 2 that roofline.avg_launch_us is "
                         "taken over (for a rocprofv3 --kernel-trace --stats run)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="launch only the dominant kernel (cold, 12 times) and a 64 MiB device "
                         "copy (3 times), for a rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the op would shard "
              "by output channel with no collective). Run with --gpus 1.",
              file=sys.stderr)
        sys.exit(2)

    sampler = None
    if args.gemm_probe and args.sustain > 0:
        sampler = start_smi_sampler()  # a child process, started before this one touches the GPU

    import torch
    from litert_amd import capi
    from litert_amd import fully_connected as fc
    from litert_amd import workloads as wl

    if not torch.cuda.is_available():
        print("bench.py needs a gfx950 GPU", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    fc._ensure_init()
    lib = capi.load()
    p = lambda t: None if t is None else C.c_void_p(t.data_ptr())
    stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)

    if args.traffic_probe:
        traffic_probe(torch, fc, wl)
        return
    if args.traffic_probe_int4:
        traffic_probe_int4(torch, fc, wl)
        return
    if args.gemm_probe:
        phases = []
        try:
            phases = gemm_probe(torch, fc, wl, args.sustain)
        finally:  # the sampler is a child process of its own: never leave it behind
            if sampler is not None:
                report_smi_samples(sampler, phases)
        return
    if args.traffic_probe_int4_single:
        traffic_probe_int4_single(torch, fc, wl)
        return

    def timed_replays(graphs, reps):
        """Average milliseconds per replay, graphs[i % len] replayed reps times."""
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(reps):
            graphs[i % len(graphs)].replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    def capture(fn):
        fn()  # warm: sets function attributes, touches lazily loaded code objects
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        return g

    if args.roofline_probe:
        roofline_probe(torch, fc, wl, capture, timed_replays)
        return

    # ---- headline workload: config 2 -------------------------------------------------
    c = wl.hybrid_fc(max(BATCHES))
    ops = []
    for i in range(WEIGHT_COPIES):
        ops.append(fc.FullyConnectedHybrid(np.roll(c["w"], i, axis=0) if i else c["w"],
                                           np.roll(c["pcs"], i) if i else c["pcs"]))
    x_all = torch.from_numpy(c["x"]).cuda()
    xs = {b: x_all[:b].contiguous() for b in BATCHES}
    outs = {b: torch.empty((b, N_OUT), dtype=torch.float32, device="cuda") for b in BATCHES}

    def step_fn(op):
        def run():
            for b in BATCHES:
                op(xs[b], out=outs[b])
        return run

    # One graph holds one step on each weight copy (6 steps, 36 kernels), so that the
    # GPU, not the host's replay call, sets the pace; K % 6 leftover steps replay
    # single-step graphs.
    step_graphs = [capture(step_fn(op)) for op in ops]
    round_fns = [step_fn(op) for op in ops]
    round_graph = capture(lambda: [f() for f in round_fns])
    hot_graph = capture(lambda: [round_fns[0]() for _ in ops])
    for i in range(args.warmup):
        step_graphs[i % len(ops)].replay()
    torch.cuda.synchronize()
    # exactly K timed steps, bracketed by synchronize on both sides
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps // len(ops)):
        round_graph.replay()
    for i in range(args.steps % len(ops)):
        step_graphs[i].replay()
    e1.record()
    torch.cuda.synchronize()
    wall_ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_cold = e0.elapsed_time(e1) / args.steps
    ms_hot = timed_replays([hot_graph], max(args.steps // len(ops), 1)) / len(ops)
    step_bytes = sum(hybrid_bytes(b) for b in BATCHES)
    value = step_bytes / (ms_cold * 1e-3) / 1e9

    # ---- per-kernel durations for the roofline -----------------------------------------
    # The op is ONE kernel (FcInt8ResidentGemvKernel, hybrid epilogue, quantization fused into
    # its prologue), so op time and dominant-kernel time coincide.
    ROUNDS = 4  # launches per graph = ROUNDS x weight copies

    def many(fns):
        """Graph of ROUNDS passes over fns; returns (graph, launches per replay)."""
        return capture(lambda: [f() for _ in range(ROUNDS) for f in fns]), ROUNDS * len(fns)

    def per_launch_us(fns, replays=25):
        g, n = many(fns)
        return timed_replays([g], replays) * 1e3 / n

    def per_launch_stats(fns, replays=25):
        """(median, min) microseconds per launch over `replays` separately timed replays."""
        g, n = many(fns)
        g.replay()
        samples = []
        for _ in range(replays):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            samples.append(e0.elapsed_time(e1) * 1e3 / n)
        samples.sort()
        return samples[len(samples) // 2], samples[0]

    per_b = {}
    for b in BATCHES:
        cold_us = per_launch_us([(lambda o: lambda: o(xs[b], out=outs[b]))(op) for op in ops])
        hot_us = per_launch_us([lambda: ops[0](xs[b], out=outs[b])] * len(ops))
        med_us, min_us = per_launch_stats([(lambda o: lambda: o(xs[b], out=outs[b]))(op) for op in ops])
        per_b[b] = dict(op_us_cold=round(cold_us, 3), op_us_cold_median=round(med_us, 3),
                        op_us_cold_min=round(min_us, 3), op_us_hot=round(hot_us, 3),
                        op_gbps_cold=round(hybrid_bytes(b) / cold_us / 1e3, 1),
                        op_gbps_hot=round(hybrid_bytes(b) / hot_us / 1e3, 1),
                        frac_of_hbm_peak_cold=round(hybrid_bytes(b) / cold_us / 1e3 / HBM_PEAK_GBPS, 4))
    # The op picks the fused kernel up to FUSED_MAX_BATCHES rows and quantizer + GEMV above;
    # both forms timed at every batch size show where the crossover lies.
    forms = {}
    for b in BATCHES:
        fused_max = fc.FullyConnectedHybrid.FUSED_MAX_BATCHES
        try:
            fc.FullyConnectedHybrid.FUSED_MAX_BATCHES = 1 << 30
            fused_us = per_launch_us([(lambda o: lambda: o(xs[b], out=outs[b]))(op) for op in ops])
        finally:
            fc.FullyConnectedHybrid.FUSED_MAX_BATCHES = fused_max
        split_us = per_launch_us([(lambda o: lambda: o.call_split(xs[b], out=outs[b]))(op)
                                  for op in ops])
        forms[b] = dict(fused_us_cold=round(fused_us, 3), split_us_cold=round(split_us, 3))
    # What the memory system alone needs for a launch of this size: a kernel that only streams
    # the same bytes (the re-tiled filter of each weight copy) with the GEMV's access pattern.
    from litert_amd import bench_probes as probes
    plib = probes.load()

    def stream_floor(buffers, nbytes):
        sink = torch.zeros(1, dtype=torch.int32, device="cuda")
        fns = [(lambda t: lambda: probes.check(plib.lrtprobe_stream_read(p(t), nbytes, p(sink),
                                                                           stream())))(t)
               for t in buffers]
        return per_launch_us(fns)

    floor2_us = stream_floor([op.packed_filter for op in ops], N_OUT * K_IN)
    b_dom = 1
    achieved = hybrid_bytes(b_dom) / per_b[b_dom]["op_us_cold"] / 1e3
    roofline = dict(bound="hbm",
                    kernel="FcInt8ResidentGemvKernel<hybrid, fused quantize> (config 2, B=1, cold)",
                    achieved=round(achieved, 1), peak=HBM_PEAK_GBPS, unit="GB/s",
                    frac=round(achieved / HBM_PEAK_GBPS, 4), traffic=measured_traffic(),
                    traffic_source="profiles/hybrid_gemv_fused_B1_hbm_traffic.txt (rocprofv3 --pmc "
                                   "FETCH_SIZE / WRITE_SIZE of `bench.py --traffic-probe`; a committed "
                                   "counter summary, not measured in this run)",
                    traffic_commit=measured_traffic("library built from commit"),
                    algorithmic_bytes_per_launch=hybrid_bytes(b_dom),
                    avg_launch_us=per_b[b_dom]["op_us_cold"],
                    stream_only_us=round(floor2_us, 3),
                    stream_only_note="a launch that only reads the same 58.7 MB filter (same "
                                     "access pattern, cold): the memory system's own time for "
                                     "this size, %.1f%% of peak" % (N_OUT * K_IN / floor2_us / 1e3 /
                                                                  HBM_PEAK_GBPS * 100))

    # Between decode and prefill (not one of the benchmark configurations): config 2's filters against 16
    # and 32 rows (row quantizer + register-resident GEMV), 64 and 128 rows (row quantizer + the
    # GEMV that walks the rows through LDS in depth chunks) and 512 rows (row quantizer + MFMA
    # GEMM).
    between = {}
    gen = torch.Generator(device="cuda").manual_seed(99)
    for rows in (16, 32, 64, 128, 512):
        xm = torch.randn((rows, K_IN), device="cuda", generator=gen)
        ym = torch.empty((rows, N_OUT), dtype=torch.float32, device="cuda")
        us = per_launch_us([(lambda o: lambda: o(xm, out=ym))(op) for op in ops])
        between["us_%d_rows" % rows] = round(us, 1)
        between["tops_%d_rows" % rows] = round(2.0 * rows * K_IN * N_OUT / us / 1e6, 1)

    also = {"config2_hybrid_per_batch": per_b, "config2_fused_vs_split": forms,
            "config2_step_ms_hot": round(ms_hot, 5),
            "config2_step_gbps_hot": round(step_bytes / (ms_hot * 1e-3) / 1e9, 1),
            "next_hybrid_between_decode_and_prefill_14336x4096": between}

    if not args.skip_extras:
        also.update(extras(torch, fc, capi, lib, wl, p, stream, capture, timed_replays, per_launch_us))

    cpu_baseline = None
    if not args.skip_cpu:
        cpu_baseline = cpu_baseline_leg(c)

    line = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_cold, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "configs[1]: hybrid f32 x int8 per-channel FULLY_CONNECTED "
                               "14336x4096, one op each at B=1,4,8 per step (one fused "
                               "quantize+GEMV kernel per op), weights rotated over %d copies (HBM-cold)"
                               % WEIGHT_COPIES,
                   "algorithmic_bytes_per_step": step_bytes,
                   "host_wall_ms_per_step": round(wall_ms_per_step, 5)},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "also": also,
    }
    print(json.dumps(line))


def mfma_rate(torch, seconds, random_operands):
    """Sustained rate (TOPS) of the matrix cores alone on this part: lrtprobe_mfma_rate (256
    workgroups x 4 wavefronts, register operands, no memory traffic) launched back to back for
    about `seconds`, wall-clock timed around device synchronisations."""
    import ctypes
    from litert_amd import bench_probes as probes
    plib = probes.load()
    sink = torch.empty(256 * 256, dtype=torch.int32, device="cuda")
    ops = ctypes.c_double(0.0)
    stream = torch.cuda.current_stream().cuda_stream

    def launch(n):
        for _ in range(n):
            probes.check(plib.lrtprobe_mfma_rate(256, 2000, int(random_operands), sink.data_ptr(),
                                                  ctypes.byref(ops), stream))
        torch.cuda.synchronize()

    launch(2)
    t0 = time.time()
    launches = 0
    while time.time() - t0 < seconds:
        launch(20)   # 20 launches of about 0.8 ms
        launches += 20
    return ops.value * launches / (time.time() - t0) / 1e12


def start_smi_sampler():
    """Starts a sampling loop (a time stamp, the socket power from the amdgpu hwmon node
    power1_input -- `rocm-smi --showpower` prints nothing for an ordinary user here --, then
    `rocm-smi --showclocks`, about three times a second) as a child process group of its own,
    writing to a temporary file. Returns (process, path)."""
    import subprocess
    import tempfile
    fd, path = tempfile.mkstemp(prefix="lrtfc_smi_", suffix=".log")
    # The loop ends by itself after five minutes, whatever becomes of this process.
    loop = ("end=$((SECONDS+300)); while [ $SECONDS -lt $end ]; do echo t=$(date +%s.%N); "
            "echo power_uw=$(cat /sys/class/drm/card*/device/hwmon/hwmon*/power1_input 2>/dev/null | head -1); "
            "rocm-smi --showclocks 2>&1; sleep 0.2; done")
    proc = subprocess.Popen(["bash", "-c", loop], stdout=fd, stderr=subprocess.STDOUT,
                            start_new_session=True)
    os.close(fd)

    def stop():  # also on an early exit of bench.py (no GPU, an import that fails)
        import signal
        try:
            os.killpg(proc.pid, signal.SIGTERM)
        except (ProcessLookupError, PermissionError):
            pass
        try:
            os.unlink(path)
        except OSError:
            pass
    import atexit
    atexit.register(stop)
    return proc, path


def report_smi_samples(sampler, phases):
    """Stops the sampler and prints, per phase of the sustained run, the median shader clock and
    socket power of the samples taken from one second into the phase on."""
    import re
    import signal
    proc, path = sampler
    try:
        os.killpg(proc.pid, signal.SIGTERM)
    except ProcessLookupError:
        pass
    proc.wait()
    samples, now = [], None
    for ln in open(path, errors="replace"):
        m = re.match(r"t=([0-9.]+)", ln)
        if m:
            now = [float(m.group(1)), None, None]
            samples.append(now)
            continue
        if now is None:
            continue
        m = re.search(r"sclk clock level:\s*\d+:?\s*\((\d+)Mhz\)", ln)
        if m and now[1] is None:
            now[1] = float(m.group(1))
        m = re.match(r"power_uw=(\d+)", ln)
        if m and now[2] is None:
            now[2] = float(m.group(1)) / 1e6
    os.unlink(path)

    def median(v):
        v = sorted(v)
        return v[len(v) // 2] if v else None

    for name, begin, end in phases:
        inside = [s for s in samples if begin + 1.0 <= s[0] <= end]
        print(json.dumps({"sustain": name, "smi_samples": len(inside),
                          "sclk_mhz_median": median([s[1] for s in inside if s[1] is not None]),
                          "power_w_median": median([s[2] for s in inside if s[2] is not None])}),
              flush=True)


def roofline_probe(torch, fc, wl, capture, timed_replays):
    """Only the launches behind roofline.avg_launch_us: config 2 at B = 1, one fused kernel per
    op, the filter copies rotated so that every launch streams from HBM, 24 launches per graph
    replayed 25 times (after one warm call per copy and one capture pass). Under
    `rocprofv3 --kernel-trace --stats` the kernel's average duration is over the same launches
    as the figure printed here, which is taken with events around the replays and so also holds
    the gaps between launches."""
    c = wl.hybrid_fc(1)
    ops = [fc.FullyConnectedHybrid(np.roll(c["w"], i, axis=0) if i else c["w"],
                                   np.roll(c["pcs"], i) if i else c["pcs"])
           for i in range(WEIGHT_COPIES)]
    x = torch.from_numpy(c["x"]).cuda()
    y = torch.empty((1, N_OUT), dtype=torch.float32, device="cuda")
    g = capture(lambda: [op(x, out=y) for _ in range(4) for op in ops])
    us = timed_replays([g], 25) * 1e3 / (4 * len(ops))
    print(json.dumps({"probe": "roofline", "launches_per_replay": 4 * len(ops), "replays": 25,
                      "avg_launch_us_by_events": round(us, 3),
                      "algorithmic_bytes": hybrid_bytes(1)}))


def traffic_probe(torch, fc, wl):
    """The launches a counter run needs and nothing else: the fused hybrid kernel at B = 1
    on rotating weight copies (so every launch streams its filter from HBM) and a plain
    device-to-device copy of 64 MiB, whose known 64 MiB read and 64 MiB written calibrate
    the counters' unit."""
    c = wl.hybrid_fc(1)
    ops = [fc.FullyConnectedHybrid(np.roll(c["w"], i, axis=0) if i else c["w"], c["pcs"])
           for i in range(WEIGHT_COPIES)]
    x = torch.from_numpy(c["x"]).cuda()
    y = torch.empty((1, N_OUT), dtype=torch.float32, device="cuda")
    src = torch.ones(64 << 20, dtype=torch.int8, device="cuda")
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for i in range(12):
        ops[i % len(ops)](x, out=y)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    print(json.dumps({"probe": "traffic", "hybrid_launches": 12, "copy_launches": 3,
                      "copy_bytes": 64 << 20, "algorithmic_bytes": hybrid_bytes(1)}))


def gemm_probe(torch, fc, wl, sustain=0.0):
    """Counter-run launches for config 4's kernel alone (FcInt8PackedGemmKernel, requantizing
    epilogue, RELU6): ten launches on the seeded U[-128,127] operands, then ten on constant
    operands (x = 3, w = 5). With `sustain` seconds, each set is then launched back to back for
    that long, so that a sampler outside the process can read the power and clocks the part
    settles at."""
    c4 = wl.prefill_int8_fc()
    y4 = torch.empty((2048, 4096), dtype=torch.int8, device="cuda")
    sets = []
    for name, w, x in (("seeded", c4["w"], torch.from_numpy(c4["x"]).cuda()),
                       ("constant", np.full_like(c4["w"], 5),
                        torch.full((2048, 4096), 3, dtype=torch.int8, device="cuda"))):
        op = fc.FullyConnectedInt8(w, c4["bias"], float(c4["in_scale"]), c4["in_zp"], c4["w_scale"],
                                   float(c4["out_scale"]), c4["out_zp"], activation="relu6")
        torch.cuda.synchronize()
        for _ in range(10):
            op(x, out=y4)
        torch.cuda.synchronize()
        sets.append((name, op, x))
    print(json.dumps({"probe": "gemm", "launches_seeded": 10, "launches_constant": 10,
                      "ops_per_launch": 2 * 2048 * 4096 * 4096}), flush=True)
    phases = []  # (name, begin, end) in unix seconds, for the power / clock samples
    if sustain > 0:
        for name, rnd in (("random", 1), ("constant", 0)):
            t0 = time.time()
            print(json.dumps({"sustain": "mfma_only_" + name, "begin_unix": round(t0, 3)}), flush=True)
            tops = mfma_rate(torch, sustain, rnd)
            phases.append(("mfma_only_" + name, t0, time.time()))
            print(json.dumps({"sustain": "mfma_only_" + name, "end_unix": round(time.time(), 3),
                              "tops": round(tops, 1)}), flush=True)
    for name, op, x in sets if sustain > 0 else []:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(50):
                op(x, out=y4)
        t0 = time.time()
        print(json.dumps({"sustain": name, "begin_unix": round(t0, 3)}), flush=True)
        launches = 0
        while time.time() - t0 < sustain:
            for _ in range(20):
                g.replay()
            torch.cuda.synchronize()
            launches += 1000
        t1 = time.time()
        phases.append((name, t0, t1))
        print(json.dumps({"sustain": name, "end_unix": round(t1, 3), "launches": launches,
                          "us_per_launch": round((t1 - t0) / launches * 1e6, 2)}), flush=True)
    return phases


def traffic_probe_int4_single(torch, fc, wl):
    """Counter-run launches for config 3's kernel alone: the fused blockwise-int4 GEMV of
    14336 x 4096 at B = 1 on rotating copies of the filter, plus the calibrating 64 MiB copy."""
    c3 = wl.blockwise_int4_fc(1)
    ops3 = [fc.FullyConnectedBlockwiseInt4(np.roll(c3["packed"], i, axis=0),
                                           np.roll(c3["scales"], i, axis=0), 4096, 32)
            for i in range(8)]
    x = torch.from_numpy(c3["x"]).cuda()
    y = torch.empty((1, 14336), dtype=torch.float32, device="cuda")
    src = torch.ones(64 << 20, dtype=torch.int8, device="cuda")
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for i in range(12):
        ops3[i % len(ops3)](x, out=y)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    print(json.dumps({"probe": "traffic-int4-single", "int4_launches": 12, "copy_launches": 3,
                      "copy_bytes": 64 << 20, "algorithmic_bytes": int4_bytes(1, 14336, 4096)}))


def traffic_probe_int4(torch, fc, wl):
    """Counter-run launches for the grouped int4 kernel: config 5's 108 nodes of depth 2048 in
    ONE launch (B = 1), four times, plus the 64 MiB copy that calibrates the counters."""
    g = torch.Generator(device="cuda").manual_seed(5)
    ops, total = [], 0
    for _ in range(wl.GEMMA2B_LAYERS):
        for name, k, n in wl.GEMMA2B_LAYER_FCS:
            if k != 2048:
                continue
            packed = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device="cuda", generator=g)
            scales = (torch.rand((n, k // 32), device="cuda", generator=g) * 1.5e-2 + 5e-3).half()
            ops.append(fc.FullyConnectedBlockwiseInt4(packed, scales, k, 32))
            total += int4_bytes(1, n, k)
    x = torch.randn((1, 2048), device="cuda", generator=g)
    ys = [torch.empty((1, op.out_depth), dtype=torch.float32, device="cuda") for op in ops]
    group = fc.GroupedBlockwiseInt4(ops).bind([x] * len(ops), ys)
    src = torch.ones(64 << 20, dtype=torch.int8, device="cuda")
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for _ in range(4):
        group()
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    print(json.dumps({"probe": "traffic-int4", "grouped_launches": 4, "nodes": len(ops),
                      "copy_launches": 3, "copy_bytes": 64 << 20, "algorithmic_bytes": total}))


def measured_traffic(field="traffic_bytes_per_launch:"):
    """HBM bytes per launch of the dominant kernel, from the committed counter summary
    (two rocprofv3 --pmc runs of `bench.py --traffic-probe`); None when it is absent.
    field "library built from commit" returns the commit the summary was taken at."""
    path = os.path.join(ROOT, "profiles", "hybrid_gemv_fused_B1_hbm_traffic.txt")
    try:
        for ln in open(path):
            if ln.startswith(field):
                tail = ln[len(field):].split()
                return int(tail[0]) if field.endswith(":") else tail[0]
    except OSError:
        pass
    return None


def extras(torch, fc, capi, lib, wl, p, stream, capture, timed_replays, per_launch_us):
    """Configs 1, 3, 4 and 5 of the benchmark contract (reported under "also")."""
    from litert_amd import bench_probes as probes
    plib = probes.load()
    out = {}
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()

    # config 1: int8 GEMV 2048 -> 2048, B = 1 (4 MiB of weights: launch-latency dominated)
    c1 = wl.int8_fc()
    op1 = fc.FullyConnectedInt8(c1["w"], c1["bias"], float(c1["in_scale"]), c1["in_zp"],
                                c1["w_scale"], float(c1["out_scale"]), c1["out_zp"])
    x1 = dev(c1["x"])
    y1 = torch.empty((1, 2048), dtype=torch.int8, device="cuda")
    us = per_launch_us([lambda: op1(x1, out=y1)] * 6)
    b1 = 2048 * 2048 + 2048 + 3 * 4 * 2048 + 2048
    out["config1_int8_gemv_2048x2048_B1"] = dict(us=round(us, 3), gbps=round(b1 / us / 1e3, 1),
                                                 frac_of_hbm_peak=round(b1 / us / 1e3 / HBM_PEAK_GBPS, 4),
                                                 note="weights fit in cache: hot figure")

    # config 3: blockwise int4 GEMV 14336 x 4096, B = 1
    c3 = wl.blockwise_int4_fc(1)
    ops3 = [fc.FullyConnectedBlockwiseInt4(np.roll(c3["packed"], i, axis=0), np.roll(c3["scales"], i, axis=0),
                                           4096, 32) for i in range(8)]
    x3 = dev(c3["x"])
    y3 = torch.empty((1, 14336), dtype=torch.float32, device="cuda")
    q3 = fc.batch_quantize_floats(x3)

    def int4_kernel_only(op):
        def run():
            capi.check(lib.lrtfc_fc_blockwise_int4_packed_quantized(
                p(q3[0]), p(q3[1]), p(q3[2]), p(op.retiled), p(op.kfsum), None, p(y3),
                1, 4096, 14336, stream()))
        return run

    def decode_rows(op, xin, yout):
        capi.check(lib.lrtfc_fc_blockwise_int4_packed(p(xin), p(op.retiled), p(op.kfsum), None, p(yout),
                                                       xin.shape[0], 4096, 14336, op.variant, stream()))

    # op = one kernel (quantizer fused into the prologue); "prequantized" = the same kernel
    # handed rows that were quantized beforehand, i.e. without the prologue's work.
    o_cold = per_launch_us([(lambda o: lambda: o(x3, out=y3))(op) for op in ops3])
    o_hot = per_launch_us([lambda: ops3[0](x3, out=y3)] * len(ops3))
    k_cold = per_launch_us([int4_kernel_only(op) for op in ops3])
    b3 = int4_bytes(1, 14336, 4096)
    sink3 = torch.zeros(1, dtype=torch.int32, device="cuda")
    floor3 = per_launch_us([(lambda o: lambda: probes.check(plib.lrtprobe_stream_read(
        p(o.retiled), o.retiled.numel(), p(sink3), stream())))(op) for op in ops3])
    out["config3_int4_gemv_14336x4096_B1"] = dict(
        stream_only_us=round(floor3, 3),
        stream_only_frac_of_hbm_peak=round(ops3[0].retiled.numel() / floor3 / 1e3 / HBM_PEAK_GBPS, 4),
        op_us_cold=round(o_cold, 3), op_us_hot=round(o_hot, 3),
        prequantized_kernel_us_cold=round(k_cold, 3),
        op_gbps_cold=round(b3 / o_cold / 1e3, 1), op_gbps_hot=round(b3 / o_hot / 1e3, 1),
        frac_of_hbm_peak_cold=round(b3 / o_cold / 1e3 / HBM_PEAK_GBPS, 4), algorithmic_bytes=b3,
        kernel="FcInt4PackedKernel<fused quantize> on the re-tiled filter")
    # Prefill batches on the blockwise int4 path (not one of the benchmark configurations): config 3's filter
    # against 2048 and 128 rows through the matrix-core GEMM (row quantizer + GEMM launches),
    # and what the decode kernel needs for the same rows in passes of four.
    op3 = fc.FullyConnectedBlockwiseInt4(c3["packed"], c3["scales"], 4096, 32)
    entry = {}
    for rows in (128, 2048):
        xg = torch.randn((rows, 4096), device="cuda", generator=torch.Generator(device="cuda").manual_seed(rows))
        yg = torch.empty((rows, 14336), dtype=torch.float32, device="cuda")
        us = per_launch_us([lambda: op3.call_gemm(xg, out=yg)] * 4, replays=5)
        entry["us_%d_rows" % rows] = round(us, 1)
        entry["tops_%d_rows" % rows] = round(2.0 * rows * 4096 * 14336 / us / 1e6, 1)
    passes = per_launch_us([lambda: [ops3[0](xg[i:i + 4], out=yg[i:i + 4]) for i in range(0, 128, 4)]],
                           replays=5)
    entry["us_128_rows_decode_kernel_passes"] = round(passes, 1)
    entry["kernel"] = "FcInt4BlockwiseGemmKernel (v_mfma_i32_16x16x32_i8 per block, float32 accumulators in block order)"
    out["next_int4_blockwise_prefill_14336x4096"] = entry
    del op3

    # Between decode and prefill on the blockwise int4 path (not one of the benchmark configurations): the
    # op as dispatched (lrtfc_fc_blockwise_int4_preferred_form picks the form per shape), filter
    # copies rotated (cold), and the forms it chose against at 8 and 16 rows.
    forms = {capi.INT4_FORM_DECODE: "decode kernel", capi.INT4_FORM_GEMM_NIBBLES: "4-bit-resident GEMM",
             capi.INT4_FORM_GEMM_INT8: "int8-expanded GEMM"}
    entry = {}
    for rows in (2, 4, 8, 16, 32):
        xg = torch.randn((rows, 4096), device="cuda", generator=torch.Generator(device="cuda").manual_seed(rows))
        yg = torch.empty((rows, 14336), dtype=torch.float32, device="cuda")
        us = per_launch_us([(lambda o: lambda: o(xg, out=yg))(o) for o in ops3])
        entry["us_%d_rows" % rows] = round(us, 2)
        entry["form_%d_rows" % rows] = forms[lib.lrtfc_fc_blockwise_int4_preferred_form(rows, 4096, 14336)]
        if rows in (8, 16):
            entry["us_%d_rows_decode_kernel_passes" % rows] = round(per_launch_us(
                [(lambda o: lambda: [decode_rows(o, xg[i:i + 4], yg[i:i + 4]) for i in range(0, rows, 4)])(o)
                 for o in ops3]), 2)
            entry["us_%d_rows_int8_expanded_gemm" % rows] = round(per_launch_us(
                [(lambda o: lambda: o.call_gemm(xg, out=yg))(o) for o in ops3]), 2)
    entry["kernel"] = ("FcInt4NibbleGemmKernel (filter stays 4 bits per weight; nibbles expanded in registers "
                       "into the v_mfma_i32_16x16x32_i8 operand; row quantizer launch + GEMM launch)")
    out["next_int4_blockwise_between_decode_and_prefill_14336x4096"] = entry

    del ops3

    # Next-row op (not one of the benchmark configurations): per-channel int4 hybrid FC (EvalHybridDense4Bit)
    # at config 3's shape, B = 1, on the 4-bit-resident filter and on its int8 expansion.
    g4 = torch.Generator(device="cuda").manual_seed(11)
    nib = [torch.randint(0, 256, (14336, 2048), dtype=torch.uint8, device="cuda", generator=g4)
           for _ in range(6)]
    fs4 = np.random.default_rng(3).uniform(0.01, 0.1, 14336).astype(np.float32)
    ops4b = [fc.FullyConnectedHybridInt4PerChannel(n, 4096, fs4) for n in nib]
    y4b = torch.empty((1, 14336), dtype=torch.float32, device="cuda")
    us_nib = per_launch_us([(lambda o: lambda: o(x3, out=y4b))(o) for o in ops4b])
    us_i8 = per_launch_us([(lambda o: lambda: o(x3, out=y4b, force_int8=True))(o) for o in ops4b])
    bytes_nib = 14336 * 2048 + 14336 * 4 + 4096 * 4 + 14336 * 4
    out["next_int4_per_channel_hybrid_14336x4096_B1"] = dict(
        us_cold_4bit_resident=round(us_nib, 3), us_cold_int8_expansion=round(us_i8, 3),
        gbps_cold=round(bytes_nib / us_nib / 1e3, 1),
        frac_of_hbm_peak_cold=round(bytes_nib / us_nib / 1e3 / HBM_PEAK_GBPS, 4),
        algorithmic_bytes=bytes_nib,
        note="4-bit-resident: one kernel (row quantizer fused into the prologue); int8 expansion: row quantizer launch + GEMV launch")
    del ops4b, nib

    # Next-row op: EMBEDDING_LOOKUP from a blockwise Int4 table of a 256000-token vocabulary,
    # 2048 columns, block size 32 (what feeds config 5's first layer): one decode token and a
    # prefill batch of 2048 tokens. Bytes per looked-up row: 1024 of nibbles + 128 of scales
    # read, 8192 of float32 written.
    from litert_amd import embedding_lookup as el
    g5 = torch.Generator(device="cuda").manual_seed(13)
    table = torch.randint(0, 256, (256000, 1024), dtype=torch.uint8, device="cuda", generator=g5)
    tscales = (torch.rand((256000, 64), device="cuda", generator=g5) * 2e-2 + 1e-3).half()
    lookup_op = el.EmbeddingLookupBlockwiseInt4(table, tscales, 2048, 32)
    entry = {}
    for count in (1, 2048):
        ids = [torch.randint(0, 256000, (count,), dtype=torch.int32, device="cuda", generator=g5)
               for _ in range(8)]
        rows_out = torch.empty((count, 2048), dtype=torch.float32, device="cuda")
        us = per_launch_us([(lambda t: lambda: lookup_op(t, out=rows_out, check=False))(t) for t in ids])
        moved = count * (1024 + 128 + 8192 + 4)
        entry["us_%d_tokens" % count] = round(us, 3)
        entry["gbps_%d_tokens" % count] = round(moved / us / 1e3, 1)
        if count == 2048:
            entry["frac_of_hbm_peak_2048_tokens"] = round(moved / us / 1e3 / HBM_PEAK_GBPS, 4)
            entry["algorithmic_bytes_2048_tokens"] = moved
    entry["kernel"] = "EmbeddingLookupKernel<Int4, float32, 8 columns per thread; from 32 rows on as two runs of 4>"
    out["next_embedding_lookup_blockwise_int4_256000x2048"] = entry
    del table, tscales, lookup_op

    # config 4: prefill int8 GEMM 2048 x 4096 x 4096, RELU6 off / on
    c4 = wl.prefill_int8_fc()
    x4 = dev(c4["x"])
    y4 = torch.empty((2048, 4096), dtype=torch.int8, device="cuda")
    ops_per_call = 2.0 * 2048 * 4096 * 4096
    # The two activations are timed in alternation, replay by replay, so that clock drift over
    # the run lands on both alike; median and minimum over the replays are reported.
    ops4 = {act: fc.FullyConnectedInt8(c4["w"], c4["bias"], float(c4["in_scale"]), c4["in_zp"],
                                       c4["w_scale"], float(c4["out_scale"]), c4["out_zp"],
                                       activation=act) for act in ("none", "relu6")}
    # 64 launches per replay (about 2.5 ms): long enough that the clock ramp after the idle gap
    # between two replays does not colour the figure.
    graphs4 = {act: (capture((lambda o: lambda: [o(x4, out=y4) for _ in range(64)])(op)), 64)
               for act, op in ops4.items()}
    samples4 = {act: [] for act in ops4}
    for g, _ in graphs4.values():
        g.replay()
    torch.cuda.synchronize()
    for _ in range(25):
        for act, (g, n) in graphs4.items():
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            samples4[act].append(e0.elapsed_time(e1) * 1e3 / n)
    for act, samples in samples4.items():
        samples.sort()
        us, us_min = samples[len(samples) // 2], samples[0]
        tops = ops_per_call / us / 1e6
        out["config4_int8_gemm_2048x4096x4096_" + act] = dict(
            us=round(us, 2), us_min=round(us_min, 2), tops=round(tops, 1),
            frac_of_int8_mfma_peak=round(tops / INT8_MFMA_PEAK_TOPS, 4),
            timing="median (us) and minimum (us_min) of 25 graph replays, alternating with the other activation")
    del graphs4
    # The same launch on constant operands (every x = 3, every w = 5). The kernel executes the same
    # instructions in the same number of cycles; only the switching activity differs. The gap
    # to the seeded U[-128,127] operands above is the clock the part sustains under that
    # activity (power limit), not something the kernel's schedule can win back.
    op4c = fc.FullyConnectedInt8(np.full_like(c4["w"], 5), c4["bias"], float(c4["in_scale"]),
                                 c4["in_zp"], c4["w_scale"], float(c4["out_scale"]), c4["out_zp"])
    x4c = torch.full_like(x4, 3)
    us_c = per_launch_us([lambda: op4c(x4c, out=y4)] * 16)
    out["config4_int8_gemm_constant_operands"] = dict(
        us=round(us_c, 2), tops=round(ops_per_call / us_c / 1e6, 1),
        frac_of_int8_mfma_peak=round(ops_per_call / us_c / 1e6 / INT8_MFMA_PEAK_TOPS, 4),
        note="same kernel and launch, x = 3 and w = 5 everywhere: lower switching activity, higher sustained clock")
    # The matrix cores alone (no operand traffic, one wavefront per SIMD as in the GEMM), 0.4 s
    # each: what this part sustains under its power limit, against the nominal 5.0 POPS.
    probe_random, probe_constant = mfma_rate(torch, 0.4, 1), mfma_rate(torch, 0.4, 0)
    out["config4_matrix_cores_alone"] = dict(
        tops_random_operands=round(probe_random, 1), tops_constant_operands=round(probe_constant, 1),
        us_for_config4_random=round(ops_per_call / probe_random / 1e6, 2),
        us_for_config4_constant=round(ops_per_call / probe_constant / 1e6, 2),
        note="lrtprobe_mfma_rate: v_mfma_i32_32x32x32_i8 back to back on register operands, "
             "256 workgroups x 4 wavefronts, sustained; the clock the part holds under this load "
             "sets the figure, and the GEMM's operand traffic draws on the same power budget")
    # Yardstick (not this library): the vendor int8 GEMM through torch._int_mm on the same
    # operands, int32 output, no requantization.
    try:
        wt = dev(c4["w"]).t()
        for _ in range(5):
            torch._int_mm(x4, wt)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(50):
            torch._int_mm(x4, wt)   # launched eagerly (the library may allocate a workspace)
        e1.record()
        torch.cuda.synchronize()
        us_lib = e0.elapsed_time(e1) * 1e3 / 50
        out["config4_yardstick_torch_int_mm"] = dict(
            us=round(us_lib, 2), tops=round(ops_per_call / us_lib / 1e6, 1),
            note="hipBLASLt via torch._int_mm(x[2048,4096], w^T): int32 out, no epilogue")
    except Exception as e:  # a torch build without _int_mm on this device
        out["config4_yardstick_torch_int_mm"] = dict(error=repr(e)[:120])
    del op4c, x4c

    # config 5: FC chain of a Gemma-2B-shaped 18-layer decoder, blockwise int4, B = 1 and 4.
    # Each node gets its own seeded N(0,1) input (FC-only chain: outputs are discarded).
    g = torch.Generator(device="cuda").manual_seed(5)
    nodes = []
    for layer in range(wl.GEMMA2B_LAYERS):
        for name, k, n in wl.GEMMA2B_LAYER_FCS:
            packed = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device="cuda", generator=g)
            scales = (torch.rand((n, k // 32), device="cuda", generator=g) * 1.5e-2 + 5e-3).half()
            nodes.append(fc.FullyConnectedBlockwiseInt4(packed, scales, k, 32))
    chain_bytes = sum(int4_bytes(0, op.out_depth, op.depth) for op in nodes)
    per_layer = len(wl.GEMMA2B_LAYER_FCS)
    aux = [torch.cuda.Stream() for _ in range(3)]  # default priority, like the delegate's

    def run_level(level, bufs):
        """Nodes that do not depend on each other, spread round-robin over the current stream
        and the auxiliary ones (what the delegate does inside a partition)."""
        main = torch.cuda.current_stream()
        lanes = [main] + aux[:max(0, min(len(level), 4) - 1)]
        for st in lanes[1:]:
            st.wait_stream(main)
        for i, (op, key) in enumerate(level):
            with torch.cuda.stream(lanes[i % len(lanes)]):
                op(bufs["x"][op.depth], out=bufs["y"][key])
        for st in lanes[1:]:
            main.wait_stream(st)

    for b in (1, 4):
        xin = {k: torch.randn((b, k), device="cuda", generator=g) for k in (2048, 16384)}
        # one output buffer per node of a layer, so that concurrent nodes never share one
        yout = {i: torch.empty((b, n), dtype=torch.float32, device="cuda")
                for i, (_, _, n) in enumerate(wl.GEMMA2B_LAYER_FCS)}
        bufs = {"x": xin, "y": yout}
        keyed = [(op, i % per_layer) for i, op in enumerate(nodes)]

        def serial():
            for op, key in keyed:
                op(xin[op.depth], out=yout[key])

        def independent():
            # As the configuration defines it (every node has its own input, outputs are
            # discarded): no node depends on another, so all of them may overlap.
            for l in range(wl.GEMMA2B_LAYERS):
                run_level(keyed[l * per_layer:(l + 1) * per_layer], bufs)

        def decoder_order():
            # The dependency structure a real decoder layer imposes on the same nodes:
            # {q, k, v} -> o -> {gate, up} -> down, layer after layer.
            for l in range(wl.GEMMA2B_LAYERS):
                layer = keyed[l * per_layer:(l + 1) * per_layer]
                run_level(layer[0:3], bufs)
                run_level(layer[3:4], bufs)
                run_level(layer[4:6], bufs)
                run_level(layer[6:7], bufs)

        # Grouped launches: independent nodes of one depth run as ONE kernel.
        def bound_group(keyed_nodes):
            ops_ = [op for op, _ in keyed_nodes]
            ys = [torch.empty((b, op.out_depth), dtype=torch.float32, device="cuda") for op in ops_]
            return fc.GroupedBlockwiseInt4(ops_).bind([xin[op.depth] for op in ops_], ys)

        layers = [keyed[l * per_layer:(l + 1) * per_layer] for l in range(wl.GEMMA2B_LAYERS)]
        # As the configuration defines it, every node is independent: all nodes of one depth
        # can share launches (groups of up to 128 nodes: one launch per depth).
        shallow = [kn for kn in keyed if kn[0].depth == 2048]
        deep = [kn for kn in keyed if kn[0].depth != 2048]
        mx = fc.GroupedBlockwiseInt4.MAX_NODES
        all_groups = [bound_group(part[i:i + mx]) for part in (shallow, deep)
                      for i in range(0, len(part), mx)]
        # Decoder dependencies: {q, k, v} | o | {gate, up} | down, layer after layer.
        decoder_groups = [[bound_group(layer[0:3]), bound_group(layer[3:4]),
                           bound_group(layer[4:6]), bound_group(layer[6:7])] for layer in layers]

        def grouped_independent():
            for grp in all_groups:
                grp()

        def grouped_decoder_order():
            for stages in decoder_groups:
                for grp in stages:
                    grp()

        res = {}
        for name, fn in (("one_launch_per_node_one_stream", serial),
                         ("one_launch_per_node_4_streams_independent", independent),
                         ("one_launch_per_node_4_streams_decoder_dependencies", decoder_order),
                         ("grouped_launches_independent_nodes", grouped_independent),
                         ("grouped_launches_decoder_dependencies", grouped_decoder_order)):
            gc = capture(fn)
            us = timed_replays([gc], 30) * 1e3
            res[name] = dict(us_per_token=round(us, 1), gbps=round(chain_bytes / us / 1e3, 1),
                             frac_of_hbm_peak=round(chain_bytes / us / 1e3 / HBM_PEAK_GBPS, 4))
            del gc
        res["launches_per_token"] = {"per_node": len(nodes),
                                     "grouped_independent": len(all_groups),
                                     "grouped_decoder_dependencies": 4 * wl.GEMMA2B_LAYERS}
        res["note"] = ("inputs are independent per node and outputs are discarded, as the "
                       "configuration states; 'decoder_dependencies' imposes the order a real "
                       "decoder layer would ({q,k,v} -> o -> {gate,up} -> down)")
        del all_groups, decoder_groups
        res.update(fc_nodes=len(nodes), weight_bytes=chain_bytes)
        out["config5_gemma2b_fc_chain_B%d" % b] = res
    out["single_node_through_delegate"] = single_node_invokes(wl)
    for b in (1, 4):
        out["config5_through_delegate_B%d" % b] = delegate_chain(torch, wl, b)
        out["config5_through_delegate_device_bound_B%d" % b] = delegate_chain(torch, wl, b, bound=True)
    return out


def delegate_chain(torch, wl, b=1, invokes=20, bound=False):
    """Config 5 end to end through the delegate plugin, driven by the stand-in interpreter
    (litert_amd/standin_host): 126 FULLY_CONNECTED nodes in one partition. Wall-clock time of
    Invoke(), final synchronization included. With host tensors in and out (bound=False) that
    includes the upload of every node's input and the download of every node's output (all 126
    are graph outputs here); with bound=True every input and output is bound to registered
    device memory through a buffer handle (litert_amd_register_device_buffer +
    Interpreter::SetBufferHandle), as an application that keeps its activations in HBM does."""
    from litert_amd.standin_host import FakeHost, FLOAT32, FLOAT16, INT4, OK
    rng = np.random.default_rng(5)
    with FakeHost() as h:
        io = []
        for layer in range(wl.GEMMA2B_LAYERS):
            for name, k, n in wl.GEMMA2B_LAYER_FCS:
                x_np = rng.standard_normal((b, k)).astype(np.float32)
                x = h.tensor(FLOAT32, (b, k), data=x_np)
                w = h.tensor(INT4, (n, k), const=True,
                             data=rng.integers(0, 256, (n, k // 2), dtype=np.uint8))
                s_ = h.tensor(FLOAT16, (n, k // 32), const=True,
                              data=(rng.random((n, k // 32), dtype=np.float32) * 1.5e-2 + 5e-3).astype(np.float16))
                h.blockwise(w, s_, 32)
                y = h.tensor(FLOAT32, (b, n))
                h.fc(x, w, None, y)
                io.append((x, x_np, y, n))
        if h.load_delegate() != 0 or h.modify_graph_with_delegate() != OK or h.allocate_tensors() != OK:
            raise RuntimeError(h.errors())
        keep = []
        if bound:
            for x, x_np, y, n in io:
                xd = torch.from_numpy(x_np).cuda()
                yd = torch.empty((b, n), dtype=torch.float32, device="cuda")
                keep += [xd, yd]
                for tensor, dev in ((x, xd), (y, yd)):
                    handle = h.register_device_buffer(dev.data_ptr(), dev.numel() * 4)
                    if handle < 0 or h.set_buffer_handle(tensor, handle) != OK:
                        raise RuntimeError("binding a device buffer failed: " + h.errors())
                h.set_data_is_stale(x)
        plan = h.plan()
        groups, _ = h.describe_partition(plan[0][2])
        for _ in range(3):
            if h.invoke() != OK:
                raise RuntimeError(h.errors())
        t0 = time.perf_counter()
        for _ in range(invokes):
            h.invoke()
        us = (time.perf_counter() - t0) / invokes * 1e6
    note = ("every input and output bound to registered device memory (buffer handles): no copies, "
            "the kernels work on the bound memory" if bound else
            "host tensors in and out: 126 uploads + 126 downloads per invoke included")
    return {"invoke_wall_us": round(us, 1), "partitions": len(plan), "grouped_launches": groups,
            "fc_nodes": wl.GEMMA2B_LAYERS * len(wl.GEMMA2B_LAYER_FCS), "note": note}


def single_node_invokes(wl, invokes=200):
    """Configs 1, 2 and 3 as ONE FULLY_CONNECTED node each through the delegate plugin with host
    tensors in and out, driven by the stand-in interpreter: median wall-clock time of Invoke()
    (gather into page-locked memory, the kernel -- which reads its input rows from that memory and
    writes its output straight into page-locked host memory --, one stream synchronisation,
    scatter), and the same invoke split into those phases by the delegate's metrics collection."""
    from litert_amd.standin_host import FakeHost, FLOAT32, FLOAT16, INT4, INT8, INT32, OK
    rng = np.random.default_rng(6)

    def timed(h):
        if h.load_delegate() != 0 or h.modify_graph_with_delegate() != OK or h.allocate_tensors() != OK:
            raise RuntimeError(h.errors())
        if [kind for kind, _, _ in h.plan()] != ["delegate"]:
            raise RuntimeError("the node was not claimed: " + h.errors())
        for _ in range(20):
            if h.invoke() != OK:
                raise RuntimeError(h.errors())
        samples = []
        for _ in range(invokes):
            t0 = time.perf_counter()
            h.invoke()
            samples.append((time.perf_counter() - t0) * 1e6)
        samples.sort()
        # The same invoke split by phase, from the delegate's own clocks (metrics collection at
        # detail level 0: clock reads only, no device events).
        if h.start_metrics() != 0:
            raise RuntimeError("metrics collection did not start")
        for _ in range(invokes):
            h.invoke()
        m = h.stop_metrics()
        phases = {p: round(m["host_%s_us" % p] / m["invokes"], 1)
                  for p in ("gather", "enqueue", "wait", "scatter")}
        return {"invoke_us": round(samples[len(samples) // 2], 1), "phases_us": phases}

    out = {}
    c1 = wl.int8_fc()
    with FakeHost() as h:
        x = h.tensor(INT8, c1["x"].shape, data=c1["x"])
        h.affine(x, [c1["in_scale"]], [c1["in_zp"]])
        w = h.tensor(INT8, c1["w"].shape, data=c1["w"], const=True)
        h.affine(w, c1["w_scale"])
        b = h.tensor(INT32, (c1["w"].shape[0],), data=c1["bias"], const=True)
        y = h.tensor(INT8, (c1["x"].shape[0], c1["w"].shape[0]))
        h.affine(y, [c1["out_scale"]], [c1["out_zp"]])
        h.fc(x, w, b, y)
        out["config1_int8_2048x2048_B1"] = timed(h)
    for batch in (1, 4):
        c2 = wl.hybrid_fc(batch)
        with FakeHost() as h:
            x = h.tensor(FLOAT32, c2["x"].shape, data=c2["x"])
            w = h.tensor(INT8, c2["w"].shape, data=c2["w"], const=True)
            h.affine(w, c2["pcs"])
            y = h.tensor(FLOAT32, (batch, c2["w"].shape[0]))
            h.fc(x, w, None, y, asymmetric=True)
            out["config2_hybrid_14336x4096_B%d" % batch] = timed(h)
    n, k = N_OUT, K_IN
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (1, k), data=rng.standard_normal((1, k)).astype(np.float32))
        w = h.tensor(INT4, (n, k), const=True, data=rng.integers(0, 256, (n, k // 2), dtype=np.uint8))
        s_ = h.tensor(FLOAT16, (n, k // 32), const=True,
                      data=(rng.random((n, k // 32), dtype=np.float32) * 1.5e-2 + 5e-3).astype(np.float16))
        h.blockwise(w, s_, 32)
        y = h.tensor(FLOAT32, (1, n))
        h.fc(x, w, None, y)
        out["config3_int4_14336x4096_B1"] = timed(h)
    out["unit"] = "us per Invoke(), median of %d, host tensors in and out" % invokes
    return out


def cpu_baseline_leg(c):
    """The reference's CPU kernels for this op, restated in oracle/ and timed on one host core
    (dense hybrid FC runs on one thread in the reference, fully_connected.cc:847-851), on a
    bounded sample: config 2 at B = 1, full 14336 x 4096 filter, row sums cached as after the
    op's first Eval, about 5 seconds per tier. Two tiers: the portable reference kernels (what
    Register_FULLY_CONNECTED_REF runs) and the optimized x86 kernel (SSE branch of
    sse_tensor_utils.cc:308-379, what a default x86 build runs). `value` is the faster one, in
    the headline unit (algorithmic GB/s of the op)."""
    import oracle
    x = c["x"][:1]
    row_sums = c["w"].astype(np.int32).sum(1).astype(np.int32)
    oracle.fc_hybrid(x, c["w"][:256], c["pcs"][:256])  # load + warm

    def timed(fn, budget=5.0, max_reps=2000):
        reps, total = 0, 0.0
        while total < budget and reps < max_reps:
            t0 = time.perf_counter()
            fn()
            total += time.perf_counter() - t0
            reps += 1
        return total / reps, reps

    sec_ref, reps_ref = timed(lambda: oracle.fc_hybrid(x, c["w"], c["pcs"], row_sums=row_sums))
    tiers = {"portable_reference_kernels": {"us_per_op": round(sec_ref * 1e6, 1),
                                            "gbps": round(hybrid_bytes(1) / sec_ref / 1e9, 3),
                                            "repetitions": reps_ref}}
    best = sec_ref
    if oracle.have_sse():
        sec_sse, reps_sse = timed(lambda: oracle.fc_hybrid_sse(x, c["w"], c["pcs"], row_sums))
        tiers["optimized_x86_sse_kernel"] = {"us_per_op": round(sec_sse * 1e6, 1),
                                             "gbps": round(hybrid_bytes(1) / sec_sse / 1e9, 3),
                                             "repetitions": reps_sse}
        best = min(best, sec_sse)
    return {"value": round(hybrid_bytes(1) / best / 1e9, 3), "unit": "GB/s", "cores": 1,
            "kind": "port", "us_per_op": round(best * 1e6, 1), "tiers": tiers,
            "sample": "config 2 at B=1 only (14336x4096 hybrid FC: BatchQuantizeFloats + int8 "
                      "row x vector product with cached row sums), about 5 s per tier on one core; "
                      "oracle built with g++ -O2 -ffp-contract=off (-msse4.1 for the SSE file)"}


if __name__ == "__main__":
    main()
