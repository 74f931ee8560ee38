#!/usr/bin/env python3
"""Benchmark of the tiled-GEMM path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--tune] [--only C2,C5,CONV] [--operands random|zeros]
                    [--sustain SECONDS] [--no-extras] [--no-cpu] [--no-vendor]

A step is one launch of the headline workload -- the bf16 8192^3 GEMM
(row-major A and B, fp32 accumulate, bf16 out, non-split tiled kernel with
the group-M swizzle) -- through the C ABI, operands resident in HBM.  Prints
one JSON line: whole-job TFLOP/s over the K timed steps, the roofline record
of the kernel (algorithmic flops / mean per-launch duration from HIP events
on the launch stream), the CPU baseline (torch fp32 matmul on the host
cores, bounded sample) and, under "per_config", the other benchmark
configurations measured the same way.  "vendor_ms" entries time torch's own
GPU matmul (rocBLAS / hipBLASLt) on the same operands in the same run, for
comparison only: nothing in the measured path calls it.

Switches for profiling and for the clock / power evidence:
  --only C2,C5       run these workloads only (the headline C2 is always what `value` reports when it is run;
                     without it the line carries per_config only and `value` is null)
  --operands zeros   all-zero operands of the same shapes: the same instruction stream without data-dependent
                     switching power, so the shader clock stays at its maximum (results are then trivially zero)
  --splitk-reduce atomic   C3 with the K slices added by fp32 atomics instead of the ordered hand-over (for the A/B);
  --splitk-reduce wave     C3 on the 16-row kernel that cuts K across the eight waves of one workgroup (no hand-over)
  --sustain S        after the timed region, keep launching the headline kernel for S seconds while sampling
                     socket power and shader clock with `amd-smi metric -p -c`; reported under "sustain"
"""
from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys
import threading
import time

PEAK = {"bf16": 2516.6, "f16": 2516.6, "i8": 5033.2}     # dense MFMA TFLOP/s (TOP/s), MI355X
HBM_PEAK_GBS = 8000.0
PRE_ROLL = 40                                            # untimed launches that bring the part out of idle clocks
NOMINAL_SCLK_MHZ = 2400.0

# L2<->fabric bytes per launch of the headline kernel come from two `rocprofv3 --pmc` runs of this file (FETCH_SIZE,
# then WRITE_SIZE; KiB per dispatch), each scaled by what the same counter reads for the 2^28-byte calibration pass
# below.  The readings live in profiles/c2_hbm_traffic.json together with the SHA-256 of the kernel sources they were
# taken from; a record taken from other sources is stale and is not reported.
TRAFFIC_RECORD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "c2_hbm_traffic.json")
KERNEL_SOURCES = ("tritonix_amd/csrc/gemm_tile.h", "tritonix_amd/csrc/capi.hip", "tritonix_amd/csrc/registry.h")


def kernel_source_hash():
    """SHA-256 over the sources the tile kernels and their launch code are built from."""
    import hashlib

    h = hashlib.sha256()
    root = os.path.dirname(os.path.abspath(__file__))
    for rel in KERNEL_SOURCES:
        with open(os.path.join(root, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def recorded_traffic(tile):
    """(bytes per launch, note) from the counter record, or (None, why) when the record does not describe this build."""
    try:
        with open(TRAFFIC_RECORD) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None, "no counter record (profiles/c2_hbm_traffic.json)"
    if rec.get("kernel_source_sha256") != kernel_source_hash():
        return None, "counter record is from other kernel sources: re-run the two --pmc passes named in it"
    if rec.get("tile") != tile:
        return None, "counter record is for another tile configuration"
    nbytes = int((rec["fetch_kib"] * rec["fetch_scale"] + rec["write_kib"] * rec["write_scale"]) * 1024)
    return nbytes, "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, profiles/c2_hbm_traffic.json"


def write_traffic_record(fetch_csv, write_csv, tile):
    """Build profiles/c2_hbm_traffic.json from the counter_collection.csv files of
        rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d DIR -o p -- python3 bench.py --only C2 --no-cpu --no-vendor
    and the same with WRITE_SIZE.  Each reading (KiB per dispatch, mean over the headline kernel's dispatches) is kept
    with the factor that makes the same counter read 2^28 bytes for the calibration pass of main()."""
    import csv

    def reading(path, counter):
        cal, kern = [], []
        with open(path) as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] != counter:
                    continue
                if "CUDAFunctorOnSelf_add<int>" in row["Kernel_Name"] and int(row["Grid_Size"]) == 1 << 24:
                    cal.append(float(row["Counter_Value"]))
                elif "gemm_tile_kernel<tnx::TagBF16" in row["Kernel_Name"]:
                    kern.append(float(row["Counter_Value"]))
        if not cal or not kern:
            raise SystemExit(f"{path}: no {counter} rows for the calibration pass or the headline kernel")
        return sum(kern) / len(kern), (1 << 28) / 1024.0 / (sum(cal) / len(cal)), len(kern)

    fetch, fetch_scale, n_f = reading(fetch_csv, "FETCH_SIZE")
    write, write_scale, n_w = reading(write_csv, "WRITE_SIZE")
    rec = {"kernel_source_sha256": kernel_source_hash(), "kernel_sources": list(KERNEL_SOURCES), "tile": tile,
           "fetch_kib": round(fetch, 1), "fetch_scale": round(fetch_scale, 3), "write_kib": round(write, 1),
           "write_scale": round(write_scale, 3), "dispatches": [n_f, n_w],
           "bytes_per_launch": int((fetch * round(fetch_scale, 3) + write * round(write_scale, 3)) * 1024),
           "algorithmic_bytes": 3 * 8192 * 8192 * 2}
    with open(TRAFFIC_RECORD, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    return rec


ALL = ("C2", "C1", "C3", "C4", "C5", "FFN", "CONV")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--tune", action="store_true", help="run the grid tuner for each workload instead of the built-in tiles")
    ap.add_argument("--only", default=None, help="comma-separated subset of " + ",".join(ALL))
    ap.add_argument("--operands", choices=("random", "zeros"), default="random")
    ap.add_argument("--splitk-reduce", choices=("ordered", "atomic", "wave"), default="ordered",
                    help="C3 only: how the K slices meet (ordered = stored apart, summed in slice order; atomic = fp32 atomic "
                         "adds; wave = the 16-row kernel whose eight waves cut K inside one workgroup and meet in LDS)")
    ap.add_argument("--sustain", type=float, default=0.0, help="seconds of sustained headline launches with power/clock sampling")
    ap.add_argument("--no-extras", action="store_true", help="headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-vendor", action="store_true", help="skip the rocBLAS/hipBLASLt timing of the same operands")
    ap.add_argument("--traffic-from", default=None, metavar="FETCH_CSV,WRITE_CSV",
                    help="no GPU: write profiles/c2_hbm_traffic.json from the counter_collection.csv files of two rocprofv3 --pmc runs")
    ap.add_argument("--tile", default=None, help="headline tile override: block_m,block_n,block_k,num_warps,num_stages,group_m")
    return ap.parse_args()


def event_times(fn, n):
    """Per-launch durations in ms from HIP events recorded on torch's current stream (the launch stream)."""
    import torch

    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(n)]
    for i in range(n):
        starts[i].record()
        fn(i)
        stops[i].record()
    torch.cuda.synchronize()
    return [s.elapsed_time(e) for s, e in zip(starts, stops)]


def region_time(fn, n):
    """Mean launch duration in ms: one HIP-event pair around n back-to-back launches on the launch stream."""
    import torch

    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(n):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / n


def cpu_time(fn, budget_s=8.0, max_reps=3):
    """Median wall time of fn() on the host: one warm-up, then up to max_reps timed runs inside the budget."""
    fn()
    ts, t_start = [], time.perf_counter()
    while len(ts) < max_reps and (not ts or time.perf_counter() - t_start < budget_s):
        t1 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t1)
    return sorted(ts)[len(ts) // 2], len(ts)


def pre_roll(fn):
    """Untimed launches until the part is out of idle clocks: PRE_ROLL of them, repeated until 50 ms have passed (after
    host-side work -- drawing operands, a CPU reference -- a short kernel would otherwise be timed at idle clocks)."""
    import torch

    t0, i = time.perf_counter(), 0
    while True:
        for _ in range(PRE_ROLL):
            fn(i)
            i += 1
        torch.cuda.synchronize()
        if time.perf_counter() - t0 > 0.05:
            return


def vendor_ms(fn, reps=20):
    """Mean per-launch ms of a torch GPU op (the vendor BLAS), same event protocol as the kernels under test."""
    pre_roll(fn)
    return round(region_time(fn, 2 * reps), 4)


def pick_config(kernel, launcher, a, b, tune, split=False):
    from tritonix_amd.ops.matmul import default_config

    if tune:
        cfg = kernel.tune(launcher, warmup=5, rep=20)
        if cfg is not None:
            return cfg
    return default_config(a, b, split=split)


def smi_sample():
    """(socket power in W, shader clock in MHz) from `amd-smi metric -p -c --json`, or None."""
    try:
        out = subprocess.run(["amd-smi", "metric", "-p", "-c", "--json"], capture_output=True, text=True, timeout=10).stdout
        gpu = json.loads(out)["gpu_data"][0]
        clocks = [v["clk"]["value"] for k, v in gpu["clock"].items() if k.startswith("gfx_") and isinstance(v.get("clk"), dict)]
        return float(gpu["power"]["socket_power"]["value"]), float(sum(clocks) / len(clocks))
    except Exception:
        return None


def power_limit_w():
    try:
        out = subprocess.run(["rocm-smi", "-M", "--json"], capture_output=True, text=True, timeout=10).stdout
        card = next(iter(json.loads(out).values()))
        return float(next(v for k, v in card.items() if "Max Graphics Package Power" in k))
    except Exception:
        return None


def sustain(step, seconds, flops):
    """Launch `step` continuously for `seconds`; a second thread samples power and clock meanwhile.

    The first second of samples is dropped (the management firmware reports moving averages)."""
    import torch

    samples, stop = [], threading.Event()

    def poll():
        while not stop.is_set():
            s = smi_sample()
            if s is not None:
                samples.append((time.perf_counter(), *s))

    th = threading.Thread(target=poll, daemon=True)
    t0 = time.perf_counter()
    th.start()
    n = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(200):
            step()
        torch.cuda.synchronize()
        n += 200
    elapsed = time.perf_counter() - t0
    stop.set()
    th.join(timeout=15)
    kept = [(p, c) for t, p, c in samples if t - t0 > 1.0 and t - t0 < elapsed]
    out = {"seconds": round(elapsed, 2), "launches": n, "tflops": round(flops * n / elapsed / 1e12, 1),
           "samples": len(kept), "power_limit_w": power_limit_w()}
    if kept:
        pw, ck = [p for p, _ in kept], [c for _, c in kept]
        out.update({"socket_power_w_mean": round(sum(pw) / len(pw), 1), "socket_power_w_max": max(pw),
                    "sclk_mhz_mean": round(sum(ck) / len(ck), 1), "sclk_mhz_min": min(ck), "sclk_mhz_max": max(ck)})
        # what a kernel that kept every MFMA pipe busy in every cycle would reach at the clock the part actually ran
        out["mfma_peak_at_sclk_tflops"] = round(PEAK["bf16"] * out["sclk_mhz_mean"] / NOMINAL_SCLK_MHZ, 1)
        out["mfma_busy_at_sclk"] = round(out["tflops"] / out["mfma_peak_at_sclk_tflops"], 4)
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2
    if args.traffic_from:
        sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
        mm = __import__("importlib").import_module("tritonix_amd.ops.matmul")
        import torch

        tile = mm.default_config(torch.empty(8192, 8192, dtype=torch.bfloat16, device="meta"),
                                 torch.empty(8192, 8192, dtype=torch.bfloat16, device="meta"))
        print(json.dumps(write_traffic_record(*args.traffic_from.split(","), tile)))
        return 0
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X: no HIP device is visible", file=sys.stderr)
        return 2
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import oracle                                  # inputs + CPU baseline only; never on the measured path
    from tritonix_amd import _C
    import importlib

    mm = importlib.import_module("tritonix_amd.ops.matmul")
    sg = importlib.import_module("tritonix_amd.ops.swiglu")

    if not os.path.exists(_C.LIB_PATH):            # nothing built yet: build it; there is nothing to fall back to
        from tritonix_amd import build as hip_build

        hip_build.build(verbose=False)
    _C.load()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    only = tuple(s.strip() for s in args.only.split(",")) if args.only else ALL
    unknown = [s for s in only if s not in ALL]
    if unknown:
        print(f"unknown workload(s) {unknown}; choose from {ALL}", file=sys.stderr)
        return 2
    if args.no_extras:
        only = tuple(s for s in only if s == "C2")
    zeros = args.operands == "zeros"

    def operands(name):
        a, b = oracle.make_inputs(name)
        if zeros:
            a, b = torch.zeros_like(a), torch.zeros_like(b)
        return a, b

    # one plain elementwise pass of known size (2^28 bytes read, 2^28 bytes written): under
    # `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` it is the dispatch the GEMM's counter readings are scaled by
    cal_src = torch.zeros(1 << 26, dtype=torch.int32, device=dev)
    cal_dst = torch.empty_like(cal_src)
    torch.add(cal_src, 1, out=cal_dst)
    torch.cuda.synchronize()
    del cal_src, cal_dst

    out = {
        "metric": "TFLOP/s + % of dense MFMA peak, bf16 GEMM 8192³ on 1×MI355X",
        "value": None, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic" if not zeros else "synthetic (all-zero operands: clock evidence, not a result)",
    }
    ok = True
    if "C2" in only:
        ok = headline(torch, dev, oracle, mm, args, operands, out)
    extras_wanted = [s for s in only if s != "C2"]
    if extras_wanted:
        out["per_config"] = extras(torch, dev, oracle, mm, sg, args, operands, extras_wanted)
    print(json.dumps(out))
    return 0 if ok else 1


def headline(torch, dev, oracle, mm, args, operands, out):
    a_cpu, b_cpu = operands("C2")
    a, b = a_cpu.to(dev), b_cpu.to(dev)
    m, k = a.shape
    n = b.shape[1]
    flops = 2.0 * m * n * k
    cfg = pick_config(mm.matmul_kernel, lambda c: mm._launch_matmul(a, b, c), a, b, args.tune)
    if args.tile:
        bm, bn, bk, nw, st, gm = (int(v) for v in args.tile.split(","))
        cfg = {"block_m": bm, "block_n": bn, "block_k": bk, "group_m": gm, "num_stages": st, "num_warps": nw}
    c = torch.empty((m, n), device=dev, dtype=torch.bfloat16)

    # one C-ABI call per step: the arguments are bound once, the step is `tnx_gemm(&args)`
    launch = mm.matmul_kernel.prepare(a, b, c, m, n, k, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0),
                                      c.stride(1), **cfg)

    def step(_i=0):
        launch()

    # the clocks settle over the first few dozen launches after idle: run those before the W warm-up steps
    pre_roll(step)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    value = flops * args.steps / wall / 1e12

    nev = max(10, min(args.steps, 100))
    durs = event_times(step, nev)                    # one event pair per launch: spread of single launches
    kern_ms = region_time(step, nev)                 # one event pair around the region: mean launch duration
    achieved = flops / kern_ms / 1e9
    traffic, traffic_note = recorded_traffic(cfg) if args.operands == "random" else (None, "not recorded for all-zero operands")
    roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK["bf16"], "unit": "TFLOP/s",
                "frac": round(achieved / PEAK["bf16"], 4), "traffic": traffic, "traffic_source": traffic_note,
                "kernel_ms": round(kern_ms, 4), "kernel_ms_single_mean": round(sum(durs) / len(durs), 4),
                "kernel_ms_single_min": round(min(durs), 4)}

    vendor = None
    if not args.no_vendor:
        cv = torch.empty_like(c)
        t = vendor_ms(lambda i: torch.matmul(a, b, out=cv))
        vendor = {"what": "torch.matmul (rocBLAS/hipBLASLt) on the same operands, same run", "kernel_ms": t,
                  "tflops": round(flops / t / 1e9, 1)}
        del cv

    # parity of what was just timed, on a sample of rows (the oracle is the checker, not the thing measured)
    rows = torch.arange(0, m, 517)
    ok, maxerr, rel = oracle.within_tolerance(c[rows.to(dev)], oracle.reference_matmul(a_cpu[rows], b_cpu))

    sustained = sustain(step, args.sustain, flops) if args.sustain > 0 else None

    # ---- CPU baseline: the reference's "pytorch" backend restated on the host ---------
    cpu = None
    if not args.no_cpu:
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        torch.set_num_threads(cores)
        rows_n = 2048                                   # bounded sample: first 2048 rows of A against all of B
        af, bf = a_cpu[:rows_n].float(), b_cpu.float()
        torch.matmul(af[:256], bf)                      # warm-up
        reps, ts = 0, []
        t_start = time.perf_counter()
        while reps < 3 and time.perf_counter() - t_start < 30:
            t1 = time.perf_counter()
            torch.matmul(af, bf)
            ts.append(time.perf_counter() - t1)
            reps += 1
        med = sorted(ts)[len(ts) // 2]
        cpu = {"value": round(2.0 * rows_n * n * k / med / 1e12, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
               "kind": "port", "sample": f"torch fp32 CPU matmul, first {rows_n} of {m} rows of A x full B, median of {reps}"}

    out.update({
        "value": round(value, 1), "ms_per_step": round(ms_per_step, 4),
        "config": {"workload": "C2: bf16 GEMM M=N=K=8192, A,B ~ N(0,1)/sqrt(K) seed 2, row-major, fp32 acc, bf16 out",
                   "tile": cfg, "operands": args.operands},
        "pct_of_peak": round(100 * value / PEAK["bf16"], 2),
        "roofline": roofline, "cpu_baseline": cpu, "vendor_blas": vendor,
        "parity": {"ok": bool(ok), "max_abs_err": maxerr, "max_err_over_max_ref": rel, "rows_checked": int(rows.numel())},
    })
    if sustained is not None:
        out["sustain"] = sustained
    return ok


def graph_replay_ms(torch, bind, per_graph=100, replays=20):
    """Per-launch ms of `per_graph` launches captured once into a HIP graph and replayed: what a launch-latency-bound
    problem costs a caller that captures its loop (the library allocates and clears nothing, so a capture is just the
    kernel nodes).  `bind()` returns the launch, bound to the stream that is current when it is called.  None if the
    capture fails."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            launch = bind()
            launch()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(per_graph):
                launch()
        pre_roll(lambda i: graph.replay())
        return round(region_time(lambda i: graph.replay(), replays) / per_graph, 5)
    except Exception as e:      # a figure beside the measurement, never a reason to fail it
        print(f"graph replay not measured: {e}", file=sys.stderr)
        return None


def default_loader(conv_args):
    """Which of the conv2d kernels a launch with these arguments runs (tnx_conv_loader), by asking the library."""
    import ctypes

    from tritonix_amd import _C

    probe = type(conv_args).from_buffer_copy(conv_args)
    if probe.loader:
        return probe.loader
    probe.loader = _C.CONV_LOADER_DMA        # with a tile given, "auto" takes the direct-to-LDS kernel whenever it is allowed
    return _C.CONV_LOADER_DMA if _C.load().tnx_conv2d_supported(ctypes.byref(probe)) == _C.OK else _C.CONV_LOADER_REGISTERS


def extras(torch, dev, oracle, mm, sg, args, operands, wanted):
    res = {}
    reps = 30
    zeros = args.operands == "zeros"

    def measure(name, fn, flops, bytes_, dt, bound, nrot=1):
        pre_roll(lambda i: fn(i % nrot))
        durs = event_times(lambda i: fn(i % nrot), reps)
        ms = region_time(lambda i: fn(i % nrot), 2 * reps)
        r = {"kernel_ms": round(ms, 4), "kernel_ms_single_mean": round(sum(durs) / len(durs), 4), "tflops": round(flops / ms / 1e9, 2), "gbs": round(bytes_ / ms / 1e6, 1)}
        if bound == "mfma":
            r["roofline"] = {"bound": "mfma", "achieved": r["tflops"], "peak": PEAK[dt], "unit": "TFLOP/s",
                             "frac": round(r["tflops"] / PEAK[dt], 4)}
        elif bound == "hbm":
            r["roofline"] = {"bound": "hbm", "achieved": r["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": round(r["gbs"] / HBM_PEAK_GBS, 4)}
        res[name] = r
        return r

    # C1: latency-bound, report only
    if "C1" in wanted:
        a, b = (t.to(dev) for t in operands("C1"))
        cfg = pick_config(mm.matmul_kernel, lambda c: mm._launch_matmul(a, b, c), a, b, args.tune)
        c = torch.empty((1024, 768), device=dev, dtype=torch.float16)
        l1 = mm.matmul_kernel.prepare(a, b, c, 1024, 768, 512, 512, 1, 768, 1, 768, 1, **cfg)
        r = measure("C1", lambda i: l1(), 805306368, 3407872, "f16", None)
        r["tile"] = cfg
        r["graph_replay_ms"] = graph_replay_ms(
            torch, lambda: mm.matmul_kernel.prepare(a, b, c, 1024, 768, 512, 512, 1, 768, 1, 768, 1, **cfg))
        if not args.no_vendor:
            cv = torch.empty_like(c)
            r["vendor_ms"] = vendor_ms(lambda i: torch.matmul(a, b, out=cv))
        if not args.no_cpu:
            af, bf = a.cpu().float(), b.cpu().float()
            t, n = cpu_time(lambda: torch.matmul(af, bf))
            r["cpu"] = {"ms": round(t * 1e3, 3), "gflops": round(805306368 / t / 1e9, 1), "cores": torch.get_num_threads(),
                        "sample": f"torch fp32 CPU matmul, whole problem, median of {n}"}

    # C3: B is streamed from HBM: rotate distinct copies of B so that none is served from the 256 MiB Infinity Cache
    if "C3" in wanted:
        a_cpu, b_cpu = operands("C3")
        a = a_cpu.to(dev)
        nrot = 4
        bs = [b_cpu.to(dev).clone() for _ in range(nrot)]
        cfg = pick_config(mm.gemm_splitk_kernel, lambda c: mm._launch_splitk(a, bs[0], c), a, bs[0], args.tune, split=True)
        if args.splitk_reduce == "atomic":
            cfg = dict(cfg, atomic_reduce=1)
        elif args.splitk_reduce == "wave":
            cfg = dict(mm.SKINNY_CONFIG)          # K cut eight ways inside one workgroup, slices meet in LDS
        c = torch.empty((16, 4096), device=dev, dtype=torch.bfloat16)
        l3 = [mm.gemm_splitk_kernel.prepare(a, bs[i], c, 16, 4096, 14336, 14336, 1, 4096, 1, 4096, 1, **cfg)
              for i in range(nrot)]
        r = measure("C3", lambda i: l3[i](), 1879048192, 118030336, "bf16", "hbm", nrot=nrot)
        r["tile"] = cfg
        r["note"] = f"{nrot} distinct copies of B rotated ({nrot * 117} MB > 256 MB Infinity Cache); one kernel, reduction fused"
        okc, _, _ = oracle.within_tolerance(c, oracle.reference_matmul(a_cpu, b_cpu))
        r["parity_ok"] = bool(okc)
        if not args.no_vendor:
            cv = torch.empty_like(c)
            r["vendor_ms"] = vendor_ms(lambda i: torch.matmul(a, bs[i % nrot], out=cv), reps=reps)
            # what plain streaming kernels of the vendor's library reach on the same rotating copies of B: a read-only
            # reduction and a copy (read + write), as context for a fraction of the nominal 8 TB/s
            flat = [t.view(-1).view(torch.float32) for t in bs]       # (bit patterns of bf16 pairs: all finite or not, the traffic is the same)
            sink = torch.empty_like(flat[0])
            t_sum = vendor_ms(lambda i: flat[i % nrot].max(), reps=reps)
            t_cp = vendor_ms(lambda i: sink.copy_(flat[i % nrot]), reps=reps)
            nb = flat[0].numel() * 4
            r["vendor_stream"] = {"max_read_gbs": round(nb / t_sum / 1e6, 1), "copy_read_plus_write_gbs": round(2 * nb / t_cp / 1e6, 1),
                                  "bytes": nb}
            del flat, sink
        if not args.no_cpu:
            af, bf = a_cpu.float(), b_cpu.float()
            t, n = cpu_time(lambda: torch.matmul(af, bf))
            r["cpu"] = {"ms": round(t * 1e3, 3), "gflops": round(1879048192 / t / 1e9, 1), "cores": torch.get_num_threads(),
                        "sample": f"torch fp32 CPU matmul, whole problem, median of {n}"}
            del af, bf
        del bs

    # C4: fused GLU, both activations; FFN: the same up-projection followed by the down-projection (two launches)
    if "C4" in wanted or "FFN" in wanted:
        x_cpu, w_cpu = operands("C4")
        x, w = x_cpu.to(dev), w_cpu.to(dev)
        cfg = pick_config(sg.glu_kernel, lambda c: sg._launch_glu(x, w, c, "silu"), x, w, args.tune)
        z = torch.empty((4096, 14336), device=dev, dtype=torch.bfloat16)
        if "C4" in wanted:
            for act in ("silu", "sigmoid"):
                l4 = sg.glu_kernel.prepare(x, w, z, 4096, 28672, 4096, 4096, 1, 28672, 1, 14336, 1, activation=act, **cfg)
                measure(f"C4_{act}", lambda i: l4(), 962072674304, 385875968, "bf16", "mfma")["tile"] = cfg
            rows = torch.arange(0, 4096, 409)
            res["C4_sigmoid"]["parity_ok"] = bool(oracle.within_tolerance(
                z[rows.to(dev)], oracle.reference_glu(x_cpu[rows], w_cpu, "sigmoid"))[0])
            if not args.no_vendor:
                g1 = torch.empty((4096, 28672), device=dev, dtype=torch.bfloat16)
                res["C4_silu"]["vendor_ms"] = vendor_ms(lambda i: torch.matmul(x, w, out=g1))
                res["C4_silu"]["vendor_note"] = "the [4096,28672] GEMM alone; gating would be a second pass over its output"
                del g1
            if not args.no_cpu:
                import torch.nn.functional as F

                nr = 256
                xf, w1, w2 = x_cpu[:nr].float(), w_cpu[:, 0::2].float(), w_cpu[:, 1::2].float()
                t, n = cpu_time(lambda: F.silu(xf @ w1) * (xf @ w2))
                res["C4_silu"]["cpu"] = {"ms": round(t * 1e3, 3), "gflops": round(962072674304 * nr / 4096 / t / 1e9, 1),
                                         "cores": torch.get_num_threads(),
                                         "sample": f"torch fp32 CPU silu(x@W1)*(x@W2), first {nr} of 4096 rows, median of {n}"}
                del xf, w1, w2
        if "FFN" in wanted:
            # the SwiGLU feed-forward block at this size: silu-GLU up-projection [4096,4096]x[4096,28672] -> [4096,14336],
            # then the down-projection [4096,14336]x[14336,4096]; the intermediate stays in HBM in bf16
            g = torch.Generator("cpu").manual_seed(44)
            w3_cpu = (0.02 * torch.randn(14336, 4096, generator=g)).bfloat16()
            if zeros:
                w3_cpu.zero_()
            w3 = w3_cpu.to(dev)
            y = torch.empty((4096, 4096), device=dev, dtype=torch.bfloat16)
            cfg_d = pick_config(mm.matmul_kernel, lambda c: mm._launch_matmul(z, w3, c), z, w3, args.tune)
            up = sg.glu_kernel.prepare(x, w, z, 4096, 28672, 4096, 4096, 1, 28672, 1, 14336, 1, activation="silu", **cfg)
            down = mm.matmul_kernel.prepare(z, w3, y, 4096, 4096, 14336, 14336, 1, 4096, 1, 4096, 1, **cfg_d)

            def ffn(_i):
                up()
                down()

            flops_ffn = 962072674304 + 2.0 * 4096 * 4096 * 14336
            bytes_ffn = 385875968 + 2 * (4096 * 14336 + 14336 * 4096 + 4096 * 4096)
            r = measure("FFN", ffn, flops_ffn, bytes_ffn, "bf16", "mfma")
            r["tiles"] = {"up": cfg, "down": cfg_d}
            r["note"] = ("swiglu_ffn = fused GLU up-projection + tiled GEMM down-projection, two launches; the [4096,14336] "
                         "bf16 intermediate (117 MB) is written and read back once")
            rows = torch.arange(0, 4096, 585)
            hidden = oracle.reference_glu(x_cpu[rows], w_cpu, "silu").bfloat16().float()
            r["parity_ok"] = bool(oracle.within_tolerance(y[rows.to(dev)], hidden @ w3_cpu.float())[0])
            # What a one-kernel fusion over the intermediate's columns has to move: every column tile of the gated
            # product (112 of them at this size) contributes a partial [rows, 4096] fp32 sum of the down-projection
            # that has to meet the others' -- the reference's draft adds them with atomics (tritonix/ops/swiglu.py:
            # 207-230).  Timed here with this library's own hand-over for K slices: the down-projection alone, K cut 56
            # ways (half the slices the fusion needs; 3.7 GB of partial sums, the most a 32-bit slice offset
            # addresses), against the same product uncut.
            cfg_cut = {"block_m": 256, "block_n": 256, "block_k": 64, "group_m": 8, "num_stages": 2, "num_warps": 4}
            try:
                cut = mm.matmul_kernel.prepare(z, w3, y, 4096, 4096, 14336, 14336, 1, 4096, 1, 4096, 1, split_k=56, **cfg_cut)
                pre_roll(lambda i: cut())
                t_cut = region_time(lambda i: cut(), 10)
                pre_roll(lambda i: down())
                t_down = region_time(lambda i: down(), 20)
                r["fused_partial_sums"] = {"down_projection_uncut_ms": round(t_down, 4), "down_projection_k_cut_56_ms": round(t_cut, 4),
                                           "partial_sum_bytes": 56 * 4096 * 4096 * 4,
                                           "note": "half the partial-sum hand-over of a fusion over 112 column tiles, and already longer than "
                                                   "the whole two-launch block"}
                del cut
            except (ValueError, RuntimeError) as e:
                r["fused_partial_sums"] = {"error": str(e)}
            del w3, y
        del x, w, z

    # CONV: conv2d forward as an implicit GEMM, a ResNet-style 3x3 layer (batch 32, 256 -> 256 channels, 56x56, padding 1):
    # GEMM_M = 100352 pixels, GEMM_N = 256, GEMM_K = 2304.  Algorithmic bytes: input + weight + bias + output once.
    if "CONV" in wanted:
        from tritonix_amd.ops.conv2d import conv2d_forward, torch_conv2d_forward
        import tritonix_amd.ops.conv2d.forward as conv

        # name: batch, c_in, h = w, c_out, filter, stride, padding.  CONV is the line quoted; the others show the two
        # kernels' ranges (small planes, a strided layer that only the register-staged kernel takes)
        layers = {"CONV": (32, 256, 56, 256, 3, 1, 1), "CONV_128x28": (32, 128, 28, 128, 3, 1, 1),
                  "CONV_512x14": (32, 512, 14, 512, 3, 1, 1), "CONV_128x56_stride2": (32, 128, 56, 128, 3, 2, 1)}
        for name, (n_, c_, hw_, k_, f_, st_, pd_) in layers.items():
            g = torch.Generator("cpu").manual_seed(66)
            x_cpu = torch.randn(n_, c_, hw_, hw_, generator=g).bfloat16()
            w_cpu = (torch.randn(k_, c_, f_, f_, generator=g) / (c_ * f_ * f_) ** 0.5).bfloat16()
            b_cpu = torch.randn(k_, generator=g).bfloat16()
            if zeros:
                x_cpu.zero_(); w_cpu.zero_(); b_cpu.zero_()
            x, w, b = x_cpu.to(dev), w_cpu.to(dev), b_cpu.to(dev)
            geo = ((st_, st_), (pd_, pd_), (1, 1))
            y = conv2d_forward(x, w, b, *geo)            # times the candidate tiles once, as the reference does
            cfg = conv._CONV_FWD_CONFIG_CACHE[(n_, c_, hw_, hw_, k_, f_, f_, *geo, torch.bfloat16)]
            ho = y.shape[2]
            flops = 2.0 * n_ * ho * ho * k_ * c_ * f_ * f_
            bytes_ = 2 * (x.numel() + w.numel() + b.numel() + y.numel())
            gm, gn, gk = n_ * ho * ho, k_, c_ * f_ * f_
            lc = conv.conv2d_forward_kernel.prepare(y, x, w, b, n_, c_, hw_, hw_, k_, ho, ho, f_, f_, st_, st_, pd_, pd_, 1, 1,
                                                    gm, gn, gk, **cfg)
            r = measure(name, lambda i: lc(), flops, bytes_, "bf16", "mfma")
            r["tile"] = cfg
            r["loader"] = {1: "registers", 2: "dma", 3: "gemm"}[default_loader(lc.args)]
            r["workload"] = (f"conv2d forward bf16: input [{n_},{c_},{hw_},{hw_}], weight [{k_},{c_},{f_},{f_}], bias, "
                             f"stride {st_}, padding {pd_}")
            ref = oracle.reference_conv2d(x_cpu[5:6], w_cpu, b_cpu, *geo)
            r["parity_ok"] = bool(oracle.within_tolerance(y[5:6], ref)[0])
            if not args.no_vendor:
                r["vendor_ms"] = vendor_ms(lambda i: torch_conv2d_forward(x, w, b, *geo))
                r["vendor_note"] = "torch.nn.functional.conv2d (MIOpen), same tensors"
            if not args.no_cpu and name == "CONV":
                xf, wf, bf = x_cpu[:2].float(), w_cpu.float(), b_cpu.float()
                t, n = cpu_time(lambda: torch.nn.functional.conv2d(xf, wf, bf, *geo))
                r["cpu"] = {"ms": round(t * 1e3, 3), "gflops": round(flops * 2 / n_ / t / 1e9, 1), "cores": torch.get_num_threads(),
                            "sample": f"torch fp32 CPU conv2d, first 2 of {n_} images, median of {n}"}
            del x, w, b, y

    # C5: int8 -> int32
    if "C5" in wanted:
        a_cpu, b_cpu = operands("C5")
        a, b = a_cpu.to(dev), b_cpu.to(dev)
        cfg = pick_config(mm.matmul_kernel, lambda c: mm._launch_matmul(a, b, c), a, b, args.tune)
        c = torch.empty((8192, 8192), device=dev, dtype=torch.int32)
        l5 = mm.matmul_kernel.prepare(a, b, c, 8192, 8192, 8192, 8192, 1, 8192, 1, 8192, 1, **cfg)
        r = measure("C5", lambda i: l5(), 1099511627776, 402653184, "i8", "mfma")
        r["tile"] = cfg
        rows = torch.arange(0, 8192, 1021)
        r["bit_exact"] = bool(torch.equal(c[rows.to(dev)].cpu(), oracle.reference_matmul(a_cpu[rows], b_cpu)))
        if not args.no_vendor and hasattr(torch, "_int_mm"):
            try:
                r["vendor_ms"] = vendor_ms(lambda i: torch._int_mm(a, b))
            except Exception as e:                      # the vendor path is optional; its absence is not an error here
                r["vendor_ms"] = None
                r["vendor_note"] = f"torch._int_mm unavailable: {type(e).__name__}"
        if not args.no_cpu:
            nr = 256
            ad, bd = a_cpu[:nr].double(), b_cpu.double()
            t, n = cpu_time(lambda: torch.matmul(ad, bd))
            r["cpu"] = {"ms": round(t * 1e3, 3), "gops": round(1099511627776 * nr / 8192 / t / 1e9, 1),
                        "cores": torch.get_num_threads(),
                        "sample": f"torch fp64 CPU matmul (exact for int8), first {nr} of 8192 rows, median of {n}"}
    return res


if __name__ == "__main__":
    sys.exit(main())
