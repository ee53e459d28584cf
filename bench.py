#!/usr/bin/env python3
"""Benchmark of the records -> Chrome-trace JSON hot path on one MI355X.

One "step" = one complete pass of the engine (dictionary, decode, clock conversion, joins, sort,
size, scan, emit) over the 10M-record configuration (10M device rows + 10M runtime rows + 2M CPU
ops, 128 streams), with the raw records already resident in HBM and the JSON document left in a
device buffer.  Prints one JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--n-device N] [--config C]
  python bench.py --logger-benchmark small|medium|large   (the reference's logger benchmark, both loggers)
  python bench.py --summarize-kernel-trace STATS.csv      (table of a `rocprofv3 --kernel-trace --stats` run)
  python bench.py --summarize-hbm FETCH_DIR WRITE_DIR STATS.csv --config C
                                                          (table of two `rocprofv3 --pmc` runs, see profiles/)
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
DOMINANT_KERNEL = "k_emit_direct"
FULL_SIZE = {1: 10000, 2: 1000000, 3: 10000000, 4: 11000000, 5: 5000000}
WORKLOAD = {
    1: "config1: 10k CPU ops + 10k launches + 10k kernels, 4 streams",
    2: "config2: 1M device rows (70% kernel / 20% memcpy / 10% memset) + 1M runtime + 1M CPU ops, 32 streams, linear clock model",
    3: "config3: 10M device + 10M runtime + 2M CPU-op records, 128 streams, block-shuffled arrival, ac2g flows",
    4: "config4: graph launches with 100-1000 kernel fan-out (~11M kernels), 5% orphans each way",
    5: "config5: 5M string-heavy generic kernel records with typed args",
}


def short_kernel_name(name):
    """ktj::gpu::k_x<...>(args) -> k_x<...>"""
    name = name.strip().strip('"')
    if name.startswith("void "):
        name = name[5:]
    depth = 0
    for i, ch in enumerate(name):
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0:
            name = name[:i]
            break
    return name.replace("ktj::gpu::", "")


def read_kernel_stats(path):
    import csv
    rows = []
    for r in csv.DictReader(open(path)):
        rows.append((short_kernel_name(r["Name"]), int(r["Calls"]), float(r["AverageNs"]) / 1e3, float(r["MinNs"]) / 1e3,
                     float(r["MaxNs"]) / 1e3, float(r["Percentage"])))
    return rows


def summarize_kernel_trace(stats_csv):
    """Prints the per-kernel table of a `rocprofv3 --kernel-trace --stats --output-format csv` run."""
    print("%-44s %6s %10s %10s %10s %6s" % ("kernel", "calls", "avg_us", "min_us", "max_us", "pct"))
    for name, calls, avg, mn, mx, pct in read_kernel_stats(stats_csv):
        print("%-44s %6d %10.1f %10.1f %10.1f %6.2f" % (name[:44], calls, avg, mn, mx, pct))


def read_counter(directory, counter):
    """Sum and launch count per kernel of one counter in a `rocprofv3 --pmc` output directory."""
    import collections
    import csv
    import glob
    files = glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise SystemExit("bench.py: no *counter_collection.csv under " + directory)
    total = collections.defaultdict(float)
    launches = collections.defaultdict(set)
    for r in csv.DictReader(open(files[0])):
        if r["Counter_Name"] != counter:
            continue
        k = short_kernel_name(r["Kernel_Name"])
        total[k] += float(r["Counter_Value"])
        launches[k].add(r["Dispatch_Id"])
    return {k: (total[k], len(launches[k])) for k in total}


def summarize_hbm(fetch_dir, write_dir, stats_csv, config, copy_bytes=1 << 30):
    """Prints HBM bytes per launch and kernel from a FETCH_SIZE run and a WRITE_SIZE run of this script
    (one pass each, both ending with the k_copy_reference launch of copy_bytes that scales the
    counters), with the kernels' average durations from a separate kernel-trace run."""
    fetch, write = read_counter(fetch_dir, "FETCH_SIZE"), read_counter(write_dir, "WRITE_SIZE")
    ref = "k_copy_reference"
    if ref not in fetch or ref not in write:
        raise SystemExit("bench.py: the counter runs hold no k_copy_reference launch to scale by")
    f_unit = copy_bytes / (fetch[ref][0] / fetch[ref][1])
    w_unit = copy_bytes / (write[ref][0] / write[ref][1])
    avg = {name: a for name, _, a, _, _, _ in read_kernel_stats(stats_csv)}
    print("scale: k_copy_reference copies %d bytes per launch: FETCH_SIZE %.1f bytes per unit, WRITE_SIZE %.1f bytes per unit"
          % (copy_bytes, f_unit, w_unit))
    print("%-36s %8s %10s %10s %9s %7s %7s" % ("kernel", "launches", "fetch_MB", "write_MB", "avg_us", "GB/s", "of_peak"))
    rows = []
    for k in set(fetch) | set(write):
        n = max(fetch.get(k, (0, 0))[1], write.get(k, (0, 0))[1]) or 1
        fb = fetch.get(k, (0, 0))[0] * f_unit / n
        wb = write.get(k, (0, 0))[0] * w_unit / n
        rows.append((k, n, fb, wb, avg.get(k)))
    rows.sort(key=lambda r: -(r[2] + r[3]) * r[1])
    for k, n, fb, wb, a in rows:
        gbs = (fb + wb) / (a * 1e-6) / 1e9 if a else 0.0
        print("%-36s %8d %10.1f %10.1f %9s %7.0f %7.3f" % (k[:36], n, fb / 1e6, wb / 1e6, "%.1f" % a if a else "-", gbs,
                                                          gbs / HBM_PEAK_GBS))
    for k, n, fb, wb, a in rows:
        if k == DOMINANT_KERNEL:
            print("traffic_json: " + json.dumps({"kernel": k, "config": config, "fetch_bytes_per_launch": round(fb),
                                                 "write_bytes_per_launch": round(wb), "hbm_bytes_per_launch": round(fb + wb)}))


def measured_traffic(config, device_rows):
    """HBM bytes per launch of the dominant kernel, from the committed summary of the counter runs
    (profiles/hbm_counters_config<C>_full.txt, written by --summarize-hbm); None when there is none
    for this workload."""
    if device_rows != FULL_SIZE[config]:
        return None
    path = os.path.join(ROOT, "profiles", "hbm_counters_config%d_full.txt" % config)
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("traffic_json:"):
            t = json.loads(line[len("traffic_json:"):])
            if t.get("kernel") == DOMINANT_KERNEL and t.get("config") == config:
                return t["hbm_bytes_per_launch"]
    return None


def name_bytes_fetched(s):
    """Sum over all records of the length of the name each one prints (the "name bytes fetched per
    record, from the dictionary" term of the emit stage's algorithmic bytes), from the raw stream:
    generic and device-kernel rows name a dictionary string, runtime rows the name of their API."""
    import numpy as np
    from kineto_amd import abi
    if s.n_strings == 0:
        return 0
    lens = np.diff(np.ctypeslib.as_array(s.str_off, shape=(s.n_strings + 1,)).astype(np.int64))

    def column(ptr, n, rec, field):
        raw = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_uint8)), shape=(n * C.sizeof(rec),)).reshape(n, C.sizeof(rec))
        o = getattr(rec, field).offset
        return raw[:, o:o + 4].copy().view(np.uint32).reshape(n)

    total = 0
    if s.n_generic:
        ids = column(s.generic, s.n_generic, abi.GenericRec, "name_id")
        total += int(lens[ids[ids < s.n_strings]].sum())
    if s.n_device:
        ids = column(s.device, s.n_device, abi.DeviceRec, "name_id")
        dom = column(s.device, s.n_device, abi.DeviceRec, "domain") & 0xFFFF
        ids = ids[dom == 0]
        total += int(lens[ids[ids < s.n_strings]].sum())
    if s.n_runtime and s.n_cids:
        cid_names = np.ctypeslib.as_array(s.cid_name_ids, shape=(s.n_cids,))
        cids = column(s.runtime, s.n_runtime, abi.RuntimeRec, "cid")
        ids = cid_names[cids[cids < s.n_cids]]
        total += int(lens[ids[ids < s.n_strings]].sum())
    return total


def host_to_file_legs(sp, n_records):
    """What a profiler pays from records in host memory to the renamed trace file, once, on a fresh
    engine: ktj_create with a file sink, every submit call, ktj_finalize (the whole GPU pass with its
    first-pass allocations, the device -> host copy streamed through two pinned buffers, write(),
    rename).  The file goes to tmpfs (/dev/shm) where there is one, so no disk is involved; the
    leg is bound by the page cache either way.  Beside it: the record submission alone from
    page-locked buffers of ktj_host_alloc (the copy into them is the producer's and not timed)."""
    import shutil
    import tempfile
    import torch
    from kineto_amd import abi
    from kineto_amd.engine import TraceEngine
    s = sp.contents
    top = "/dev/shm" if os.path.isdir("/dev/shm") and os.access("/dev/shm", os.W_OK) else None
    d = tempfile.mkdtemp(prefix="ktj_bench_", dir=top)
    out = {"file_system": "tmpfs (/dev/shm)" if top else "default temporary directory"}
    try:
        path = os.path.join(d, "trace.json")
        t0 = time.perf_counter()
        eng = TraceEngine(path, device=0, no_file=False)
        eng.submit_stream(sp)
        t1 = time.perf_counter()
        n = eng.finalize()
        t2 = time.perf_counter()
        st = eng.stats()
        eng.close()
        out.update({"e2e_host_to_file_s": t2 - t0, "submit_s": t1 - t0, "finalize_s": t2 - t1, "file_bytes": int(n),
                    "file_write_and_copy_s": st.stage_ms[9] * 1e-3, "records_per_s": n_records / (t2 - t0),
                    "file_gb_per_s": n / (st.stage_ms[9] * 1e-3) / 1e9 if st.stage_ms[9] > 0 else None,
                    "file_size_on_disk_matches": os.path.getsize(path) == n})
    finally:
        shutil.rmtree(d, ignore_errors=True)
    # the same records from page-locked buffers
    eng = TraceEngine(s.trace_name.decode(), device=0)
    bufs = []
    total = 0
    for cls, ptr, cnt, rec in ((abi.REC_GENERIC, s.generic, s.n_generic, abi.GenericRec), (abi.REC_RUNTIME, s.runtime, s.n_runtime, abi.RuntimeRec),
                               (abi.REC_DEVICE, s.device, s.n_device, abi.DeviceRec), (abi.REC_EXTCORR, s.extcorr, s.n_extcorr, abi.ExtCorrRec)):
        nb = cnt * C.sizeof(rec)
        if not nb:
            continue
        p = C.c_void_p()
        if eng.lib.ktj_host_alloc(eng.h, nb, C.byref(p)) != 0:
            break
        C.memmove(p, C.cast(ptr, C.c_void_p), nb)
        bufs.append((cls, p, cnt))
        total += nb
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for cls, p, cnt in bufs:
        eng.lib.ktj_submit_records(eng.h, cls, p, cnt)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for _, p, _ in bufs:
        eng.lib.ktj_host_free(eng.h, p)
    eng.close()
    out.update({"h2d_records_from_pinned_s": dt, "h2d_records_from_pinned_gb_per_s": total / dt / 1e9 if dt > 0 else None,
                "h2d_record_bytes": int(total)})
    return out


def small_trace_legs():
    """What a trace of a few records and configuration 1 at its full size (30 000 records) cost: the
    fixed cost of the pass (some forty short kernels and two read-backs), not throughput.  Median over
    repeated passes on a warm engine, with and without the events between the stages
    (KTJ_CREATE_NO_STAGE_TIMES, which the ActivityLogger shim sets), and from ktj_create to
    ktj_destroy on engines that start from what the previous one left behind."""
    import statistics
    from kineto_amd import abi
    from kineto_amd.engine import TraceEngine
    out = {}
    for label, cfg, n in (("fifteen_records", 1, 5), ("config1_full", 1, FULL_SIZE[1])):
        sp, release = abi.synth_stream(cfg, n, host_name="bench")
        s = sp.contents
        leg = {"records": int(s.n_generic + s.n_runtime + s.n_device)}
        for key, nst in (("warm_pass_ms", False), ("warm_pass_no_stage_times_ms", True)):
            with TraceEngine(s.trace_name.decode(), device=0, no_stage_times=nst) as eng:
                eng.submit_stream(sp)
                for _ in range(5):
                    eng.process()
                ts = []
                for _ in range(100):
                    t0 = time.perf_counter()
                    eng.process()
                    ts.append((time.perf_counter() - t0) * 1e3)
                leg[key] = statistics.median(ts)
        ts = []
        for k in range(30):
            t0 = time.perf_counter()
            with TraceEngine(s.trace_name.decode(), device=0, no_stage_times=True) as eng:
                eng.submit_stream(sp)
                eng.process()
                eng.output()
            if k >= 5:
                ts.append((time.perf_counter() - t0) * 1e3)
        leg["create_to_destroy_ms"] = statistics.median(ts)   # includes this script's ctypes calls
        release()
        out[label] = leg
    return out


def host_cpu():
    model = None
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count()
    return {"model": model, "logical_cpus": os.cpu_count(), "usable_cpus": usable}


def reference_logger_leg(sp, ora, engine_bytes):
    """The reference's own ChromeTraceLogger (oracle/_ref/libktj_ref.so, built from the reference's
    sources) fed the sample's joined activities, timed from logger construction to the end of
    finalizeTrace, file included; None where that library is not built."""
    import oracle_glue as og
    if not og.have_ref():
        return None
    t0 = time.perf_counter()
    data = og.ref_render(sp, ora, call_order=0)
    dt = time.perf_counter() - t0
    _, n_acts = ora.activities()
    return {"value": n_acts / dt, "unit": "activities/s", "cores": 1, "kind": "reference",
            "seconds": dt, "activities": int(n_acts), "output_bytes": len(data),
            "note": "logger only: the reference's join stages need a profiling session and are not part of this leg; "
                    "includes building the activity objects and writing the file to a temporary directory",
            "identical_to_engine_output_on_sample": bool(data == engine_bytes)}


def cpu_baseline(config, sample_device_rows):
    """Times the single-threaded CPU restatement of the reference path (oracle/) on a bounded
    sample of the same workload, and checks the engine against it on that sample."""
    from kineto_amd import abi
    from kineto_amd.engine import TraceEngine
    import oracle_glue as og
    # with the reference logger at hand the sample takes its base time and host name, so that the
    # three documents (engine, port, reference logger) can be compared byte for byte
    stream_args = og.ref_stream_args() if og.have_ref() else dict(host_name="bench")
    sp, release = abi.synth_stream(config, sample_device_rows, **stream_args)
    s = sp.contents
    n_records = s.n_generic + s.n_runtime + s.n_device
    t0 = time.perf_counter()
    ora = og.OracleRun(sp)
    dt = time.perf_counter() - t0
    import numpy as np
    want = ora.output_view()
    with TraceEngine(s.trace_name.decode(), base_time_ns=s.base_time_ns, device=0) as eng:
        eng.submit_stream(sp)
        eng.process()
        got = eng.output_view()
        same = got.shape == want.shape and bool(np.array_equal(got, want))
        engine_bytes = bytes(got) if same else eng.output()
    stages = ora.timings()
    ref_leg = reference_logger_leg(sp, ora, engine_bytes)
    del engine_bytes
    ora.close()
    release()
    return ref_leg, {
        "value": n_records / dt, "unit": "records/s", "cores": 1, "kind": "port", "host_cpu": host_cpu(),
        "sample": f"same workload scaled to {sample_device_rows} device rows ({n_records} records, "
                  f"{len(want)} output bytes) in {dt:.2f} s on one host core "
                  f"(join {stages[0]:.2f} s, sort {stages[1]:.2f} s, emit {stages[2]:.2f} s)",
        "output_gb_per_s": len(want) / dt / 1e9,
        "engine_output_identical_on_sample": bool(same),
    }


def logger_benchmark(scenario, iterations, threads):
    """The reference's own logger benchmark (benchmarks/json_output_benchmark.cpp: a fixed-seed stream
    of GenericTraceActivity objects, timed from logger construction to the end of finalizeTrace,
    file included) run on the reference's ChromeTraceLogger and on the GpuChromeTraceLogger shim in
    the same process.  Needs oracle/_ref/libktj_shim_test.so (built where the reference is present).
    Prints one JSON line; the shim's file is compared byte for byte with the reference's."""
    import statistics
    import tempfile
    so = os.path.join(ROOT, "oracle", "_ref", "libktj_shim_test.so")
    if not os.path.exists(so):
        print("bench.py: oracle/_ref/libktj_shim_test.so is not built (it needs the reference's sources)", file=sys.stderr)
        sys.exit(1)
    lib = C.CDLL(so)
    lib.ktj_logger_bench_create.restype = C.c_void_p
    lib.ktj_logger_bench_create.argtypes = [C.c_uint64, C.c_uint32]
    lib.ktj_logger_bench_destroy.argtypes = [C.c_void_p]
    lib.ktj_logger_bench_run.restype = C.c_double
    lib.ktj_logger_bench_run.argtypes = [C.c_void_p, C.c_int, C.c_char_p, C.c_int, C.c_int]
    n = {"small": 5, "medium": 6000, "large": 6000000}[scenario]
    if iterations <= 0:
        iterations = {"small": 100, "medium": 20, "large": 2}[scenario]
    w = lib.ktj_logger_bench_create(n, 42)
    legs = {"reference": 0, "reference_sorted_input": 1, "shim_per_activity": 2, "shim_bulk": 3}
    out = {}
    digests = {}
    with tempfile.TemporaryDirectory() as top:
        for name, which in legs.items():
            d = os.path.join(top, name)
            os.makedirs(d)
            path = os.path.join(d, "benchmark_%s.json" % scenario)
            times = []
            for it in range(iterations + 1):  # the first iteration is a warm-up for every leg
                ms = lib.ktj_logger_bench_run(w, which, path.encode(), 0, threads)
                if ms < 0:
                    print("bench.py: logger benchmark leg %s failed (%g)" % (name, ms), file=sys.stderr)
                    sys.exit(1)
                if it:
                    times.append(ms)
            size = os.path.getsize(path)
            with open(path, "rb") as f:
                data = f.read().replace(path.encode(), b"FILE")
            import hashlib
            digests[name] = hashlib.blake2b(data).hexdigest()
            del data
            os.remove(path)
            mean = statistics.mean(times)
            out[name] = {"mean_ms": mean, "min_ms": min(times), "stddev_ms": statistics.pstdev(times), "file_bytes": size,
                         "activities_per_s": n / (mean / 1e3), "mib_per_s": size / 1048576.0 / (mean / 1e3)}
    lib.ktj_logger_bench_destroy(w)
    print(json.dumps({
        "metric": "logger_benchmark_activities_per_s", "scenario": scenario, "activities": n, "iterations": iterations,
        "packing_threads": threads, "legs": out,
        "shim_identical_to_reference": digests["shim_per_activity"] == digests["reference_sorted_input"]
        and digests["shim_bulk"] == digests["reference_sorted_input"],
        "speedup_bulk_vs_reference": out["reference"]["mean_ms"] / out["shim_bulk"]["mean_ms"],
        "note": "file output included in every leg; the shim writes activities in (device, resource, start) order, "
                "so its file is compared with the reference logger fed in that order"}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", type=int, default=3)
    ap.add_argument("--n-device", type=int, default=0, help="device rows (0 = the configuration's full size)")
    ap.add_argument("--cpu-sample", type=int, default=0, help="device rows of the CPU-baseline sample (0 = auto)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-host-legs", action="store_true", help="skip the host-records-to-file leg")
    ap.add_argument("--copy-bytes", type=int, default=1 << 30, help="size of the reference copy kernel run (0 = skip)")
    ap.add_argument("--summarize-kernel-trace", metavar="STATS_CSV", default=None)
    ap.add_argument("--summarize-hbm", nargs=3, metavar=("FETCH_DIR", "WRITE_DIR", "STATS_CSV"), default=None)
    ap.add_argument("--logger-benchmark", choices=["small", "medium", "large"], default=None,
                    help="run the reference's logger benchmark on both loggers instead of the hot-path bench")
    ap.add_argument("--iterations", type=int, default=0, help="iterations of --logger-benchmark (0 = the reference's defaults)")
    ap.add_argument("--threads", type=int, default=16, help="packing workers of the shim's bulk leg")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path runs on exactly one GPU (no sharding, no collectives); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    if args.summarize_kernel_trace:
        summarize_kernel_trace(args.summarize_kernel_trace)
        return
    if args.summarize_hbm:
        summarize_hbm(*args.summarize_hbm, config=args.config, copy_bytes=args.copy_bytes)
        return
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if args.logger_benchmark:
        logger_benchmark(args.logger_benchmark, args.iterations, args.threads)
        return
    from kineto_amd import abi
    from kineto_amd.engine import TraceEngine

    cfg = args.config
    n_dev = args.n_device or FULL_SIZE[cfg]
    t0 = time.perf_counter()
    sp, release = abi.synth_stream(cfg, n_dev, host_name="bench")
    s = sp.contents
    n_records = s.n_generic + s.n_runtime + s.n_device
    gen_s = time.perf_counter() - t0
    raw_bytes = s.n_generic * 64 + s.n_runtime * 96 + s.n_device * 64 + s.n_extcorr * 16 + s.n_args * 8

    eng = TraceEngine(s.trace_name.decode(), device=0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eng.submit_stream(sp)          # host -> HBM; not part of the timed steps
    torch.cuda.synchronize()
    h2d_s = time.perf_counter() - t0
    name_bytes = name_bytes_fetched(s)

    cold_first_step_ms = None
    for w in range(args.warmup):
        t0 = time.perf_counter()
        eng.process()              # the first pass allocates every working buffer and the document
        if w == 0:
            torch.cuda.synchronize()
            cold_first_step_ms = (time.perf_counter() - t0) * 1e3
    torch.cuda.synchronize()
    stage_sum = [0.0] * abi.N_STAGES
    t0 = time.perf_counter()
    for _ in range(args.steps):
        eng.process()
        st = eng.stats()
        for k in range(abi.N_STAGES):
            stage_sum[k] += st.stage_ms[k]
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    st = eng.stats()
    out_bytes = st.output_bytes
    stage_ms = {abi.STAGE_NAMES[k]: stage_sum[k] / args.steps for k in range(abi.N_STAGES) if stage_sum[k] > 0}
    stage_gbs = {abi.STAGE_NAMES[k]: st.stage_bytes[k] / (stage_sum[k] / args.steps * 1e-3) / 1e9
                 for k in range(abi.N_STAGES) if stage_sum[k] > 0 and st.stage_bytes[k] > 0}

    # PCIe-inclusive figure, reported on the side: one device -> pinned host copy of the document
    t0 = time.perf_counter()
    host_copy_ok = True
    try:
        p, n = C.c_void_p(), C.c_uint64()
        rc = eng.lib.ktj_output_host(eng.h, C.byref(p), C.byref(n))
        host_copy_ok = rc == 0
    except Exception:
        host_copy_ok = False
    d2h_s = time.perf_counter() - t0
    d2h_ms = eng.stats().stage_ms[8] if host_copy_ok else None
    copy_gbs = None
    if args.copy_bytes:
        ms = C.c_float()
        if eng.lib.ktj_debug_copy_reference(eng.h, args.copy_bytes, C.byref(ms)) == 0 and ms.value > 0:
            copy_gbs = 2 * args.copy_bytes / (ms.value * 1e-3) / 1e9   # read + write
    eng.close()
    host_legs = None if args.no_host_legs else host_to_file_legs(sp, n_records)
    release()
    small = None if args.no_host_legs else small_trace_legs()

    # algorithmic bytes of a stage / its time, as a fraction of the HBM peak (the three stages the
    # per-kernel target of this path is stated for, and the rest beside them)
    stage_frac = {k: v / HBM_PEAK_GBS for k, v in stage_gbs.items()}
    emit_ms = stage_ms.get("emit", 0.0)
    emit_alg = int(st.stage_bytes[7])
    achieved = emit_alg / (emit_ms * 1e-3) / 1e9 if emit_ms > 0 else 0.0
    result = {
        "metric": "trace_records_per_s",
        "value": n_records / (ms_per_step * 1e-3),
        "unit": "records/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "cold_first_step_ms": cold_first_step_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8/int64",
        "data": "synthetic",
        "config": {"workload": WORKLOAD[cfg], "records": int(n_records), "device_rows": int(n_dev),
                   "output_bytes": int(out_bytes), "raw_input_bytes": int(raw_bytes),
                   "output_placement": "device buffer (HBM)"},
        "output_gb_per_s": out_bytes / (ms_per_step * 1e-3) / 1e9,
        "output_frac_of_hbm_peak": out_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "stage_ms": stage_ms,
        "stage_algorithmic_gb_per_s": stage_gbs,
        "stage_frac_of_peak": stage_frac,
        "roofline": {"bound": "hbm", "kernel": DOMINANT_KERNEL, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes_per_launch": emit_alg, "avg_launch_ms": emit_ms,
                     # the same with every record's name counted as fetched once per record (each distinct
                     # string is counted once in `achieved`: the dictionary is a few MB and stays cached)
                     "algorithmic_bytes_with_name_bytes_per_record": emit_alg + name_bytes,
                     "achieved_with_name_bytes_per_record": (emit_alg + name_bytes) / (emit_ms * 1e-3) / 1e9 if emit_ms > 0 else 0.0},
        "pcie": {"h2d_submit_s": h2d_s, "d2h_document_ms": d2h_ms, "d2h_wall_s": d2h_s,
                 "records_per_s_incl_d2h": (n_records / (ms_per_step * 1e-3 + (d2h_ms or 0) * 1e-3)) if d2h_ms else None},
        "host_legs": host_legs,
        "small_traces": small,
        "generate_s": gen_s,
        "copy_kernel_gb_per_s": copy_gbs,
    }
    if copy_gbs:
        result["roofline"]["frac_of_copy_kernel"] = achieved / copy_gbs
    result["roofline"]["traffic"] = measured_traffic(cfg, n_dev)
    if not args.no_cpu_baseline:
        sample = args.cpu_sample or max(1000, min(n_dev, {1: 10000, 2: 1000000, 3: 2500000, 4: 4000000, 5: 1000000}[cfg]))
        ref_leg, result["cpu_baseline"] = cpu_baseline(cfg, sample)
        if ref_leg:
            result["reference_logger"] = ref_leg
    print(json.dumps(result))


if __name__ == "__main__":
    main()
