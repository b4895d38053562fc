#!/usr/bin/env python3
"""Benchmark of the MI355X-native ROC_SHMEM data path.

    python bench.py --gpus 1 --steps K --warmup W

One "step" is one pass of the hot path over one batch of synthetic input: a
`roc_shmem_ctx_float_sum_wg_to_all` over 8 PE slices of 2^26 elements each
(the configuration the HBM-roofline target is quoted on), all slices resident
in the one GPU's HBM before the timed region starts.  The JSON line also
carries the other workloads of the metric (bf16 / int64 reductions, wg putmem,
small puts and AMOs, broadcast, alltoall), the roofline of the dominant kernel
and the CPU oracle timed on the host cores of the same box.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published peak

# HBM bytes per launch of the headline kernel come from two rocprofv3 --pmc runs (FETCH_SIZE, then
# WRITE_SIZE) of `bench.py --counter-pair`, each counter scaled by what it reads for a wg-putmem copy
# of known size in the same run.  `bench.py --record-traffic FETCH.csv WRITE.csv` turns the two
# counter files into TRAFFIC_JSON together with a fingerprint of the kernel's sources; when the
# sources have changed since, `roofline.traffic` is reported as null instead of a stale figure.
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "to_all_float_sum_8pe_2e26.traffic.json")
KERNEL_SOURCES = ["roc_shmem_amd/csrc/rocshmem_device/reduce.hpp", "roc_shmem_amd/csrc/rocshmem_device/copy.hpp",
                  "roc_shmem_amd/csrc/rocshmem_device/sync.hpp", "roc_shmem_amd/csrc/cabi/drv_reduce.hip"]

# Launch shapes chosen by measurement on MI355X (256 CUs).
TO_ALL_LAUNCH = dict(wgs_per_pe=32, wg_size=1024)
# The headline: the unchanged roc_shmem_ctx_float_sum_wg_to_all, one call per workgroup over a
# tile of 2^21 elements (32 tiles per PE dealt to the PE's 32 workgroups of 1024 lanes; each call
# is 8 passes of 128 KiB per member)
TO_ALL_STANDARD_LAUNCH = dict(wgs_per_pe=32, wg_size=1024, tile=1 << 21)
# Shapes the pacing tuner is tried with (256 workgroups either way: 128 KiB or 64 KiB per member per pass).
TUNE_SHAPES = (dict(wgs_per_pe=32, wg_size=1024), dict(wgs_per_pe=32, wg_size=512))
PUT_LAUNCH = dict(wgs_per_pe=32, wg_size=512)
# one large message shared by the PE's workgroups (sharded extension): 1024-lane workgroups
# (6.36 against 6.17 TB/s with 512 lanes; standard 256 KiB calls prefer 512: 6.12 against 5.87)
PUT_SHARED_LAUNCH = dict(wgs_per_pe=32, wg_size=1024)
PUT_TILE = 256 << 10


def random_payload(rs, arr, n_pes, seed):
    """Uniform random bytes in every PE's copy of `arr` (one random block, rotated per PE)."""
    block = np.random.default_rng(seed).integers(0, 256, min(arr.nbytes, 64 << 20), dtype=np.uint8)
    reps = -(-arr.nbytes // block.size)
    for p in range(n_pes):
        data = np.tile(np.roll(block, 4099 * p), reps)[:arr.nbytes]
        arr.write(p, data.view(arr.dtype))


def event_time_ms(rs, fn, iters):
    start, stop = rs.Event(), rs.Event()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    ms = start.elapsed_ms(stop)
    start.destroy()
    stop.destroy()
    return ms


def per_launch_ms(rs, fn, iters):
    """Duration of each of `iters` launches: an event between every two launches."""
    marks = [rs.Event() for _ in range(iters + 1)]
    marks[0].record()
    for i in range(iters):
        fn()
        marks[i + 1].record()
    out = [marks[i].elapsed_ms(marks[i + 1]) for i in range(iters)]
    for m in marks:
        m.destroy()
    return out


def kernel_fingerprint():
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic():
    """(bytes per launch or None, note) from the tracked counter summary."""
    try:
        with open(TRAFFIC_JSON) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None, "no counter summary (%s)" % os.path.relpath(TRAFFIC_JSON, ROOT)
    if rec.get("kernel_sources_sha256_16") != kernel_fingerprint():
        return None, "stale: the kernel's sources changed after the counters were read; rerun the --pmc pair"
    return int(rec["traffic_bytes_per_launch"]), "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, see profiles/"


def record_traffic(fetch_csv, write_csv):
    """Reads the two rocprofv3 counter files of `bench.py --counter-pair` and writes TRAFFIC_JSON."""
    import csv

    def mean_kib(path, counter, kernel_prefix):
        # only launches that fill the chip: the copy of known size is issued by 256 workgroups, the
        # same kernel's one-workgroup-per-PE rows of the put sweep move other amounts
        vals = []
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] == counter and row["Kernel_Name"].startswith(kernel_prefix) and \
                        int(row["Grid_Size"]) // int(row["Workgroup_Size"]) >= 256:
                    vals.append(float(row["Counter_Value"]))
        if not vals:
            raise SystemExit("%s: no %s rows for %s" % (path, counter, kernel_prefix))
        return sum(vals) / len(vals), len(vals)

    known = 8 * (256 << 20)                          # the copy reads and writes 2 GiB
    reduce_kernel = "void (anonymous namespace)::to_all_kernel<float"
    copy_kernel = "(anonymous namespace)::rma_kernel"
    out = {"kernel": "to_all_kernel<float, ROC_SHMEM_SUM, kTiled> (standard calls, one per workgroup)",
           "copy_bytes_known": known}
    total = 0.0
    for name, path in (("FETCH_SIZE", fetch_csv), ("WRITE_SIZE", write_csv)):
        k, n_k = mean_kib(path, name, reduce_kernel)
        c, n_c = mean_kib(path, name, copy_kernel)
        scale = known / (c * 1024.0)
        out[name] = {"to_all_kib_per_dispatch": k, "dispatches": n_k, "copy_kib_per_dispatch": c,
                     "copy_dispatches": n_c, "scale_known_over_counter": scale,
                     "to_all_bytes": k * 1024.0 * scale}
        total += k * 1024.0 * scale
    out["traffic_bytes_per_launch"] = int(round(total))
    out["algorithmic_bytes_per_launch"] = 2 * 8 * (1 << 26) * 4
    out["kernel_sources_sha256_16"] = kernel_fingerprint()
    out["kernel_sources"] = KERNEL_SOURCES
    with open(TRAFFIC_JSON, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(json.dumps(out))


def timeline_summary(path):
    """Summary of the clock readings a timeline build of the library leaves in ROC_SHMEM_TIMELINE_FILE
    (csrc/Makefile: EXTRA=-DROCSHMEM_TIMELINE; the readings of the last large reduction before the
    runtime went): microseconds after the first wave entered the call, per mark, for the waves on
    even and on odd XCDs - first wave, median, last wave - and the same for wave 0 and the last
    wave of every workgroup."""
    raw = np.fromfile(path, dtype=np.uint64).reshape(-1, 8)
    rows = raw[raw[:, 0] != 0]
    if not len(rows):
        return {"waves": 0}
    t0 = rows[:, 0].min()
    us = (rows[:, :6].astype(np.int64) - np.int64(t0)) / 100.0      # 100 MHz clock
    xcd = (rows[:, 6] & 15).astype(int)
    wave_of_wg = np.nonzero(raw[:, 0] != 0)[0] % 16
    names = ["entered", "entry_barrier_done", "first_burst_stored", "last_pass_stored", "own_stores_landed",
             "closing_barrier_done"]
    out = {"waves": int(len(rows)), "period_ticks": int(rows[0, 6] >> 16)}
    for label, sel in (("even_xcds", xcd % 2 == 0), ("odd_xcds", xcd % 2 == 1),
                       ("first_wave_of_each_workgroup", wave_of_wg == 0),
                       ("last_wave_of_each_workgroup", wave_of_wg == wave_of_wg.max())):
        if not sel.any():
            continue
        out[label] = {n: [round(float(np.min(us[sel, i])), 1), round(float(np.median(us[sel, i])), 1),
                          round(float(np.max(us[sel, i])), 1)] for i, n in enumerate(names)}
    # how many waves are still streaming (own stores not landed) at 10 us steps before the end
    end = us[:, 4].max()
    out["waves_still_streaming_at_us_before_end"] = {str(d): int((us[:, 4] > end - d).sum()) for d in (5, 10, 20, 30, 40, 60, 80)}
    out["per_xcd_last_store_landed_us"] = {str(x): round(float(us[xcd == x, 4].max()), 1) for x in sorted(set(xcd))}
    return out


class ClockSampler:
    """Clock and power readings while a loop of launches runs: the driver's files
    (/sys/class/drm/card0/device: the GFX clock level marked current, socket power in microwatts)
    read by a thread every 20 ms, and `amd-smi metric -c -p --json` (the GFX clock of every XCD)
    run by a child process meanwhile."""

    SYS = "/sys/class/drm/card0/device"

    def __init__(self):
        import glob
        self.power_files = glob.glob(self.SYS + "/hwmon/*/power1_input") + glob.glob(self.SYS + "/hwmon/*/power1_average")
        self.sclk, self.power, self.xcd_clocks, self.smi_power = [], [], [], []
        self.stop = False

    def _sys_loop(self):
        import re
        while not self.stop:
            try:
                with open(self.SYS + "/pp_dpm_sclk") as f:
                    m = re.search(r"(\d+)Mhz \*", f.read())
                if m:
                    self.sclk.append(int(m.group(1)))
                if self.power_files:
                    with open(self.power_files[0]) as f:
                        self.power.append(int(f.read()) / 1e6)
            except (OSError, ValueError):
                pass
            time.sleep(0.02)

    def _smi_loop(self):
        import subprocess
        while not self.stop:
            try:
                txt = subprocess.run(["amd-smi", "metric", "-c", "-p", "--json"], capture_output=True, text=True,
                                     timeout=20).stdout
                rec = json.loads(txt)
                rec = rec[0] if isinstance(rec, list) else rec
                rec = rec.get("gpu_data", [rec])[0] if isinstance(rec, dict) and "gpu_data" in rec else rec
                clocks = [v["clk"]["value"] for k, v in sorted(rec.get("clock", {}).items())
                          if k.startswith("gfx_") and isinstance(v.get("clk"), dict) and isinstance(v["clk"].get("value"), (int, float))]
                if clocks:
                    self.xcd_clocks.append(clocks)
                pw = rec.get("power", {}).get("socket_power", {})
                if isinstance(pw, dict) and isinstance(pw.get("value"), (int, float)):
                    self.smi_power.append(pw["value"])
            except Exception:   # the tool is optional, its output format differs between releases
                time.sleep(0.2)

    def __enter__(self):
        import threading
        self.threads = [threading.Thread(target=self._sys_loop, daemon=True), threading.Thread(target=self._smi_loop, daemon=True)]
        for t in self.threads:
            t.start()
        return self

    def __exit__(self, *exc):
        self.stop = True
        for t in self.threads:
            t.join(timeout=30)
        return False

    def summary(self):
        def stats(v):
            return None if not v else {"mean": round(float(np.mean(v)), 1), "min": round(float(np.min(v)), 1),
                                       "max": round(float(np.max(v)), 1), "samples": len(v)}
        out = {"sysfs_gfx_clock_MHz": stats(self.sclk), "sysfs_socket_power_W": stats(self.power),
               "amd_smi_socket_power_W": stats(self.smi_power)}
        if self.xcd_clocks:
            arr = np.array([c for c in self.xcd_clocks if len(c) == len(self.xcd_clocks[0])], dtype=float)
            out["amd_smi_gfx_clock_MHz_by_xcd_mean"] = [round(float(x), 0) for x in arr.mean(axis=0)]
            out["amd_smi_gfx_clock_MHz_mean"] = round(float(arr.mean()), 1)
            out["amd_smi_samples"] = int(len(arr))
        return out


def bench_clock_ab(rs, oracle, variants, seconds, launches_only=0):
    """The GFX clock (which the L2 runs at) and the socket power under loops of one kernel each.
    Every variant moves 4 GiB per launch (the one-way probes 2 GiB).  seconds: length of each sampled loop; launches_only > 0:
    no sampling, that many launches per variant (for a rocprofv3 --pmc run, whose TCC_CYCLE_sum /
    128 / duration is the L2 clock the kernel saw)."""
    out = {}
    total_elems = 1 << 29                      # 8 x 2^26 four-byte elements
    for name in variants:
        kind, _, arg = name.partition(":")
        n_pes = int(arg) if kind == "members" else 8
        n = total_elems // n_pes
        rs.roc_shmem_init(n_pes, 2 * n * 4 + (64 << 20), 64, 1024)
        dtype, op = (rs.FLOAT, rs.MAX) if kind == "float_max" else (rs.INT, rs.SUM) if kind == "int_sum" else (rs.FLOAT, rs.SUM)
        npd = rs.NP_DTYPE[dtype]
        src = rs.sym_array(n, npd)
        dst = rs.sym_array(n, npd, fill=0)
        psync = rs.sym_array(max(64, 256 // n_pes) * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
        rng = np.random.default_rng(3)
        block = rng.standard_normal(min(n, 1 << 24), dtype=np.float32)
        for p in range(n_pes):
            vals = np.tile(np.roll(block, 977 * p), -(-n // block.size))[:n]
            src.write(p, vals.astype(npd) if dtype == rs.FLOAT else (vals * 1000).astype(npd))
        wgs = 256 // n_pes
        shard = rs.Launch(wgs, 1024)
        tiled = rs.Launch(wgs, 1024, n // wgs)
        if kind == "free":
            rs.set_pacing(0, 0)
        if kind == "put":
            fn = lambda: rs.roc_shmem_rma(rs.PUT, rs.WG_SHARED, dst, src, n * 4, 1, n * 4, n * 4, 1, shard)
        elif kind in ("read", "write"):
            fn = lambda: rs.stream_probe(rs.STREAM_READ if kind == "read" else rs.STREAM_WRITE, src, n * 4, None, 7, shard)
        elif kind == "standard":
            fn = lambda: rs.roc_shmem_to_all(dtype, op, dst, src, n, 0, 0, n_pes, None, psync, tiled)
        else:
            fn = lambda: rs.roc_shmem_to_all(dtype, op, dst, src, n, 0, 0, n_pes, None, psync, shard)
        for _ in range(3):
            fn()
        rs.synchronize()
        if launches_only:
            for _ in range(launches_only):
                fn()
            rs.synchronize()
            out[name] = {"launches": launches_only}
        else:
            ms1 = event_time_ms(rs, fn, 10) / 10
            reps = max(10, int(seconds * 1e3 / ms1))
            with ClockSampler() as sampler:
                time.sleep(0.1)
                ms = event_time_ms(rs, fn, reps) / reps
            # (the one-way probes move half as much per launch: 2 GiB)
            row = {"GBps": round((1.0 if kind in ("read", "write") else 2.0) * total_elems * 4 / ms / 1e6, 1),
                   "ms_per_launch": round(ms, 4), "launches": reps}
            row.update(sampler.summary())
            out[name] = row
            print(name, json.dumps(row), file=sys.stderr, flush=True)
        if rs.take_status():
            raise RuntimeError("device status word raised")
        rs.roc_shmem_finalize()
    return out


def host_threads():
    """Threads for the CPU legs: the cores this process may run on, capped by the box's
    per-GPU share of host cores where the environment states one (OMP_NUM_THREADS)."""
    avail = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    share = os.environ.get("OMP_NUM_THREADS", "")
    share = int(share) if share.isdigit() and int(share) > 0 else None
    used = min(avail, share) if share else avail
    return used, {"os_cpu_count": os.cpu_count(), "cores_this_process_may_use": avail,
                  "OMP_NUM_THREADS": share}


def device_report():
    """Clock and power state of the GPU as rocm-smi prints it (run as a child process)."""
    import subprocess
    try:
        txt = subprocess.run(["rocm-smi", "--showclocks", "--showpower", "--showperflevel"],
                             capture_output=True, text=True, timeout=30).stdout
    except Exception as e:  # the tool is optional
        return {"rocm_smi": "unavailable: %s" % e}
    keep = [ln.strip() for ln in txt.splitlines() if ln.startswith("GPU[0]")]
    return {"rocm_smi": keep[:16]}


def bench_to_all(rs, oracle, steps, warmup, dtype, n_pes, n, seed, check=True, cpu=False,
                 spread=False, launch_shape=None, tune=False, pace=None):
    """Returns a dict with ms_per_step, GB/s (algorithmic 2*P*N*s bytes) and optional CPU figures.
    pace: None = the pacing rates the library holds (its defaults: 6.7 TB/s, 6.3 with short passes),
    0 = workgroups run free, another value = that rate in bytes per tick.
    tune: let the library measure, outside the timed region, which rate suits this reduction on
    this card, with the launch shapes of TUNE_SHAPES; the timed steps then run with the better
    shape and the rate the tuner set (0 = free running).  The library's rate is put back at the end."""
    npd = rs.NP_DTYPE[dtype]
    es = np.dtype(npd).itemsize
    src = rs.sym_array(n, npd)
    dst = rs.sym_array(n, npd, fill=0x5A)
    launch = rs.Launch(**(launch_shape or TO_ALL_LAUNCH))
    psync = rs.sym_array(max(launch.wgs_per_pe, 64) * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
    rng = np.random.default_rng(seed)
    host = []
    for p in range(n_pes):
        if dtype in (rs.LONG, rs.LONGLONG):
            vals = rng.integers(-(1 << 30), (1 << 30) + 1, size=n, dtype=np.int64)
        elif dtype == rs.BF16:
            vals = oracle.float_to_bf16(rng.standard_normal(n, dtype=np.float32))
        else:
            vals = rng.standard_normal(n, dtype=np.float32).astype(npd)
        src.write(p, vals)
        host.append(vals)

    def step():
        rs.roc_shmem_to_all(dtype, rs.SUM, dst, src, n, 0, 0, n_pes, None, psync, launch)

    tuning = None
    pacing_before = rs.get_pacing()
    if pace is not None:
        rs.set_pacing(pacing_before[0], pace)
    if tune:
        tuning, best = {}, None
        for shape in ([launch_shape] if launch_shape else TUNE_SHAPES):
            res = rs.tune_reduce_pacing(dtype, rs.SUM, dst, src, n, 0, 0, n_pes, psync, rs.Launch(**shape))
            tuning["%dx%d" % (shape["wgs_per_pe"], shape["wg_size"])] = {k: round(v, 4) for k, v in res.items()}
            if best is None or res["paced_ms"] < best[1]["paced_ms"]:
                best = (shape, res)
        launch = rs.Launch(**best[0])
        rs.set_pacing(pacing_before[0], best[1]["rate"])
    for _ in range(warmup):
        step()
    rs.synchronize()
    ms = event_time_ms(rs, step, steps)
    rs.synchronize()
    status = rs.take_status()
    if status:
        raise RuntimeError("device status word raised: %d" % status)
    out = {"ms_per_step": ms / steps, "GBps": 2.0 * n_pes * n * es / (ms / steps) / 1e6,
           "bytes_per_step": 2 * n_pes * n * es,
           "launch": {"wgs_per_pe": launch.wgs_per_pe, "wg_size": launch.wg_size, "tile": launch.tile},
           "pacing_bytes_per_tick": rs.get_pacing()[1]}
    if tuning is not None:
        out["pacing_tuner"] = tuning
    if spread:
        each = sorted(per_launch_ms(rs, step, steps))
        rs.synchronize()
        out["ms_median"] = each[len(each) // 2]
        out["ms_min"] = each[0]
        out["ms_max"] = each[-1]
    rs.set_pacing(*pacing_before)

    heap = None
    if check or cpu:
        heap = oracle.Heap(n_pes, 2 * n * es)
        for p in range(n_pes):
            heap.view(p, 0, n, npd)[:] = host[p]
    if check:
        # Three windows of the result (the first elements, an odd place in the middle, the last
        # elements) on every PE: bit for bit against the oracle's statement of the library's
        # arithmetic (integers exact; float folded in double, bfloat16 in float, ascending member
        # order, one rounding), and for floating point within the stated tolerance of the fp64 sum.
        m = min(n, 1 << 16)
        checked = 0
        for at in sorted({0, max(0, (n // 2 + 12345) // 8 * 8 - m // 2), n - m}):
            sample = oracle.Heap(n_pes, 2 * m * es)
            for p in range(n_pes):
                sample.view(p, 0, m, npd)[:] = host[p][at:at + m]
            got = [dst.read(p, m, at) for p in range(n_pes)]
            oracle.to_all_rounded_once(sample, dtype, oracle.SUM, m * es, 0, m)
            for p in range(n_pes):
                assert np.array_equal(got[p].view(np.uint8), sample.view(p, m * es, m, npd).view(np.uint8)), \
                    "parity check failed (bit-exact, window at %d, PE %d)" % (at, p)
            if dtype not in (rs.LONG, rs.LONGLONG):
                ref = oracle.to_all_f64(sample, dtype, oracle.SUM, 0, m)
                scale = oracle.abs_sum_f64(sample, dtype, 0, m)
                tol, eps = (1e-6, 2.0 ** -24) if dtype == rs.FLOAT else (1e-2, 2.0 ** -8)
                for p in range(n_pes):
                    g = (oracle.bf16_to_float(got[p]) if dtype == rs.BF16 else got[p]).astype(np.float64)
                    assert (np.abs(g - ref) <= tol * np.maximum(np.abs(ref), eps * scale)).all(), \
                        "parity check failed (tolerance, window at %d, PE %d)" % (at, p)
            checked += m
        out["parity_checked_elements"] = checked
        out["parity"] = "bit-exact against the oracle in %d windows of %d elements on every PE" % (checked // m, m)
    if cpu:
        cores, host = host_threads()

        def cpu_rate(threads, passes):
            best = None
            for i in range(passes + 1):          # the first pass warms the pages
                t0 = time.perf_counter()
                oracle.to_all(heap, dtype, oracle.SUM, n * es, 0, n, threads=threads)
                dt = time.perf_counter() - t0
                if i and (best is None or dt < best):
                    best = dt
            return 2.0 * n_pes * n * es / best / 1e9

        out["cpu"] = {"value": cpu_rate(cores, 3), "unit": "GB/s", "cores": cores,
                      "kind": "port",
                      "sample": "same workload, full size (%d slices x 2^%d %s, sum), CPU oracle "
                                "chunked over %d host threads, best of 3 passes after one warm-up"
                                % (n_pes, int(np.log2(n)), np.dtype(npd).name, cores),
                      "host": host,
                      "one_thread_per_pe": {"value": round(cpu_rate(min(n_pes, cores), 2), 2),
                                            "cores": min(n_pes, cores)},
                      "single_thread": {"value": round(cpu_rate(1, 1), 2), "cores": 1}}
    src.free()
    dst.free()
    psync.free()
    return out


def cpu_other_legs(oracle):
    """The other two legs of the metric on the host cores, next to the reduction's: what the
    reference's host-centric path does for them on one node (MPI_Put -> memcpy,
    MPI_Fetch_and_op -> an atomic add, host_helpers.hpp:52-88, host_templates.hpp:285-307), and
    the scalar 64-byte WQE builder."""
    cores, _ = host_threads()
    out = {}
    # putmem: 8 PEs each move one 64 MiB message to the next PE's slice
    n_pes, msg = 8, 64 << 20
    src = np.full(n_pes * msg, 7, dtype=np.uint8)
    dst = np.zeros(n_pes * msg, dtype=np.uint8)

    def copy_rate(threads):
        best = None
        for i in range(4):
            t0 = time.perf_counter()
            oracle.copy_mt(dst, src, threads)
            dt = time.perf_counter() - t0
            if i and (best is None or dt < best):
                best = dt
        return 2.0 * n_pes * msg / best / 1e9

    out["putmem_64MiB_8pe"] = {"value": round(copy_rate(cores), 2), "unit": "GB/s (read + write)", "cores": cores,
                               "single_thread": round(copy_rate(1), 2), "kind": "port",
                               "sample": "8 x 64 MiB memcpy, best of 3 passes after one warm-up"}
    del src, dst
    # small operations: 5 M 8-byte puts + 5 M int64 fetch-adds, 16 slices x 64 MiB, random targets
    n_ops, n_slices, words = 10_000_000, 16, (64 << 20) // 8
    rng = np.random.default_rng(4)
    ops = np.zeros(n_ops, oracle.SMALL_OP_DTYPE)
    is_put = np.arange(n_ops) % 2 == 0
    ops["kind"] = np.where(is_put, oracle.OP_P64, oracle.OP_FADD64)
    ops["pe"] = rng.integers(0, n_slices, n_ops)
    ops["offset"] = np.where(is_put, rng.integers(0, words // 2, n_ops), words // 2 + rng.integers(0, words // 2, n_ops)) * 8
    ops["value"] = rng.integers(-1000, 1000, n_ops)
    heap = oracle.Heap(n_slices, 64 << 20)
    t0 = time.perf_counter()
    oracle.small_ops(heap, ops[:2_000_000], np.zeros(2_000_000, np.uint32))
    one = 2_000_000 / (time.perf_counter() - t0) / 1e6
    best = None
    for i in range(3):
        t0 = time.perf_counter()
        oracle.small_ops_mt(heap, ops, cores)
        dt = time.perf_counter() - t0
        if i and (best is None or dt < best):
            best = dt
    out["small_ops_put8_fetch_add"] = {"value": round(n_ops / best / 1e6, 1), "unit": "Mops/s", "cores": cores,
                                       "single_thread": round(one, 1), "kind": "port",
                                       "sample": "10 M operations (half 8-byte puts, half int64 fetch-adds) on 16 x "
                                                 "64 MiB host slices with hardware atomics, best of 2 passes after "
                                                 "one warm-up; single thread: the sequential model on 2 M of them"}
    del heap
    # WQE builder: 10 M entries (1 M distinct requests, ten laps) into a 1024-entry ring
    import ctypes
    n_req = 1_000_000
    reqs = (oracle.WqeReq * n_req)()
    view = np.frombuffer(reqs, dtype=np.uint8).reshape(n_req, ctypes.sizeof(oracle.WqeReq))
    view[:] = 0
    view[:, oracle.WqeReq.opcode.offset] = np.where(np.arange(n_req) % 2 == 0, 0x08, 0x12)
    view[:, oracle.WqeReq.size.offset] = 8
    raddr = (0x7F0000000000 + rng.integers(0, 1 << 30, n_req) * 8).astype(np.uint64)
    view[:, oracle.WqeReq.raddr.offset:oracle.WqeReq.raddr.offset + 8] = raddr.view(np.uint8).reshape(n_req, 8)
    qp = oracle.Qp()
    qp.ctrl_qp_sq, qp.lkey, qp.atomic_lkey, qp.atomic_ret_base, qp.max_nwqe = 0x000100, 0x2000, 0x3000, 1 << 40, 1024
    ring = np.zeros(1024 * 64, np.uint8)
    t0 = time.perf_counter()
    for lap in range(10):
        oracle.wqe_build_many(ring, qp, lap * n_req, reqs)
    out["wqe_build"] = {"value": round(10 * n_req / (time.perf_counter() - t0) / 1e6, 1), "unit": "M entries/s",
                        "cores": 1, "kind": "port",
                        "sample": "10 M entries (inline 8-byte writes and fetch-adds alternating) by the scalar "
                                  "builder into a 1024-entry ring, one thread"}
    return out


def bench_putmem(rs, steps, n_pes, msg_bytes_list, get_sweep=False):
    """wg putmem from every PE p to PE p+1: GB/s counted as 2*m bytes per message (read+write).
    get_sweep: the same sweep with roc_shmemx_ctx_getmem_wg (the reference's tester walks every
    size for every test type, tester.cpp:503-563), under keys "getmem_<bytes>"."""
    total = 256 << 20
    src = rs.sym_array(total, np.uint8)
    dst = rs.sym_array(total, np.uint8, fill=0)
    random_payload(rs, src, n_pes, seed=2)
    res = {}
    for kind, prefix in ((rs.PUT, ""), (rs.GET, "getmem_")) if get_sweep else ((rs.PUT, ""),):
        for m in msg_bytes_list:
            if m >= PUT_TILE:
                tile, n_msgs = PUT_TILE, total // PUT_TILE      # large messages tiled across workgroups
            else:
                tile, n_msgs = m, min(total // max(m, 256), 1 << 16)
            stride = max(tile, 256)
            # A few large workgroups stream best.  A blocking put returns when its loads have, so short
            # messages are bound by load latency and want as many resident workgroups as the CUs hold
            # (4 KiB: 2.6 TB/s with 64 x 256 lanes per PE, 4.6 with 256 x 128).
            # (32 KiB - 128 KiB per call: one or two accesses per lane of 1024 in flight, 3-4 % above the
            # smaller workgroups' rate on one card)
            launch = rs.Launch(**PUT_LAUNCH) if tile >= (256 << 10) else \
                rs.Launch(32, 1024) if tile >= (32 << 10) else \
                rs.Launch(64, 256) if tile > 4096 else rs.Launch(256, 128)

            def step():
                rs.roc_shmem_rma(kind, rs.WG, dst, src, tile, n_msgs, stride, stride, 1, launch)

            step()
            rs.synchronize()
            ms = event_time_ms(rs, step, steps) / steps
            moved = 2.0 * n_pes * tile * n_msgs
            res[prefix + str(m)] = {"GBps": moved / ms / 1e6, "ms": ms, "calls_per_pe": n_msgs, "bytes_per_call": tile,
                                    "Mmsgs_per_s": n_pes * n_msgs / ms / 1e3}
    # getmem in the same shape as the largest put
    launch = rs.Launch(**PUT_LAUNCH)

    def get_step():
        rs.roc_shmem_rma(rs.GET, rs.WG, dst, src, PUT_TILE, total // PUT_TILE, PUT_TILE, PUT_TILE, 1, launch)

    get_step()
    rs.synchronize()
    ms = event_time_ms(rs, get_step, steps) / steps
    res["getmem_67108864"] = {"GBps": 2.0 * n_pes * total / ms / 1e6, "ms": ms,
                              "calls_per_pe": total // PUT_TILE, "bytes_per_call": PUT_TILE}
    # one 64 MiB message per PE moved by all of the PE's workgroups together (sharded extension)
    msg = 64 << 20
    launch = rs.Launch(**PUT_SHARED_LAUNCH)

    def shared():
        rs.roc_shmem_rma(rs.PUT, rs.WG_SHARED, dst, src, msg, total // msg, msg, msg, 1, launch)

    shared()
    rs.synchronize()
    ms = event_time_ms(rs, shared, steps) / steps
    res["67108864_shared"] = {"GBps": 2.0 * n_pes * total / ms / 1e6, "ms": ms, "calls_per_pe": total // msg,
                              "bytes_per_call": msg, "note": "roc_shmemx_ctx_putmem_wg_shard", "launch": PUT_SHARED_LAUNCH}

    def shared_get():
        rs.roc_shmem_rma(rs.GET, rs.WG_SHARED, dst, src, msg, total // msg, msg, msg, 1, launch)

    shared_get()
    rs.synchronize()
    ms = event_time_ms(rs, shared_get, steps) / steps
    res["getmem_67108864_shared"] = {"GBps": 2.0 * n_pes * total / ms / 1e6, "ms": ms, "calls_per_pe": total // msg,
                                     "bytes_per_call": msg, "note": "roc_shmemx_ctx_getmem_wg_shard",
                                     "launch": PUT_SHARED_LAUNCH}
    # the reference's own launch model (driver.sh: one workgroup per PE issues the whole message with
    # one roc_shmemx_ctx_putmem_wg call): what one compute unit moves
    one = {}
    launch = rs.Launch(1, 1024)
    for m in (64 << 10, 1 << 20, 64 << 20):
        def one_call():
            rs.roc_shmem_rma(rs.PUT, rs.WG, dst, src, m, 1, m, m, 1, launch)

        one_call()
        rs.synchronize()
        ms = event_time_ms(rs, one_call, steps) / steps
        one[str(m)] = {"GBps": 2.0 * n_pes * m / ms / 1e6, "us": ms * 1e3}
    res["one_workgroup_per_pe_one_call_per_message"] = one
    # the sharded put in the launch shape of the fastest plain copy: one 256 MiB message per PE, one
    # small workgroup per share of a few KiB ("<share bytes>x<lanes>"; one, two or four accesses per lane)
    small = {}
    for share, lanes in ((4096, 256), (4096, 128), (8192, 256), (2048, 64), (8192, 128)):
        launch = rs.Launch(total // share, lanes)

        def small_shares():
            rs.roc_shmem_rma(rs.PUT, rs.WG_SHARED, dst, src, total, 1, total, total, 1, launch)

        small_shares()
        rs.synchronize()
        ms = event_time_ms(rs, small_shares, steps) / steps
        small["%dx%d" % (share, lanes)] = round(2.0 * n_pes * total / ms / 1e6, 1)
    res["268435456_shared_one_small_workgroup_per_share"] = small
    src.free()
    dst.free()
    return res


def bench_nbi_windows(rs, steps, n_pes, msg_bytes_list, max_windows=1):
    """The reference's message-rate pattern (primitive_mr_tester.cpp:32-58: 64 putmem_nbi, one
    quiet) at workgroup and at wavefront granularity: every workgroup (every wave) issues a window
    of 64 roc_shmemx_ctx_putmem_nbi_wg (_wave) calls of one size to the next PE, then the
    workgroup's waves meet and one lane issues the quiet (a wave's first lane for the wave forms);
    a kernel is one such window per workgroup (wave), or up to max_windows of them, as many as the
    buffers hold (the reference's kernel runs 64 x loop windows; every quiet between two windows
    drains the workgroup's memory pipeline and writes this XCD's L2 back).  GB/s counted as 2*m
    bytes per message, M messages/s; the launch shape is the best of a few for each size (named in
    the row)."""
    total = 256 << 20
    src = rs.sym_array(total, np.uint8)
    dst = rs.sym_array(total, np.uint8, fill=0)
    random_payload(rs, src, n_pes, seed=2)
    shapes = {"wg": ((256, 128), (128, 256), (64, 256), (64, 512), (32, 512), (32, 1024)),
              "wave": ((64, 256), (32, 512), (32, 1024), (64, 512))}
    res = {}
    for gran, gname in ((rs.WG, "wg"), (rs.WAVE, "wave")):
        rows = {}
        for kind, kname in ((rs.PUT_NBI, "putmem_nbi"), (rs.GET_NBI, "getmem_nbi")):
            for m in msg_bytes_list:
                stride, best = max(m, 256), None
                for wgs, lanes in shapes[gname]:
                    per_window = 64 * (wgs if gname == "wg" else wgs * (lanes // 64))
                    n_windows = min(max_windows, total // (per_window * stride))
                    if n_windows == 0:
                        continue
                    n_msgs = per_window * n_windows
                    launch = rs.Launch(wgs, lanes)

                    def step():
                        rs.roc_shmem_rma(kind, gran, dst, src, m, n_msgs, stride, stride, 1, launch)

                    step()
                    rs.synchronize()
                    ms = event_time_ms(rs, step, steps) / steps
                    rate = 2.0 * n_pes * m * n_msgs / ms / 1e6
                    if best is None or rate > best["GBps"]:
                        best = {"GBps": round(rate, 1), "Mmsgs_per_s": round(n_pes * n_msgs / ms / 1e3, 1),
                                "us_per_kernel": round(ms * 1e3, 2), "windows_per_kernel": n_windows,
                                "launch": "%dx%d" % (wgs, lanes)}
                if best:
                    rows["%s_%d" % (kname, m)] = best
        res[gname] = rows
    if rs.take_status():
        raise RuntimeError("device status word raised")
    src.free()
    dst.free()
    return res


def bench_streams(rs, n_pes, steps=10):
    """What this card's memory system gives plain streams (rsm_stream_probe): reads alone, writes
    alone and a copy, for two shapes of launch.  `staying`: workgroups that stay and take pass after
    pass, the shape a device-side collective has (32 or 64 workgroups of 1024 or 512 lanes per PE,
    two to eight accesses per lane and pass; the best of them for each kind).  `one_per_pass`: as many small workgroups as passes, handed out by the hardware in address
    order, which only a kernel launched for the purpose can have.  The harmonic mean of a shape's
    two one-way rates, 2 / (1/read + 1/write), is what a stream that reads and writes as much would
    reach if mixing the directions cost nothing; the copy rows show what it costs.  Also the HIP
    runtime's own fill and device-to-device copy over the same buffers."""
    per_pe = 512 << 20          # 4 GiB per launch among 8 PEs, the headline's traffic
    buf = rs.sym_array(per_pe, np.uint8)

    def rate(kind, launch):
        def fn():
            rs.stream_probe(kind, buf, per_pe, None, 7, launch)

        fn()
        rs.synchronize()
        ms = event_time_ms(rs, fn, steps) / steps
        return n_pes * per_pe / ms / 1e6, ms

    def shapes(staying, span):
        if staying:
            # (workgroups, lanes, bytes per pass): two, four or eight accesses per lane in flight
            return [(wgs, lanes, lanes * 16 * u) for wgs, lanes in ((32, 1024), (64, 1024), (64, 512))
                    for u in (2, 4, 8)]
        # one workgroup per pass: (lanes, accesses per lane)
        return [(span // (lanes * 16 * u), lanes, lanes * 16 * u) for lanes, u in ((256, 1), (1024, 1), (256, 4))]

    # The memory system is faster on zeros (a bare reduction over zero-filled arrays ran 1.8 % faster
    # than over floats): give the buffers contents before anything is read or copied.
    rs.stream_probe(rs.STREAM_WRITE, buf, per_pe, None, 7, rs.Launch(32, 1024))
    rs.synchronize()
    out = {}
    for shape_name, staying in (("staying", True), ("one_per_pass", False)):
        rows = {}
        for name, kind in (("read_only", rs.STREAM_READ), ("write_only", rs.STREAM_WRITE), ("copy", rs.STREAM_COPY)):
            best = None
            for wgs, lanes, tile in shapes(staying, per_pe // 2 if kind == rs.STREAM_COPY else per_pe):
                r, ms = rate(kind, rs.Launch(wgs, lanes, tile))
                if best is None or r > best["GBps"]:
                    best = {"GBps": round(r, 1), "ms": round(ms, 4),
                            "launch": {"wgs_per_pe": wgs, "wg_size": lanes, "pass_bytes": tile or lanes * 128}}
            rows[name] = best
        r, w = rows["read_only"]["GBps"], rows["write_only"]["GBps"]
        rows["harmonic_mean_GBps"] = round(2.0 / (1.0 / r + 1.0 / w), 1)
        out[shape_name] = rows
    # the shape the library's collectives have is the one their rates are compared with
    out["read_only"] = out["staying"]["read_only"]
    out["write_only"] = out["staying"]["write_only"]
    out["harmonic_mean_GBps"] = out["staying"]["harmonic_mean_GBps"]
    for name, kind in (("runtime_fill_hipMemsetAsync", rs.STREAM_RUNTIME_FILL),
                       ("runtime_copy_hipMemcpyAsync", rs.STREAM_RUNTIME_COPY)):
        r, ms = rate(kind, rs.Launch(32, 1024))
        out[name] = {"GBps": round(r, 1), "ms": round(ms, 4)}
    out["bytes_per_launch"] = n_pes * per_pe
    if rs.take_status():
        raise RuntimeError("device status word raised")
    buf.free()
    return out


def bench_pacing_sweep(rs, n_pes):
    """Rate of the headline reduction and of a sharded 256 MiB put, running free and paced at fixed
    rates (no tuner), for two launch shapes: GB/s by rate in bytes per tick of the 100 MHz clock."""
    out = {"float_sum_to_all_8x2^26": {}, "putmem_wg_shard_256MiB": {}}
    n = 1 << 26
    src = rs.sym_array(n, np.float32)
    dst = rs.sym_array(n, np.float32, fill=0)
    psync = rs.sym_array(64 * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
    rng = np.random.default_rng(3)
    for p in range(n_pes):                     # N(0,1) like the headline's inputs, not zeros
        src.write(p, rng.standard_normal(n, dtype=np.float32))
    rates = [0] + list(range(58000, 70001, 1000)) + [75000, 80000, 90000]
    pacing_before = rs.get_pacing()
    for shape in TUNE_SHAPES:
        launch = rs.Launch(**shape)
        key = "%dx%d" % (shape["wgs_per_pe"], shape["wg_size"])

        def reduce():
            rs.roc_shmem_to_all(rs.FLOAT, rs.SUM, dst, src, n, 0, 0, n_pes, None, psync, launch)

        def put():
            rs.roc_shmem_rma(rs.PUT, rs.WG_SHARED, dst, src, 256 << 20, 1, 256 << 20, 256 << 20, 1, launch)

        for name, fn, nbytes, which in (("float_sum_to_all_8x2^26", reduce, 2.0 * n_pes * n * 4, 1),
                                        ("putmem_wg_shard_256MiB", put, 2.0 * n_pes * (256 << 20), 0)):
            row = {}
            for r in rates:
                rs.set_pacing(r if which == 0 else 0, r if which == 1 else 0)
                fn()
                rs.synchronize()
                row["free" if r == 0 else str(r)] = round(nbytes / (event_time_ms(rs, fn, 10) / 10) / 1e6, 1)
            out[name][key] = row
    rs.set_pacing(*pacing_before)
    if rs.take_status():
        raise RuntimeError("device status word raised")
    for a in (psync, dst, src):
        a.free()
    return out


def bench_granularities(rs, steps, n_pes):
    """putmem / getmem issued per wave and per thread (every wave or lane moves its own message to
    or from the next PE): GB/s counted as 2*m bytes per message, and messages per second."""
    total = 256 << 20
    src = rs.sym_array(total, np.uint8)
    dst = rs.sym_array(total, np.uint8, fill=0)
    random_payload(rs, src, n_pes, seed=2)
    res = {}
    shapes = [(rs.WAVE, "wave", m) for m in (256, 4096, 65536, 1 << 20)] + \
             [(rs.THREAD, "thread", m) for m in (8, 256, 4096)]
    for gran, name, m in shapes:
        stride = max(m, 256)
        n_msgs = min(total // stride, 1 << 16)
        # short per-wave messages are bound by load latency: sixteen waves per workgroup
        launch = rs.Launch(64, 1024) if gran == rs.WAVE and m <= 1024 else rs.Launch(64, 256)
        for kind, kname in ((rs.PUT, "putmem"), (rs.GET, "getmem")):
            def step():
                rs.roc_shmem_rma(kind, gran, dst, src, m, n_msgs, stride, stride, 1, launch)

            step()
            rs.synchronize()
            ms = event_time_ms(rs, step, steps) / steps
            res["%s_%s_%d" % (kname, name, m)] = {
                "GBps": round(2.0 * n_pes * m * n_msgs / ms / 1e6, 1), "ms": round(ms, 4),
                "calls_per_pe": n_msgs, "Mmsgs_per_s": round(n_pes * n_msgs / ms / 1e3, 1)}
    if rs.take_status():
        raise RuntimeError("device status word raised")
    src.free()
    dst.free()
    return res


def bench_small_ops(rs, n_pes, n_ops, wgs_total, wg_size, slice_bytes, seed, live_queue=True):
    """10 M 8-byte puts (unique targets, lower half) and int64 fetch-adds (upper half)."""
    rng = np.random.default_rng(seed)
    words = slice_bytes // 8
    mem = rs.sym_array(words, np.int64, fill=0)
    res = {}
    for name, kinds in (("put8", (rs.OP_P64,)), ("fetch_add", (rs.OP_FADD64,)),
                        ("mixed", (rs.OP_P64, rs.OP_FADD64))):
        ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
        is_put = np.ones(n_ops, bool) if kinds == (rs.OP_P64,) else \
            np.zeros(n_ops, bool) if kinds == (rs.OP_FADD64,) else (np.arange(n_ops) % 2 == 0)
        ops["kind"] = np.where(is_put, rs.OP_P64, rs.OP_FADD64)
        ops["pe"] = rng.integers(0, n_pes, n_ops)
        uniq = rng.permutation(n_pes * (words // 2))[:n_ops]
        ops["pe"][is_put] = uniq[is_put] // (words // 2)
        ops["offset"] = np.where(is_put, (uniq % (words // 2)) * 8,
                                 (words // 2 + rng.integers(0, words // 2, n_ops)) * 8) + mem.offset
        ops["value"] = rng.integers(-1000, 1000, n_ops)
        dev = rs.device_array(ops)
        launch = rs.Launch(wgs_total // n_pes, wg_size)

        def step():
            rs.roc_shmem_small_ops(dev, n_ops, None, launch)

        step()
        rs.synchronize()
        ms = event_time_ms(rs, step, 3) / 3
        res[name] = {"Mops_per_s": n_ops / ms / 1e3, "ms": ms}
        dev.free()
    # Fetch-adds that collide: every op on one word, and on 16 words (one per PE).  Lanes of a wave
    # that name the same word share one atomic.
    for name, n_words in (("fetch_add_one_word", 1), ("fetch_add_16_words", 16)):
        ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
        word = rng.integers(0, n_words, n_ops)
        ops["kind"] = rs.OP_FADD64
        ops["pe"] = word % n_pes
        ops["offset"] = mem.offset + (words - 1) * 8
        ops["value"] = rng.integers(1, 5, n_ops)
        mem.fill(0)
        dev = rs.device_array(ops)

        def hot():
            rs.roc_shmem_small_ops(dev, n_ops, None, launch)

        hot()
        rs.synchronize()
        ms = event_time_ms(rs, hot, 3) / 3
        total = sum(int(mem.read(p)[words - 1]) for p in range(min(n_pes, n_words)))
        if total != 4 * int(ops["value"].sum()):
            raise RuntimeError("%s: the words hold %d, expected %d" % (name, total, 4 * int(ops["value"].sum())))
        res[name] = {"Mops_per_s": n_ops / ms / 1e3, "ms": ms}
        dev.free()
    # Lane-contiguous 8-byte putmems: the coalescer merges each wave's 64 messages into one 512-byte
    # WQE (wf_coal_policy.cpp:57-172); every lane still moves its own 8 bytes.
    half = words // 2
    ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
    i = np.arange(n_ops)
    ops["kind"] = rs.OP_PUTMEM
    ops["pe"] = (i // 64) % n_pes
    ops["offset"] = mem.offset + (i % half) * 8
    ops["value"] = mem.offset + (half + i % half) * 8
    ops["aux"] = 8
    dev = rs.device_array(ops)

    def coalesced():
        rs.roc_shmem_small_ops(dev, n_ops, None, launch)

    coalesced()
    rs.synchronize()
    ms = event_time_ms(rs, coalesced, 3) / 3
    res["putmem8_lane_contiguous"] = {"Mops_per_s": n_ops / ms / 1e3, "ms": ms,
                                      "note": "64 lanes x 8 B coalesced into one 512-byte WQE per wave"}
    dev.free()
    # The mixed stream through queues with a live consumer: a consumer kernel retires entries while
    # the producers post (1024-entry rings, producers wait for space, quiet collects completions).
    ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
    is_put = np.arange(n_ops) % 2 == 0
    uniq = rng.permutation(n_pes * (words // 2))[:n_ops]
    ops["kind"] = np.where(is_put, rs.OP_P64, rs.OP_FADD64)
    ops["pe"] = np.where(is_put, uniq // (words // 2), rng.integers(0, n_pes, n_ops))
    ops["offset"] = np.where(is_put, (uniq % (words // 2)) * 8,
                             (words // 2 + rng.integers(0, words // 2, n_ops)) * 8) + mem.offset
    ops["value"] = rng.integers(-1000, 1000, n_ops)
    if live_queue:
        dev = rs.device_array(ops)
        stream = rs.Stream()
        live_launch = rs.Launch(wgs_total // n_pes, wg_size, 0, stream)
        rs.synchronize()
        rs.sq_reset()
        rs.sq_consumer_start()
        try:
            rs.roc_shmem_small_ops(dev, n_ops, None, live_launch)
            stream.synchronize()
            start, stop, reps = rs.Event(), rs.Event(), 3
            start.record(stream)
            for _ in range(reps):
                rs.roc_shmem_small_ops(dev, n_ops, None, live_launch)
            stop.record(stream)
            ms = start.elapsed_ms(stop) / reps
            stream.synchronize()
        finally:
            totals = rs.sq_consumer_stop()
        # every workgroup's closing quiet posts one zero-byte read per launch besides the operations
        if totals["lost"] or totals["rejected"] or totals["retired"] != (reps + 1) * (n_ops + wgs_total):
            raise RuntimeError("live consumer: %r" % (totals,))
        res["mixed_through_live_queues"] = {"Mops_per_s": n_ops / ms / 1e3, "ms": ms, "retired": totals["retired"],
                                            "lost": 0, "rejected": 0,
                                            "note": "1024-entry rings in queue mode, consumer kernel running beside the "
                                                    "producers, entries written through to memory"}
        start.destroy()
        stop.destroy()
        stream.destroy()
        dev.free()
    # The same stream once more with the rings as logs, for the consumer pass below.
    dev = rs.device_array(ops)
    rs.sq_reset()
    rs.roc_shmem_small_ops(dev, n_ops, None, launch)
    rs.synchronize()
    dev.free()
    # Consumer pass over what the last stream left in the rings (each ring keeps its newest
    # sq_size entries): check + complete only, host-timed around the synchronous call.
    t0 = time.perf_counter()
    totals = rs.sq_consume()
    dt = time.perf_counter() - t0
    if totals["rejected"]:
        raise RuntimeError("the consumer pass rejected %d ring entries" % totals["rejected"])
    res["consume_check_only"] = {"entries": totals["retired"], "rejected": totals["rejected"],
                                 "lost_to_wraparound": totals["lost"], "ms": dt * 1e3,
                                 "Mentries_per_s": totals["retired"] / dt / 1e6}
    status = rs.take_status()
    if status:
        raise RuntimeError("device status word raised: %d" % status)
    mem.free()
    return res


def bench_amo_kinds(rs, n_pes, n_ops, wgs_total, wg_size, slice_bytes, seed):
    """One stream of n_ops operations per kind, uniformly random (PE, word) targets: M ops/s."""
    rng = np.random.default_rng(seed)
    words = slice_bytes // 8
    mem = rs.sym_array(words, np.int64, fill=0)
    ops = np.zeros(n_ops, rs.SMALL_OP_DTYPE)
    ops["pe"] = rng.integers(0, n_pes, n_ops)
    ops["offset"] = mem.offset + rng.integers(0, words // 2, n_ops) * 8
    ops["value"] = rng.integers(1, 1000, n_ops)
    launch = rs.Launch(wgs_total // n_pes, wg_size)
    res = {}
    kinds = [("p64", rs.OP_P64), ("p32", rs.OP_P32), ("fetch_add64", rs.OP_FADD64), ("fetch_add32", rs.OP_FADD32),
             ("add64", rs.OP_ADD64), ("fetch_inc64", rs.OP_FINC64), ("inc64", rs.OP_INC64),
             ("compare_swap64", rs.OP_CSWAP64), ("fetch64", rs.OP_FETCH64), ("set64", rs.OP_SET64),
             ("swap64", rs.OP_SWAP64), ("fetch_and64", rs.OP_FAND64), ("fetch_or64", rs.OP_FOR64),
             ("fetch_xor64", rs.OP_FXOR64), ("getmem8_nbi", rs.OP_GETMEM), ("putmem8_nbi", rs.OP_PUTMEM)]
    for name, kind in kinds:
        ops["kind"] = kind
        if kind in (rs.OP_GETMEM, rs.OP_PUTMEM):
            # `value` names the local buffer: a word of the upper half, one per operation
            ops["value"] = mem.offset + (words // 2 + np.arange(n_ops) % (words // 2)) * 8
            ops["aux"] = 8
        dev = rs.device_array(ops)

        def step():
            rs.roc_shmem_small_ops(dev, n_ops, None, launch)

        step()
        rs.synchronize()
        ms = event_time_ms(rs, step, 3) / 3
        res[name] = {"Mops_per_s": round(n_ops / ms / 1e3, 1), "ms": round(ms, 4)}
        dev.free()
    status = rs.take_status()
    if status:
        raise RuntimeError("device status word raised: %d" % status)
    mem.free()
    return res


def bench_small_latencies(rs, n_pes):
    """Fixed cost of a collective: 4 KiB per PE, one workgroup of 256 lanes per PE, back-to-back
    launches, microseconds per call."""
    src = rs.sym_array(1 << 16, np.uint8, fill=1)
    dst = rs.sym_array(1 << 16, np.uint8, fill=0)
    psync = rs.sym_array(rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
    world = rs.roc_shmem_team_world()
    launch, nbytes, out = rs.Launch(1, 256), 4096, {}
    calls = {
        "int_sum_to_all": lambda: rs.roc_shmem_to_all(rs.INT, rs.SUM, dst, src, nbytes // 4, 0, 0, n_pes, None,
                                                      psync, launch),
        "broadcast": lambda: rs.roc_shmem_team_broadcast(1, world, dst, src, nbytes, 0, launch),
        "alltoall": lambda: rs.roc_shmem_alltoall(1, world, dst, src, nbytes // n_pes, launch),
        "fcollect": lambda: rs.roc_shmem_fcollect(1, world, dst, src, nbytes // n_pes, launch),
    }
    for name, fn in calls.items():
        fn()
        rs.synchronize()
        out[name + "_us"] = round(event_time_ms(rs, fn, 50) / 50 * 1e3, 2)
    if rs.take_status():
        raise RuntimeError("device status word raised")
    for a in (psync, dst, src):
        a.free()
    return out


def bench_small_collectives(rs, n_pes, n, calls):
    """A launch-bound sequence: `calls` int64 sum_to_all of `n` elements back to back, issued call by
    call and as one recorded graph.  Microseconds per collective."""
    stream = rs.Stream()
    src = rs.sym_array(n, np.int64, fill=1)
    dst = rs.sym_array(n, np.int64, fill=0)
    psync = rs.sym_array(rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
    launch = rs.Launch(1, 512, 0, stream)

    def eager():
        for _ in range(calls):
            rs.roc_shmem_to_all(rs.LONG, rs.SUM, dst, src, n, 0, 0, n_pes, None, psync, launch)

    with rs.Graph.capture(stream) as graph:
        eager()
    out = {}
    for name, fn in (("eager_us", eager), ("graph_us", graph.launch)):
        fn()
        rs.synchronize()
        start, stop = rs.Event(), rs.Event()
        start.record(stream)
        for _ in range(5):
            fn()
        stop.record(stream)
        out[name] = start.elapsed_ms(stop) / 5 / calls * 1e3
        start.destroy()
        stop.destroy()
    got = dst.read(n_pes - 1)
    # every source byte is 1, so every byte of the sum over n_pes <= 255 slices is n_pes
    if not (got.view(np.uint8) == n_pes).all() or rs.take_status():
        raise RuntimeError("small collectives: wrong sum after the graph replays")
    graph.destroy()
    stream.destroy()
    for a in (psync, dst, src):
        a.free()
    return out


def bench_bcast_a2a(rs, n_pes, slice_bytes):
    world = rs.roc_shmem_team_world()
    res = {}
    src = rs.sym_array(slice_bytes, np.uint8)
    dst = rs.sym_array(slice_bytes, np.uint8, fill=0)
    random_payload(rs, src, n_pes, seed=5)
    # best of a sweep over 8/16/32 workgroups per PE x 512/1024 threads for each
    launch = rs.Launch(16, 512)
    bcast_launch = fcollect_launch = rs.Launch(8, 1024)
    nelem = slice_bytes // 4

    def bcast():
        rs.roc_shmem_team_broadcast(4, world, dst, src, nelem, 0, bcast_launch)

    bcast()
    rs.synchronize()
    ms = event_time_ms(rs, bcast, 5) / 5
    res["broadcast"] = {"GBps": (slice_bytes + (n_pes - 1) * slice_bytes) / ms / 1e6, "ms": ms}
    block = nelem // n_pes

    def a2a():
        rs.roc_shmem_alltoall(4, world, dst, src, block, launch)

    a2a()
    rs.synchronize()
    ms = event_time_ms(rs, a2a, 5) / 5
    res["alltoall"] = {"GBps": 2.0 * n_pes * slice_bytes / ms / 1e6, "ms": ms}
    # the same with the copies' schedule switched on (off by default: it pays here and costs in other shapes)
    pacing_before = rs.get_pacing()
    rs.set_pacing(67000, pacing_before[1])
    a2a()
    rs.synchronize()
    ms = event_time_ms(rs, a2a, 5) / 5
    rs.set_pacing(*pacing_before)
    res["alltoall_copies_paced_at_67000"] = {"GBps": 2.0 * n_pes * slice_bytes / ms / 1e6, "ms": ms}

    def fcollect():
        rs.roc_shmem_fcollect(4, world, dst, src, block, fcollect_launch)

    fcollect()
    rs.synchronize()
    ms = event_time_ms(rs, fcollect, 5) / 5
    # every member's block is read once and written into all n_pes dests
    res["fcollect"] = {"GBps": float(n_pes + 1) * slice_bytes / ms / 1e6, "ms": ms}
    if rs.take_status():
        raise RuntimeError("device status word raised")
    src.free()
    dst.free()
    return res


def bench_alignment(rs, n_pes):
    """Large put, broadcast and reduction with source and destination shifted off their natural
    alignment: (source shift, destination shift) in bytes -> GB/s."""
    out = {"put_64MiB_messages": {}, "broadcast_64MiB": {}, "float_sum_to_all_2^26": {}}
    src = rs.sym_array(256 << 20, np.uint8, fill=1)
    dst = rs.sym_array(256 << 20, np.uint8, fill=0)
    world = rs.roc_shmem_team_world()
    psync = rs.sym_array(TO_ALL_LAUNCH["wgs_per_pe"] * rs.ROC_SHMEM_REDUCE_SYNC_SIZE, np.int64, fill=0)
    total, msg, n = 192 << 20, 64 << 20, (1 << 26) - 1024
    for ss, ds in ((0, 0), (16, 16), (128, 128), (256, 256), (1024, 1024), (4, 4), (4, 8), (16, 32), (1, 0)):
        key = "%d/%d" % (ss, ds)

        def put():
            rs.roc_shmem_rma(rs.PUT, rs.WG_SHARED, dst.addr + ds, src.addr + ss, msg, total // msg, msg, msg, 1,
                             rs.Launch(**PUT_LAUNCH))

        def bcast():
            rs.roc_shmem_team_broadcast(1, world, dst.addr + ds, src.addr + ss, msg, 0, rs.Launch(8, 1024))

        def reduce():
            rs.roc_shmem_to_all(rs.FLOAT, rs.SUM, dst.addr + ds, src.addr + ss, n, 0, 0, n_pes, None, psync,
                                rs.Launch(**TO_ALL_LAUNCH))

        for name, fn, nbytes in (("put_64MiB_messages", put, 2.0 * n_pes * total),
                                 ("broadcast_64MiB", bcast, float(n_pes) * msg),
                                 ("float_sum_to_all_2^26", reduce, 2.0 * n_pes * n * 4)):
            if name.startswith("float") and (ss % 4 or ds % 4):
                continue
            fn()
            rs.synchronize()
            out[name][key] = round(nbytes / (event_time_ms(rs, fn, 5) / 5) / 1e6, 1)
    if rs.take_status():
        raise RuntimeError("device status word raised")
    for a in (psync, dst, src):
        a.free()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--quick", action="store_true", help="headline workload only")
    ap.add_argument("--counter-pair", action="store_true",
                    help="for rocprofv3 --pmc: a few launches of the headline kernel and of a "
                         "plain wg putmem copy of known size (2 GiB read + 2 GiB written), nothing else")
    ap.add_argument("--stream-probes", action="store_true",
                    help="read-only and write-only streams over the heap (rsm_stream_probe), nothing else")
    ap.add_argument("--small-ops", action="store_true",
                    help="for rocprofv3 --pmc: the 10 M-operation streams and the consumer pass, nothing else")
    ap.add_argument("--skip-live-queue", action="store_true",
                    help="with --small-ops under rocprofv3 --pmc: leave out the stream through queues with a live "
                         "consumer (counter collection runs one kernel at a time, and a consumer kernel cannot run "
                         "beside the producers then)")
    ap.add_argument("--granularities", action="store_true",
                    help="putmem / getmem per wave and per thread, nothing else")
    ap.add_argument("--amo-kinds", action="store_true",
                    help="10 M operations of every small-operation kind, random targets, nothing else")
    ap.add_argument("--collectives", action="store_true",
                    help="for rocprofv3: broadcast, alltoall and fcollect over 16 slices x 64 MiB, nothing else")
    ap.add_argument("--alignment", action="store_true",
                    help="large put / broadcast / reduction with shifted source and destination, nothing else")
    ap.add_argument("--pace-reduce", type=int, default=0, metavar="BYTES_PER_TICK",
                    help="run the headline kernel paced at this rate instead of the library's default "
                         "(also with --counter-pair)")
    ap.add_argument("--pacing-sweep", action="store_true",
                    help="the headline reduction and a sharded 64 MiB put, free and paced at fixed rates, nothing else")
    ap.add_argument("--reduce-lds", action="store_true",
                    help="headline workload only, through the LDS-staged form of the reduction "
                         "(ROC_SHMEM_REDUCE_LDS=1), running free, for 32 x 512 and 32 x 1024 lanes per PE")
    ap.add_argument("--tune", action="store_true",
                    help="let the library's pacing tuner pick launch shape and rate for the headline reduction")
    ap.add_argument("--no-pacing", action="store_true",
                    help="pacing off: every reduction runs free (no schedule, no tuner)")
    ap.add_argument("--record-traffic", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: read the two rocprofv3 --pmc counter files of --counter-pair runs and "
                         "write the tracked traffic summary under profiles/")
    ap.add_argument("--clock-ab", metavar="VARIANTS", nargs="?", const="default",
                    help="GFX (L2) clock and socket power under two-second loops of one 4 GiB kernel each, nothing "
                         "else.  VARIANTS: comma-separated among sharded, standard, free, float_max, int_sum, "
                         "members:2, members:4, members:16, put, read, write (default: all of them)")
    ap.add_argument("--clock-ab-launches", type=int, default=0, metavar="N",
                    help="with --clock-ab under rocprofv3 --pmc: N launches per variant, no sampling")
    ap.add_argument("--sharded", action="store_true",
                    help="with --counter-pair: launch the sharded extension instead of the headline's standard calls")
    ap.add_argument("--timeline", metavar="FILE",
                    help="no GPU work: summarise the clock readings a timeline build of the library wrote "
                         "(ROC_SHMEM_TIMELINE_FILE)")
    args = ap.parse_args()
    if args.timeline:
        print(json.dumps(timeline_summary(args.timeline)))
        return
    if args.record_traffic:
        record_traffic(*args.record_traffic)
        return
    if args.gpus != 1:
        print("bench.py: every PE slice lives in one GPU's HBM; this build measures one GPU only "
              "(--gpus %d is not supported)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import oracle
    import roc_shmem_amd as rs

    if args.clock_ab:
        names = ["sharded", "standard", "free", "float_max", "int_sum", "members:2", "members:4", "members:16",
                 "put", "read", "write"] if args.clock_ab == "default" else args.clock_ab.split(",")
        print(json.dumps({"clock_and_power_by_kernel": bench_clock_ab(rs, oracle, names, 2.0, args.clock_ab_launches),
                          "library": os.environ.get("ROC_SHMEM_LIBRARY", "librocshmem_mi355x.so")}))
        return
    if args.reduce_lds:
        out = {}
        for staged in (1, 0):
            os.environ["ROC_SHMEM_REDUCE_LDS"] = str(staged)
            rs.roc_shmem_init(8, 1 << 30, 64, 1024)
            for shape in TUNE_SHAPES:
                r = bench_to_all(rs, oracle, 10, 3, rs.FLOAT, 8, 1 << 26, seed=3, launch_shape=shape, pace=0)
                out["%s_%dx%d" % ("lds_staged" if staged else "registers", shape["wgs_per_pe"], shape["wg_size"])] = \
                    {"GBps": round(r["GBps"], 1), "ms": round(r["ms_per_step"], 4),
                     "parity_checked_elements": r["parity_checked_elements"]}
            rs.roc_shmem_finalize()
        del os.environ["ROC_SHMEM_REDUCE_LDS"]
        print(json.dumps({"to_all_float_sum_8x2^26_free_running": out}))
        return
    if args.pacing_sweep:
        rs.roc_shmem_init(8, 1 << 30, 64, 1024)
        out = bench_pacing_sweep(rs, 8)
        rs.roc_shmem_finalize()
        print(json.dumps({"GBps_by_pacing_rate_8pe": out}))
        return
    if args.small_ops:
        rs.roc_shmem_init(16, 256 << 20, 64, 1024)
        out = bench_small_ops(rs, 16, 10_000_000, 1024, 256, 64 << 20, seed=4,
                              live_queue=not args.skip_live_queue)
        rs.roc_shmem_finalize()
        print(json.dumps({"small_ops_16x64MiB_1024wg_x256": out}))
        return
    if args.amo_kinds:
        rs.roc_shmem_init(16, 256 << 20, 64, 1024)
        out = bench_amo_kinds(rs, 16, 10_000_000, 1024, 256, 64 << 20, seed=5)
        rs.roc_shmem_finalize()
        print(json.dumps({"small_op_kinds_16x64MiB_1024wg_x256": out}))
        return
    if args.granularities:
        rs.roc_shmem_init(8, 1 << 30, 64, 1024)
        out = bench_granularities(rs, 5, 8)
        rs.roc_shmem_finalize()
        print(json.dumps({"putmem_getmem_per_wave_and_thread_8pe": out}))
        return
    if args.collectives:
        rs.roc_shmem_init(16, 256 << 20, 64, 1024)
        out = bench_bcast_a2a(rs, 16, 64 << 20)
        rs.roc_shmem_finalize()
        print(json.dumps({"collectives_16x64MiB": out}))
        return
    if args.alignment:
        rs.roc_shmem_init(8, 1 << 30, 64, 1024)
        out = bench_alignment(rs, 8)
        rs.roc_shmem_finalize()
        print(json.dumps({"GBps_by_source_shift/destination_shift_8pe": out}))
        return
    if args.stream_probes:
        rs.roc_shmem_init(8, 1 << 30, 64, 1024)
        out = bench_streams(rs, 8)
        rs.roc_shmem_finalize()
        print(json.dumps({"hbm_streams_on_this_card": out}))
        return
    device = device_report() if not args.counter_pair else {}
    # ---- headline: fp32 sum_to_all, 8 slices x 2^26 elements (4 GiB algorithmic traffic) ----
    n_pes, n = 8, 1 << 26
    if not args.counter_pair:     # a runtime of its own: one 512 MiB block per PE on a fresh heap
        rs.roc_shmem_init(n_pes, 1 << 30, 64, 1024)
        streams = bench_streams(rs, n_pes)
        rs.roc_shmem_finalize()
    rs.roc_shmem_init(n_pes, 1 << 30, 64, 1024)
    if args.counter_pair:
        out = bench_to_all(rs, oracle, 3, 1, rs.FLOAT, n_pes, n, seed=3, check=False,
                           launch_shape=None if args.sharded else TO_ALL_STANDARD_LAUNCH,
                           pace=0 if args.no_pacing else (args.pace_reduce or None))
        put = bench_putmem(rs, 3, n_pes, [64 << 20])
        rs.roc_shmem_finalize()
        print(json.dumps({"to_all": out, "putmem_copy": put,
                          "copy_bytes_read": n_pes * (256 << 20), "copy_bytes_written": n_pes * (256 << 20)}))
        return
    # The headline runs as a caller's loop would: the reference's own symbol
    # (roc_shmem_ctx_float_sum_wg_to_all), one call per workgroup over its tile of the array, the
    # library's default pacing rates, no tuning.
    # --tune lets the library's tuner pick the rate first (outside the timed region),
    # --pace-reduce R / --no-pacing fix the rate (0 = workgroups run free).
    head = bench_to_all(rs, oracle, args.steps, args.warmup, rs.FLOAT, n_pes, n, seed=3, cpu=True,
                        spread=True, launch_shape=TO_ALL_STANDARD_LAUNCH, tune=args.tune,
                        pace=None if args.tune else (0 if args.no_pacing else (args.pace_reduce or None)))
    extra = {}
    # against workgroups that stay, the shape the reduction's own workgroups have, and against the
    # best plain copy the card did in any shape (a 1:1 stream like the reduction's)
    streams["headline_over_harmonic_mean"] = round(head["GBps"] / streams["harmonic_mean_GBps"], 4)
    streams["headline_over_best_plain_copy"] = round(
        head["GBps"] / max(streams["staying"]["copy"]["GBps"], streams["one_per_pass"]["copy"]["GBps"]), 4)
    extra["hbm_streams_on_this_card"] = streams
    # the sharded extension (the PE's 32 workgroups share one call), same launch shape and rates
    extra["to_all_float_sum_8x2^26_sharded_extension"] = bench_to_all(
        rs, oracle, args.steps, 3, rs.FLOAT, n_pes, n, seed=3, spread=True,
        pace=0 if args.no_pacing else (args.pace_reduce or None))
    extra["to_all_float_sum_8x2^26_sharded_extension"]["api"] = "roc_shmemx_ctx_float_sum_wg_to_all_shard"
    if not args.quick:
        extra["to_all_float_sum_8x2^26_free_running"] = bench_to_all(
            rs, oracle, max(args.steps // 2, 3), 2, rs.FLOAT, n_pes, n, seed=3, check=False, pace=0,
            launch_shape=TO_ALL_STANDARD_LAUNCH)
        extra["to_all_float_sum_8x2^26_rate_from_the_tuner"] = bench_to_all(
            rs, oracle, max(args.steps // 2, 3), 2, rs.FLOAT, n_pes, n, seed=3, check=False, tune=True)
        # workgroups of 512 lanes (passes of 64 KiB per member) at the library's rate for short passes
        extra["to_all_float_sum_8x2^26_standard_api_32x512"] = bench_to_all(
            rs, oracle, max(args.steps // 2, 3), 2, rs.FLOAT, n_pes, n, seed=3, check=False,
            launch_shape=dict(wgs_per_pe=32, wg_size=512, tile=1 << 21))
        extra["to_all_float_sum_8x2^26_sharded_32x512"] = bench_to_all(
            rs, oracle, max(args.steps // 2, 3), 2, rs.FLOAT, n_pes, n, seed=3, check=False,
            launch_shape=dict(wgs_per_pe=32, wg_size=512))
        extra["to_all_bf16_sum_8x2^26"] = {k: v for k, v in bench_to_all(
            rs, oracle, max(args.steps // 2, 3), 2, rs.BF16, n_pes, n, seed=3,
            launch_shape=dict(wgs_per_pe=32, wg_size=1024, tile=1 << 21),
            pace=0 if args.no_pacing else None).items() if k != "cpu"}
        extra["to_all_bf16_sum_8x2^26_sharded_extension"] = {k: v for k, v in bench_to_all(
            rs, oracle, max(args.steps // 2, 3), 2, rs.BF16, n_pes, n, seed=3, check=False,
            pace=0 if args.no_pacing else None).items() if k != "cpu"}
        # every power of two from 8 B to 64 MiB, put and get (BASELINE configs[1]; the reference's
        # own sweep, clients/functional_tests/tester.cpp:503-563)
        extra["putmem_wg_8pe"] = bench_putmem(rs, 5, n_pes, [1 << k for k in range(3, 27)], get_sweep=True)
        # windows of 64 non-blocking puts / gets and one quiet (primitive_mr_tester.cpp:32-58)
        extra["nbi_windows_8pe"] = bench_nbi_windows(rs, 5, n_pes, [1 << k for k in range(3, 19)])
        extra["nbi_windows_8pe_up_to_8_per_kernel"] = bench_nbi_windows(rs, 5, n_pes, [8, 512, 4096, 65536], 8)
        extra["putmem_getmem_per_wave_and_thread_8pe"] = bench_granularities(rs, 5, n_pes)
        extra["collectives_4KiB_8pe_one_wg_of_256"] = bench_small_latencies(rs, n_pes)
    rs.roc_shmem_finalize()

    if not args.quick:
        rs.roc_shmem_init(4, 64 << 20, 64, 1024)
        # 64 MiB of traffic: launch, two flag barriers and 10 us of streaming (64 x 256 lanes per PE:
        # 17.3-17.5 us on one card, 64 x 1024 17.7, 64 x 512 18.5, 32 x 512 20.0-21.8)
        extra["to_all_int64_sum_4x2^20"] = bench_to_all(rs, oracle, 50, 10, rs.LONG, 4, 1 << 20, seed=1,
                                                        launch_shape=dict(wgs_per_pe=64, wg_size=256))
        barrier_launch, rounds = rs.Launch(1, 256), 500

        def barriers():
            rs.roc_shmem_wg_barrier_all(rounds, barrier_launch)

        barriers()
        rs.synchronize()
        extra["wg_barrier_all_4pe_us"] = event_time_ms(rs, barriers, 3) / 3 / rounds * 1e3
        extra["sum_to_all_4096_int64_x100"] = bench_small_collectives(rs, 4, 4096, 100)
        rs.roc_shmem_finalize()

        rs.roc_shmem_init(16, 256 << 20, 64, 1024)
        extra["small_ops_16x64MiB_1024wg_x256"] = bench_small_ops(rs, 16, 10_000_000, 1024, 256,
                                                                  64 << 20, seed=4)
        extra["collectives_16x64MiB"] = bench_bcast_a2a(rs, 16, 64 << 20)
        rs.roc_shmem_finalize()

    cpu = head.pop("cpu")
    if not args.quick:
        cpu["other_legs"] = cpu_other_legs(oracle)
    traffic, traffic_note = measured_traffic()

    def pick(*path):
        node = extra
        for key in path:
            if not isinstance(node, dict) or key not in node:
                return None
            node = node[key]
        return round(node, 1) if isinstance(node, float) else node

    line = {
        "metric": "to_all reduce + putmem GB/s (% of HBM peak); small-put/AMO Mops/s",
        "value": round(head["GBps"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "float sum_to_all over 8 PE slices x 2^26 elements, N(0,1) inputs, "
                               "all slices in one GPU's HBM (BASELINE configs[2], fp32 sum)",
                   "api": "roc_shmem_ctx_float_sum_wg_to_all (the reference's symbol, library/include/roc_shmem.hpp:"
                          "837-851), one call per workgroup over a tile of 2^21 elements, 32 workgroups of 1024 "
                          "lanes per PE; the sharded extension is extra.to_all_float_sum_8x2^26_sharded_extension",
                   "pes": n_pes, "elements_per_pe": n, "algorithmic_bytes_per_step": head["bytes_per_step"],
                   "launch": head["launch"], "pacing_bytes_per_tick": head["pacing_bytes_per_tick"],
                   "pacing_tuner": head.get("pacing_tuner"),
                   "parity_checked_elements": head.get("parity_checked_elements"), "parity": head.get("parity")},
        "roofline": {"bound": "hbm", "achieved": round(head["GBps"], 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(head["GBps"] / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_source": traffic_note},
        "cpu_baseline": {k: (round(v, 2) if isinstance(v, float) else v) for k, v in cpu.items()},
        "per_launch_ms": {"median": round(head["ms_median"], 4), "min": round(head["ms_min"], 4),
                          "max": round(head["ms_max"], 4)},
        # the legs of the metric in one place (GB/s unless named otherwise; null = not run with --quick)
        "standard_api_GBps": round(head["GBps"], 1),
        "sharded_extension_GBps": pick("to_all_float_sum_8x2^26_sharded_extension", "GBps"),
        "bf16_GBps": pick("to_all_bf16_sum_8x2^26", "GBps"),
        "standard_api_32x512_GBps": pick("to_all_float_sum_8x2^26_standard_api_32x512", "GBps"),
        "putmem_64MiB_GBps": pick("putmem_wg_8pe", "67108864", "GBps"),
        "getmem_64MiB_GBps": pick("putmem_wg_8pe", "getmem_67108864", "GBps"),
        "putmem_64MiB_shard_GBps": pick("putmem_wg_8pe", "67108864_shared", "GBps"),
        "putmem_4KiB_GBps": pick("putmem_wg_8pe", "4096", "GBps"),
        "putmem_64KiB_GBps": pick("putmem_wg_8pe", "65536", "GBps"),
        "putmem_nbi_wg_4KiB_GBps": pick("nbi_windows_8pe", "wg", "putmem_nbi_4096", "GBps"),
        "putmem_nbi_wg_64KiB_GBps": pick("nbi_windows_8pe", "wg", "putmem_nbi_65536", "GBps"),
        "putmem_nbi_wave_4KiB_GBps": pick("nbi_windows_8pe", "wave", "putmem_nbi_4096", "GBps"),
        "small_put_Mops": pick("small_ops_16x64MiB_1024wg_x256", "put8", "Mops_per_s"),
        "fetch_add_Mops": pick("small_ops_16x64MiB_1024wg_x256", "fetch_add", "Mops_per_s"),
        "mixed_live_queue_Mops": pick("small_ops_16x64MiB_1024wg_x256", "mixed_through_live_queues", "Mops_per_s"),
        "broadcast_GBps": pick("collectives_16x64MiB", "broadcast", "GBps"),
        "alltoall_GBps": pick("collectives_16x64MiB", "alltoall", "GBps"),
        "fcollect_GBps": pick("collectives_16x64MiB", "fcollect", "GBps"),
        "int64_sum_4x2^20_us": pick("to_all_int64_sum_4x2^20", "ms_per_step"),
        "device": device,
        "extra": extra,
    }
    if line["int64_sum_4x2^20_us"] is not None:
        line["int64_sum_4x2^20_us"] = round(extra["to_all_int64_sum_4x2^20"]["ms_per_step"] * 1e3, 2)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
