#!/usr/bin/env python3
"""SGEMM benchmark of the MI355X library: prints ONE JSON line.

    python bench.py [--gpus 1] [--steps 100] [--warmup 10] [--no-layouts] [--no-cpu] [--no-counters] [--counters]

Workload (the reference README's identity-multiply methodology, reference README.md:27-47):
M = N = K = 4096, A, B, C row-major, A uniform[-1, 1) from mt19937(seed 0), B = identity; the output
must equal A bit for bit.  A "step" is one rocm_sgemm::gemm call on operands already resident in HBM.
Timing follows the reference bench (reference benchmark/gemm/bench.cpp:74-106): every launch is
bracketed by an event pair on the launch stream; avg and min over the timed launches are reported,
`value` is the whole-run figure 2*M*N*K*steps / wall time of the timed region.  Unlike the
reference's gpu_timer the host does not wait after every launch: the launches are queued back to
back and the region is closed by one device synchronisation.

Also in the line:
  roofline      MFMA-bound: achieved = 2MNK / mean launch duration, peak = 157.3 TFLOP/s (dense FP32
                matrix peak of MI355X); traffic = HBM bytes per launch from rocprofv3 --pmc passes
                of this run (four short child processes; skipped with --no-counters or where
                rocprofv3 is missing, then read from the summary under profiles/; traffic_source
                says which)
  counters      from the same passes: matrix-pipe busy %, LDS bank conflicts %, HBM bytes per launch
  dense_4096    the same 4096^3 product on uniform[-1, 1) A and B (identity B draws less power and
                runs about 1 % faster): NN / NT / TN / TT (A, B column- or row-major in BLAS terms:
                row-major = T) with C row-major, avg and min-time TFLOP/s each
  held_out      shapes that are not entries of the tuned table, in mixed layouts: the config the
                planner chose, its rate, and the vendor library's on the same operands
  layouts       the reference bench's default cubes, 1024^3 to 8192^3, in the four A/B storage
                combinations (NN/NT/TN/TT) with C row- and column-major, uniform[-1, 1) A and B.
                Per row: avg / min-time TFLOP/s of the per-launch event pairs, the sustained rate
                (first start event to last stop event) and the back-to-back rate (one event pair
                around the same number of launches: no event packets between the kernels)
  shapes_row_major  the rectangular, unaligned and 16384^3 row-major configurations, with the
                vendor library on the same operands, by the same protocol, beside them
  context       hipBLASLt / rocBLAS (through torch.matmul, fp32, TF32 off) on the same GPU, and
                the rate of a kernel that issues MFMAs only (the ceiling of this GPU sample)
  cpu_baseline  the reference's CPU GEMM (the oracle's restatement of sgemm_cpu): one thread at
                1024^3 as the reference runs it, all usable threads at 1024^3 and on a bounded
                sample of 4096^3 (labelled extrapolated when cut), timed on this host; plus, where
                it has been built, the reference's own GPU kernel on this GPU for context
--counters also writes the counter summary to profiles/sgemm_mfma_4096_rrr_counters.txt.
"""

import argparse
import csv
import glob
import json
import os
import shutil
import subprocess
import sys
import tempfile
import time

REPO = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, REPO)

PEAK_TFLOPS = 157.3  # 256 CU x 4 SIMD x 64 FLOP/clk x 2.4 GHz
M = N = K = 4096
COUNTER_SUMMARY = os.path.join(REPO, "profiles", "sgemm_mfma_4096_rrr_counters.txt")
KERNEL_NAME_TAG = "sgemm_mfma_kernel"
COPY_PROBE_TAG = "MulFunctor"  # torch.mul(x, 1.0, out=y): a plain read-one-write-one kernel


def tflops(m, n, k, ms):
    return 2.0 * m * n * k / (ms * 1e-3) * 1e-12


WARMUP_MIN_MS = 40.0   # sustained launches before any timed region (the clocks need tens of ms)
WARMUP_MAX_MS = 600.0  # ... and at most this long while the launch time is still falling


def timed_launches(fn, steps, warmup, min_warm_ms=WARMUP_MIN_MS, max_warm_ms=WARMUP_MAX_MS):
    """The one timing protocol of this file.  Warm-up: at least `warmup` launches AND at least
    `min_warm_ms` of sustained launches, continued in batches of about 10 ms until two batches in
    a row agree within 1 % (after an idle gap the GPU needs tens of milliseconds of work to reach
    its full clock, more for some kernels: 1024 x 1024 x 16384 launches fell from 302 to 245 us
    over the 100 launches that followed a 40 ms warm-up).  Then `steps` launches queued back to
    back, each bracketed by an event pair on the launch stream, closed by ONE synchronisation.
    Returns the per-launch durations (ms), the wall time (ms) of the timed region, and the device
    time (ms) from the first launch's start event to the last one's stop event - the sustained
    rate, which unlike the per-launch figures includes launch gaps."""
    import torch
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]  # before the warm-up:
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]   # no idle gap after it
    warmed_ms, launched, batch, previous = 0.0, 0, 5, None
    w0, w1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    while True:
        w0.record()
        for _ in range(batch):
            fn()
        w1.record()
        w1.synchronize()
        took = max(w0.elapsed_time(w1), 1e-3)
        warmed_ms += took
        launched += batch
        per_launch = took / batch
        settled = previous is not None and abs(per_launch - previous) <= 0.01 * previous
        previous = per_launch
        if launched >= warmup and warmed_ms >= min_warm_ms and (settled or warmed_ms >= max_warm_ms):
            break
        # next batch: about 10 ms at the rate just seen (at least what `warmup` still asks for)
        batch = int(max(warmup - launched, min(10.0 / per_launch, 5000), 2))
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        fn()
        stops[i].record()
    torch.cuda.synchronize()  # one synchronisation for the whole timed region
    wall_ms = (time.perf_counter() - t0) * 1e3
    return [s.elapsed_time(e) for s, e in zip(starts, stops)], wall_ms, starts[0].elapsed_time(stops[-1])


def summary(m, n, k, ms, span_ms, burst_ms=None):
    avg = sum(ms) / len(ms)
    out = {"avg_tflops": round(tflops(m, n, k, avg), 2),
           "min_time_tflops": round(tflops(m, n, k, min(ms)), 2),
           "pct_peak_avg": round(100 * tflops(m, n, k, avg) / PEAK_TFLOPS, 1),
           "avg_ms": round(avg, 5),
           "sustained_tflops": round(tflops(m, n, k, span_ms / len(ms)), 2)}
    if burst_ms is not None:
        out["back_to_back_tflops"] = round(tflops(m, n, k, burst_ms), 2)
        out["back_to_back_ms"] = round(burst_ms, 5)
    return out


def burst_ms(fn, steps):
    """Mean duration of `steps` launches queued back to back between ONE event pair (right after
    a timed region, so the GPU is warm): no event packets between the kernels, which cost a few
    microseconds each - what a caller that just issues products sees."""
    import torch
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / steps


def measure(fn, m, n, k, steps, warmup):
    ms, _, span = timed_launches(fn, steps, warmup)
    return summary(m, n, k, ms, span, burst_ms(fn, steps))


def uniform_device(count, seed):
    import torch
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    return torch.rand(count, generator=g, device="cuda:0", dtype=torch.float32) * 2.0 - 1.0


def bench_layouts(rs, sizes, steps, warmup):
    """The reference bench's default shapes (reference benchmark/gemm/bench.cpp:240-303,
    docs/square.md:9-24): cubes x the four A/B storage orders x both C orders, uniform inputs."""
    import torch
    out = {}
    names = {0: "row", 1: "col"}
    for size in sizes:
        dA, dB = uniform_device(size * size, 1), uniform_device(size * size, 2)
        dC = torch.empty(size * size, dtype=torch.float32, device="cuda:0")
        stream = torch.cuda.current_stream()
        n_steps = steps if size <= 4096 else max(10, steps // 5)
        for lc in (0, 1):
            for la in (0, 1):
                for lb in (0, 1):
                    def fn():
                        rs.gemm(dC, dA, dB, size, size, size, lc, la, lb, stream=stream)
                    key = f"{size}^3 A={names[la]} B={names[lb]} C={names[lc]}"
                    out[key] = measure(fn, size, size, size, n_steps, warmup)
        del dA, dB, dC
    return out


RECT_SHAPES = [(8192, 8192, 1024), (1024, 1024, 16384), (128, 4096, 4096), (4096, 128, 4096),
               (4095, 4097, 4093), (1000, 3000, 777), (16384, 16384, 16384)]


def bench_shapes(rs, steps, warmup):
    """The rectangular, unaligned and large row-major configurations, with the vendor library
    (torch.matmul) timed on the same operands, by the same protocol, for context."""
    import torch
    torch.backends.cuda.matmul.allow_tf32 = False
    out = {}
    stream = torch.cuda.current_stream()
    for (m, n, k) in RECT_SHAPES:
        dA, dB = uniform_device(m * k, 5), uniform_device(k * n, 6)
        dC = torch.empty(m * n, dtype=torch.float32, device="cuda:0")
        flop_ms = 2.0 * m * n * k / 140e9  # rough duration, to keep every shape to a fraction of a second
        n_steps = max(5, min(steps, int(200 / max(flop_ms, 0.01))))
        row = measure(lambda: rs.gemm(dC, dA, dB, m, n, k, stream=stream), m, n, k, n_steps, warmup)
        a2, b2 = dA.view(m, k), dB.view(k, n)
        vendor = measure(lambda: torch.matmul(a2, b2), m, n, k, n_steps, warmup)
        row["vendor_avg_tflops"] = vendor["avg_tflops"]
        row["vendor_sustained_tflops"] = vendor["sustained_tflops"]
        row["vendor_back_to_back_tflops"] = vendor["back_to_back_tflops"]
        row["kernel_config"] = rs.find_config(m, n, k).as_dict()
        out[f"{m}x{n}x{k}"] = row
        del dA, dB, dC, a2, b2
    return out


# Shapes that are NOT entries of the tuned table (config/gemm_config.json must never list them):
# (M, N, K, layout of A, B, C; 0 = row-major, 1 = column-major).  What runs is the planner's choice.
HELD_OUT = [(3072, 5120, 2048, 0, 1, 0), (1536, 1200, 900, 1, 1, 0), (6000, 6000, 6000, 0, 0, 0),
            (2304, 768, 12288, 1, 0, 1), (5000, 1500, 2500, 0, 0, 1), (640, 9000, 3100, 1, 0, 0)]


def vendor_operands(dA, dB, m, n, k, la, lb, lc):
    """torch views such that torch.matmul(x, y) is the product in the caller's storage orders: a
    column-major C (M x N) is the row-major N x M matrix C^T = B^T A^T."""
    a = dA.view(m, k) if la == 0 else dA.view(k, m).t()
    b = dB.view(k, n) if lb == 0 else dB.view(n, k).t()
    return (a, b) if lc == 0 else (b.t(), a.t())


def bench_held_out(rs, steps, warmup):
    import torch
    torch.backends.cuda.matmul.allow_tf32 = False
    names = {0: "r", 1: "c"}
    table = {key for key, _ in rs.table()}
    table |= {(n, m, k, 1 - lb, 1 - la, 1 - lc) for (m, n, k, la, lb, lc) in table}  # mirror images: the same launch
    out = {}
    stream = torch.cuda.current_stream()
    for (m, n, k, la, lb, lc) in HELD_OUT:
        dA, dB = uniform_device(m * k, 7), uniform_device(k * n, 8)
        dC = torch.empty(m * n, dtype=torch.float32, device="cuda:0")
        flop_ms = 2.0 * m * n * k / 140e9
        n_steps = max(5, min(steps, int(200 / max(flop_ms, 0.01))))
        row = measure(lambda: rs.gemm(dC, dA, dB, m, n, k, lc, la, lb, stream=stream), m, n, k, n_steps, warmup)
        x, y = vendor_operands(dA, dB, m, n, k, la, lb, lc)
        vendor = measure(lambda: torch.matmul(x, y), m, n, k, n_steps, warmup)
        row["vendor_avg_tflops"] = vendor["avg_tflops"]
        row["vendor_back_to_back_tflops"] = vendor["back_to_back_tflops"]
        row["planned_config"] = rs.find_config(m, n, k, la, lb, lc).as_dict()
        row["in_tuned_table"] = (m, n, k, la, lb, lc) in table
        out[f"{m}x{n}x{k} {names[la]}{names[lb]}{names[lc]}"] = row
        del dA, dB, dC, x, y
    return out


def bench_dense_4096(rs, steps, warmup):
    """4096^3 on uniform operands, C row-major, the four A / B storage orders under their BLAS
    names (a row-major operand is a transposed one: reference test/rocblas/test.cpp:4-14)."""
    import torch
    dA, dB = uniform_device(M * K, 1), uniform_device(K * N, 2)
    dC = torch.empty(M * N, dtype=torch.float32, device="cuda:0")
    stream = torch.cuda.current_stream()
    out = {}
    for name, la, lb in (("NN", 1, 1), ("NT", 1, 0), ("TN", 0, 1), ("TT", 0, 0)):
        ms, _, span = timed_launches(lambda: rs.gemm(dC, dA, dB, M, N, K, 0, la, lb, stream=stream), steps, warmup)
        row = summary(M, N, K, ms, span)
        out[name] = {"avg_tflops": row["avg_tflops"], "min_time_tflops": row["min_time_tflops"],
                     "pct_peak_avg": row["pct_peak_avg"]}
    return out


def bench_context(sizes, steps, warmup):
    """hipBLASLt / rocBLAS SGEMM on the same GPU for context (vendor library, via torch.matmul)."""
    import torch
    torch.backends.cuda.matmul.allow_tf32 = False
    out = {}
    for size in sizes:
        a = uniform_device(size * size, 3).view(size, size)
        b = uniform_device(size * size, 4).view(size, size)
        n_steps = steps if size <= 4096 else max(10, steps // 5)
        out[f"torch.matmul fp32 {size}^3 (hipBLASLt/rocBLAS)"] = measure(lambda: torch.matmul(a, b), size, size, size,
                                                                          n_steps, warmup)
    return out


def mfma_only_kernel():
    """What the matrix pipes reach with nothing else to do (`bench_float --mfma_ceiling`: a kernel
    of MFMAs only, one workgroup per CU) and the shader clock of every XCD meanwhile - the ceiling
    every SGEMM kernel on this GPU sample works under.  None where the bench program is not built."""
    import re
    import subprocess
    exe = os.path.join(REPO, "rocm_sgemm_amd", "benchmark", "bench_float")
    if not os.path.exists(exe):
        return None
    out = subprocess.run([exe, "--mfma_ceiling"], capture_output=True, text=True, timeout=120)
    whole = re.search(r"= ([\d.]+) TFLOP/s = ([\d.]+) % of", out.stdout)
    if out.returncode != 0 or whole is None:
        return None
    clocks = [int(v) for v in re.findall(r"shader clock (\d+) MHz", out.stdout)]
    return {"tflops": float(whole.group(1)), "pct_peak": float(whole.group(2)), "xcd_shader_clock_mhz": clocks,
            "note": "256 workgroups of 4 waves issuing v_mfma_f32_32x32x2_f32 only; the launch ends with the slowest XCD"}


def cpu_baseline(max_seconds=12.0):
    """The reference CPU GEMM on this host (reference test/test.hpp:30-45: i-j-k, fp32
    accumulator): one thread at 1024^3, as the reference runs it; the same loop nest with the rows
    of C dealt out to threads at 1024^3; and the all-threads leg at 4096^3 on a bounded sample -
    the first R rows of C against the whole of B, which keeps the real access pattern (a
    column-strided walk over a 64 MiB B), with R sized to about `max_seconds` and the figure for
    all 4096 rows extrapolated by row count and labelled so.
    This leg is the only place where the benchmark touches the oracle (as a baseline, never as the
    thing measured): the CPU restatement, and - where it has been built - the reference's own GPU
    kernel timed on this GPU at 4096^3 row-major for context."""
    import oracle
    n = 1024
    a, b = oracle.fill_uniform_pair(n, n, n, 0, 0, seed=0)
    t0 = time.perf_counter()
    oracle.sgemm_f32(a, b, n, n, n, 0, 0, 0, threads=1)
    one = time.perf_counter() - t0
    host_cores = os.cpu_count() or 1
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = host_cores
    # threads actually used: what this process may run on, at most the 16 a one-GPU box grants
    cores = max(1, min(usable, 16))
    t0 = time.perf_counter()
    oracle.sgemm_f32(a, b, n, n, n, 0, 0, 0, threads=cores)
    many = time.perf_counter() - t0
    flops = 2.0 * n ** 3
    out = {"value": round(flops / one * 1e-12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
           "sample": "one 1024^3 row-major SGEMM, uniform[-1,1) seed 0, reference loop nest "
                     "(i-j-k, fp32 accumulator), 1 thread as the reference runs it",
           "seconds": round(one, 3),
           "host_cores": host_cores, "usable_cores": usable,
           "all_cores": {"value": round(flops / many * 1e-12, 6), "cores": cores,
                         "seconds": round(many, 3),
                         "note": "same loop nest at 1024^3, rows of C dealt out to threads"}}
    # 4096^3 on all threads, bounded
    big = 4096
    a4, b4 = oracle.fill_uniform_pair(big, big, big, 0, 0, seed=0)
    rows = cores  # one row of C per thread first, to size the sample
    t0 = time.perf_counter()
    oracle.sgemm_f32(a4[:rows * big], b4, rows, big, big, 0, 0, 0, threads=cores)
    probe = time.perf_counter() - t0
    rows = int(min(big, max(cores, cores * int(max_seconds / max(probe, 1e-3)))))
    t0 = time.perf_counter()
    oracle.sgemm_f32(a4[:rows * big], b4, rows, big, big, 0, 0, 0, threads=cores)
    took = time.perf_counter() - t0
    out["all_cores_4096"] = {
        "value": round(2.0 * rows * big * big / took * 1e-12, 6), "unit": "TFLOP/s", "cores": cores,
        "rows_timed": rows, "seconds": round(took, 3),
        "seconds_for_4096_rows": round(took * big / rows, 1),
        "extrapolated": rows < big,
        "note": ("the whole 4096^3 product" if rows == big else
                 f"first {rows} of 4096 rows of C against the whole of B (the full access pattern); "
                 "seconds_for_4096_rows is extrapolated by row count")}
    del a4, b4
    ref = oracle.ref_kernel()
    if ref is not None:
        import torch
        dA, dB = uniform_device(M * K, 1), uniform_device(K * N, 2)
        dC = torch.empty(M * N, dtype=torch.float32, device="cuda:0")
        stream = torch.cuda.current_stream()

        def fn():
            ref.ref_kernel_sgemm(0, 0, 0, dC.data_ptr(), dA.data_ptr(), dB.data_ptr(), M, N, K,
                                 stream.cuda_stream)
        ms, _, span = timed_launches(fn, 30, 10)
        out["reference_gpu_kernel_same_gpu"] = dict(
            summary(M, N, K, ms, span),
            note="the reference's kernel_gemm with its own tuned 4096^3 row-major parameters, "
                 "compiled for gfx950 from the reference sources (context, not a target)")
    return out


def read_traffic():
    """HBM bytes per launch from the committed counter summary (written by an earlier
    `bench.py --counters` run of this same workload), or None."""
    try:
        with open(COUNTER_SUMMARY) as f:
            for line in f:
                if line.startswith("hbm_bytes_per_launch:"):
                    return float(line.split(":")[1].split()[0])
    except OSError:
        pass
    return None


# ---- rocprofv3 counter passes (north-star bench extension) -----------------------------------------

PMC_PASSES = {
    "mfma": ["SQ_VALU_MFMA_BUSY_CYCLES", "SQ_BUSY_CU_CYCLES", "GRBM_GUI_ACTIVE", "SQ_INSTS_MFMA",
             "SQ_WAIT_INST_ANY", "SQ_WAVE_CYCLES"],
    "lds": ["SQ_LDS_BANK_CONFLICT", "SQ_LDS_IDX_ACTIVE", "SQ_INSTS_LDS"],
    "fetch": ["FETCH_SIZE"],
    "write": ["WRITE_SIZE"],
}


def run_counter_passes(steps=5, warmup=3):
    """Runs the inner loop of this script under rocprofv3 once per counter set and returns
    {counter: mean value per dispatch} for the SGEMM kernel and for a copy kernel of known size."""
    rocprof = shutil.which("rocprofv3")
    if rocprof is None:
        raise RuntimeError("rocprofv3 not found")
    results = {}
    env = dict(os.environ, TMPDIR="/tmp")
    for name, counters in PMC_PASSES.items():
        out_dir = tempfile.mkdtemp(prefix=f"rsg_pmc_{name}_", dir="/tmp")
        cmd = [rocprof, "--pmc", *counters, "--output-format", "csv", "-d", out_dir, "--",
               sys.executable, os.path.abspath(__file__), "--inner", "--steps", str(steps),
               "--warmup", str(warmup)]
        subprocess.run(cmd, check=True, env=env, cwd="/tmp", timeout=300,
                       stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        for path in glob.glob(os.path.join(out_dir, "**", "*counter_collection.csv"), recursive=True):
            per = {}
            with open(path) as f:
                for row in csv.DictReader(f):
                    kname = row["Kernel_Name"]
                    tag = "sgemm" if KERNEL_NAME_TAG in kname else ("copy" if COPY_PROBE_TAG in kname else None)
                    if tag is None:
                        continue
                    per.setdefault((tag, row["Counter_Name"]), []).append(float(row["Counter_Value"]))
            for (tag, cname), vals in per.items():
                results[f"{tag}:{cname}"] = sum(vals) / len(vals)
        shutil.rmtree(out_dir, ignore_errors=True)
    return results


def counters_report(steps, warmup):
    raw = run_counter_passes()
    rep = {}
    busy, gui = raw.get("sgemm:SQ_VALU_MFMA_BUSY_CYCLES"), raw.get("sgemm:GRBM_GUI_ACTIVE")
    if busy and gui:
        # GRBM_GUI_ACTIVE is summed over the 8 XCDs, MFMA busy cycles over the 1024 SIMDs
        rep["mfma_busy_pct"] = round(100.0 * busy / (gui / 8.0 * 1024.0), 2)
    cu_busy = raw.get("sgemm:SQ_BUSY_CU_CYCLES")
    if busy and cu_busy:
        # SQ_BUSY_CU_CYCLES is summed over the CUs: cycles in which a CU holds waves of the kernel
        # (GRBM_GUI_ACTIVE also counts the dispatch overhead around a launch under the profiler)
        rep["mfma_busy_pct_of_cu_busy"] = round(100.0 * busy / (cu_busy * 4.0), 2)
    conf, act = raw.get("sgemm:SQ_LDS_BANK_CONFLICT"), raw.get("sgemm:SQ_LDS_IDX_ACTIVE")
    if conf is not None and act:
        rep["lds_bank_conflict_pct"] = round(100.0 * conf / act, 2)
    copy_bytes = 2 * 4 * M * K  # the copy probe reads and writes one 4096 x 4096 fp32 matrix
    f_s, w_s = raw.get("sgemm:FETCH_SIZE"), raw.get("sgemm:WRITE_SIZE")
    f_c, w_c = raw.get("copy:FETCH_SIZE"), raw.get("copy:WRITE_SIZE")
    if f_s is not None and w_s is not None:
        # counters are in KiB per dispatch; scale by what the same counter reads for the copy probe
        f_scale = (copy_bytes / 2) / (f_c * 1024.0) if f_c else 1.0
        w_scale = (copy_bytes / 2) / (w_c * 1024.0) if w_c else 1.0
        rep["fetch_scale_from_copy"] = round(f_scale, 4)
        rep["write_scale_from_copy"] = round(w_scale, 4)
        rep["hbm_bytes_per_launch"] = (f_s * f_scale + w_s * w_scale) * 1024.0
    rep["raw"] = {k: v for k, v in sorted(raw.items())}
    return rep


def write_counter_summary(rep, avg_ms):
    os.makedirs(os.path.dirname(COUNTER_SUMMARY), exist_ok=True)
    with open(COUNTER_SUMMARY, "w") as f:
        f.write("# rocprofv3 --pmc summary: sgemm_mfma_kernel, 4096^3 row-major, identity B\n")
        f.write("# command: python bench.py --counters   (runs `rocprofv3 --pmc <set> --output-format csv "
                "-d <tmp> -- python3 bench.py --inner --steps 5 --warmup 3` once per counter set)\n")
        for name, counters in PMC_PASSES.items():
            f.write(f"# pass {name}: {' '.join(counters)}\n")
        for k in ("mfma_busy_pct", "mfma_busy_pct_of_cu_busy", "lds_bank_conflict_pct", "fetch_scale_from_copy",
                  "write_scale_from_copy"):
            if k in rep:
                f.write(f"{k}: {rep[k]}\n")
        if "hbm_bytes_per_launch" in rep:
            f.write(f"hbm_bytes_per_launch: {rep['hbm_bytes_per_launch']:.0f}\n")
            f.write(f"algorithmic_bytes_per_launch: {4 * (M * K + K * N + M * N)}\n")
            if avg_ms:
                f.write(f"achieved_hbm_GBps: {rep['hbm_bytes_per_launch'] / (avg_ms * 1e-3) * 1e-9:.1f}\n")
        for k, v in rep.get("raw", {}).items():
            f.write(f"raw {k}: {v:.6g}\n")


# ---- main --------------------------------------------------------------------------------------------

def uniform_mt19937(count, seed):
    """uniform[-1, 1) float32 values as std::uniform_real_distribution<float>(-1, 1) draws them
    from std::mt19937(seed) in libstdc++ (one 32-bit output per value, x / 2^32 in float, a result
    of 1.0 replaced by the float below it, then 2 * u - 1): the generator of the reference's
    test inputs (reference test/test.hpp:11-25), restated with numpy's MT19937."""
    import numpy as np
    bits = np.random.MT19937()
    bits._legacy_seeding(seed)
    u = bits.random_raw(count).astype(np.uint32).astype(np.float32) / np.float32(2.0 ** 32)
    u = np.where(u >= np.float32(1.0), np.nextafter(np.float32(1.0), np.float32(0.0)), u)
    return (np.float32(2.0) * u - np.float32(1.0)).astype(np.float32)


def identity_workload():
    """A uniform[-1,1) (mt19937 seed 0), B = I, both row-major, resident on the GPU."""
    import numpy as np
    import torch
    a = uniform_mt19937(M * K, 0)
    dA = torch.from_numpy(a).to("cuda:0")
    dB = torch.eye(K, dtype=torch.float32, device="cuda:0").reshape(-1).contiguous()
    dC = torch.full((M * N,), float("nan"), dtype=torch.float32, device="cuda:0")
    return np, dA, dB, dC


def inner(steps, warmup):
    """Body run under rocprofv3: the timed loop plus one copy kernel of known size."""
    import torch
    import rocm_sgemm_amd as rs
    _, dA, dB, dC = identity_workload()
    stream = torch.cuda.current_stream()
    for _ in range(warmup + steps):
        rs.gemm(dC, dA, dB, M, N, K, stream=stream)
    torch.cuda.synchronize()
    probe = torch.empty_like(dA)
    for _ in range(3):
        torch.mul(dA, 1.0, out=probe)  # plain copy kernel: reads 64 MiB, writes 64 MiB
    torch.cuda.synchronize()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-layouts", action="store_true", help="skip the per-layout and 8192^3 table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-context", action="store_true", help="skip the vendor-library context")
    ap.add_argument("--counters", action="store_true",
                    help="also write the counter summary under profiles/ (the counters themselves are "
                         "collected by default)")
    ap.add_argument("--no-counters", action="store_true", help="skip the rocprofv3 counter passes")
    ap.add_argument("--inner", action="store_true", help=argparse.SUPPRESS)
    args = ap.parse_args()

    if args.gpus != 1:
        sys.exit("bench.py: this library drives one GPU per call; --gpus must be 1 "
                 "(no multi-GPU figure exists for this path)")
    if args.inner:
        inner(args.steps, args.warmup)
        return

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import rocm_sgemm_amd as rs

    np, dA, dB, dC = identity_workload()
    stream = torch.cuda.current_stream()

    def step():
        rs.gemm(dC, dA, dB, M, N, K, stream=stream)

    times, wall_ms, _ = timed_launches(step, args.steps, args.warmup)
    if not torch.equal(dC.view(torch.int32), dA.view(torch.int32)):
        sys.exit("bench.py: identity-B result differs from A - refusing to report a number")
    avg_ms = sum(times) / len(times)
    min_ms = min(times)
    ms_per_step = wall_ms / args.steps
    cfg = rs.find_config(M, N, K).as_dict()

    counters, counters_error = None, None
    if not args.no_counters:
        try:
            counters = counters_report(args.steps, args.warmup)
        except (RuntimeError, OSError, subprocess.SubprocessError) as e:
            counters_error = f"{type(e).__name__}: {e}"[:200]
            if args.counters:
                sys.exit(f"bench.py: --counters asked for, but the rocprofv3 passes failed ({counters_error})")
    if counters is not None and counters.get("hbm_bytes_per_launch") is not None:
        if args.counters:
            write_counter_summary(counters, avg_ms)
        counters.pop("raw", None)
        traffic = counters["hbm_bytes_per_launch"]
        traffic_source = "this run: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE passes"
    else:
        traffic = read_traffic()
        traffic_source = (None if traffic is None else
                          "profiles/sgemm_mfma_4096_rrr_counters.txt: rocprofv3 --pmc passes of an "
                          "earlier `bench.py --counters` run of this workload, not measured in this run"
                          + (f" ({counters_error})" if counters_error else ""))

    line = {
        "metric": "SGEMM TFLOPS (avg & min) at 4096^3 NN/NT/TN/TT; % of MI355X FP32 MFMA peak",
        "value": round(tflops(M, N, K, ms_per_step), 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "SGEMM M=N=K=4096, A/B/C row-major, A uniform[-1,1) mt19937 seed 0, "
                               "B = identity (output checked bit-exact against A)",
                   "kernel_config": cfg},
        "avg_tflops": round(tflops(M, N, K, avg_ms), 2),
        "min_time_tflops": round(tflops(M, N, K, min_ms), 2),
        "avg_ms": round(avg_ms, 5),
        "min_ms": round(min_ms, 5),
        "pct_of_fp32_mfma_peak": {"avg": round(100 * tflops(M, N, K, avg_ms) / PEAK_TFLOPS, 1),
                                  "min_time": round(100 * tflops(M, N, K, min_ms) / PEAK_TFLOPS, 1)},
        "roofline": {"bound": "mfma", "achieved": round(tflops(M, N, K, avg_ms), 2),
                     "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops(M, N, K, avg_ms) / PEAK_TFLOPS, 4), "traffic": traffic,
                     "traffic_source": traffic_source},
    }
    if counters is not None:
        line["counters"] = counters
        for k in ("mfma_busy_pct", "mfma_busy_pct_of_cu_busy", "lds_bank_conflict_pct"):
            if k in counters:
                line["roofline"][k] = counters[k]
    line["dense_4096"] = bench_dense_4096(rs, args.steps, args.warmup)
    if not args.no_layouts:
        line["layouts"] = bench_layouts(rs, (1024, 2048, 4096, 8192), args.steps, args.warmup)
        line["shapes_row_major"] = bench_shapes(rs, args.steps, args.warmup)
        line["held_out"] = bench_held_out(rs, args.steps, args.warmup)
    if not args.no_context:
        line["context"] = bench_context((4096, 8192), args.steps, args.warmup)
        ceiling = mfma_only_kernel()
        if ceiling is not None:
            line["context"]["kernel of MFMAs only (bench_float --mfma_ceiling)"] = ceiling
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
