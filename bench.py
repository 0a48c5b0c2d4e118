#!/usr/bin/env python3
"""Benchmark of the brick-blocked SpMM hot path on one MI355X.

A step is one SpMM (C = A.B) over the headline workload: the 65536-row 9-point-stencil
matrix with a dense 65536 x 128 fp32 B, inputs resident in HBM before timing starts -- in HBM,
not in a cache: the timed steps cycle through enough (B, C) buffer sets that the 256 MB Infinity
Cache cannot hold them, so `value` and `roofline` are what a product on fresh data costs.  The same
launches on one buffer set (served by that cache) are reported beside them as `cache_resident`.
Prints ONE JSON line: GFLOP/s = 2.nnz.N / t, the HBM roofline of the dominant kernel
(algorithmic bytes / average launch duration from HIP events around the timed launches), the
other four benchmark configurations (`other_configs`) and the CPU oracle timed on the host cores
as a reported baseline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--no-cpu] [--no-others] [--rotate R] [--detail FILE]
                    [--path auto|mfma|rows] [--mfma-shape 0|1|2] [--pipeline 0|1|2] [--calibrate-copy]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def algorithmic_bytes(M, K, N, nnz):
    """CSR values + column indices + row pointers read once, B read once, C written once."""
    return nnz * 8 + (M + 1) * 4 + K * N * 4 + M * N * 4


KERNEL_SOURCES = ("cutespmm_ae_amd/csrc/kernels.hip.hpp", "cutespmm_ae_amd/csrc/device.hip")


def kernel_sources_sha16():
    """Fingerprint of the device code the counters under profiles/ were taken with."""
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def recorded_traffic(workload, kernel):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE): read from the record
    committed under profiles/ -- but only if that record was taken with the kernel sources as they are now
    and for the kernel that ran; otherwise the traffic is unknown (None) and the source says why."""
    rel = "profiles/hbm_traffic_%s.json" % workload
    try:
        rec = json.load(open(os.path.join(ROOT, rel))).get(workload)
        for name, other in (rec.get("other_kernels") or {}).items():      # a second kernel profiled on the same workload
            if kernel and str(name).startswith(kernel):
                rec = other
        total = float(rec["fetch_bytes"]) + float(rec["write_bytes"])
    except (OSError, ValueError, KeyError, TypeError, AttributeError):
        return None, None
    source = dict(file=rel, kernel=rec.get("kernel"), kernel_sources_sha16=rec.get("kernel_sources_sha16"),
                  recorded_at_commit=rec.get("commit"))
    if rec.get("kernel_sources_sha16") != kernel_sources_sha16():
        source["stale"] = "kernel sources changed since the counters were recorded"
        return None, source
    if kernel and rec.get("kernel") and not str(rec["kernel"]).startswith(kernel):
        source["stale"] = "recorded for another kernel"
        return None, source
    if rec.get("mfma_busy_pct") is not None:
        source["mfma_busy_pct"] = rec["mfma_busy_pct"]
    return total, source


def cpu_baseline(A, B, budget_s=10.0):
    """The CPU oracle (row-parallel CSR restatement of inc.h:71-83) on the host cores:
    repeated full passes over the same workload for about `budget_s` seconds."""
    import oracle
    out = np.empty((A.M, B.shape[1]), np.float32)
    oracle.spmm_csr(A.rowPtr, A.cols, A.vals, B, out=out)           # warm-up pass
    times = []
    t_end = time.perf_counter() + budget_s
    while time.perf_counter() < t_end or len(times) < 3:
        t0 = time.perf_counter()
        oracle.spmm_csr(A.rowPtr, A.cols, A.vals, B, out=out)
        times.append(time.perf_counter() - t0)
    t = float(np.median(times))
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    res = dict(value=2.0 * A.nnz * B.shape[1] / t / 1e9, unit="GFLOP/s", cores=cores, kind="port",
               sample="%d full passes of the same workload (median)" % len(times))
    if A.nnz <= 100000:
        # the reference's own loop placement (inc.h:71-83: the thread team is forked inside the loop
        # over nonzeros), once, on workloads small enough for it: why it is not the timed baseline
        rows = np.repeat(np.arange(A.M, dtype=np.uint32), np.diff(A.rowPtr.astype(np.int64)))
        t0 = time.perf_counter()
        same = oracle.spmm_coo(rows, A.cols, A.vals, B, A.M, inner_parallel=True)
        t1 = time.perf_counter() - t0
        res["reference_loop_placement"] = dict(value=2.0 * A.nnz * B.shape[1] / t1 / 1e9, unit="GFLOP/s", seconds=t1,
                                               equal_to_baseline=bool((same == out).all()))
    return res, out


INFINITY_CACHE_BYTES = 256 << 20
ORACLE_BUILD = "gcc -O3 -mavx2 -ffp-contract=off -fopenmp (portable build: AVX2, not -march=native, so the library built in one container runs on another host)"


def buffer_sets_for(set_bytes):
    """How many (B, C) buffer sets the timed steps cycle through so that no cache holds them: five times the
    Infinity Cache in all (at most 64 sets); one when a single set already exceeds that cache."""
    if set_bytes > INFINITY_CACHE_BYTES:
        return 1
    return int(min(64, max(2, -(-5 * INFINITY_CACHE_BYTES // set_bytes))))


def timed_steps(torch, plan, dBs, dCs, steps, warmup, ramp_ms, stream):
    """`warmup` untimed steps (after `ramp_ms` of the same launches, which bring the clocks up), then exactly `steps`
    timed ones, synchronised on both sides; HIP events on the launch stream bracket the same launches.
    Returns (wall ms per step, event ms per step)."""
    R, i = len(dBs), 0
    ramp_end = time.perf_counter() + ramp_ms * 1e-3
    while time.perf_counter() < ramp_end:
        for _ in range(50):
            plan.run(dBs[i % R], dCs[i % R]); i += 1
        torch.cuda.synchronize()
    for _ in range(warmup):
        plan.run(dBs[i % R], dCs[i % R]); i += 1
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for _ in range(steps):
        plan.run(dBs[i % R], dCs[i % R]); i += 1
    ev1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall * 1e3 / steps, ev0.elapsed_time(ev1) / steps


def timed_steps_graph(torch, plan, dBs, dCs, steps):
    """The same `steps` launches recorded once into a HIP graph and replayed: no host time between them.  For launches of a
    few microseconds, which the host cannot issue as fast as the device runs them.  Returns event ms per step (best of 3
    replays after one untimed replay)."""
    R = len(dBs)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for i in range(steps):
            plan.run(dBs[i % R], dCs[i % R], stream=torch.cuda.current_stream())
    graph.replay()
    torch.cuda.synchronize()
    best = None
    for _ in range(3):
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        graph.replay()
        ev1.record()
        torch.cuda.synchronize()
        ms = ev0.elapsed_time(ev1) / steps
        best = ms if best is None else min(best, ms)
    return best


def plan_kernels(plan):
    kernels = []
    if plan.info["numChunks"]:
        kernels.append(plan.kernel_name)
    if (plan.info["numRowPanelsSparse"] or plan.info["numEmptyPanels"]) and not plan.info["fusedLaunch"]:
        kernels.append("csr_rows_batched")
    if plan.info["numAtomicChunks"]:
        kernels.append("reduce_partials")
    return kernels, (plan.kernel_name if plan.info["numChunks"] else "csr_rows_batched")


def simple_csr_us(cs, h, dB, dC, nnz, stream):
    """The three plain CSR kernels on the same inputs (one buffer set): median us of single launches."""
    out = {}
    for alg, name in ((0, "thread_per_element"), (1, "wave_per_row_scalar"), (2, "wave_per_row_vector")):
        iters = 30 if nnz < 10_000_000 else 5
        out[name] = float(np.median(cs.csr_spmm_time(alg, h, dB, dC, warmup=3, iters=iters, stream=stream))) * 1e3
    return out


def other_config(torch, cs, config, stream, precision=None):
    """One of the other benchmark configurations through the planner's default: us per step over rotating buffer
    sets (HBM-fed) and on one set, GFLOP/s, share of the HBM roofline, kernel, speed-up over the best plain CSR kernel."""
    cfg = cs.CONFIGS[config]
    A = cs.gen_config(config)
    N = cfg["N"]
    B = cs.gen_dense(cs.SEED_BASE + 100 + config, A.K, N, 2)
    h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    dB = torch.from_numpy(B).cuda()
    del B
    dC = torch.empty((A.M, N), device="cuda")
    set_bytes = (A.K + A.M) * N * 4
    R = buffer_sets_for(set_bytes)
    dBs = [dB] + [dB.clone() for _ in range(R - 1)]
    dCs = [dC] + [torch.empty_like(dC) for _ in range(R - 1)]
    kw = dict(precision=cs.PREC_BF16X3) if precision == "bf16x3" else {}
    plan = cs.SPMM_TC(h, N, **kw)
    big = A.nnz >= 10_000_000
    steps = 20 if big else 200
    abytes, flops = algorithmic_bytes(A.M, A.K, N, A.nnz), 2.0 * A.nnz * N
    ms, kernel_ms = timed_steps(torch, plan, dBs, dCs, steps, 5 if big else 50, 30.0, stream)
    kernels, dominant = plan_kernels(plan)
    traffic, source = recorded_traffic(cfg["name"], dominant)
    host_bound = None
    if kernel_ms < 0.015:
        # launches this short are issued more slowly than they run (7-8 us per call from Python against a 4 us
        # kernel): the figure is taken from a replayed graph of the same steps, the eager one is reported beside it
        host_bound = dict(us_per_step_eager=ms * 1e3, event_us_per_step_eager=kernel_ms * 1e3)
        kernel_ms = timed_steps_graph(torch, plan, dBs, dCs, steps)
        ms = kernel_ms
    res = dict(workload=cfg["name"], M=A.M, K=A.K, N=N, nnz=A.nnz, kernel=dominant, kernels_per_step=kernels,
               precision=precision or "fp32", buffer_sets=R, steps=steps, us_per_step=ms * 1e3, kernel_us=kernel_ms * 1e3,
               value=flops / (ms * 1e-3) / 1e9, unit="GFLOP/s", algorithmic_bytes=abytes,
               achieved_GBps=abytes / (kernel_ms * 1e-3) / 1e9, frac=abytes / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
               traffic=traffic, mfma_busy_pct=(source or {}).get("mfma_busy_pct"))
    if host_bound:
        res["steps_replayed_from_a_graph"] = host_bound
    if R > 1:
        ms1, kernel_ms1 = timed_steps(torch, plan, dBs[:1], dCs[:1], steps, 50, 0.0, stream)
        if host_bound:
            ms1 = kernel_ms1 = timed_steps_graph(torch, plan, dBs[:1], dCs[:1], steps)
        res["cache_resident"] = dict(us_per_step=ms1 * 1e3, kernel_us=kernel_ms1 * 1e3,
                                     frac_of_hbm_peak=abytes / (kernel_ms1 * 1e-3) / 1e9 / HBM_PEAK_GBS)
    if precision is None:
        csr = simple_csr_us(cs, h, dB, dC, A.nnz, stream)
        each = float(np.median(plan.time(dB, dC, warmup=3, iters=30 if not big else 5, stream=stream))) * 1e3
        res["simple_csr_kernels_us"] = csr
        res["speedup_over_best_simple_csr"] = min(csr.values()) / each     # both: single launches on one buffer set
    return res


def memory_pattern_probe():
    """Runs cutespmm_ae_amd/membw_probe (plain streaming kernels, no SpMM) as a child process and returns its
    HBM-fed ("rotating") times in microseconds, keyed by pattern; None if the program is not built or fails.
    Called before this process touches the GPU."""
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cutespmm_ae_amd", "membw_probe")
    if not os.path.exists(exe):
        return None
    try:
        text = subprocess.run([exe], capture_output=True, text=True, timeout=120, check=True).stdout
    except (OSError, subprocess.SubprocessError):
        return None
    out = {}
    for line in text.splitlines():
        parts = line.rsplit("rotating", 1)
        if len(parts) == 2 and " us" in parts[1]:
            out[" ".join(parts[0].split())] = float(parts[1].split("us")[0])
    return out or None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--ramp-ms", type=float, default=50.0,
                    help="run the same launches for this long before the warm-up steps: the GPU takes a few milliseconds of "
                         "continuous work to reach its steady clocks (0 switches it off)")
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration 1..5 (2 = headline)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--detail", default=None, help="also time every path and the CSR kernels; write JSON here")
    ap.add_argument("--path", choices=("auto", "mfma", "rows"), default="auto", help="kernel family (default: the planner's choice)")
    ap.add_argument("--mfma-shape", type=int, default=0, help="1: 16x16x4 brick kernel, 2: 4x4x1 quad kernel, 0: planner's choice")
    ap.add_argument("--pipeline", type=int, default=0, help="brick kernel variant: 1 rolling, 2 pipelined, 0: default")
    ap.add_argument("--precision", choices=("fp32", "bf16x3"), default="fp32",
                    help="bf16x3: the brick kernel on the bf16 matrix pipeline (opt-in, error below 2^-15); default fp32")
    ap.add_argument("--residency", type=int, default=0, help="cute_tunables.operand_residency: 0 unknown (default), 1 from HBM, 2 cache-resident")
    ap.add_argument("--no-csr", action="store_true", help="skip the three plain CSR comparison kernels")
    ap.add_argument("--rotate", type=int, default=0,
                    help="number of (B, C) buffer sets the timed steps cycle through; 0 (default): enough that the 256 MB Infinity "
                         "Cache cannot hold them (five times its size in all); 1: the same buffers every step, which that cache "
                         "then serves when they fit it")
    ap.add_argument("--no-resident-leg", "--no-hbm-leg", dest="no_resident_leg", action="store_true",
                    help="skip the second measurement of the same launches on one buffer set, and the forced-kernel comparison")
    ap.add_argument("--no-others", action="store_true", help="skip the other four benchmark configurations")
    ap.add_argument("--chunk-order", type=int, default=0,
                    help="MFMA work items: 0 planner's choice, 1 panel order, 2 dealt to the SIMDs longest first")
    ap.add_argument("--graph", action="store_true",
                    help="record the K launches of the timed region into one HIP graph and replay it (launch-bound workloads; one buffer set)")
    ap.add_argument("--no-probe", action="store_true", help="skip the memory-pattern microbenchmark (hbm_fed.plain_streaming_kernels_us)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run 10 plain device copies of 32 MiB and exit (reference point for HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (got --gpus %d); nothing here shards across GPUs" % args.gpus)

    # plain streaming kernels of the headline's size for scale; a child process, started before this one uses the GPU
    # (not under a profiler: its preloaded library would profile the child as well)
    profiled = any("rocprof" in v.lower() for v in (os.environ.get("LD_PRELOAD", ""), os.environ.get("ROCP_TOOL_LIBRARIES", "")))
    probe = None
    if args.config == 2 and not (args.no_probe or args.calibrate_copy or args.graph or args.no_resident_leg or profiled):
        probe = memory_pattern_probe()

    import torch
    import cutespmm_ae_amd as cs

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    if args.calibrate_copy:
        src = torch.arange(8 << 20, dtype=torch.float32, device="cuda")      # 32 MiB read, 32 MiB written per copy
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps(dict(copy_bytes_read=src.numel() * 4, copy_bytes_written=dst.numel() * 4, copies=10)))
        return
    cfg = cs.CONFIGS[args.config]
    A = cs.gen_config(args.config)
    N = cfg["N"]
    B = cs.gen_dense(cs.SEED_BASE + 100 + args.config, A.K, N, 2)
    h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    dB = torch.from_numpy(B).cuda()
    dC = torch.empty((A.M, N), device="cuda")
    set_bytes = (A.K + A.M) * N * 4
    if args.rotate < 0:
        sys.exit("bench.py: --rotate needs 0 (automatic) or a number of buffer sets")
    R = 1 if args.graph else (args.rotate or buffer_sets_for(set_bytes))
    dBs = [dB] + [dB.clone() for _ in range(R - 1)]
    dCs = [dC] + [torch.empty_like(dC) for _ in range(R - 1)]
    tun = dict(path={"auto": cs.PATH_AUTO, "mfma": cs.PATH_BRICK, "rows": cs.PATH_ROWS}[args.path],
               mfma_shape=args.mfma_shape, pipeline=args.pipeline, chunk_order=args.chunk_order, operand_residency=args.residency,
               precision=cs.PREC_BF16X3 if args.precision == "bf16x3" else cs.PREC_FP32)
    plan = cs.SPMM_TC(h, N, **tun)
    stream = torch.cuda.current_stream()
    flops = 2.0 * A.nnz * N
    abytes = algorithmic_bytes(A.M, A.K, N, A.nnz)

    if args.graph:
        # cute_spmm_run only enqueues kernels, so the K launches can be captured once and replayed
        timed_steps(torch, plan, dBs, dCs, 1, args.warmup, args.ramp_ms, stream)
        side = torch.cuda.Stream()
        side.wait_stream(stream)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(args.steps):
                plan.run(dB, dC, stream=torch.cuda.current_stream())
        graph.replay()                                  # one untimed replay: the first one uploads the graph
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record(stream)
        graph.replay()
        ev1.record(stream)
        torch.cuda.synchronize()
        ms_per_step, kernel_ms = (time.perf_counter() - t0) * 1e3 / args.steps, ev0.elapsed_time(ev1) / args.steps
    else:
        # the timed region: exactly K steps, synchronised on both sides; HIP events on the launch
        # stream bracket the same K launches and give the average launch duration for the roofline
        ms_per_step, kernel_ms = timed_steps(torch, plan, dBs, dCs, args.steps, args.warmup, args.ramp_ms, stream)
    value = flops / (ms_per_step * 1e-3) / 1e9

    # the same launches one by one on one buffer set, each inside its own event pair (adds the cost of the bracket):
    # the figure the plain CSR kernels are compared with, so only taken with them
    each = None if args.no_csr else plan.time(dB, dC, warmup=5, iters=max(20, min(args.steps, 200)), stream=stream)
    achieved = abytes / (kernel_ms * 1e-3) / 1e9
    kernels, dominant = plan_kernels(plan)
    traffic, traffic_source = recorded_traffic(cfg["name"], dominant)
    hbm_fed = R > 1 or set_bytes > INFINITY_CACHE_BYTES
    if R > 1:
        operands = ("HBM: the timed steps cycle through %d (B, C) buffer sets, %.2f GB in all, which the 256 MB Infinity Cache "
                    "cannot hold" % (R, R * set_bytes / 1e9))
    elif hbm_fed:
        operands = "HBM: one set of B and C (%.0f MB) exceeds the 256 MB Infinity Cache" % (set_bytes / 1e6)
    else:
        operands = ("the 256 MB Infinity Cache: the same %.0f MB of B and C every step -- NOT an HBM-fed figure" % (set_bytes / 1e6))
    roofline = dict(bound="hbm", achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s", frac=achieved / HBM_PEAK_GBS,
                    traffic=traffic, traffic_source=traffic_source, mfma_busy_pct=(traffic_source or {}).get("mfma_busy_pct"),
                    kernel=dominant, kernels_per_step=kernels, kernel_ms=kernel_ms, operands_fed_from=operands,
                    kernel_ms_single_bracketed_median_one_set=None if each is None else float(np.median(each)), algorithmic_bytes=abytes)

    out = dict(metric="SpMM GFLOP/s (2*nnz*N/t) on 1 MI355X", value=value, unit="GFLOP/s", n_gpus=1,
               steps=args.steps, warmup=args.warmup, ms_per_step=ms_per_step, higher_is_better=True,
               scaling="weak", vs_baseline=None, dtype="f32" if plan.info["precision"] == cs.PREC_FP32 else "bf16x3 (f32 accumulate)",
               data="synthetic (seeded generator)",
               launch="hip graph replay" if args.graph else "stream launches", ramp_ms=args.ramp_ms, buffer_sets=R,
               config=dict(workload=cfg["name"], M=A.M, K=A.K, N=N, nnz=A.nnz, blocks=h.numBlocks,
                           bricks=h.num_bricks, plan={k: plan.info[k] for k in
                                                      ("slabWidth", "numSlabs", "numChunks", "numAtomicChunks",
                                                       "numBrickPanels", "numRowPanelsSparse", "dealtChunks")}),
               roofline=roofline)

    if R > 1 and not args.no_resident_leg:
        # the protocol of the earlier figures: one buffer set, which the Infinity Cache then serves
        steps1 = max(args.steps, 200)
        ms1, kernel_ms1 = timed_steps(torch, plan, dBs[:1], dCs[:1], steps1, 50, 0.0, stream)
        res = dict(note="the same launches on ONE buffer set (%.0f MB of B and C), which the 256 MB Infinity Cache serves after the "
                        "first step: what a caller sees who multiplies the same operands again and again; not an HBM figure"
                        % (set_bytes / 1e6),
                   steps=steps1, ms_per_step=ms1, kernel_ms=kernel_ms1, value=flops / (ms1 * 1e-3) / 1e9, unit="GFLOP/s",
                   kernel=plan.kernel_name, algorithmic_GBps=abytes / (kernel_ms1 * 1e-3) / 1e9,
                   frac_of_hbm_peak=abytes / (kernel_ms1 * 1e-3) / 1e9 / HBM_PEAK_GBS)
        if plan.info["numChunks"] and args.residency == 0 and args.mfma_shape == 0:
            told = cs.SPMM_TC(h, N, **dict(tun, operand_residency=2))
            t_ms, t_kernel_ms = timed_steps(torch, told, dBs[:1], dCs[:1], steps1, 50, 0.0, stream)
            res["planner_told_operands_stay_resident"] = dict(kernel=told.kernel_name, ms_per_step=t_ms, value=flops / (t_ms * 1e-3) / 1e9,
                                                              frac_of_hbm_peak=abytes / (t_kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS)
        out["cache_resident"] = res
    if hbm_fed and not args.graph:
        # the HBM-fed figures under the name earlier records used for them
        fed = dict(note="the main measurement of this line (value, ms_per_step, roofline) is HBM-fed", sets=R, bytes_cycled=R * set_bytes,
                   ms_per_step=ms_per_step, kernel_ms=kernel_ms, value=value, frac=achieved / HBM_PEAK_GBS, kernel=plan.kernel_name,
                   planner="default tunables" if (args.residency == 0 and args.mfma_shape == 0 and args.path == "auto") else "forced by flags")
        if R > 1 and plan.info["numChunks"] and not args.no_resident_leg:
            # either MFMA kernel forced, under the same conditions
            steps2 = max(min(args.steps, 500), 200)
            fed["mfma_kernels_forced_us"] = {name: timed_steps(torch, cs.SPMM_TC(h, N, mfma_shape=shape), dBs, dCs, steps2, 50, 0.0, stream)[1] * 1e3
                                             for name, shape in (("quad", 2), ("brick", 1))}
            fed["device_copy_of_B_onto_C_us"] = timed_steps(torch, type("Copy", (), {"run": staticmethod(lambda b, c: c.copy_(b))}), dBs, dCs,
                                                            steps2, 50, 0.0, stream)[1] * 1e3
        if probe:
            fed["plain_streaming_kernels_us"] = dict(
                note="cutespmm_ae_amd/membw_probe: 4 096 wavefronts that stream private regions, rotating buffer sets (HBM-fed); "
                     "for scale against this launch's bytes beyond the L2s (roofline.traffic)", **probe)
        out["hbm_fed"] = fed
    plan.run(dB, dC)
    torch.cuda.synchronize()

    if not args.no_csr:
        # the plain CSR kernels on the same inputs and clocks: the "best simple CSR kernel" a caller would write instead
        csr_us = simple_csr_us(cs, h, dB, dC, A.nnz, stream)
        out["simple_csr_kernels_us"] = csr_us
        out["speedup_over_best_simple_csr"] = min(csr_us.values()) / (float(np.median(each)) * 1e3)     # both timed one launch per event pair
        plan.run(dB, dC)                                # the output checked below is the planned path's
        torch.cuda.synchronize()

    ref = None
    if not args.no_cpu:
        out["cpu_baseline"], ref = cpu_baseline(A, B)
        out["cpu_baseline"]["build"] = ORACLE_BUILD
        got = dC.cpu().numpy()
        out["backward_error_vs_oracle"] = cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, got)
        out["reference_metric_vs_oracle"] = cs.check_gemm_correctness_coo(ref, got)
        out["parity_note"] = ("checked against this build's CPU oracle (inc.h:71-83 restated); the reference's own comparison path, "
                              "cuSPARSE CSR SpMM (spmm.cu:912-938), is a closed binary with no stored outputs: parity with its bits is unpinned")

    if args.config == 2 and not args.no_others and not args.graph:
        # the other four benchmark configurations, each through the planner's default (present_gflops.py:30-42 prints one
        # line per matrix and width the same way); free this config's buffers first
        del dBs, dCs, plan
        dB = dC = None
        torch.cuda.empty_cache()
        others = {}
        for c in (1, 3, 4, 5):
            others["cfg%d" % c] = other_config(torch, cs, c, stream)
            if c == 3:
                others["cfg3_bf16x3"] = other_config(torch, cs, 3, stream, precision="bf16x3")
            torch.cuda.empty_cache()
        out["other_configs"] = others

    if args.detail:
        dB = torch.from_numpy(B).cuda()
        dC = torch.empty((A.M, N), device="cuda")
        detail = dict(workload=cfg["name"], paths={}, csr={})
        for name, kw in (("quad", dict(path=cs.PATH_BRICK, mfma_shape=2)),
                         ("brick_rolling", dict(path=cs.PATH_BRICK, mfma_shape=1, pipeline=1)),
                         ("brick_pipelined", dict(path=cs.PATH_BRICK, mfma_shape=1, pipeline=2)),
                         ("rows", dict(path=cs.PATH_ROWS)), ("auto", dict())):
            p = cs.SPMM_TC(h, N, **kw)
            t = p.time(dB, dC, warmup=5, iters=50, stream=stream)
            detail["paths"][name] = dict(median_us=float(np.median(t)) * 1e3, mean_us=float(np.mean(t)) * 1e3,
                                         gflops=flops / (float(np.median(t)) * 1e-3) / 1e9, info=p.info)
        for alg, name in ((0, "thread_per_element"), (1, "wave_per_row_scalar"), (2, "wave_per_row_vector")):
            t = cs.csr_spmm_time(alg, h, dB, dC, warmup=3, iters=30, stream=stream)
            detail["csr"][name] = dict(median_us=float(np.median(t)) * 1e3,
                                       gflops=flops / (float(np.median(t)) * 1e-3) / 1e9)
        # the comparison format of the reference's harness: Blocked-ELL, block sizes 16 and 32
        detail["blocked_ell"] = {}
        csr = cs.CSR_Matrix(nrows=A.M, ncols=A.K, rowPtr=A.rowPtr.astype(np.int32), cols=A.cols.astype(np.int32), values=A.vals)
        for bs in (16, 32):
            if A.M % bs or A.K % bs:
                continue
            ell = cs.preprocess(csr, bs)
            dCe = torch.empty((ell.get_ellColIdx_height() * bs, N), device="cuda")
            for _ in range(3):
                ell.spmm(dB, dCe, stream=stream)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(30):
                ell.spmm(dB, dCe, stream=stream)
            e1.record(stream)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / 30 * 1e3
            stored = ell.get_num_blocks() * bs * bs
            detail["blocked_ell"]["block_%d" % bs] = dict(
                mean_us=us, gflops=flops / us / 1e3, width=ell.get_ellColIdx_width(), blocks=ell.get_num_blocks(),
                stored_tflops=2.0 * stored * N / us / 1e6, fill=A.nnz / stored)
        best = max(v["gflops"] for v in detail["csr"].values())
        detail["best_simple_csr_gflops"] = best
        detail["speedup_over_best_simple_csr"] = detail["paths"]["auto"]["gflops"] / best
        with open(args.detail, "w") as f:
            json.dump(detail, f, indent=1)

    print(json.dumps(out))


if __name__ == "__main__":
    main()
