#!/usr/bin/env python3
"""Benchmark of the brick-blocked SpMM hot path on one MI355X.

A step is one SpMM (C = A.B) over the headline workload: the 65536-row 9-point-stencil
matrix with a dense 65536 x 128 fp32 B, inputs resident in HBM before timing starts.
Prints ONE JSON line: GFLOP/s = 2.nnz.N / t, the HBM roofline of the dominant kernel
(algorithmic bytes / average launch duration from HIP events around the timed launches) and
the CPU oracle timed on the host cores as a reported baseline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--no-cpu] [--detail FILE]
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
        total = float(rec["fetch_bytes"]) + float(rec["write_bytes"])
    except (OSError, ValueError, KeyError, TypeError):
        return None, None
    source = dict(file=rel, kernel=rec.get("kernel"), kernel_sources_sha16=rec.get("kernel_sources_sha16"),
                  recorded_at_commit=rec.get("commit"))
    if rec.get("kernel_sources_sha16") != kernel_sources_sha16():
        source["stale"] = "kernel sources changed since the counters were recorded"
        return None, source
    if kernel and rec.get("kernel") and not str(rec["kernel"]).startswith(kernel):
        source["stale"] = "recorded for another kernel"
        return None, source
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


def hbm_fed_leg(torch, cs, plan, h, dB, dC, N, set_bytes, abytes, flops, steps):
    """The same launches over enough rotating (B, C) buffer sets that no cache can hold them (1.25 GB, five times
    the Infinity Cache): every B row then comes from HBM and every C row goes there.  The main measurement
    re-runs one set; when that set fits the 256 MB Infinity Cache, the cache serves most of it."""
    if set_bytes > INFINITY_CACHE_BYTES:
        return dict(sets=1, note="one set of B and C (%.0f MB) already exceeds the Infinity Cache: the main measurement is HBM-fed"
                                 % (set_bytes / 1e6))
    sets = max(2, -(-5 * INFINITY_CACHE_BYTES // set_bytes))
    dBs = [dB] + [dB.clone() for _ in range(sets - 1)]
    dCs = [dC] + [torch.empty_like(dC) for _ in range(sets - 1)]

    def timed(p):
        i = 0
        for _ in range(max(sets, 50)):
            p.run(dBs[i % sets], dCs[i % sets]); i += 1
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            p.run(dBs[i % sets], dCs[i % sets]); i += 1
        e1.record()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps

    ms, kernel_ms = timed(plan)
    res = dict(sets=sets, bytes_cycled=sets * set_bytes, steps=steps, ms_per_step=ms, kernel_ms=kernel_ms,
               value=flops / (ms * 1e-3) / 1e9, unit="GFLOP/s", achieved_GBps=abytes / (kernel_ms * 1e-3) / 1e9,
               frac=abytes / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, kernel=plan.kernel_name)
    if plan.info["numChunks"]:
        # either MFMA kernel forced, under the same conditions: the planner's choice assumes nothing about residency
        alt = {}
        for name, shape in (("quad", 2), ("brick", 1)):
            alt[name] = timed(cs.SPMM_TC(h, N, mfma_shape=shape))[1] * 1e3
        res["mfma_kernels_forced_us"] = alt
        # the planner told that its operands come from HBM (cute_tunables.operand_residency = 1); by default it goes by size
        told = cs.SPMM_TC(h, N, operand_residency=1)
        t_ms, t_kernel_ms = timed(told)
        res["planner_told_operands_are_cold"] = dict(kernel=told.kernel_name, ms_per_step=t_ms, value=flops / (t_ms * 1e-3) / 1e9,
                                                     frac=abytes / (t_kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS)
    plan.run(dB, dC)
    torch.cuda.synchronize()
    return res


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
    ap.add_argument("--no-csr", action="store_true", help="skip the three plain CSR comparison kernels")
    ap.add_argument("--rotate", type=int, default=1,
                    help="number of (B, C) buffer sets the timed steps cycle through (default 1: the same buffers every step, "
                         "which the 256 MB Infinity Cache then serves when they fit it)")
    ap.add_argument("--no-hbm-leg", action="store_true",
                    help="skip the second measurement over enough rotating buffer sets to exceed the Infinity Cache")
    ap.add_argument("--chunk-order", type=int, default=0,
                    help="MFMA work items: 0 planner's choice, 1 panel order, 2 dealt to the SIMDs longest first")
    ap.add_argument("--graph", action="store_true",
                    help="record the K launches of the timed region into one HIP graph and replay it (launch-bound workloads)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run 10 plain device copies of 32 MiB and exit (reference point for HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (got --gpus %d); nothing here shards across GPUs" % args.gpus)

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
    if args.rotate < 1:
        sys.exit("bench.py: --rotate needs at least one buffer set")
    dBs = [dB] + [dB.clone() for _ in range(args.rotate - 1)]
    dCs = [dC] + [torch.empty_like(dC) for _ in range(args.rotate - 1)]
    plan = cs.SPMM_TC(h, N, path={"auto": cs.PATH_AUTO, "mfma": cs.PATH_BRICK, "rows": cs.PATH_ROWS}[args.path],
                      mfma_shape=args.mfma_shape, pipeline=args.pipeline, chunk_order=args.chunk_order,
                      precision=cs.PREC_BF16X3 if args.precision == "bf16x3" else cs.PREC_FP32)
    stream = torch.cuda.current_stream()

    ramp_end = time.perf_counter() + args.ramp_ms * 1e-3
    while time.perf_counter() < ramp_end:
        for _ in range(50):
            plan.run(dB, dC)
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        plan.run(dB, dC)
    torch.cuda.synchronize()
    # the timed region: exactly K steps, synchronised on both sides; HIP events on the launch
    # stream bracket the same K launches and give the average launch duration for the roofline
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    graph = None
    if args.graph:
        # cute_spmm_run only enqueues kernels, so the K launches can be captured once and replayed
        side = torch.cuda.Stream()
        side.wait_stream(stream)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(args.steps):
                plan.run(dB, dC, stream=torch.cuda.current_stream())
        graph.replay()                                  # one untimed replay: the first one uploads the graph
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record(stream)
    if graph is not None:
        graph.replay()
    elif args.rotate == 1:
        for _ in range(args.steps):
            plan.run(dB, dC)
    else:
        for i in range(args.steps):
            plan.run(dBs[i % args.rotate], dCs[i % args.rotate])
    ev1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    flops = 2.0 * A.nnz * N
    value = flops / (ms_per_step * 1e-3) / 1e9

    kernel_ms = ev0.elapsed_time(ev1) / args.steps
    # the same launches one by one, each inside its own event pair (adds the cost of the bracket)
    each = plan.time(dB, dC, warmup=5, iters=max(20, min(args.steps, 200)), stream=stream)
    abytes = algorithmic_bytes(A.M, A.K, N, A.nnz)
    achieved = abytes / (kernel_ms * 1e-3) / 1e9
    kernels = []
    if plan.info["numChunks"]:
        kernels.append(plan.kernel_name)
    if (plan.info["numRowPanelsSparse"] or plan.info["numEmptyPanels"]) and not plan.info["fusedLaunch"]:
        kernels.append("csr_rows_batched")
    if plan.info["numAtomicChunks"]:
        kernels.append("reduce_partials")
    dominant = plan.kernel_name if plan.info["numChunks"] else "csr_rows_batched"
    traffic, traffic_source = recorded_traffic(cfg["name"], dominant)
    roofline = dict(bound="hbm", achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s", frac=achieved / HBM_PEAK_GBS,
                    traffic=traffic, traffic_source=traffic_source, kernel=dominant,
                    kernels_per_step=kernels, kernel_ms=kernel_ms, kernel_ms_single_bracketed_median=float(np.median(each)),
                    algorithmic_bytes=abytes)

    out = dict(metric="SpMM GFLOP/s (2*nnz*N/t) on 1 MI355X", value=value, unit="GFLOP/s", n_gpus=1,
               steps=args.steps, warmup=args.warmup, ms_per_step=ms_per_step, higher_is_better=True,
               scaling="weak", vs_baseline=None, dtype="f32" if plan.info["precision"] == cs.PREC_FP32 else "bf16x3 (f32 accumulate)",
               data="synthetic (seeded generator)",
               launch="hip graph replay" if args.graph else "stream launches", ramp_ms=args.ramp_ms, buffer_sets=args.rotate,
               config=dict(workload=cfg["name"], M=A.M, K=A.K, N=N, nnz=A.nnz, blocks=h.numBlocks,
                           bricks=h.num_bricks, plan={k: plan.info[k] for k in
                                                      ("slabWidth", "numSlabs", "numChunks", "numAtomicChunks",
                                                       "numBrickPanels", "numRowPanelsSparse", "dealtChunks")}),
               roofline=roofline)

    set_bytes = (A.K + A.M) * N * 4
    if not args.no_hbm_leg and args.rotate == 1 and not args.graph:
        out["hbm_fed"] = hbm_fed_leg(torch, cs, plan, h, dB, dC, N, set_bytes, abytes, flops, min(args.steps, 500))

    if not args.no_csr:
        # the plain CSR kernels on the same inputs and clocks: the "best simple CSR kernel" a caller would write instead
        csr_us = {}
        for alg, name in ((0, "thread_per_element"), (1, "wave_per_row_scalar"), (2, "wave_per_row_vector")):
            iters = 30 if A.nnz < 10_000_000 else 5
            t = cs.csr_spmm_time(alg, h, dB, dC, warmup=3, iters=iters, stream=stream)
            csr_us[name] = float(np.median(t)) * 1e3
        best = min(csr_us.values())
        out["simple_csr_kernels_us"] = csr_us
        out["speedup_over_best_simple_csr"] = best / (float(np.median(each)) * 1e3)     # both timed one launch per event pair
        plan.run(dB, dC)                                # the output checked below is the planned path's
        torch.cuda.synchronize()

    ref = None
    if not args.no_cpu:
        out["cpu_baseline"], ref = cpu_baseline(A, B)
        got = dC.cpu().numpy()
        out["backward_error_vs_oracle"] = cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, got)
        out["reference_metric_vs_oracle"] = cs.check_gemm_correctness_coo(ref, got)
        out["parity_note"] = ("checked against this build's CPU oracle (inc.h:71-83 restated); the reference's own comparison path, "
                              "cuSPARSE CSR SpMM (spmm.cu:912-938), is a closed binary with no stored outputs: parity with its bits is unpinned")

    if args.detail:
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
