"""Benchmark sweep over a directory of MatrixMarket files.

Counterpart of the reference's two scripts (run_kernel.py:16-25 profiles ``run_cute_16_4`` on
every matrix of ./ae_matrices with Nsight Compute; present_gflops.py:19-45 turns the recorded
kernel times into a table): here ``run_cute`` times its own launches with HIP events, so one
pass gives the same table

    matrix, N(feature size), cuTeSpMM GFLOPS, CSR GFLOPS

for N in 32, 128, 512 (run.cu:16), GFLOPS = 2 * nnz * N / t (present_gflops.py:30-34).  The CSR
column is the best hand-written CSR kernel of this library (the reference's is cuSPARSE).
With ``--rocprof`` every (matrix, N) is also run once under ``rocprofv3 --kernel-trace --stats`` -- the
profiler in the place of the reference's Nsight Compute -- and the table is made from the recorded kernel
durations (the kernels of one step added up) instead of the event times.

    python -m cutespmm_ae_amd.sweep ROOT [--n 32,128,512] [--iters 20] [--json FILE] [--cache-dir DIR] [--rocprof]

ROOT holds either ``name/name.mtx`` sub-directories (the layout of ae_matrices/) or ``*.mtx``
files; ``gen:1`` .. ``gen:5`` name the built-in benchmark generators.
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

HERE = os.path.dirname(os.path.abspath(__file__))
DRIVER = os.path.join(HERE, "run_cute")


def find_matrices(root):
    if root.startswith("gen:"):
        return [(root, root)]
    found = []
    for entry in sorted(os.listdir(root)):
        path = os.path.join(root, entry)
        nested = os.path.join(path, entry + ".mtx")
        if os.path.isdir(path) and os.path.isfile(nested):
            found.append((entry, nested))
        elif entry.endswith(".mtx") and os.path.isfile(path):
            found.append((entry[:-4], path))
    return found


def run_one(path, widths, iters, cache=None, check=True, extras=False):
    if not os.path.isfile(DRIVER):
        raise RuntimeError("run_cute is not built; run python -m cutespmm_ae_amd.build")
    cmd = [DRIVER, path, "--n", ",".join(str(n) for n in widths), "--iters", str(iters)]
    if cache:
        cmd += ["--cache", cache]
    if not check:
        cmd.append("--no-check")
    if extras:
        cmd.append("--extras")      # also the device-built format and the hybrid call, per width
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("%s: %s" % (path, proc.stderr.strip() or "exit %d" % proc.returncode))
    return [json.loads(line) for line in proc.stdout.splitlines() if line.startswith("{")]


PLAN_KERNELS = ("hrpb_", "csr_rows_batched", "reduce_partials")      # what one step of a plan launches
CSR_KERNEL = "csr_rows<"                                              # the comparison column's kernel


def kernel_durations(path, n, iters):
    """One (matrix, N) under rocprofv3 --kernel-trace --stats: microseconds per step of the plan's kernels (their
    average durations added up: each runs once per step) and of the CSR comparison kernel, from *_kernel_stats.csv."""
    prof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not path.startswith("gen:"):
        path = os.path.abspath(path)              # the profiler runs from /tmp
    out = tempfile.mkdtemp(prefix="cute_sweep_", dir="/tmp")
    try:
        cmd = [prof, "--kernel-trace", "--stats", "--output-format", "csv", "-d", out, "--",
               DRIVER, path, "--n", str(n), "--iters", str(iters), "--ramp-ms", "0"]
        proc = subprocess.run(cmd, capture_output=True, text=True, cwd="/tmp", env=dict(os.environ, TMPDIR="/tmp"))
        if proc.returncode != 0:
            raise RuntimeError("%s under rocprofv3: %s" % (path, proc.stderr.strip()[-300:] or "exit %d" % proc.returncode))
        plan_ns, csr_ns = 0.0, 0.0
        for stats in glob.glob(os.path.join(out, "**", "*_kernel_stats.csv"), recursive=True):
            for row in csv.DictReader(open(stats)):
                name = row["Name"].replace("void ", "")
                if not name.startswith("cute_dev::"):
                    continue
                name = name[len("cute_dev::"):]
                if name.startswith(PLAN_KERNELS):
                    plan_ns += float(row["AverageNs"])
                elif name.startswith(CSR_KERNEL):
                    csr_ns += float(row["AverageNs"])
        if plan_ns <= 0:
            raise RuntimeError("%s under rocprofv3: no kernel of the plan in the trace" % path)
        return plan_ns / 1e3, csr_ns / 1e3
    finally:
        shutil.rmtree(out, ignore_errors=True)


def table(rows, rocprof=False):
    lines = ["matrix, N(feature size), cuTeSpMM GFLOPS, CSR GFLOPS"]
    for name, r in rows:
        t, t_csr = (r["kernel_us_rocprof"], r["csr_kernel_us_rocprof"]) if rocprof else (r["kernel_us"], r["csr_kernel_us"])
        flops = 2.0 * r["nnz"] * r["N"]
        csr = flops / (t_csr * 1e-6) / 1e9 if t_csr > 0 else float("nan")
        lines.append("%s, %d, %.2f, %.2f" % (name, r["N"], r["gflops"] if not rocprof else flops / (t * 1e-6) / 1e9, csr))
    return "\n".join(lines)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("roots", nargs="+", help="directories of .mtx files, single .mtx files, or gen:1..gen:5")
    ap.add_argument("--n", default="32,128,512")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--json", default=None, help="also write every per-launch record here")
    ap.add_argument("--cache-dir", default=None, help="keep converted matrices here and reuse them")
    ap.add_argument("--rocprof", action="store_true",
                    help="also run every (matrix, N) under rocprofv3 --kernel-trace --stats and make the table from the kernel durations")
    args = ap.parse_args(argv)
    widths = [int(x) for x in args.n.split(",")]
    jobs = []
    for root in args.roots:
        if os.path.isfile(root):
            jobs.append((os.path.basename(root)[:-4] if root.endswith(".mtx") else root, root))
        else:
            jobs.extend(find_matrices(root))
    rows, failures = [], []
    for i, (name, path) in enumerate(jobs):
        print("%d out of %d done" % (i, len(jobs)), file=sys.stderr)
        cache = None
        if args.cache_dir:
            os.makedirs(args.cache_dir, exist_ok=True)
            cache = os.path.join(args.cache_dir, name.replace(":", "_") + ".hrpb")
        try:
            got = run_one(path, widths, args.iters, cache)
            if args.rocprof:
                for r in got:
                    r["kernel_us_rocprof"], r["csr_kernel_us_rocprof"] = kernel_durations(path, r["N"], args.iters)
            rows.extend((name, r) for r in got)
        except RuntimeError as e:
            failures.append(str(e))
    print(table(rows, args.rocprof))
    for f in failures:
        print("FAILED", f, file=sys.stderr)
    if args.json:
        with open(args.json, "w") as f:
            json.dump([dict(r, name=name) for name, r in rows], f, indent=1)
    return 1 if failures else 0


if __name__ == "__main__":
    sys.exit(main())
