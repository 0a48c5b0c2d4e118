"""The library's host sources under the compiler's sanitizers: tests/cpp/host_sanitize_check.cpp walks the
readers, the format builders, the cache file, the generators and the second API family on the reference's G67
matrix, on generated matrices, on hand-made shapes (empty, one entry, a full row, a full column, a dense panel),
on damaged cache files and on malformed MatrixMarket files; it is compiled with the five host translation units
once with AddressSanitizer + UndefinedBehaviorSanitizer and once with ThreadSanitizer (the builders run on all
host threads).  The reference has no such target; its builders hold two latent faults of exactly this kind
(data.cu:312-317 writes work_space[0] of an empty array when a thread's share holds no block;
inc/prepareBlkEll.hpp:100,155 count under `omp parallel for` without synchronisation).  No GPU call is made."""
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "cutespmm_ae_amd", "csrc")
HOST_UNITS = ["host_format.cpp", "host_formats2.cpp", "host_quad.cpp", "host_cache.cpp", "gen.cpp"]
COMMON = ["-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer", "-pthread", "-ffp-contract=off", "-Wno-unknown-pragmas", "-I", os.path.join(ROOT, "include")]
FLAVOURS = {
    # the address sanitizer's runtime is linked statically: a dynamic one insists on being the first library loaded
    "address+undefined": (["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined"], ["-static-libasan"]),
    "thread": (["-fsanitize=thread"], []),
}


def build(flavour, outdir):
    flags, link = FLAVOURS[flavour]
    sources = [os.path.join(CSRC, u) for u in HOST_UNITS] + [os.path.join(ROOT, "tests", "cpp", "host_sanitize_check.cpp")]
    objects = [os.path.join(outdir, os.path.basename(s) + ".o") for s in sources]

    def compile_one(pair):
        src, obj = pair
        subprocess.run(["g++", "-c", src, "-o", obj] + COMMON + flags, check=True, capture_output=True, text=True)

    with ThreadPoolExecutor(max_workers=3) as pool:
        list(pool.map(compile_one, zip(sources, objects)))
    exe = os.path.join(outdir, "host_sanitize_check")
    subprocess.run(["g++", "-o", exe] + objects + COMMON + flags + link, check=True, capture_output=True, text=True)
    return exe


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
@pytest.mark.parametrize("flavour", sorted(FLAVOURS))
def test_host_sources_under_sanitizers(flavour, tmp_path):
    outdir = str(tmp_path / "build")
    work = str(tmp_path / "files")
    os.makedirs(outdir)
    os.makedirs(work)
    try:
        exe = build(flavour, outdir)
    except subprocess.CalledProcessError as e:
        if "sanitize" in (e.stderr or "") and ("cannot find" in e.stderr or "unrecognized" in e.stderr):
            pytest.skip("this g++ has no %s sanitizer runtime" % flavour)
        raise AssertionError(e.stderr[-2000:])
    env = dict(os.environ, CUTE_NUM_THREADS="8", ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", TSAN_OPTIONS="halt_on_error=1")
    run = subprocess.run([exe, os.path.join(ROOT, "tests", "golden", "G67.mtx"), work], capture_output=True, text=True, env=env,
                         timeout=300)
    assert run.returncode == 0, (run.stdout + run.stderr)[-3000:]
    assert "0 failures" in run.stdout
    assert "runtime error" not in run.stderr and "Sanitizer" not in run.stderr, run.stderr[-3000:]
