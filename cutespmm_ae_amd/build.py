"""Builds libcutespmm.so (gfx950 only) and the C++ driver with hipcc, in-tree."""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libcutespmm.so")
DRIVER = os.path.join(HERE, "run_cute")
PROBE = os.path.join(HERE, "membw_probe")

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

# -packed-fp32-ops is switched off for device code: the compiler then never forms
# v_pk_{add,mul,fma}_f32 from scalar float code.
# -amdgpu-kernarg-preload-count: the first kernel arguments arrive in scalar registers when a wavefront starts
# instead of being fetched by its first instructions (gfx940 and later; the compiler keeps a prologue that
# fetches them for firmware without the feature).  Every wavefront's first dependent loads start that much
# earlier: 2.6 % on the headline launch.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-mllvm", "-amdgpu-kernarg-preload-count=16"]
COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
          "-pthread"]

LIB_SOURCES = ["host_format.cpp", "host_formats2.cpp", "host_quad.cpp", "host_cache.cpp", "gen.cpp", "device.hip"]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_library():
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    for s in LIB_SOURCES:
        path = os.path.join(CSRC, s)
        obj = os.path.join(objdir, s + ".o")
        if s.endswith(".cpp"):               # host-only translation units
            _run([HIPCC, "-x", "c++", path, "-c", "-o", obj] + COMMON)
        else:
            _run([HIPCC, "-x", "hip", path, "-c", "-o", obj] + COMMON + DEVICE_FLAGS)
        objs.append(obj)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-pthread", "-o", LIB] + objs)
    return LIB


def build_driver():
    src = os.path.join(CSRC, "run_cute.cpp")
    if not os.path.exists(src):
        return None
    rocm = os.path.dirname(os.path.dirname(os.path.realpath(HIPCC)))
    _run([HIPCC, "-x", "c++", src, "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(rocm, "include")] + COMMON +
         ["-I", os.path.join(ROOT, "include"), "-o", DRIVER, "-L", HERE, "-lcutespmm",
          "-L", os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath,$ORIGIN"])
    return DRIVER


def build_probe():
    """The memory-pattern microbenchmark (a stand-alone HIP program; nothing of the library links to it)."""
    src = os.path.join(CSRC, "membw_probe.hip")
    _run([HIPCC, "-x", "hip", src, "-o", PROBE] + COMMON + DEVICE_FLAGS)
    return PROBE


def build_all():
    build_library()
    build_driver()
    build_probe()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
