"""The C++ face of the boundary (include/cutespmm.hpp): a host-only program written against the
reference's class names is compiled with g++, linked with libcutespmm.so and run."""
import os
import shutil
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_reference_style_host_program(cs, orc, tmp_path):
    exe = str(tmp_path / "host_api_check")
    libdir = os.path.join(ROOT, "cutespmm_ae_amd")
    subprocess.check_call(["g++", "-std=c++17", "-O1", os.path.join(ROOT, "tests", "cpp", "host_api_check.cpp"),
                           "-I", os.path.join(ROOT, "include"), "-L", libdir, "-lcutespmm",
                           "-Wl,-rpath," + libdir, "-o", exe])
    mtx = os.path.join(ROOT, "tests", "golden", "G67.mtx")
    out = subprocess.run([exe, mtx, str(tmp_path / "g67.hrpb")], check=True, capture_output=True, text=True).stdout.split()
    got = dict(kv.split("=") for kv in out)
    M, K, nnz, rp, cl, vl = orc.mtx_read(mtx)
    h = orc.hrpb_build(M, K, rp, cl, vl)
    assert (int(got["M"]), int(got["K"]), int(got["nnz"])) == (M, K, nnz)
    assert (int(got["panels"]), int(got["blocks"]), int(got["words"])) == (h["numRowPanels"], h["numBlocks"], h["numWords"])
    assert got["bcsr"] == "8750" and got["tiles"] == "4325" and got["heavy"] == "1875/33800" and got["light"] == "2450/6200"
    assert got["densediff"] == "0" and got["grown"] == "2,1" and got["cache"] == "0"
    assert got["registry"] == "111" and got["coo"] == "1" and got["fit"] == "01"
    dy, dx, _, r, c, v = orc.coo_read(mtx)
    rp2, cl2, _ = orc.coo_to_csr(dy, r, c, v)
    want = orc.get_stats(dy, dx, rp2, cl2, 16)
    assert [np.float32(x) for x in got["stats"].split(",")] == want.tolist()
    assert [np.float32(x) for x in got["anxs"].split(",")] == [np.float32(orc.get_anxs(dy, rp2, cl2, 16, a)) for a in (True, False)]
