"""Format construction on the device (cute_hrpb_upload_device_csr and the late builds inside a plan) against the
host builders: the brick tiles must equal cute_hrpb_retile(cute_hrpb_build(..)) and the quad lists cute_quad_pack(..)
word for word -- index, bitmap and value content -- on the edge cases of the format tests, on the reference's G67
and on the five benchmark configurations; products through device-built layouts are checked against the oracle."""
import os

import numpy as np
import pytest

from helpers import random_csr
from test_oracle_pins import GOLD, _edge_cases

pytestmark = pytest.mark.gpu

BERR = 2e-6


def _to_gpu(torch, rp, cl, vl):
    return (torch.from_numpy(rp.astype(np.int64).astype(np.int32)).cuda(), torch.from_numpy(cl.view(np.int32).copy()).cuda(),
            torch.from_numpy(vl.copy()).cuda())


def _check_bricks(cs, got, M, K, rp, cl, vl):
    want = cs.HRPB(M, K, rp, cl, vl).retile()
    assert (got["blockedRowPtr"] == want["blockedRowPtr"]).all()
    assert got["hdr"].shape == want["hdr"].shape and (got["hdr"] == want["hdr"]).all()
    assert got["tileVals"].tobytes() == want["vals"].tobytes()


def _check_quads(cs, got, M, rp, cl, vl):
    want = cs.quad_pack(M, rp, cl, vl, strips=got["rowsPerList"] == 4)
    assert (got["groupPtr"] == want["groupPtr"]).all()
    assert got["recs"].shape == want["recs"].shape and (got["recs"] == want["recs"]).all()
    assert got["quadVals"].tobytes() == want["packed"].tobytes()


def _both_layouts(cs, torch, M, K, rp, cl, vl, quad_layout):
    """Device-built handle with both layouts forced into existence (the upload builds one, a plan the other)."""
    d = cs.DeviceHRPB(M, K, *_to_gpu(torch, rp, cl, vl), quad_layout=quad_layout)
    cs.SPMM_TC(d, 16, path=cs.PATH_BRICK, mfma_shape=1)
    cs.SPMM_TC(d, 16, path=cs.PATH_BRICK, mfma_shape=2)
    return d


@pytest.mark.parametrize("name", sorted(_edge_cases().keys()))
@pytest.mark.parametrize("quad_layout", [1, 2])
def test_edge_cases_equal_host_built(cs, orc, torch_cuda, name, quad_layout):
    M, K, rp, cl, vl = _edge_cases()[name]
    d = _both_layouts(cs, torch_cuda, M, K, rp, cl, vl, quad_layout)
    got = d.layouts()
    _check_bricks(cs, got, M, K, rp, cl, vl)
    _check_quads(cs, got, M, rp, cl, vl)
    assert got["rowsPerList"] == (16 if quad_layout == 1 else 4)
    # and a product through each device-built layout
    N = 48
    B = np.random.default_rng(7).standard_normal((K, N)).astype(np.float32)
    ref = orc.spmm_csr(rp, cl, vl, B)
    dB = torch_cuda.from_numpy(B).cuda()
    for kw in (dict(path=cs.PATH_BRICK, mfma_shape=1), dict(path=cs.PATH_BRICK, mfma_shape=2), dict()):
        dC = torch_cuda.full((M, N), float("nan"), device="cuda")
        cs.SPMM_TC(d, N, **kw).run(dB, dC)
        torch_cuda.cuda.synchronize()
        assert cs.backward_error(rp, cl, vl, B, ref, dC.cpu().numpy()) <= BERR, (name, kw)


def test_explicit_zeros_and_empty_matrix(cs, torch_cuda):
    """An explicit zero keeps its bitmap bit in the brick tiles and is an empty slot of the quad lists, as on the host;
    a matrix without entries builds empty layouts."""
    rng = np.random.default_rng(5)
    M, K = 64, 80
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 9)
    vl[::3] = 0.0
    vl[1::7] = -0.0
    for quad_layout in (1, 2):
        got = _both_layouts(cs, torch_cuda, M, K, rp, cl, vl, quad_layout).layouts()
        _check_bricks(cs, got, M, K, rp, cl, vl)
        _check_quads(cs, got, M, rp, cl, vl)
    empty = cs.DeviceHRPB(32, 32, *_to_gpu(torch_cuda, np.zeros(33, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32)))
    g = empty.layouts()
    assert g["hdr"].size == 0 and g["recs"].size == 0 and (g["blockedRowPtr"] == 0).all()
    dC = torch_cuda.full((32, 8), float("nan"), device="cuda")
    cs.SPMM_TC(empty, 8).run(torch_cuda.ones((32, 8), device="cuda"), dC)
    torch_cuda.cuda.synchronize()
    assert (dC == 0).all().item()


def test_preconditions_are_checked_on_the_device(cs, torch_cuda):
    rng = np.random.default_rng(6)
    M, K = 32, 48
    rp, cl, vl = random_csr(rng, M, K, row_nnz=lambda r: 5)
    bad = cl.copy()
    s = int(rp[3])
    bad[s], bad[s + 1] = bad[s + 1], bad[s]                          # one row out of order
    with pytest.raises(cs.CuteError) as e:
        cs.DeviceHRPB(M, K, *_to_gpu(torch_cuda, rp, bad, vl))
    assert e.value.status == -3
    dup = cl.copy()
    dup[s + 1] = dup[s]                                              # a duplicate column
    with pytest.raises(cs.CuteError) as e:
        cs.DeviceHRPB(M, K, *_to_gpu(torch_cuda, rp, dup, vl))
    assert e.value.status == -3
    far = cl.copy()
    far[int(rp[8]) - 1] = K                                          # a column outside the matrix (last of its row: still sorted)
    with pytest.raises(cs.CuteError) as e:
        cs.DeviceHRPB(M, K, *_to_gpu(torch_cuda, rp, far, vl))
    assert e.value.status == -4
    broken = rp.copy()
    broken[5] = broken[6] + 1                                        # row pointers that do not ascend
    with pytest.raises(cs.CuteError) as e:
        cs.DeviceHRPB(M, K, *_to_gpu(torch_cuda, broken, cl, vl))
    assert e.value.status == -4
    with pytest.raises(cs.CuteError) as e:
        cs.DeviceHRPB(M + 8, K, *_to_gpu(torch_cuda, np.concatenate([rp, np.full(8, rp[-1], np.uint32)]), cl, vl))
    assert e.value.status == -2                                      # M not a multiple of 16


def test_g67_equal_host_built(cs, orc, torch_cuda):
    r = cs.MTX_READER(os.path.join(GOLD, "G67.mtx"))
    for quad_layout in (1, 2):
        got = _both_layouts(cs, torch_cuda, r.M, r.K, r.rowPtr, r.cols, r.vals, quad_layout).layouts()
        _check_bricks(cs, got, r.M, r.K, r.rowPtr, r.cols, r.vals)
        _check_quads(cs, got, r.M, r.rowPtr, r.cols, r.vals)


@pytest.mark.parametrize("config", [1, 2, 3, 4, 5])
def test_benchmark_configs_equal_host_built(cs, orc, torch_cuda, config):
    """Full size for every configuration; the layout the library would choose for the quad lists (lockstep, or strips
    for the R-MAT graph), both MFMA layouts, word for word; then the default plan's product against the oracle."""
    A = cs.gen_config(config)
    d = cs.DeviceHRPB(A.M, A.K, *_to_gpu(torch_cuda, A.rowPtr, A.cols, A.vals))
    host = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    host.upload()
    # the same default choice of layout as the host path makes, before any plan asks for another
    first = d.layouts()
    want_first = host.device_layouts()
    assert first["rowsPerList"] == want_first["rowsPerList"]
    assert first["hdr"].shape == want_first["hdr"].shape and first["recs"].shape == want_first["recs"].shape
    cs.SPMM_TC(d, 16, path=cs.PATH_BRICK, mfma_shape=1)
    cs.SPMM_TC(d, 16, path=cs.PATH_BRICK, mfma_shape=2)
    got = d.layouts()
    _check_bricks(cs, got, A.M, A.K, A.rowPtr, A.cols, A.vals)
    _check_quads(cs, got, A.M, A.rowPtr, A.cols, A.vals)
    del got, first, want_first
    N = cs.CONFIGS[config]["N"] if config != 5 else 32
    B = cs.gen_dense(11, A.K, N, 2)
    ref = orc.spmm_csr(A.rowPtr, A.cols, A.vals, B)
    dB = torch_cuda.from_numpy(B).cuda()
    dC = torch_cuda.full((A.M, N), float("nan"), device="cuda")
    plan = cs.SPMM_TC(d, N)
    plan.run(dB, dC)
    torch_cuda.cuda.synchronize()
    out = dC.cpu().numpy()
    assert cs.backward_error(A.rowPtr, A.cols, A.vals, B, ref, out) <= (BERR if config != 4 else 6e-6)
    # the host-built handle gives the same bits through the same plan
    dC2 = torch_cuda.full((A.M, N), float("nan"), device="cuda")
    plan2 = cs.SPMM_TC(host, N)
    assert plan2.kernel_name == plan.kernel_name
    plan2.run(dB, dC2)
    torch_cuda.cuda.synchronize()
    assert torch_cuda.equal(dC, dC2)
