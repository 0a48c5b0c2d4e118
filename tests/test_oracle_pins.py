"""Pins the CPU oracle: each check here is a fact that does not come from the oracle's own
formula -- the reference's shipped table and inputs, a recorded print-out of the reference's
host code, closed forms, an independent decoder, float64 numpy/scipy."""
import json
import os

import numpy as np
import pytest

from helpers import (csr_from_dense, dense_from_csr, hrpb_check_invariants, hrpb_decode, random_csr)

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden")
REF_MATS = "/root/reference/ae_matrices"


def _meta():
    out = {}
    with open(os.path.join(GOLD, "meta.data")) as f:
        for line in f:
            p = line.strip().split(",")
            if len(p) == 4:
                out[p[0]] = tuple(int(x) for x in p[1:])
    return out


# ---------------------------------------------------------------- reader (IO.cu:10-87)
def test_reader_matches_reference_table_on_committed_fixture(orc):
    M, K, nnz, rp, cl, vl = orc.mtx_read(os.path.join(GOLD, "G67.mtx"))
    assert (M, K, nnz) == _meta()["G67"] == (10000, 10000, 40000)
    assert rp[-1] == nnz and (vl == 1.0).all()
    g = json.load(open(os.path.join(GOLD, "g67_block0.json")))
    assert cl[rp[0]:rp[1]].tolist() == g["row0_cols"]
    assert cl[rp[1]:rp[2]].tolist() == g["row1_cols"]


@pytest.mark.skipif(not os.path.isdir(REF_MATS), reason="reference matrices not mounted")
def test_reader_matches_reference_table_on_all_shipped_matrices(orc):
    meta = _meta()
    names = sorted(os.listdir(REF_MATS))
    assert len(names) >= 40
    for n in names:
        M, K, nnz, rp, cl, vl = orc.mtx_read(os.path.join(REF_MATS, n, n + ".mtx"))
        assert (M, K, nnz) == meta[n], n
        assert rp[-1] == nnz and cl.max() < K


def test_reader_closed_forms(orc, tmp_path):
    # general, real values, 5x7 -> padded 16x16; values forced to 1.0 (IO.cu:68); file order kept
    p = tmp_path / "g.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real general\n% c\n%c2\n5 7 4\n3 7 2.5\n1 2 -1e3\n3 1 4\n5 5 9\n")
    M, K, nnz, rp, cl, vl = orc.mtx_read(str(p))
    assert (M, K, nnz) == (16, 16, 4)
    assert rp.tolist() == [0, 1, 1, 3, 3, 4] + [4] * 11
    assert cl.tolist() == [1, 6, 0, 4] and (vl == 1.0).all()
    # symmetric pattern: off-diagonals mirrored, diagonal not; nnz = 2*offdiag + diag
    p = tmp_path / "s.mtx"
    p.write_text("%%MatrixMarket matrix coordinate pattern symmetric\n17 17 3\n2 1\n3 3\n17 2\n")
    M, K, nnz, rp, cl, vl = orc.mtx_read(str(p))
    assert (M, K, nnz) == (32, 32, 5)
    D = dense_from_csr(M, K, rp, cl, vl)
    E = np.zeros((32, 32))
    for r, c in [(1, 0), (0, 1), (2, 2), (16, 1), (1, 16)]:
        E[r, c] = 1
    assert (D == E).all()
    # "symmetric" is only looked for on the first line (IO.cu:16)
    p = tmp_path / "n.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real general\n% symmetric\n16 16 1\n2 1 1.0\n")
    assert orc.mtx_read(str(p))[2] == 1


# ---------------------------------------------------------------- HRPB (data.cu:94-335)
def test_hrpb_recorded_first_block_of_G67(orc):
    """Values printed by the reference's own host code for ae_matrices/G67."""
    g = json.load(open(os.path.join(GOLD, "g67_block0.json")))
    M, K, nnz, rp, cl, vl = orc.mtx_read(os.path.join(GOLD, "G67.mtx"))
    h = orc.hrpb_build(M, K, rp, cl, vl)
    assert (h["numRowPanels"], h["numBlocks"], h["numWords"]) == (g["numRowPanels"], g["numBlocks"], g["numWords"])
    assert h["blockedRowPtr"][:5].tolist() == g["blockedRowPtr_head"]
    assert h["sizePtr"][:4].tolist() == g["sizePtr_head"]
    b0 = g["block0"]
    rec = h["blocksData"][:128]
    assert h["activeCols"][:16].tolist() == b0["activeCols"]
    assert int(rec[0:2].view(np.uint64)[0]) == b0["next_addr"]
    assert int(rec[2:4].view(np.uint64)[0]) == int(b0["col_ptr"], 16)
    assert [int(x) for x in rec[4:8]] == [int(x, 16) for x in b0["nnz_words"]]
    assert rec[8:24].tolist() == b0["next_cols"]
    assert rec[24:26].view(np.uint16).tolist() == b0["prefix"]
    assert (rec[26], rec[27]) == (b0["fetch"], b0["next_fetch"])
    assert [int(x) for x in rec[28:36].view(np.uint64)] == [int(x, 16) for x in b0["bitmaps"]]
    v = rec[36:].view(np.float32)
    assert (v[:b0["num_values"]] == b0["value"]).all() and (v[b0["num_values"]:] == 0).all()


def _edge_cases():
    rng = np.random.default_rng(1234)
    cases = {}
    cases["random_sparse"] = (64, 96) + random_csr(rng, 64, 96, density=0.06)
    cases["empty_rows_and_panel"] = (64, 64) + random_csr(rng, 64, 64, row_nnz=lambda r: 0 if 16 <= r < 32 or r % 5 == 0 else 3)
    # exactly 16 active columns in panel 0, 17 in panel 1
    D = np.zeros((32, 48), np.float32)
    D[0:16, 8:24] = np.eye(16)
    D[16:32, 3:20] = (rng.random((16, 17)) < 0.4)
    D[16, 3:20] = 1
    cases["exactly16_and_17_cols"] = (32, 48) + csr_from_dense(D * rng.standard_normal(D.shape).astype(np.float32))
    # a fully dense 16x16 block: 256 values -> 3 chunks; plus one trailing column
    D = np.zeros((16, 32), np.float32)
    D[:, :16] = rng.standard_normal((16, 16))
    D[3, 20] = 2.0
    D[D == 0] = 0
    cases["dense_block_256"] = (16, 32) + csr_from_dense(D)
    cases["rectangular_wide"] = (16, 160) + random_csr(rng, 16, 160, density=0.3)
    cases["single_entry"] = (16, 16) + csr_from_dense(np.pad(np.ones((1, 1), np.float32), ((5, 10), (7, 8))))
    cases["dense_rows"] = (48, 64) + random_csr(rng, 48, 64, row_nnz=lambda r: 64 if r % 7 == 0 else 2)
    return cases


@pytest.mark.parametrize("name", sorted(_edge_cases().keys()))
def test_hrpb_invariants_and_dense_roundtrip(orc, name):
    M, K, rp, cl, vl = _edge_cases()[name]
    h = orc.hrpb_build(M, K, rp, cl, vl)
    hrpb_check_invariants(h, rp, cl)
    r, c, v = hrpb_decode(h)
    rows = np.repeat(np.arange(M), np.diff(rp.astype(np.int64)))
    assert (r == rows).all() and (c == cl).all() and (v == vl).all()


def test_hrpb_roundtrip_on_G67(orc):
    M, K, nnz, rp, cl, vl = orc.mtx_read(os.path.join(GOLD, "G67.mtx"))
    # MTX_READER keeps file order; the shipped inputs happen to be sorted within rows
    for r in range(M):
        assert (np.diff(cl[rp[r]:rp[r + 1]].astype(np.int64)) > 0).all()
    h = orc.hrpb_build(M, K, rp, cl, vl)
    hrpb_check_invariants(h, rp, cl)
    r, c, v = hrpb_decode(h)
    rows = np.repeat(np.arange(M), np.diff(rp.astype(np.int64)))
    assert (r == rows).all() and (c == cl).all()


def test_hrpb_rejects_bad_shape(orc):
    rp, cl, vl = random_csr(np.random.default_rng(0), 16, 16, density=0.2)
    with pytest.raises(ValueError):
        orc.hrpb_build(16, 24, rp, cl, vl)


# ---------------------------------------------------------------- partition (spmm.cu:776-812)
def test_partition_worked_examples(orc):
    # 4096 panels of 4 blocks (but 16352 in total: 32 short ones) on 864 resident blocks, one N tile:
    # waves = ceil(4096/864) = 5, avg = floor(16352/4096) = 3, loads = 2, ratio = 1 -> nothing is split
    nblk = np.full(4096, 4, np.uint32)
    nblk[:32] = 3
    brp = np.concatenate([[0], np.cumsum(nblk)]).astype(np.uint32)
    assert brp[-1] == 16352
    q = orc.partition(brp, 1, 864)
    assert len(q) == 4096 and (q[:, 3] == 0).all()
    assert (q[:, 0] == brp[:-1]).all() and (q[:, 1] == brp[1:]).all() and (q[:, 2] == np.arange(4096)).all()
    # one long panel: 300 blocks at avg 10, 5 waves -> loads 30, ratio 6, chunks of 50, atomic
    nblk = np.full(864 * 5, 10, np.uint32)
    nblk[7] = 300
    # keep the floor average at 10: remove the surplus elsewhere
    nblk[100:129] = 0
    brp = np.concatenate([[0], np.cumsum(nblk)]).astype(np.uint32)
    assert brp[-1] // len(nblk) == 10
    q = orc.partition(brp, 1, 864)
    mine = q[q[:, 2] == 7]
    assert len(mine) == 6 and (mine[:, 3] == 1).all()
    assert (mine[:, 1] - mine[:, 0] == 50).all() and mine[0, 0] == brp[7] and mine[-1, 1] == brp[8]
    assert not (q[:, 2] == 100).any()           # empty panels are skipped
    assert (q[q[:, 2] != 7][:, 3] == 0).all()


def test_partition_tiles_every_panel_exactly(orc):
    rng = np.random.default_rng(5)
    nblk = rng.integers(0, 40, 500).astype(np.uint32)
    nblk[rng.integers(0, 500, 5)] = rng.integers(200, 2000, 5)
    brp = np.concatenate([[0], np.cumsum(nblk)]).astype(np.uint32)
    for nbN, slots in [(1, 64), (2, 864), (4, 8192)]:
        q = orc.partition(brp, nbN, slots)
        for p in range(500):
            mine = q[q[:, 2] == p]
            if nblk[p] == 0:
                assert len(mine) == 0
                continue
            assert mine[0, 0] == brp[p] and mine[-1, 1] == brp[p + 1]
            assert (mine[1:, 0] == mine[:-1, 1]).all() and (mine[:, 1] > mine[:, 0]).all()
            assert (mine[:, 3] == (1 if len(mine) > 1 else 0)).all()


# ---------------------------------------------------------------- CPU SpMM (inc.h:71-83)
def test_spmm_against_float64_dense_and_scipy(orc):
    import scipy.sparse as sp
    rng = np.random.default_rng(7)
    M, K, N = 48, 80, 24
    rp, cl, vl = random_csr(rng, M, K, density=0.1)
    B = rng.standard_normal((K, N)).astype(np.float32)
    D = dense_from_csr(M, K, rp, cl, vl)
    exact = D @ B.astype(np.float64)
    bound = (np.abs(D) @ np.abs(B.astype(np.float64))) * (K * 2.0 ** -24) + 1e-30
    rows = np.repeat(np.arange(M), np.diff(rp.astype(np.int64))).astype(np.uint32)
    c_coo = orc.spmm_coo(rows, cl, vl, B, M)
    c_csr = orc.spmm_csr(rp, cl, vl, B)
    assert (c_coo == c_csr).all()                       # same sums in the same order
    assert (orc.spmm_coo(rows, cl, vl, B, M, inner_parallel=True) == c_coo).all()   # the reference's loop placement
    assert (np.abs(c_csr - exact) <= bound).all()
    s = sp.csr_matrix((vl.astype(np.float64), cl.astype(np.int64), rp.astype(np.int64)), shape=(M, K)) @ B.astype(np.float64)
    assert np.allclose(c_csr, s, rtol=1e-5, atol=1e-5)
    # a transposed operand, a dropped nonzero or a wrong sign would fail these exact cases:
    I = csr_from_dense(np.eye(K, dtype=np.float32))
    assert (orc.spmm_csr(*I, B) == B).all()
    ones = np.ones((K, 3), np.float32)
    rp1, cl1, vl1 = random_csr(rng, M, K, density=0.2, values="ones")
    assert (orc.spmm_csr(rp1, cl1, vl1, ones)[:, 0] == np.diff(rp1.astype(np.int64))).all()


def test_spmm_from_hrpb_stream_equals_csr(orc):
    rng = np.random.default_rng(11)
    M, K, N = 64, 96, 20
    rp, cl, vl = random_csr(rng, M, K, density=0.12, values="ints")
    B = rng.integers(-4, 5, (K, N)).astype(np.float32)   # every product and sum exact in fp32
    h = orc.hrpb_build(M, K, rp, cl, vl)
    assert (orc.spmm_hrpb(h, B) == orc.spmm_csr(rp, cl, vl, B)).all()
    assert (orc.spmm_hrpb(h, B) == dense_from_csr(M, K, rp, cl, vl) @ B.astype(np.float64)).all()


# ---------------------------------------------------------------- metric (inc.h:84-109)
def test_check_gemm_hand_cases(orc):
    ref = np.array([[1.0, 0.0], [-4.0, 2.0]], np.float32)
    out = np.array([[1.5, 123.0], [-3.0, 2.0]], np.float32)
    # element (0,1) has a zero reference and is skipped; max(0.5/1, 1/4, 0) = 0.5
    assert orc.check_gemm(ref, out) == pytest.approx(0.5)
    assert orc.check_gemm(ref, ref) == 0.0
    # not symmetric: the first argument is the trusted one
    assert orc.check_gemm(out, ref) == pytest.approx(max(0.5 / 1.5, 123.0 / 123.0, 1.0 / 3.0))
