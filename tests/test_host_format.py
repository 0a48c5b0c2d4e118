"""Host side of libcutespmm through its C ABI against the oracle: bit-exact for every
index, bitmap and value word; also the ABI surface, error behaviour and the re-tile
bijection.  No GPU needed."""
import ctypes as C
import os
import re

import numpy as np
import scipy.sparse
import pytest

from helpers import dense_from_csr, hrpb_check_invariants, random_csr
from test_oracle_pins import _edge_cases, GOLD, REF_MATS

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KEYS = ["blockedRowPtr", "activeCols", "sizePtr", "blocksData"]


def _same(h, o):
    for k in KEYS:
        a, b = getattr(h, k), o[k]
        assert a.dtype == b.dtype and a.shape == b.shape and (a == b).all(), k


# ---------------------------------------------------------------- ABI surface
def test_library_exports_every_declared_symbol(cs):
    lib = cs.load_library()
    text = open(os.path.join(ROOT, "include", "cutespmm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(cute_[a-z0-9_]+)\s*\(", text)))
    assert len(declared) >= 25
    for name in declared:
        assert hasattr(lib, name), name
    assert sorted(cs.ABI_SYMBOLS) == declared


def test_struct_sizes_match_header(cs):
    # layout the C header implies on LP64
    assert C.sizeof(cs.cute_csr) == 40
    assert C.sizeof(cs.cute_hrpb_host) == 88
    assert C.sizeof(cs.cute_hrpb_tiled) == 48
    assert C.sizeof(cs.cute_tunables) == 48
    assert C.sizeof(cs.cute_plan_info) == 68


def test_status_strings(cs):
    lib = cs.load_library()
    assert lib.cute_status_string(0) == b"ok"
    assert b"unsorted" in lib.cute_status_string(-3)


# ---------------------------------------------------------------- reader
def test_reader_equals_oracle_on_fixture(cs, orc):
    path = os.path.join(GOLD, "G67.mtx")
    r = cs.MTX_READER(path)
    M, K, nnz, rp, cl, vl = orc.mtx_read(path)
    assert (r.M, r.K, r.nnz) == (M, K, nnz)
    assert (r.rowPtr == rp).all() and (r.cols == cl).all() and (r.vals == vl).all()


@pytest.mark.skipif(not os.path.isdir(REF_MATS), reason="reference matrices not mounted")
def test_reader_equals_oracle_on_all_shipped_matrices(cs, orc):
    for n in sorted(os.listdir(REF_MATS)):
        path = os.path.join(REF_MATS, n, n + ".mtx")
        r = cs.MTX_READER(path)
        M, K, nnz, rp, cl, vl = orc.mtx_read(path)
        assert (r.M, r.K, r.nnz) == (M, K, nnz), n
        assert (r.rowPtr == rp).all() and (r.cols == cl).all() and (r.vals == vl).all(), n


def test_reader_flags_and_errors(cs, tmp_path):
    p = tmp_path / "v.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real symmetric\n4 4 3\n2 1 2.5\n3 3 -7\n4 2 1e-2\n\n")
    ones = cs.MTX_READER(str(p))
    assert (ones.vals == 1.0).all() and ones.nnz == 5 and (ones.M, ones.K) == (16, 16)
    kept = cs.MTX_READER(str(p), keep_values=True)
    D = dense_from_csr(16, 16, kept.rowPtr, kept.cols, kept.vals)
    assert D[1, 0] == D[0, 1] == 2.5 and D[2, 2] == -7 and D[3, 1] == D[1, 3] == np.float32(1e-2)
    with pytest.raises(cs.CuteError) as e:
        cs.MTX_READER(str(tmp_path / "missing.mtx"))
    assert e.value.status == -1
    q = tmp_path / "bad.mtx"
    q.write_text("%%MatrixMarket matrix coordinate real general\n4 4 1\n9 1 1.0\n")
    with pytest.raises(cs.CuteError) as e:
        cs.MTX_READER(str(q))
    assert e.value.status == -4
    q.write_text("%%MatrixMarket matrix coordinate real general\n4 4 1\nx y 1.0\n")
    with pytest.raises(cs.CuteError) as e:
        cs.MTX_READER(str(q))
    assert e.value.status == -1


# ---------------------------------------------------------------- builder
@pytest.mark.parametrize("name", sorted(_edge_cases().keys()))
def test_builder_equals_oracle_on_edge_cases(cs, orc, name):
    M, K, rp, cl, vl = _edge_cases()[name]
    h = cs.HRPB(M, K, rp, cl, vl)
    _same(h, orc.hrpb_build(M, K, rp, cl, vl))
    hrpb_check_invariants(h.as_dict(), rp, cl)


@pytest.mark.parametrize("seed", range(6))
def test_builder_equals_oracle_on_random_matrices(cs, orc, seed):
    rng = np.random.default_rng(100 + seed)
    M = 16 * int(rng.integers(1, 40))
    K = 16 * int(rng.integers(1, 40))
    dens = float(rng.choice([0.002, 0.02, 0.1, 0.5]))
    rp, cl, vl = random_csr(rng, M, K, density=dens)
    h = cs.HRPB(M, K, rp, cl, vl)
    o = orc.hrpb_build(M, K, rp, cl, vl)
    _same(h, o)
    assert h.numNNZ == len(cl)


def test_builder_equals_oracle_on_fixture_and_configs(cs, orc):
    r = cs.MTX_READER(os.path.join(GOLD, "G67.mtx"))
    _same(cs.HRPB(r.M, r.K, r.rowPtr, r.cols, r.vals), orc.hrpb_build(r.M, r.K, r.rowPtr, r.cols, r.vals))
    for cfg, scale in [(1, 1.0), (2, 0.25), (3, 0.1), (4, 1 / 16.0), (5, 1 / 64.0)]:
        A = cs.gen_config(cfg, scale)
        h = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
        _same(h, orc.hrpb_build(A.M, A.K, A.rowPtr, A.cols, A.vals))


def test_builder_thread_count_does_not_change_a_word(cs, monkeypatch):
    A = cs.gen_config(4, 1 / 16.0)
    monkeypatch.setenv("CUTE_NUM_THREADS", "1")
    h1 = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    monkeypatch.setenv("CUTE_NUM_THREADS", "7")
    h7 = cs.HRPB(A.M, A.K, A.rowPtr, A.cols, A.vals)
    for k in KEYS:
        assert (getattr(h1, k) == getattr(h7, k)).all()
    assert h1.num_bricks == h7.num_bricks


def test_builder_rejects_what_the_reference_silently_assumes(cs):
    rng = np.random.default_rng(3)
    rp, cl, vl = random_csr(rng, 32, 32, density=0.2)
    with pytest.raises(cs.CuteError) as e:
        cs.HRPB(32, 40, rp, cl, vl)
    assert e.value.status == -2
    bad = cl.copy()
    r = int(np.argmax(np.diff(rp.astype(np.int64)) >= 2))
    s = int(rp[r])
    bad[s], bad[s + 1] = bad[s + 1], bad[s]
    with pytest.raises(cs.CuteError) as e:
        cs.HRPB(32, 32, rp, bad, vl)
    assert e.value.status == -3
    dup = cl.copy()
    dup[s + 1] = dup[s]
    with pytest.raises(cs.CuteError) as e:
        cs.HRPB(32, 32, rp, dup, vl)
    assert e.value.status == -3
    big = cl.copy()
    big[-1] = 32
    with pytest.raises(cs.CuteError) as e:
        cs.HRPB(32, 32, rp, big, vl)
    assert e.value.status == -4


def test_sort_rows_makes_file_order_input_valid(cs, tmp_path):
    p = tmp_path / "u.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real general\n3 20 4\n1 9 1\n1 2 2\n1 17 3\n2 5 4\n")
    r = cs.MTX_READER(str(p), keep_values=True)
    assert r.cols[:3].tolist() == [8, 1, 16]
    r.sort_rows()
    assert r.cols[:3].tolist() == [1, 8, 16] and r.vals[:3].tolist() == [2.0, 1.0, 3.0]
    cs.HRPB(r.M, r.K, r.rowPtr, r.cols, r.vals)


# ---------------------------------------------------------------- re-tile bijection
@pytest.mark.parametrize("name", sorted(_edge_cases().keys()))
def test_retile_is_a_bijection(cs, name):
    M, K, rp, cl, vl = _edge_cases()[name]
    h = cs.HRPB(M, K, rp, cl, vl)
    back = h.retile_roundtrip()
    for k in KEYS:
        assert (back[k] == getattr(h, k)).all(), k
    assert back["nnz"] == len(cl) and back["numBricks"] == h.num_bricks


def test_tiled_layout_is_what_the_kernel_reads(cs):
    """Lane L of a wavefront owns A[row L%16][k L/16] of a 16x16x4 fp32 MFMA: tiled bit L,
    value rank = popcount of lower bits, column word k*4+brick."""
    rng = np.random.default_rng(9)
    M, K = 32, 64
    rp, cl, vl = random_csr(rng, M, K, density=0.15)
    h = cs.HRPB(M, K, rp, cl, vl)
    t = h.retile()
    D = dense_from_csr(M, K, rp, cl, vl)
    rebuilt = np.zeros_like(D)
    for p in range(h.numRowPanels):
        for b in range(int(h.blockedRowPtr[p]), int(h.blockedRowPtr[p + 1])):
            hd = t["hdr"][b]
            bms = hd[16:24].view(np.uint64)
            assert (hd[29:32] == 0).all()
            n = 0
            for j in range(4):
                rank = 0
                for lane in range(64):
                    if (int(bms[j]) >> lane) & 1:
                        row, k = lane % 16, lane // 16
                        col = int(hd[k * 4 + j])
                        rebuilt[p * 16 + row, col] += t["vals"][int(hd[24 + j]) + rank]
                        rank += 1
                n += rank
            assert hd[28] == n
    assert (rebuilt == D).all()


# ---------------------------------------------------------------- partition + metrics
def test_partition_equals_oracle(cs, orc):
    rng = np.random.default_rng(21)
    for trial in range(8):
        P = int(rng.integers(1, 600))
        nblk = rng.integers(0, 30, P).astype(np.uint32)
        if P > 3:
            nblk[rng.integers(0, P, 3)] = rng.integers(100, 3000, 3)
        if nblk.sum() == 0:
            nblk[0] = 1
        brp = np.concatenate([[0], np.cumsum(nblk)]).astype(np.uint32)
        for nbN, slots in [(1, 864), (2, 1024), (4, 8192), (1, 7)]:
            assert (cs.partition(brp, nbN, slots) == orc.partition(brp, nbN, slots)).all()


def test_metric_equals_oracle(cs, orc):
    rng = np.random.default_rng(2)
    ref = rng.standard_normal((37, 19)).astype(np.float32)
    ref[rng.random(ref.shape) < 0.2] = 0
    out = ref + 1e-4 * rng.standard_normal(ref.shape).astype(np.float32)
    assert cs.check_gemm_correctness_coo(ref, out) == orc.check_gemm(ref, out)
    assert cs.check_gemm_correctness_coo(ref, ref) == 0.0


def test_backward_error_hand_case(cs):
    rp = np.array([0, 2, 2], np.uint32)
    cl = np.array([0, 1], np.uint32)
    vl = np.array([2.0, -3.0], np.float32)
    B = np.array([[1.0, 4.0], [1.0, -2.0]], np.float32)
    ref = np.array([[-1.0, 14.0], [0.0, 0.0]], np.float32)
    out = ref.copy()
    out[0, 0] += 0.5          # scale |2||1| + |3||1| = 5  -> 0.1
    out[0, 1] -= 1.4          # scale |2||4| + |3||2| = 14 -> 0.1
    assert cs.backward_error(rp, cl, vl, B, ref, out) == pytest.approx(0.1, rel=1e-6)
    out[1, 1] = 1e-3          # empty row: any difference is infinitely large relative to a zero scale
    assert cs.backward_error(rp, cl, vl, B, ref, out) == float("inf")


# ---------------------------------------------------------------- generators
def test_generators_match_their_specification(cs):
    A = cs.gen_config(1)
    assert (A.M, A.K, A.nnz) == (4096, 4096, 65536) and (np.diff(A.rowPtr.astype(np.int64)) == 16).all()
    assert np.abs(A.vals).max() <= 1.0
    S = cs.gen_config(2)
    assert (S.M, S.nnz) == (65536, 766 * 766)
    def sparse(m):
        return scipy.sparse.csr_matrix((m.vals.astype(np.float64), m.cols.astype(np.int64), m.rowPtr.astype(np.int64)), shape=(m.M, m.K))

    def pattern_is_symmetric(a):
        p = (a != 0).astype(np.int8)
        return (p != p.T).nnz == 0

    D = sparse(cs.gen_matrix(2, 5, 64))
    assert D.shape == (64 * 64, 64 * 64) and (np.abs(D.diagonal() - 8) <= 0.01).all()
    off = (D - scipy.sparse.diags(D.diagonal())).tocsr()
    off.eliminate_zeros()
    assert (np.abs(off.data + 1) <= 0.01).all() and pattern_is_symmetric(off)
    F = cs.gen_config(3, 0.05)
    Df = sparse(F)
    assert pattern_is_symmetric(Df)
    assert (np.abs(Df.diagonal()) > np.asarray(abs(Df).sum(1)).ravel() - np.abs(Df.diagonal())).all()
    R = cs.gen_config(4, 1 / 64.0)
    Dr = sparse(R)
    assert (Dr.data != 0).all()
    deg = np.diff(Dr.indptr)
    assert (Dr.diagonal() > 0).all() and pattern_is_symmetric(Dr)
    i, j = Dr.nonzero()
    assert np.allclose(np.asarray(Dr[i, j]).ravel(), 1 / np.sqrt(deg[i] * deg[j]), rtol=1e-6)
    Bd = cs.gen_config(5, 1 / 256.0)
    assert (np.diff(Bd.rowPtr.astype(np.int64)) == 32).all()
    rows = np.repeat(np.arange(Bd.M), 32)
    assert (np.abs(Bd.cols.astype(np.int64) - rows) <= 2048).all()
    for m in (A, S, F, R, Bd):
        for r in range(0, m.M, max(1, m.M // 200)):
            assert (np.diff(m.cols[m.rowPtr[r]:m.rowPtr[r + 1]].astype(np.int64)) > 0).all()


def test_generators_are_deterministic_and_thread_independent(cs, monkeypatch):
    monkeypatch.setenv("CUTE_NUM_THREADS", "1")
    a = cs.gen_config(5, 1 / 256.0)
    b1 = cs.gen_dense(77, 100, 33, 2)
    monkeypatch.setenv("CUTE_NUM_THREADS", "5")
    b = cs.gen_config(5, 1 / 256.0)
    b5 = cs.gen_dense(77, 100, 33, 2)
    assert (a.cols == b.cols).all() and (a.vals == b.vals).all() and (b1 == b5).all()
    assert abs(float(b1.mean())) < 0.1 and abs(float(b1.std()) - 1.0) < 0.1
    u = cs.gen_dense(78, 1000, 10, 0)
    assert 0.0 <= u.min() and u.max() < 1.0 and abs(float(u.mean()) - 0.5) < 0.02
