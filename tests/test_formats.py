"""Second host API family (SparseCoo, CSR_Matrix, Blocked-ELL preprocess, Splitter, block
classifier, double-precision CPU SpMM): oracle pins first, then product against oracle.
No GPU needed."""
import json
import os

import numpy as np
import pytest

from helpers import dense_from_csr, random_csr
from test_oracle_pins import GOLD

G67 = os.path.join(GOLD, "G67.mtx")


def _csr_case(seed, M=70, K=90, density=0.08):
    rng = np.random.default_rng(seed)
    rp, cl, vl = random_csr(rng, M, K, density=density)
    return M, K, rp.astype(np.int32), cl.astype(np.int32), vl


# ---------------------------------------------------------------- oracle pins
def test_oracle_coo_reader(orc, tmp_path):
    import scipy.io
    dy, dx, nnz, r, c, v = orc.coo_read(G67)
    m = scipy.io.mmread(G67).tocsr()          # independent reader: symmetric expansion, values kept
    m.sort_indices()
    assert (dy, dx, nnz) == (m.shape[0], m.shape[1], m.nnz)
    rows = np.repeat(np.arange(m.shape[0]), np.diff(m.indptr))
    assert (r == rows).all() and (c == m.indices).all() and (v == m.data.astype(np.float32)).all()
    # the other loader's pattern, once sorted, is the same set of positions
    M, K, nnz2, rp, cl, _ = orc.mtx_read(G67)
    assert nnz2 == nnz and (np.diff(rp.astype(np.int64))[:dy] == np.bincount(r, minlength=dy)).all()
    # pattern file: value defaults to 1.0; general file keeps order-independent sorting
    p = tmp_path / "p.mtx"
    p.write_text("%%MatrixMarket matrix coordinate pattern general\n% c\n3 5 3\n3 1\n1 4\n1 2\n")
    dy, dx, nnz, r, c, v = orc.coo_read(str(p))
    assert (dy, dx, nnz) == (3, 5, 3) and r.tolist() == [0, 0, 2] and c.tolist() == [1, 3, 0] and (v == 1).all()


def test_oracle_coo2csr_bcsr_and_counts(orc):
    g = json.load(open(os.path.join(GOLD, "g67_block0.json")))
    dy, dx, nnz, r, c, v = orc.coo_read(G67)
    rp, cl, vl = orc.coo_to_csr(dy, r, c, v)
    assert rp[-1] == nnz and (cl == c).all()
    assert orc.count_blocks(dy, dx, rp, cl, 16, 4) == g["csr_count_blocks_16x4"]      # value recorded from the reference
    M, K, rp, cl, vl = _csr_case(1, 64, 96)
    D = dense_from_csr(M, K, rp, cl, vl)
    for R, Cc in [(16, 4), (8, 8), (4, 32)]:
        brute = sum(1 for i in range(M // R) for j in range(K // Cc) if np.any(D[i * R:(i + 1) * R, j * Cc:(j + 1) * Cc]))
        assert orc.count_blocks(M, K, rp, cl, R, Cc) == brute
        brp, bc, bv = orc.to_bcsr(M, K, rp, cl, vl, R, Cc)
        rebuilt = np.zeros_like(D)
        for i in range(M // R):
            for b in range(brp[i], brp[i + 1]):
                rebuilt[i * R:(i + 1) * R, bc[b] * Cc:(bc[b] + 1) * Cc] += bv[b * R * Cc:(b + 1) * R * Cc].reshape(R, Cc)
        assert brp[-1] == brute and (rebuilt == D.astype(np.float32)).all()


def test_oracle_blocked_ell_roundtrip_and_shape(orc):
    for seed, B in [(2, 16), (3, 8), (4, 32)]:
        M, K, rp, cl, vl = _csr_case(seed, 64, 96, 0.05)
        e = orc.blocked_ell(M, K, rp, cl, vl, B)
        D = dense_from_csr(M, K, rp, cl, vl).astype(np.float32)
        occupied = [[j for j in range(K // B) if np.any(D[i * B:(i + 1) * B, j * B:(j + 1) * B])] for i in range(M // B)]
        assert e["height"] == M // B and e["width"] == max(len(o) for o in occupied)
        assert e["num_blocks"] == sum(len(o) for o in occupied) and e["num_elems"] == len(cl)
        for i, o in enumerate(occupied):
            assert e["ellColIdx"][i, :len(o)].tolist() == o and (e["ellColIdx"][i, len(o):] == -1).all()
        assert (orc.blocked_ell_to_dense(e, B, K) == D).all()
    # a trailing partial block row still gets its own row of ellColIdx (ceil(nrows/B))
    M, K, rp, cl, vl = _csr_case(5, 40, 64, 0.1)
    assert orc.blocked_ell(M, K, rp, cl, vl, 16)["height"] == 3


def test_oracle_splitter(orc):
    g = json.load(open(os.path.join(GOLD, "g67_block0.json")))["splitter_tile16_thr8"]
    dy, dx, nnz, r, c, v = orc.coo_read(G67)
    rp, cl, vl = orc.coo_to_csr(dy, r, c, v)
    which, cnt = orc.split(dy, dx, rp, cl, 16, 8)
    assert cnt.tolist() == [g["tiles"], g["heavy_tiles"], g["heavy_elems"], g["light_tiles"], g["light_elems"]]
    M, K, rp, cl, vl = _csr_case(6, 64, 80, 0.1)
    D = dense_from_csr(M, K, rp, cl, vl)
    which, cnt = orc.split(M, K, rp, cl, 16, 20)
    rows = np.repeat(np.arange(M), np.diff(rp))
    tile_nnz = {}
    for rr, cc in zip(rows, cl):
        tile_nnz[(rr // 16, cc // 16)] = tile_nnz.get((rr // 16, cc // 16), 0) + 1
    assert cnt[0] == len(tile_nnz) and cnt[1] == sum(1 for n in tile_nnz.values() if n >= 20)
    assert cnt[3] == cnt[0] - cnt[1] and cnt[2] + cnt[4] == len(cl)
    assert (which == np.array([tile_nnz[(rr // 16, cc // 16)] >= 20 for rr, cc in zip(rows, cl)])).all()


def test_oracle_block_stats_hand_cases(orc):
    # one row, B = 8 (two 4-wide bands per block), columns 5, 6, 7 and 17:
    #   band 0 (block 0) is the implicit start band with 0 nonzeros -> underloaded
    #   band 1 (block 0) holds 3 nonzeros -> overloaded when the walk leaves it
    #   bands 2, 3 (block 1) are skipped -> two underloads; band 4 (block 2) is the last band: never booked
    rp = np.array([0, 4] + [4] * 7, np.int32)
    cl = np.array([5, 6, 7, 17], np.int32)
    st = orc.block_stats(8, 24, rp, cl, 8)[0]
    assert st[0].tolist() == [3, 1, 1] and st[1].tolist() == [0, 2, 0] and st[2].tolist() == [1, 0, 0]
    # a row that starts in band 0 with exactly two nonzeros books nothing for it
    rp = np.array([0, 3] + [3] * 7, np.int32)
    cl = np.array([0, 3, 4], np.int32)
    st = orc.block_stats(8, 8, rp, cl, 8)[0]
    assert st[0].tolist() == [3, 0, 0]
    # rule (inc/preprocess.hpp:172-193) with B = 16: distance = 4 (u + o) / 256
    assert orc.classify(10, 30, 10, 16, 0.5, 0.8) == 0        # 0.625 > 0.5, ratio 0.75 <= 0.8 -> dense
    assert orc.classify(10, 36, 4, 16, 0.5, 0.8) == 2         # ratio 0.9 > 0.8 -> very sparse
    assert orc.classify(10, 10, 10, 16, 0.5, 0.8) == 1        # 0.3125 <= 0.5 -> 2:4 candidate
    assert orc.classify(5, 0, 0, 16, 0.5, 0.8) == 1


def test_oracle_double_spmm(orc):
    M, K, rp, cl, vl = _csr_case(7, 30, 40, 0.2)
    B = np.random.default_rng(0).standard_normal((K, 11))
    out = orc.spmm_csr_f64(rp, cl, vl.astype(np.float64), B)
    assert np.allclose(out, dense_from_csr(M, K, rp, cl, vl) @ B, rtol=1e-13, atol=1e-13)


# ---------------------------------------------------------------- product against oracle
def test_product_coo_and_csr_equal_oracle(cs, orc, tmp_path):
    coo = cs.SparseCoo(G67)
    dy, dx, nnz, r, c, v = orc.coo_read(G67)
    assert (coo.dimY, coo.dimX, coo.nnz) == (dy, dx, nnz)
    assert (coo.rows == r).all() and (coo.cols == c).all() and (coo.values == v).all()
    csr = cs.CSR_Matrix(coo)
    rp, cl, vl = orc.coo_to_csr(dy, r, c, v)
    assert (csr.rowPtr == rp).all() and (csr.cols == cl).all() and (csr.values == vl).all()
    # unsorted COO input is sorted by coo2CSR; save_mtx / re-read is the identity
    rng = np.random.default_rng(3)
    perm = rng.permutation(nnz)[:5000]
    shuffled = cs.SparseCoo(dy, dx, r[perm], c[perm], v[perm])
    again = cs.CSR_Matrix(shuffled)
    order = np.lexsort((c[perm], r[perm]))
    assert (again.cols == c[perm][order]).all() and (again.values == v[perm][order]).all()
    path = str(tmp_path / "out.mtx")
    shuffled.save_mtx(path)
    back = cs.SparseCoo(path)
    assert back.nnz == 5000 and (back.cols == c[perm][order]).all() and (back.values == v[perm][order]).all()
    with pytest.raises(cs.CuteError):
        cs.SparseCoo(str(tmp_path / "none.mtx"))


@pytest.mark.parametrize("seed", range(4))
def test_product_blocked_formats_equal_oracle(cs, orc, seed):
    M, K, rp, cl, vl = _csr_case(20 + seed, 16 * (2 + seed), 32 * (1 + seed), [0.02, 0.1, 0.3, 0.6][seed])
    csr = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp, cols=cl, values=vl)
    assert (csr.ToDense() == dense_from_csr(M, K, rp, cl, vl).astype(np.float32)).all()
    for R, Cc in [(16, 4), (8, 8), (16, 16)]:
        assert csr.csr_count_blocks(R, Cc) == orc.count_blocks(M, K, rp, cl, R, Cc)
        b = csr.to_BCSR(R, Cc)
        brp, bc, bv = orc.to_bcsr(M, K, rp, cl, vl, R, Cc)
        assert (b["BCSR_rowPtr"] == brp).all() and (b["BCSR_cols"] == bc).all() and (b["BCSR_values"] == bv).all()
    for B in (8, 16):
        e, o = cs.preprocess(csr, B), orc.blocked_ell(M, K, rp, cl, vl, B)
        assert (e.get_ellColIdx_height(), e.get_ellColIdx_width()) == (o["height"], o["width"])
        assert (e.get_num_blocks(), e.get_num_elems()) == (o["num_blocks"], o["num_elems"])
        assert (e.get_ellColIdx() == o["ellColIdx"]).all() and (e.get_ellValues() == o["ellValues"]).all()
        assert (e.blockedELLToDense() == csr.ToDense()).all()
    for tile, thr in [(16, 8), (8, 3), (16, 1), (16, 1000)]:
        s = cs.Splitter(csr, tile, thr)
        which, cnt = orc.split(M, K, rp, cl, tile, thr)
        assert [s.get_total_tiles(), s.get_num_heavy_tiles(), s.get_num_heavy_elems(), s.get_num_light_tiles(),
                s.get_num_light_elems()] == cnt.tolist()
        rows = np.repeat(np.arange(M), np.diff(rp))
        h, l = s.get_heavyMatrix(), s.get_lightMatrix()
        assert (h.rows == rows[which]).all() and (h.cols == cl[which]).all() and (h.values == vl[which]).all()
        assert (l.rows == rows[~which]).all() and (l.cols == cl[~which]).all() and (l.values == vl[~which]).all()


def test_product_classifier_equals_oracle(cs, orc):
    for seed, B, thr, dom in [(30, 16, 0.5, 0.8), (31, 8, 0.25, 0.5), (32, 32, 0.1, 0.9)]:
        M, K, rp, cl, vl = _csr_case(seed, 64, 128, 0.15)
        csr = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp, cols=cl, values=vl)
        got = cs.classify_blocks(csr, B, thr, dom)
        st = orc.block_stats(M, K, rp, cl, B)
        want = []
        for br in range(st.shape[0]):
            for bc in range(st.shape[1]):
                n, u, o = st[br, bc]
                if n:
                    want.append([br, bc, n, u, o, orc.classify(n, u, o, B, thr, dom)])
        assert got.tolist() == want
        assert got[:, 2].sum() == len(cl)


def test_product_double_spmm_equals_oracle(cs, orc):
    M, K, rp, cl, vl = _csr_case(40, 25, 33, 0.2)
    csr = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp, cols=cl, values=vl)
    B = np.random.default_rng(1).standard_normal((K, 7))
    out, ms = csr.sequentioal_spmm(B)
    assert ms >= 0 and (out == orc.spmm_csr_f64(rp, cl, vl.astype(np.float64), B)).all()
