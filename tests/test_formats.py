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


def _block_stats_brute(D, bs, ncols):
    """Per key r_blk * (ncols // bs) + c_blk (gpu_kernels.cu:1064-1067): nonzeros, distinct rows, distinct columns."""
    rows, cols = {}, {}
    for r, c in zip(*np.nonzero(D)):
        key = (r // bs) * (ncols // bs) + c // bs
        rows.setdefault(key, []).append(r)
        cols.setdefault(key, []).append(c)
    nnz = np.array([len(rows[k]) for k in sorted(rows)], np.float64)
    nr = np.array([len(set(rows[k])) for k in sorted(rows)], np.float64)
    nc = np.array([len(set(cols[k])) for k in sorted(rows)], np.float64)
    return np.array([(nnz / nr).mean(), (nnz / nc).mean(), len(nnz), (nnz / (bs * bs)).mean()])


def test_oracle_get_stats_and_anxs(orc):
    # closed forms.  Identity: every diagonal block holds bs nonzeros in bs rows and bs columns.
    n, bs = 64, 16
    rp, cl = np.arange(n + 1, dtype=np.int32), np.arange(n, dtype=np.int32)
    assert orc.get_stats(n, n, rp, cl, bs).tolist() == [1.0, 1.0, 4.0, np.float32(1 / 16)]
    assert orc.get_anxs(n, rp, cl, bs, True) == 1.0 and orc.get_anxs(n, rp, cl, bs, False) == 1.0
    # all ones, 32 x 48: 6 full blocks; each block row holds 48 distinct columns, each block column 32 distinct rows
    rp, cl = np.arange(33, dtype=np.int32) * 48, np.tile(np.arange(48, dtype=np.int32), 32)
    assert orc.get_stats(32, 48, rp, cl, bs).tolist() == [16.0, 16.0, 6.0, 1.0]
    assert orc.get_anxs(32, rp, cl, bs, True) == np.float32(32 * 48) / np.float32(2 * 48)
    assert orc.get_anxs(32, rp, cl, bs, False) == np.float32(32 * 48) / np.float32(3 * 32)
    # only the first row of every block row is full: 16 nonzeros in one row and 16 columns per block
    rp = np.zeros(33, np.int32)
    rp[1:17], rp[17:] = 48, 96
    cl = np.tile(np.arange(48, dtype=np.int32), 2)
    assert orc.get_stats(32, 48, rp, cl, bs).tolist() == [16.0, 1.0, 6.0, np.float32(1 / 16)]
    # dense-matrix brute force, also where the block size does not divide the column count (the last block
    # column then counts into the next block row's first block) and where it exceeds it (one block in all)
    for seed, M, K, b, dens in [(50, 64, 96, 16, 0.05), (51, 48, 64, 8, 0.3), (52, 70, 90, 16, 0.08), (53, 40, 12, 16, 0.3),
                                (54, 33, 50, 7, 0.15)]:
        M, K, rp, cl, vl = _csr_case(seed, M, K, dens)
        D = dense_from_csr(M, K, rp, cl, np.ones_like(vl))
        want = _block_stats_brute(D, b, K)
        got = orc.get_stats(M, K, rp, cl, b)
        assert got[2] == want[2] and np.allclose(got, want, rtol=2e-6, atol=0)
        per_band_cols = sum(int(np.any(D[i:i + b], axis=0).sum()) for i in range(0, M, b))
        per_band_rows = sum(int(np.any(D[:, j:j + b], axis=1).sum()) for j in range(0, K, b))
        assert orc.get_anxs(M, rp, cl, b, True) == np.float32(len(cl)) / np.float32(per_band_cols)
        assert orc.get_anxs(M, rp, cl, b, False) == np.float32(len(cl)) / np.float32(per_band_rows)


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


def test_product_split_by_class_equals_oracle(cs, orc):
    """The split the classifier implies: an entry is heavy iff its block is not "very sparse" (kind 2) by the oracle's
    band statistics and rule (inc/preprocess.hpp:64-193 restated); heavy and light together are the matrix, in CSR order."""
    for seed, B, thr, dom in [(30, 16, 0.5, 0.8), (31, 8, 0.25, 0.5), (32, 32, 0.1, 0.9), (33, 16, 0.9, 0.3)]:
        M, K, rp, cl, vl = _csr_case(seed, 64, 128, 0.15)
        csr = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp, cols=cl, values=vl)
        s = cs.ClassSplitter(csr, B, thr, dom)
        st = orc.block_stats(M, K, rp, cl, B)
        kind = np.full(st.shape[:2], -1)
        for br in range(st.shape[0]):
            for bc in range(st.shape[1]):
                n, u, o = st[br, bc]
                if n:
                    kind[br, bc] = orc.classify(n, u, o, B, thr, dom)
        rows = np.repeat(np.arange(M), np.diff(rp))
        which = kind[rows // B, cl // B] != 2
        assert (kind[rows // B, cl // B] >= 0).all()
        h, l = s.get_heavyMatrix(), s.get_lightMatrix()
        assert (h.rows == rows[which]).all() and (h.cols == cl[which]).all() and (h.values == vl[which]).all()
        assert (l.rows == rows[~which]).all() and (l.cols == cl[~which]).all() and (l.values == vl[~which]).all()
        assert s.get_total_tiles() == (kind >= 0).sum() and s.get_num_light_tiles() == (kind == 2).sum()
        assert s.get_num_heavy_tiles() == ((kind == 0) | (kind == 1)).sum()
        assert s.get_num_heavy_elems() == which.sum() and s.get_num_light_elems() == (~which).sum()


def test_product_double_spmm_equals_oracle(cs, orc):
    M, K, rp, cl, vl = _csr_case(40, 25, 33, 0.2)
    csr = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp, cols=cl, values=vl)
    B = np.random.default_rng(1).standard_normal((K, 7))
    out, ms = csr.sequentioal_spmm(B)
    assert ms >= 0 and (out == orc.spmm_csr_f64(rp, cl, vl.astype(np.float64), B)).all()


def test_product_block_statistics_equal_oracle(cs, orc):
    cases = [(60, 64, 96, 16, 0.05), (61, 48, 64, 8, 0.3), (62, 70, 90, 16, 0.08), (63, 40, 12, 16, 0.3), (64, 33, 50, 7, 0.15),
             (65, 200, 333, 32, 0.02), (66, 16, 16, 1, 0.5)]
    for seed, M, K, b, dens in cases:
        M, K, rp, cl, vl = _csr_case(seed, M, K, dens)
        csr = cs.CSR_Matrix(nrows=M, ncols=K, rowPtr=rp, cols=cl, values=vl)
        assert cs.GET_STATS(csr, b).tolist() == orc.get_stats(M, K, rp, cl, b).tolist()      # same order of additions
        for axis in (True, False):
            assert np.float32(cs.GET_ANXS(csr, b, axis)) == np.float32(orc.get_anxs(M, rp, cl, b, axis))
    coo = cs.SparseCoo(G67)
    csr = cs.CSR_Matrix(coo)
    for b in (16, 32):
        assert cs.GET_STATS(csr, b).tolist() == orc.get_stats(csr.nrows, csr.ncols, csr.rowPtr, csr.cols, b).tolist()
        assert np.float32(cs.GET_ANXS(csr, b, True)) == np.float32(orc.get_anxs(csr.nrows, csr.rowPtr, csr.cols, b, True))
    # 16x16 blocks of G67 hold 4 325 tiles, the count the splitter reports for the same tiling
    assert cs.GET_STATS(csr, 16)[2] == 4325
    empty = cs.CSR_Matrix(nrows=8, ncols=8, rowPtr=np.zeros(9, np.int32), cols=np.zeros(0, np.int32), values=np.zeros(0, np.float32))
    st = cs.GET_STATS(empty, 4)
    assert st[2] == 0 and np.isnan(st[0]) and np.isnan(cs.GET_ANXS(empty, 4, True))
    with pytest.raises(cs.CuteError):
        cs.GET_STATS(csr, 0)
    with pytest.raises(cs.CuteError):
        cs.GET_ANXS(csr, -1, True)
