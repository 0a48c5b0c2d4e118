"""The value-keeping MatrixMarket readers on every banner flavour, pinned by scipy.io.mmread on small
hand-written files; duplicate merging; the CPU COO product; the planner's addressing predicate.
No GPU needed."""
import os

import numpy as np
import pytest
import scipy.io
import scipy.sparse

from helpers import random_csr
from test_oracle_pins import GOLD

FILES = {
    "real_general": "%%MatrixMarket matrix coordinate real general\n% comment\n4 5 4\n1 1 1.5\n4 5 -2\n2 3 0.25\n2 1 7\n",
    "real_symmetric": "%%MatrixMarket matrix coordinate real symmetric\n4 4 4\n1 1 2\n3 1 -1.5\n4 2 3\n4 4 5\n",
    "real_skew": "%%MatrixMarket matrix coordinate real skew-symmetric\n4 4 3\n2 1 5\n4 1 -2.5\n4 3 1\n",
    "integer_symmetric": "%%MatrixMarket matrix coordinate integer symmetric\n3 3 3\n1 1 4\n2 1 -3\n3 3 9\n",
    "pattern_symmetric": "%%MatrixMarket matrix coordinate pattern symmetric\n3 3 2\n2 1\n3 3\n",
    "pattern_general_caps": "%%MatrixMarket MATRIX Coordinate Pattern General\n3 4 2\n2 4\n3 1\n",
    "array_general": "%%MatrixMarket matrix array real general\n3 2\n1\n0\n2.5\n0\n-4\n6\n",
    "array_symmetric": "%%MatrixMarket matrix array real symmetric\n3 3\n1\n2\n0\n3\n-4\n5\n",
    "array_skew": "%%MatrixMarket matrix array integer skew-symmetric\n3 3\n2\n0\n-7\n",
}
REFUSED = {
    "complex_general": "%%MatrixMarket matrix coordinate complex general\n2 2 1\n1 2 1.0 2.0\n",
    "complex_hermitian": "%%MatrixMarket matrix coordinate complex hermitian\n2 2 1\n2 1 1.0 2.0\n",
    "real_hermitian": "%%MatrixMarket matrix coordinate real hermitian\n2 2 1\n2 1 1.0\n",
    "unknown_field": "%%MatrixMarket matrix coordinate quaternion general\n2 2 1\n2 1 1.0\n",
    "unknown_format": "%%MatrixMarket matrix banded real general\n2 2 1\n2 1 1.0\n",
    "short_banner": "%%MatrixMarket matrix coordinate real\n2 2 1\n2 1 1.0\n",
    "array_pattern": "%%MatrixMarket matrix array pattern general\n2 2\n1\n1\n1\n1\n",
    "array_too_short": "%%MatrixMarket matrix array real general\n2 2\n1\n1\n1\n",
    "array_too_long": "%%MatrixMarket matrix array real general\n2 2\n1\n1\n1\n1\n1\n",
    "symmetric_not_square": "%%MatrixMarket matrix coordinate real symmetric\n2 3 1\n2 1 1.0\n",
    "fewer_entries_than_announced": "%%MatrixMarket matrix coordinate real general\n3 3 3\n1 1 1.0\n",
    "more_entries_than_announced": "%%MatrixMarket matrix coordinate real general\n3 3 1\n1 1 1.0\n2 2 1.0\n",
    "no_entry_count": "%%MatrixMarket matrix coordinate real general\n3 3\n1 1 1.0\n",
}


def _scipy_dense(path):
    m = scipy.io.mmread(path)
    return np.asarray(m.todense() if scipy.sparse.issparse(m) else m, np.float64)


def _dense_of_csr(r):
    D = np.zeros((r.M, r.K))
    for i in range(r.M):
        s, e = int(r.rowPtr[i]), int(r.rowPtr[i + 1])
        np.add.at(D[i], r.cols[s:e].astype(np.int64), r.vals[s:e].astype(np.float64))
    return D


@pytest.mark.parametrize("name", sorted(FILES))
def test_flavours_against_scipy(cs, tmp_path, name):
    p = tmp_path / (name + ".mtx")
    p.write_text(FILES[name])
    want = _scipy_dense(str(p))
    # CSR family: dimensions padded to 16 (IO.cu:30-31), values kept
    r = cs.MTX_READER(str(p), keep_values=True)
    D = _dense_of_csr(r)
    assert r.M % 16 == 0 and r.K % 16 == 0 and r.M - want.shape[0] < 16 and r.K - want.shape[1] < 16
    assert (D[:want.shape[0], :want.shape[1]] == want).all() and np.count_nonzero(D) == np.count_nonzero(want)
    assert r.nnz == np.count_nonzero(want)
    # COO family: dimensions as in the file, sorted by (row, column)
    c = cs.SparseCoo(str(p))
    assert (c.dimY, c.dimX, c.nnz) == (want.shape[0], want.shape[1], np.count_nonzero(want))
    D2 = np.zeros(want.shape)
    D2[c.rows, c.cols] = c.values
    assert (D2 == want).all()
    assert (np.lexsort((c.cols, c.rows)) == np.arange(c.nnz)).all()


def test_skew_symmetric_sign_is_what_the_reference_gets_wrong(cs, orc, tmp_path):
    """(2,1) = 5 mirrors to (1,2) = -5; the reference's readers (and therefore the oracle) give +5."""
    p = tmp_path / "s.mtx"
    p.write_text(FILES["real_skew"])
    c = cs.SparseCoo(str(p))
    D = np.zeros((4, 4))
    D[c.rows, c.cols] = c.values
    assert D[1, 0] == 5 and D[0, 1] == -5 and (D == -D.T).all()
    _, _, _, r, cl, v = orc.coo_read(str(p))                      # inc/SparseCoo.hpp:113,141-149 restated
    O = np.zeros((4, 4))
    O[r, cl] = v
    assert O[0, 1] == 5 and (O == O.T).all()
    # keep_values=0 stays the reference's reader: same pattern either way, all ones
    r0 = cs.MTX_READER(str(p))
    M, K, nnz, rp, cl0, vl0 = orc.mtx_read(str(p))
    assert (r0.M, r0.K, r0.nnz) == (M, K, nnz) and (r0.rowPtr == rp).all() and (r0.cols == cl0).all() and (r0.vals == 1).all()


@pytest.mark.parametrize("name", sorted(REFUSED))
def test_refused_files(cs, tmp_path, name):
    p = tmp_path / (name + ".mtx")
    p.write_text(REFUSED[name])
    for read in (lambda: cs.MTX_READER(str(p), keep_values=True), lambda: cs.SparseCoo(str(p))):
        with pytest.raises(cs.CuteError) as e:
            read()
        assert e.value.status == -9, name


@pytest.mark.parametrize("dims", ["4000000000 4000000000 1", "2147483648 5 1", "5 2147483648 1"])
def test_size_lines_beyond_int_are_refused(cs, tmp_path, dims):
    """The reference parses the size line with stoi (IO.cu:23-29), which throws beyond INT_MAX; here every reader
    returns a status instead of allocating row pointers for four billion rows."""
    p = tmp_path / "huge.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real general\n" + dims + "\n1 1 1.0\n")
    for read in (lambda: cs.MTX_READER(str(p)), lambda: cs.MTX_READER(str(p), keep_values=True), lambda: cs.SparseCoo(str(p))):
        with pytest.raises(cs.CuteError) as e:
            read()
        assert e.value.status == -2, dims


def test_entry_count_is_ignored_by_the_reference_mode_only(cs, orc, tmp_path):
    """keep_values=0 stays the reference's reader, which never looks at the announced count (IO.cu:23-29)."""
    p = tmp_path / "short.mtx"
    p.write_text(REFUSED["fewer_entries_than_announced"])
    r = cs.MTX_READER(str(p))
    M, K, nnz, rp, cl, _ = orc.mtx_read(str(p))
    assert (r.M, r.K, r.nnz) == (M, K, nnz) == (16, 16, 1) and (r.rowPtr == rp).all() and (r.cols == cl).all()


def test_no_banner_reads_like_the_reference(cs, orc, tmp_path):
    p = tmp_path / "nb.mtx"
    p.write_text("% a file whose first line only mentions symmetric\n3 3 2\n2 1 4\n3 3 1\n")
    r = cs.MTX_READER(str(p), keep_values=True)
    M, K, nnz, rp, cl, _ = orc.mtx_read(str(p))
    assert (r.M, r.K, r.nnz) == (M, K, nnz) == (16, 16, 3) and (r.rowPtr == rp).all() and (r.cols == cl).all()
    assert sorted(r.vals.tolist()) == [1.0, 4.0, 4.0]


def test_valued_reader_keeps_the_reference_order(cs, orc):
    """On a file the reference reads correctly, keep_values changes the values and nothing else."""
    g = os.path.join(GOLD, "G67.mtx")
    a, b = cs.MTX_READER(g), cs.MTX_READER(g, keep_values=True)
    assert (a.M, a.K, a.nnz) == (b.M, b.K, b.nnz) and (a.rowPtr == b.rowPtr).all() and (a.cols == b.cols).all()
    m = scipy.io.mmread(g).tocsr()
    mine = scipy.sparse.csr_matrix((b.vals.astype(np.float64), b.cols.astype(np.int64), b.rowPtr.astype(np.int64)), shape=(b.M, b.K))
    assert b.rowPtr[m.shape[0]] == b.nnz and b.cols.max() < m.shape[1]           # nothing in the padding
    diff = mine[:m.shape[0], :m.shape[1]] - m
    assert diff.nnz == 0 or abs(diff).max() == 0


def test_merge_duplicates(cs, tmp_path):
    p = tmp_path / "d.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real general\n3 4 7\n2 3 1\n1 1 2\n2 3 4\n2 1 8\n2 3 16\n1 1 32\n3 4 64\n")
    want = scipy.io.mmread(str(p)).tocsr()                        # scipy adds duplicates up on conversion
    want.sum_duplicates()
    r = cs.MTX_READER(str(p), keep_values=True)
    assert r.nnz == 7
    with pytest.raises(cs.CuteError) as e:
        cs.MTX_READER(str(p), keep_values=True).sort_rows()       # sorting alone still reports the duplicates
    assert e.value.status == -3
    r.merge_duplicates()
    assert r.nnz == want.nnz == 4
    assert (r.rowPtr[:4] == want.indptr).all() and (r.rowPtr[3:] == 4).all()
    assert (r.cols == want.indices).all() and (r.vals == want.data.astype(np.float32)).all()
    cs.HRPB(r.M, r.K, r.rowPtr, r.cols, r.vals)                   # now a legal input of the format builder
    c = cs.SparseCoo(str(p))
    assert c.nnz == 7
    c.merge_duplicates()
    assert c.nnz == 4 and c.rows.tolist() == [0, 1, 1, 2] and c.cols.tolist() == [0, 0, 2, 3]
    assert c.values.tolist() == [34.0, 8.0, 21.0, 64.0]
    # sums are taken in file order: 1e8 + 1 - 1e8 is 0 in fp32 that way round
    p.write_text("%%MatrixMarket matrix coordinate real general\n1 1 3\n1 1 1e8\n1 1 1\n1 1 -1e8\n")
    assert cs.MTX_READER(str(p), keep_values=True).merge_duplicates().vals.tolist() == [0.0]
    assert cs.SparseCoo(str(p)).merge_duplicates().values.tolist() == [0.0]


def test_spmm_coo_equals_the_oracle_bit_for_bit(cs, orc):
    rng = np.random.default_rng(11)
    for M, K, N, dens in ((64, 96, 33, 0.2), (32, 32, 128, 0.5), (160, 48, 7, 0.05)):
        rp, cl, vl = random_csr(rng, M, K, density=dens)
        rows = np.repeat(np.arange(M, dtype=np.uint32), np.diff(rp.astype(np.int64)))
        perm = rng.permutation(len(cl))                            # array order, not row order, decides the sums
        rows, cols, vals = rows[perm], cl[perm], vl[perm]
        B = rng.standard_normal((K, N)).astype(np.float32)
        want = orc.spmm_coo(rows, cols, vals, B, M)
        got = cs.spmm_coo(rows, cols, vals, B, M)
        assert got.tobytes() == want.tobytes()
    # duplicates are legal here and add up in array order; empty rows come out as zeros
    rows = np.array([1, 1, 1], np.uint32)
    cols = np.array([0, 0, 0], np.uint32)
    vals = np.array([1e8, 1.0, -1e8], np.float32)
    B = np.ones((1, 2), np.float32)
    assert cs.spmm_coo(rows, cols, vals, B, 3).tolist() == [[0, 0], [0, 0], [0, 0]]
    with pytest.raises(cs.CuteError) as e:
        cs.spmm_coo(np.array([3], np.uint32), cols[:1], vals[:1], B, 3)
    assert e.value.status == -4


def test_offsets_predicate(cs):
    """Synthetic sizes around every limit of the fast kernels' 32-bit / 24-bit addressing."""
    fit = cs.offsets_fit
    assert fit(65536, 65536, 128, 586756, 0)
    assert fit(65536, 65536, 128, 0, (1 << 24) - 1) is False       # partial rows x pitch beyond 4 GiB
    assert fit(4096, 4096, 32, 0, (1 << 24) - 1)                   # 2^24 - 1 rows of 128 bytes: 2 GiB, fine
    assert fit(4096, 4096, 32, 0, 1 << 24) is False                # the row operand itself
    assert fit(4096, 4096, 16, 0, (1 << 20) * 16) is False         # 2^20 pieces of 16 rows at N = 16: bytes fit, rows do not
    assert fit(4096, 4096, 16, 0, (1 << 20) * 16 - 16)
    assert fit((1 << 24) - 16, 4096, 4, 0, 0) is False and fit((1 << 24) - 32, 4096, 4, 0, 0)
    assert fit(4096, 1 << 24, 4, 0, 0) is False and fit(4096, (1 << 24) - 16, 4, 0, 0)
    assert fit(16, 16, 1 << 22, 0, 0) is False                     # row pitch of 2^24 bytes
    assert fit((1 << 20) - 32, (1 << 20) - 16, 1024, 0, 0)         # B and C just below 4 GiB
    assert fit((1 << 20) - 32, 1 << 20, 1024, 0, 0) is False       # B of 4 GiB
    assert fit((1 << 20) - 16, (1 << 20) - 16, 1024, 0, 0) is False  # C plus one spare panel of 4 GiB
    assert fit(4096, 4096, 64, (1 << 30) - 65, 0) and fit(4096, 4096, 64, (1 << 30) - 64, 0) is False
