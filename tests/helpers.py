"""Test-side helpers that are independent of both the oracle and the product:
a pure-numpy HRPB stream decoder, structural checks and small CSR builders."""
import numpy as np


def csr_from_dense(D):
    D = np.asarray(D, np.float32)
    M, K = D.shape
    rowPtr = np.zeros(M + 1, np.uint32)
    cols, vals = [], []
    for r in range(M):
        nz = np.nonzero(D[r])[0]
        cols.extend(nz.tolist())
        vals.extend(D[r, nz].tolist())
        rowPtr[r + 1] = len(cols)
    return rowPtr, np.asarray(cols, np.uint32), np.asarray(vals, np.float32)


def dense_from_csr(M, K, rowPtr, cols, vals):
    D = np.zeros((M, K), np.float64)
    for r in range(M):
        s, e = int(rowPtr[r]), int(rowPtr[r + 1])
        D[r, cols[s:e]] += vals[s:e]
    return D


def random_csr(rng, M, K, density=None, row_nnz=None, empty_rows=(), values="normal"):
    """Sorted distinct columns per row; M, K multiples of 16 expected by the caller."""
    rowPtr = np.zeros(M + 1, np.uint32)
    cols = []
    for r in range(M):
        if r in empty_rows:
            n = 0
        elif row_nnz is not None:
            n = int(row_nnz(r)) if callable(row_nnz) else int(row_nnz)
        else:
            n = int(rng.binomial(K, density))
        n = min(n, K)
        c = np.sort(rng.choice(K, size=n, replace=False)) if n else np.zeros(0, np.int64)
        cols.append(c)
        rowPtr[r + 1] = rowPtr[r] + n
    cols = np.concatenate(cols).astype(np.uint32) if cols else np.zeros(0, np.uint32)
    nnz = len(cols)
    if values == "ones":
        vals = np.ones(nnz, np.float32)
    elif values == "ints":
        vals = rng.integers(-8, 9, nnz).astype(np.float32)
        vals[vals == 0] = 1
    else:
        vals = rng.standard_normal(nnz).astype(np.float32)
        vals[vals == 0] = 1
    return rowPtr, cols, vals


def popcount64(x):
    x = np.asarray(x, np.uint64)
    return np.array([bin(int(v)).count("1") for v in x.ravel()], np.int64).reshape(x.shape)


def hrpb_decode(h):
    """Decode the canonical stream into sorted COO triplets using only the documented layout
    (record words 0-35 + values; bit row*4+k; values brick-column-major in bitmap order)."""
    brp, ac, sp, bd = h["blockedRowPtr"], h["activeCols"], h["sizePtr"], h["blocksData"]
    rows, cols, vals = [], [], []
    P = len(brp) - 1
    for p in range(P):
        for b in range(int(brp[p]), int(brp[p + 1])):
            rec = bd[int(sp[b]):int(sp[b + 1])]
            bitmaps = rec[28:36].view(np.uint64)
            fv = rec[36:].view(np.float32)
            n = 0
            for j in range(4):
                bm = int(bitmaps[j])
                for bit in range(64):
                    if (bm >> bit) & 1:
                        r, k = bit // 4, bit % 4
                        rows.append(p * 16 + r)
                        cols.append(int(ac[b * 16 + j * 4 + k]))
                        vals.append(fv[n])
                        n += 1
    rows, cols, vals = np.asarray(rows, np.int64), np.asarray(cols, np.int64), np.asarray(vals, np.float32)
    order = np.lexsort((cols, rows))
    return rows[order], cols[order], vals[order]


def hrpb_check_invariants(h, rowPtr, cols):
    """Facts any correct serialisation must satisfy, none of which restates the builder."""
    brp, ac, sp, bd = h["blockedRowPtr"], h["activeCols"], h["sizePtr"], h["blocksData"]
    P = len(brp) - 1
    nb = int(brp[-1])
    assert len(ac) == nb * 16 and len(sp) == nb + 1 and len(bd) == int(sp[-1])
    assert sp[0] == 0
    steps = np.diff(sp.astype(np.int64))
    assert (steps > 0).all() and (steps % 128 == 0).all()
    total = 0
    for p in range(P):
        s, e = int(rowPtr[p * 16]), int(rowPtr[(p + 1) * 16])
        distinct = np.unique(cols[s:e])
        nblk = int(brp[p + 1]) - int(brp[p])
        assert nblk == (len(distinct) + 15) // 16
        a = ac[int(brp[p]) * 16:int(brp[p + 1]) * 16]
        assert (a[:len(distinct)] == distinct).all() and (a[len(distinct):] == 0).all()
        for i, b in enumerate(range(int(brp[p]), int(brp[p + 1]))):
            rec = bd[int(sp[b]):int(sp[b + 1])]
            bitmaps = rec[28:36].view(np.uint64)
            pc = popcount64(bitmaps)
            prefix = rec[24:26].view(np.uint16)
            assert prefix[0] == 0 and (np.diff(prefix.astype(np.int64)) == pc[:3]).all()
            for j in range(4):
                lo = bin(int(bitmaps[j]) & 0xFFFFFFFF).count("1")
                hi = bin(int(bitmaps[j]) >> 32).count("1")
                assert int(rec[4 + j]) == (lo | (hi << 8))
            col_ptr = int(rec[2:4].view(np.uint64)[0])
            assert col_ptr == sum((1 << (4 * j)) for j in range(4) if bitmaps[j])
            nnz_blk = int(pc.sum())
            words = ((nnz_blk + 1) // 2) * 2 + 36
            assert len(rec) == ((words + 127) // 128) * 128 and rec[26] == len(rec) // 128
            assert int(rec[0:2].view(np.uint64)[0]) == int(sp[b + 1])
            if i + 1 < nblk:
                nxt = ac[(b + 1) * 16:(b + 2) * 16]
                assert (rec[8:24] == nxt).all()
                assert rec[27] == (int(sp[b + 2]) - int(sp[b + 1])) // 128
            else:
                assert (rec[8:24] == 0).all() and rec[27] == 0
            assert (rec[36 + nnz_blk:] == 0).all()
            total += nnz_blk
    assert total == int(rowPtr[-1])
