"""Quad lists (the 4x4x1 MFMA kernel's layout): structure and exact content, on the CPU.

The layout has no counterpart in the reference, so it is pinned by what defines it: decoding it
must give back the CSR matrix bit for bit, each row group's columns must ascend strictly over its
real steps, the four lists of a panel must be padded to one common length, and that length must be
the shortest one possible (some row group really has that many distinct columns)."""
import numpy as np
import pytest

from helpers import random_csr


def _decode(M, K, q):
    """(row, col) -> value for every non-padding slot, plus per-(panel, row group) real lengths."""
    gp = q["groupPtr"].astype(np.int64)
    entries = {}
    for p in range(len(gp) - 1):
        for g in range(gp[p], gp[p + 1]):
            for pair in range(16):
                rg, col = pair % 4, int(q["cols"][g, pair])
                for i in range(4):
                    v = q["vals"][g, 4 * pair + i]
                    if v != 0:
                        key = (16 * p + 4 * rg + i, col)
                        assert key not in entries, "a matrix entry appears twice"
                        entries[key] = v
    return entries


def _cases():
    rng = np.random.default_rng(11)
    yield "random", (64, 96) + random_csr(rng, 64, 96, density=0.1)
    yield "empty_rows", (48, 64) + random_csr(rng, 48, 64, density=0.2, empty_rows=set(range(16, 32)) | {3, 40})
    yield "dense_panel", (16, 32) + random_csr(rng, 16, 32, density=1.0)
    yield "single", (16, 16) + random_csr(rng, 16, 16, row_nnz=lambda r: 1 if r == 5 else 0)
    yield "all_empty", (32, 16) + random_csr(rng, 32, 16, row_nnz=0)
    yield "long_row", (32, 4096) + random_csr(rng, 32, 4096, row_nnz=lambda r: 3000 if r == 17 else 2)


@pytest.mark.parametrize("name,case", list(_cases()), ids=[n for n, _ in _cases()])
def test_quad_lists_hold_exactly_the_matrix(cs, name, case):
    M, K, rp, cl, vl = case
    q = cs.quad_lists(M, K, rp, cl, vl)
    gp = q["groupPtr"].astype(np.int64)
    assert gp[0] == 0 and gp[-1] == q["numGroups"] and len(gp) == M // 16 + 1 and (np.diff(gp) >= 0).all()
    assert q["cols"].shape == (q["numGroups"], 16) and q["vals"].shape == (q["numGroups"], 64)
    assert (q["cols"] < K).all()
    entries = _decode(M, K, q)
    expect = {(r, int(cl[k])): vl[k] for r in range(M) for k in range(rp[r], rp[r + 1]) if vl[k] != 0}
    assert entries.keys() == expect.keys()
    assert all(np.float32(entries[k]).tobytes() == np.float32(expect[k]).tobytes() for k in expect)
    # structure of every panel
    for p in range(M // 16):
        longest = 0
        for rg in range(4):
            rows = range(16 * p + 4 * rg, 16 * p + 4 * rg + 4)
            want = sorted({int(c) for r in rows for c in cl[rp[r]:rp[r + 1]]})
            longest = max(longest, len(want))
            steps = [int(q["cols"][g, 4 * s + rg]) for g in range(gp[p], gp[p + 1]) for s in range(4)]
            assert steps[:len(want)] == want, (name, p, rg)                       # ascending, complete
            pad = want[-1] if want else 0
            assert all(c == pad for c in steps[len(want):]), (name, p, rg)        # padding repeats the last column
            for t in range(len(want), len(steps)):                                # ... with zero values
                g, s = gp[p] + t // 4, t % 4
                assert not q["vals"][g, 4 * (4 * s + rg):4 * (4 * s + rg) + 4].any()
        assert gp[p + 1] - gp[p] == (longest + 3) // 4, (name, p)


def test_quad_lists_of_the_golden_matrix(cs):
    import os
    from test_oracle_pins import GOLD
    r = cs.MTX_READER(os.path.join(GOLD, "G67.mtx"))
    q = cs.quad_lists(r.M, r.K, r.rowPtr, r.cols, r.vals)
    assert np.count_nonzero(q["vals"]) == r.nnz
    # a toroidal 4-neighbour grid: a 4-row group of consecutive vertices touches at most 16 columns
    assert q["numGroups"] <= 4 * (r.M // 16)


def test_quad_build_rejects_null_arguments(cs):
    import ctypes as C
    lib = cs.load_library()
    assert lib.cute_quad_build(16, 16, None, None, None, None) == -5


@pytest.mark.parametrize("name,case", list(_cases()), ids=[n for n, _ in _cases()])
def test_strip_lists_hold_exactly_the_matrix(cs, name, case):
    """One list per 4-row strip: same content, no padding beyond a strip's own last group."""
    M, K, rp, cl, vl = case
    q = cs.quad_lists(M, K, rp, cl, vl, strips=True)
    gp = q["groupPtr"].astype(np.int64)
    assert q["rowsPerList"] == 4 and len(gp) == M // 4 + 1 and gp[-1] == q["numGroups"]
    entries, pairs = {}, 0
    for st in range(M // 4):
        rows = range(4 * st, 4 * st + 4)
        want = sorted({int(c) for r in rows for c in cl[rp[r]:rp[r + 1]]})
        pairs += len(want)
        assert gp[st + 1] - gp[st] == (len(want) + 15) // 16, (name, st)
        assert q["tail"][st] == (len(want) - 16 * ((len(want) + 15) // 16 - 1) if want else 0)
        slots = [int(c) for g in range(gp[st], gp[st + 1]) for c in q["cols"][g]]
        assert slots[:len(want)] == want and all(c == want[-1] for c in slots[len(want):])
        for g in range(gp[st], gp[st + 1]):
            for p in range(16):
                for i in range(4):
                    v = q["vals"][g, 4 * p + i]
                    if v != 0:
                        assert (16 * (g - gp[st]) + p) < len(want)
                        entries[(4 * st + i, int(q["cols"][g, p]))] = v
    expect = {(r, int(cl[k])): vl[k] for r in range(M) for k in range(rp[r], rp[r + 1]) if vl[k] != 0}
    assert entries.keys() == expect.keys() and q["numPairs"] == pairs
    assert all(np.float32(entries[k]).tobytes() == np.float32(expect[k]).tobytes() for k in expect)


def test_lockstep_tail_and_pair_count(cs):
    rng = np.random.default_rng(2)
    M, K = 64, 128
    rp, cl, vl = random_csr(rng, M, K, density=0.07)
    q = cs.quad_lists(M, K, rp, cl, vl)
    gp = q["groupPtr"].astype(np.int64)
    pairs = 0
    for p in range(M // 16):
        lens = [len({int(c) for r in range(16 * p + 4 * rg, 16 * p + 4 * rg + 4) for c in cl[rp[r]:rp[r + 1]]}) for rg in range(4)]
        pairs += sum(lens)
        L = max(lens)
        assert q["tail"][p] == (4 * (L - 4 * ((L + 3) // 4 - 1)) if L else 0)
    assert q["numPairs"] == pairs and q["rowsPerList"] == 16
    import ctypes as C
    g, n = C.c_uint64(), C.c_uint64()
    rp32, cl32 = np.ascontiguousarray(rp, np.uint32), np.ascontiguousarray(cl, np.uint32)
    assert cs.load_library().cute_quad_fill(M, rp32.ctypes.data_as(C.POINTER(C.c_uint32)), cl32.ctypes.data_as(C.POINTER(C.c_uint32)),
                                            C.byref(g), C.byref(n)) == 0
    assert (g.value, n.value) == (q["numGroups"], pairs)


def test_direct_packing_equals_packing_the_lists(cs):
    """cute_quad_pack (what the upload sends to the device, written straight from the CSR matrix) against the
    same records made here from the inspectable host form of the lists: per group 16 columns, the mask of
    nonzero value slots, the running index of the first stored value, and the stored values in slot order."""
    rng = np.random.default_rng(31)
    cases = [(64, 96, dict(density=0.1)), (32, 64, dict(row_nnz=0)), (48, 2048, dict(row_nnz=lambda r: 900 if r == 3 else 5)),
             (160, 64, dict(density=0.4, empty_rows=set(range(16, 40))))]
    for M, K, kw in cases:
        rp, cl, vl = random_csr(rng, M, K, **kw)
        if len(vl) > 4:
            vl[rng.choice(len(vl), 3, replace=False)] = 0.0          # explicit zeros are empty slots, not stored values
        for strips in (False, True):
            q = cs.quad_lists(M, K, rp, cl, vl, strips=strips)
            got = cs.quad_pack(M, rp, cl, vl, strips=strips)
            assert np.array_equal(got["groupPtr"], q["groupPtr"])
            G = q["numGroups"]
            recs = np.zeros((G, 20), np.uint32)
            packed = []
            for g in range(G):
                recs[g, :16] = q["cols"][g]
                recs[g, 18] = len(packed)
                mask = 0
                for slot in range(64):
                    v = q["vals"][g, slot]
                    if v != 0.0:
                        mask |= 1 << slot
                        packed.append(v)
                recs[g, 16], recs[g, 17] = mask & 0xFFFFFFFF, mask >> 32
            assert np.array_equal(got["recs"], recs), (M, K, strips)
            assert got["packed"].tobytes() == np.asarray(packed, np.float32).tobytes(), (M, K, strips)
            assert int(got["stripPairs"].sum()) == q["numPairs"] and int(got["stripVals"].sum()) == len(packed)
