"""Binary cache of a preprocessed matrix: exact round trip and rejection of anything damaged."""
import os
import struct

import numpy as np
import pytest

from helpers import random_csr


def _same(a, b):
    for f in ("M", "K", "numRowPanels", "numBlocks", "numWords", "num_bricks", "numNNZ"):
        assert getattr(a, f) == getattr(b, f), f
    for f in ("blockedRowPtr", "activeCols", "sizePtr", "blocksData", "rowPtr", "cols"):
        assert np.array_equal(getattr(a, f), getattr(b, f)), f
    assert a.vals.tobytes() == b.vals.tobytes()


def test_round_trip_is_bit_exact(cs, tmp_path):
    rng = np.random.default_rng(5)
    for i, (M, K, kw) in enumerate([(64, 96, dict(density=0.1)), (32, 16, dict(row_nnz=0)),
                                    (48, 4096, dict(row_nnz=lambda r: 700 if r == 3 else 5))]):
        rp, cl, vl = random_csr(rng, M, K, **kw)
        h = cs.HRPB(M, K, rp, cl, vl)
        path = str(tmp_path / ("m%d.hrpb" % i))
        h.save(path)
        back = cs.HRPB.load(path)
        _same(h, back)
        # the loaded object is a full citizen: it re-tiles like the original
        t0, t1 = h.retile(), back.retile()
        assert np.array_equal(t0["hdr"], t1["hdr"]) and t0["vals"].tobytes() == t1["vals"].tobytes()


def test_golden_matrix_round_trip(cs, tmp_path):
    from test_oracle_pins import GOLD
    r = cs.MTX_READER(os.path.join(GOLD, "G67.mtx"))
    h = cs.HRPB(r.M, r.K, r.rowPtr, r.cols, r.vals)
    path = str(tmp_path / "g67.hrpb")
    h.save(path)
    assert os.path.getsize(path) == 64 + 4 * (626 + 2500 * 16 + 320000 + 10001 + 2 * 40000) + 8 * 2501
    _same(h, cs.HRPB.load(path))


def test_damaged_files_are_rejected(cs, tmp_path):
    rng = np.random.default_rng(6)
    rp, cl, vl = random_csr(rng, 32, 64, density=0.2)
    path = str(tmp_path / "a.hrpb")
    cs.HRPB(32, 64, rp, cl, vl).save(path)
    good = open(path, "rb").read()

    def rejected(data, status=-9):
        p = str(tmp_path / "bad.hrpb")
        open(p, "wb").write(data)
        with pytest.raises(cs.CuteError) as e:
            cs.HRPB.load(p)
        assert e.value.status == status

    rejected(b"NOTAFILE" + good[8:])                               # magic
    rejected(good[:8] + struct.pack("<I", 2) + good[12:])          # version
    rejected(good[:-1])                                            # truncated
    rejected(good + b"\0")                                         # trailing bytes
    rejected(good[:100] + bytes([good[100] ^ 1]) + good[101:])     # one flipped payload bit
    rejected(good[:24] + struct.pack("<I", 48) + good[28:])        # header disagrees with the payload length
    rejected(good[:30])                                            # shorter than the header
    with pytest.raises(cs.CuteError) as e:
        cs.HRPB.load(str(tmp_path / "missing.hrpb"))
    assert e.value.status == -1
