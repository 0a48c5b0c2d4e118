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
    rejected(good[:8] + struct.pack("<I", 1) + good[12:])          # version
    rejected(good[:-1])                                            # truncated
    rejected(good + b"\0")                                         # trailing bytes
    rejected(good[:100] + bytes([good[100] ^ 1]) + good[101:])     # one flipped payload bit
    rejected(good[:24] + struct.pack("<I", 48) + good[28:])        # header disagrees with the payload length
    rejected(good[:30])                                            # shorter than the header
    with pytest.raises(cs.CuteError) as e:
        cs.HRPB.load(str(tmp_path / "missing.hrpb"))
    assert e.value.status == -1


def _fnv1a(data):
    h = 0xcbf29ce484222325
    for b in data:
        h = ((h ^ b) * 0x100000001b3) & 0xFFFFFFFFFFFFFFFF
    return h


def _resealed(data):
    """The same bytes with the checksum field recomputed, as a forger (not an accident) would leave them."""
    return data[:56] + struct.pack("<Q", _fnv1a(data[:56] + data[64:])) + data[64:]


def test_header_is_covered_by_the_checksum(cs, tmp_path):
    rng = np.random.default_rng(7)
    rp, cl, vl = random_csr(rng, 32, 64, density=0.2)
    path = str(tmp_path / "a.hrpb")
    cs.HRPB(32, 64, rp, cl, vl).save(path)
    good = open(path, "rb").read()
    assert _resealed(good) == good                                 # the test's idea of the checksum is the library's
    for off, val in ((28, 48), (28, 80), (44, 1)):                 # K smaller, K larger, brick count
        bad = good[:off] + struct.pack("<I", val) + good[off + 4:]
        p = str(tmp_path / "bad.hrpb")
        open(p, "wb").write(bad)
        with pytest.raises(cs.CuteError) as e:
            cs.HRPB.load(p)
        assert e.value.status == -9


def test_forged_contents_are_rejected(cs, tmp_path):
    """A file whose checksum is right but whose arrays would send a consumer out of bounds."""
    rng = np.random.default_rng(8)
    M, K = 32, 64
    rp, cl, vl = random_csr(rng, M, K, density=0.2)
    h = cs.HRPB(M, K, rp, cl, vl)
    path = str(tmp_path / "a.hrpb")
    h.save(path)
    good = open(path, "rb").read()
    nb, P, nnz, words = h.numBlocks, h.numRowPanels, h.numNNZ, h.numWords
    off_brp = 64
    off_act = off_brp + 4 * (P + 1)
    off_sp = off_act + 4 * nb * 16
    off_data = off_sp + 8 * (nb + 1)
    off_rp = off_data + 4 * words
    off_cols = off_rp + 4 * (M + 1)

    def patched(off, fmt, val):
        return _resealed(good[:off] + struct.pack(fmt, val) + good[off + struct.calcsize(fmt):])

    assert cl.max() >= 48
    cases = {
        "K below the largest column": patched(28, "<I", 48),
        "a column beyond K": patched(off_cols, "<I", K),
        "an active column beyond K": patched(off_act + 4, "<I", K + 5),
        "nnz in the header": patched(32, "<I", nnz - 1),
        "row pointers that descend": patched(off_rp + 4 * 3, "<I", nnz + 7),
        "panel pointers that descend": patched(off_brp + 4, "<I", nb + 1),
        "a record offset off the chunk grid": patched(off_sp + 8, "<Q", 64),
        "a record offset beyond the stream": patched(off_sp + 8, "<Q", words + 128),
        "a record that states another size": patched(off_data + 4 * 26, "<I", 9),
        "a bitmap with one more bit": patched(off_data + 4 * 28, "<I", 0xFFFFFFFF),
    }
    for what, data in cases.items():
        p = str(tmp_path / "forged.hrpb")
        open(p, "wb").write(data)
        with pytest.raises(cs.CuteError) as e:
            cs.HRPB.load(p)
        assert e.value.status == -9, what
