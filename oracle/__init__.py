"""ctypes/numpy front end of the CPU oracle (``cute_oracle.c``).

TEST INFRASTRUCTURE ONLY: importable from ``tests/``, the smoke check and the
benchmark's CPU-baseline leg.  The shipped package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcute_oracle.so")
_lib = None


def build(force=False):
    """Compile ``cute_oracle.c`` with the Makefile beside it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_partition.restype = C.c_uint32
        _lib.orc_check_gemm.restype = C.c_float
        _lib.orc_free.argtypes = [C.c_void_p]
    return _lib


def _p(a, t):
    return a.ctypes.data_as(C.POINTER(t))


def _take(ptr, n, dtype):
    """Copy n items from a malloc'ed pointer into a numpy array and free it."""
    out = np.ctypeslib.as_array(ptr, shape=(max(int(n), 1),)).astype(dtype, copy=True)[: int(n)]
    lib().orc_free(C.cast(ptr, C.c_void_p))
    return out


def mtx_read(path):
    """IO.cu:10-87 -> (M, K, nnz, rowPtr, cols, vals)."""
    M, K, nnz = C.c_uint32(), C.c_uint32(), C.c_uint32()
    rp, cl, vl = C.POINTER(C.c_uint32)(), C.POINTER(C.c_uint32)(), C.POINTER(C.c_float)()
    rc = lib().orc_mtx_read(os.fsencode(path), C.byref(M), C.byref(K), C.byref(nnz),
                            C.byref(rp), C.byref(cl), C.byref(vl))
    if rc:
        raise IOError("orc_mtx_read(%s) failed: %d" % (path, rc))
    total = rp[M.value]
    return (M.value, K.value, nnz.value, _take(rp, M.value + 1, np.uint32),
            _take(cl, total, np.uint32), _take(vl, total, np.float32))


def hrpb_build(M, K, rowPtr, cols, vals):
    """data.cu:94-335 -> dict of the four canonical arrays."""
    rowPtr = np.ascontiguousarray(rowPtr, np.uint32)
    cols = np.ascontiguousarray(cols, np.uint32)
    vals = np.ascontiguousarray(vals, np.float32)
    brp, ac, bd = (C.POINTER(C.c_uint32)() for _ in range(3))
    sp = C.POINTER(C.c_uint64)()
    nb, nw = C.c_uint32(), C.c_uint64()
    rc = lib().orc_hrpb_build(C.c_uint32(M), C.c_uint32(K), _p(rowPtr, C.c_uint32), _p(cols, C.c_uint32),
                              _p(vals, C.c_float), C.byref(brp), C.byref(ac), C.byref(sp), C.byref(bd),
                              C.byref(nb), C.byref(nw))
    if rc:
        raise ValueError("orc_hrpb_build failed: %d" % rc)
    P = M // 16
    return dict(M=M, K=K, numRowPanels=P, numBlocks=nb.value, numWords=nw.value,
                blockedRowPtr=_take(brp, P + 1, np.uint32),
                activeCols=_take(ac, nb.value * 16, np.uint32),
                sizePtr=_take(sp, nb.value + 1, np.uint64),
                blocksData=_take(bd, nw.value, np.uint32))


def partition(blockedRowPtr, nbN, slots):
    """spmm.cu:776-812 -> uint32 array [n,4] of {start,end,panel,atomic}."""
    brp = np.ascontiguousarray(blockedRowPtr, np.uint32)
    P = len(brp) - 1
    cap = int(brp[-1]) + P + 1
    out = np.zeros((cap, 4), np.uint32)
    n = lib().orc_partition(C.c_uint32(P), _p(brp, C.c_uint32), C.c_uint32(nbN), C.c_uint32(slots),
                            _p(out, C.c_uint32), C.c_uint32(cap))
    assert n <= cap
    return out[:n].copy()


def spmm_coo(rows, cols, vals, B, M, inner_parallel=False):
    """inc.h:71-83.  inner_parallel=True keeps the reference's placement of the parallel loop
    (inside the loop over nonzeros); the result is the same, bit for bit."""
    rows = np.ascontiguousarray(rows, np.uint32)
    cols = np.ascontiguousarray(cols, np.uint32)
    vals = np.ascontiguousarray(vals, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    K, N = B.shape
    Cm = np.empty((M, N), np.float32)
    fn = lib().orc_spmm_coo_inner_parallel if inner_parallel else lib().orc_spmm_coo
    fn(_p(rows, C.c_uint32), _p(cols, C.c_uint32), _p(vals, C.c_float), _p(B, C.c_float),
       _p(Cm, C.c_float), C.c_uint32(M), C.c_uint32(K), C.c_uint32(N), C.c_uint32(len(vals)))
    return Cm


def spmm_csr(rowPtr, cols, vals, B, out=None):
    rowPtr = np.ascontiguousarray(rowPtr, np.uint32)
    cols = np.ascontiguousarray(cols, np.uint32)
    vals = np.ascontiguousarray(vals, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    M, N = len(rowPtr) - 1, B.shape[1]
    Cm = np.empty((M, N), np.float32) if out is None else out
    lib().orc_spmm_csr(_p(rowPtr, C.c_uint32), _p(cols, C.c_uint32), _p(vals, C.c_float), _p(B, C.c_float),
                       _p(Cm, C.c_float), C.c_uint32(M), C.c_uint32(N))
    return Cm


def spmm_hrpb(h, B):
    B = np.ascontiguousarray(B, np.float32)
    N = B.shape[1]
    Cm = np.empty((h["M"], N), np.float32)
    lib().orc_spmm_hrpb(C.c_uint32(h["M"]), C.c_uint32(N), _p(h["blockedRowPtr"], C.c_uint32),
                        _p(h["activeCols"], C.c_uint32), _p(h["sizePtr"], C.c_uint64),
                        _p(h["blocksData"], C.c_uint32), _p(B, C.c_float), _p(Cm, C.c_float))
    return Cm


def check_gemm(C_ref, C_test):
    """inc.h:84-109; the first argument is the trusted result."""
    a = np.ascontiguousarray(C_ref, np.float32)
    b = np.ascontiguousarray(C_test, np.float32)
    assert a.shape == b.shape
    M, N = a.shape
    return float(lib().orc_check_gemm(_p(a, C.c_float), _p(b, C.c_float), C.c_uint32(M), C.c_uint32(N)))


# ---------------------------------------------------------------- second API family
def coo_read(path):
    """inc/SparseCoo.hpp:91-157 -> (dimY, dimX, nnz, rows, cols, values)."""
    dy, dx, nnz = C.c_int(), C.c_int(), C.c_int()
    r, c, v = C.POINTER(C.c_int)(), C.POINTER(C.c_int)(), C.POINTER(C.c_float)()
    rc = lib().orc_coo_read(os.fsencode(path), C.byref(dy), C.byref(dx), C.byref(nnz), C.byref(r), C.byref(c), C.byref(v))
    if rc:
        raise IOError("orc_coo_read(%s) failed: %d" % (path, rc))
    return (dy.value, dx.value, nnz.value, _take(r, nnz.value, np.int32), _take(c, nnz.value, np.int32),
            _take(v, nnz.value, np.float32))


def coo_to_csr(nrows, rows, cols, vals):
    rows, cols, vals = (np.ascontiguousarray(rows, np.int32), np.ascontiguousarray(cols, np.int32),
                        np.ascontiguousarray(vals, np.float32))
    rp, co, vo = np.zeros(nrows + 1, np.int32), np.zeros(len(cols), np.int32), np.zeros(len(cols), np.float32)
    lib().orc_coo_to_csr(C.c_int(nrows), C.c_int(len(cols)), _p(rows, C.c_int), _p(cols, C.c_int), _p(vals, C.c_float),
                         _p(rp, C.c_int), _p(co, C.c_int), _p(vo, C.c_float))
    return rp, co, vo


def _csr_i32(rowPtr, cols):
    return np.ascontiguousarray(rowPtr, np.int32), np.ascontiguousarray(cols, np.int32)


def count_blocks(nrows, ncols, rowPtr, cols, R, Cc):
    rowPtr, cols = _csr_i32(rowPtr, cols)
    return int(lib().orc_count_blocks(C.c_int(nrows), C.c_int(ncols), _p(rowPtr, C.c_int), _p(cols, C.c_int), C.c_int(R), C.c_int(Cc)))


def to_bcsr(nrows, ncols, rowPtr, cols, vals, R, Cc):
    rowPtr, cols = _csr_i32(rowPtr, cols)
    vals = np.ascontiguousarray(vals, np.float32)
    nb = count_blocks(nrows, ncols, rowPtr, cols, R, Cc)
    brp, bc, bv = np.zeros(nrows // R + 1, np.int32), np.zeros(nb, np.int32), np.zeros(nb * R * Cc, np.float32)
    lib().orc_to_bcsr(C.c_int(nrows), C.c_int(ncols), _p(rowPtr, C.c_int), _p(cols, C.c_int), _p(vals, C.c_float),
                      C.c_int(R), C.c_int(Cc), _p(brp, C.c_int), _p(bc, C.c_int), _p(bv, C.c_float))
    return brp, bc, bv


def blocked_ell(nrows, ncols, rowPtr, cols, vals, B):
    rowPtr, cols = _csr_i32(rowPtr, cols)
    vals = np.ascontiguousarray(vals, np.float32)
    H, W, nb, ne = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    args = (C.c_int(nrows), C.c_int(ncols), _p(rowPtr, C.c_int), _p(cols, C.c_int), _p(vals, C.c_float), C.c_int(B))
    lib().orc_blocked_ell(*args, C.byref(H), C.byref(W), None, None, C.byref(nb), None)
    idx = np.zeros((H.value, max(W.value, 0)), np.int32)
    val = np.zeros((H.value * B, W.value * B), np.float32)
    lib().orc_blocked_ell(*args, C.byref(H), C.byref(W), _p(idx, C.c_int), _p(val, C.c_float), C.byref(nb), C.byref(ne))
    return dict(height=H.value, width=W.value, num_blocks=nb.value, num_elems=ne.value, ellColIdx=idx, ellValues=val)


def blocked_ell_to_dense(e, B, ncols):
    dense = np.zeros((e["height"] * B, ncols), np.float32)
    lib().orc_blocked_ell_to_dense(C.c_int(e["height"]), C.c_int(e["width"]), C.c_int(B), C.c_int(ncols),
                                   _p(e["ellColIdx"], C.c_int), _p(e["ellValues"], C.c_float), _p(dense, C.c_float))
    return dense


def split(nrows, ncols, rowPtr, cols, tile, threshold):
    rowPtr, cols = _csr_i32(rowPtr, cols)
    which = np.zeros(len(cols), np.uint8)
    counters = np.zeros(5, np.int32)
    lib().orc_split(C.c_int(nrows), C.c_int(ncols), _p(rowPtr, C.c_int), _p(cols, C.c_int), C.c_int(tile),
                    C.c_int(threshold), _p(which, C.c_uint8), _p(counters, C.c_int))
    return which.astype(bool), counters


def block_stats(nrows, ncols, rowPtr, cols, B):
    rowPtr, cols = _csr_i32(rowPtr, cols)
    nbr, nbc = (nrows + B - 1) // B, (ncols + B - 1) // B + 1
    stats = np.zeros((nbr, nbc, 3), np.int32)
    lib().orc_block_stats(C.c_int(nrows), C.c_int(ncols), _p(rowPtr, C.c_int), _p(cols, C.c_int), C.c_int(B), _p(stats, C.c_int))
    return stats


def classify(nnz, under, over, B, deviation_threshold, underload_dominance):
    return int(lib().orc_classify(C.c_int(nnz), C.c_int(under), C.c_int(over), C.c_int(B), C.c_float(deviation_threshold),
                                  C.c_float(underload_dominance)))


def get_stats(nrows, ncols, rowPtr, cols, blocksize):
    """GET_STATS (gpu_kernels.cu:1049-1137): [ANRS, ANCS, non-empty blocks, mean block density] as float32."""
    rowPtr, cols = _csr_i32(rowPtr, cols)
    out = np.zeros(4, np.float32)
    lib().orc_get_stats(C.c_int(nrows), C.c_int(ncols), _p(rowPtr, C.c_int), _p(cols, C.c_int), C.c_int(blocksize),
                        _p(out, C.c_float))
    return out


def get_anxs(nrows, rowPtr, cols, blocksize, axis):
    """GET_ANXS (gpu_kernels.cu:1139-1186)."""
    rowPtr, cols = _csr_i32(rowPtr, cols)
    f = lib().orc_get_anxs
    f.restype = C.c_float
    return float(f(C.c_int(nrows), _p(rowPtr, C.c_int), _p(cols, C.c_int), C.c_int(blocksize), C.c_int(1 if axis else 0)))


def spmm_csr_f64(rowPtr, cols, vals, B):
    rowPtr, cols = _csr_i32(rowPtr, cols)
    vals, B = np.ascontiguousarray(vals, np.float64), np.ascontiguousarray(B, np.float64)
    m, n = len(rowPtr) - 1, B.shape[1]
    out = np.zeros((m, n), np.float64)
    lib().orc_spmm_csr_f64(C.c_int(m), C.c_int(n), _p(rowPtr, C.c_int), _p(cols, C.c_int), _p(vals, C.c_double),
                           _p(B, C.c_double), _p(out, C.c_double))
    return out
