"""Python face of libcutespmm.so (ctypes).  Class and field names follow the reference's
host API: ``MTX_READER`` (IO.cu:2-88), ``HRPB`` (data.cu:54-340), ``SPMM_TC``
(spmm.cu:258-840), ``check_gemm_correctness_coo`` (inc.h:84-109) and
``GPU_CSR_cuSPARSE_NEW`` (spmm.cu:860-960, here a hand-written HIP CSR kernel).

The shared library is the product; this module only marshals numpy arrays and device
pointers into its C ABI.  There is no CPU fallback: device entry points raise
``CuteError`` when the library or a gfx950 device is missing.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("CUTESPMM_LIBRARY") or os.path.join(_HERE, "libcutespmm.so")

# every symbol declared in include/cutespmm.h
ABI_SYMBOLS = [
    "cute_status_string", "cute_last_hip_error", "cute_free",
    "cute_mtx_read", "cute_csr_release", "cute_csr_sort_rows", "cute_csr_merge_duplicates", "cute_coo_merge_duplicates",
    "cute_spmm_coo", "cute_offsets_fit",
    "cute_hrpb_build", "cute_hrpb_host_release",
    "cute_hrpb_retile", "cute_hrpb_untile", "cute_hrpb_tiled_release",
    "cute_quad_build", "cute_quad_fill", "cute_quad_build_strips", "cute_quad_release", "cute_quad_census", "cute_quad_pack", "cute_hrpb_save", "cute_hrpb_load",
    "cute_partition", "cute_check_gemm_correctness", "cute_backward_error",
    "cute_gen_matrix", "cute_gen_dense",
    "cute_hrpb_upload", "cute_hrpb_upload_layout", "cute_hrpb_upload_device_csr", "cute_hrpb_dev_layout_sizes",
    "cute_hrpb_dev_read_layouts", "cute_hrpb_dev_free", "cute_hrpb_dev_bytes", "cute_hrpb_dev_csr",
    "cute_spmm_plan_create", "cute_spmm_plan_info", "cute_spmm_plan_free", "cute_spmm_run", "cute_spmm_run_static",
    "cute_spmm_run_scratch", "cute_spmm_plan_scratch_bytes", "cute_device_layout",
    "cute_csr_spmm_dev", "cute_gpu_csr_spmm", "cute_spmm_time", "cute_csr_spmm_time",
    "cute_device_info",
    "cute_coo_read", "cute_coo_save_mtx", "cute_coo_release", "cute_coo_to_csr", "cute_csr_i32_release",
    "cute_csr_to_dense", "cute_csr_count_blocks", "cute_csr_to_bcsr", "cute_bcsr_release",
    "cute_blocked_ell_build", "cute_blocked_ell_to_dense", "cute_blocked_ell_release",
    "cute_blocked_ell_upload", "cute_blocked_ell_dev_free", "cute_blocked_ell_spmm",
    "cute_splitter_split", "cute_split_release", "cute_classify_blocks", "cute_sequential_spmm",
    "cute_block_stats", "cute_anxs",
    "cute_split_by_class", "cute_hybrid_create", "cute_hybrid_get_info", "cute_hybrid_spmm", "cute_hybrid_free",
]

u32p = C.POINTER(C.c_uint32)
u64p = C.POINTER(C.c_uint64)
f32p = C.POINTER(C.c_float)


class CuteError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = "%s: %s (%d)" % (where, _status_string(status), status)
        if status in (-7, -8, -10):
            msg += " -- " + _last_hip_error()
        super().__init__(msg)


class cute_csr(C.Structure):
    _fields_ = [("M", C.c_uint32), ("K", C.c_uint32), ("nnz", C.c_uint32),
                ("rowPtr", u32p), ("cols", u32p), ("vals", f32p)]


class cute_hrpb_host(C.Structure):
    _fields_ = [("M", C.c_uint32), ("K", C.c_uint32), ("numRowPanels", C.c_uint32), ("numBlocks", C.c_uint32),
                ("numWords", C.c_uint64), ("blockedRowPtr", u32p), ("activeCols", u32p), ("sizePtr", u64p),
                ("blocksData", u32p), ("rowPtr", u32p), ("cols", u32p), ("vals", f32p),
                ("nnz", C.c_uint32), ("numBricks", C.c_uint32)]


class cute_hrpb_tiled(C.Structure):
    _fields_ = [("M", C.c_uint32), ("K", C.c_uint32), ("numRowPanels", C.c_uint32), ("numBlocks", C.c_uint32),
                ("numVals", C.c_uint64), ("blockedRowPtr", u32p), ("hdr", u32p), ("vals", f32p)]


class cute_quad_lists(C.Structure):
    _fields_ = [("M", C.c_uint32), ("K", C.c_uint32), ("numRowPanels", C.c_uint32), ("numGroups", C.c_uint64),
                ("groupPtr", u32p), ("cols", u32p), ("vals", f32p), ("tail", u32p), ("numPairs", C.c_uint64),
                ("rowsPerList", C.c_uint32)]


class cute_tunables(C.Structure):
    _fields_ = [("path", C.c_int32), ("precision", C.c_int32), ("min_reuse", C.c_float), ("slots", C.c_uint32),
                ("max_chunk_blocks", C.c_uint32), ("brick_groups", C.c_uint32), ("pipeline", C.c_uint32), ("mfma_shape", C.c_uint32), ("max_row_nnz", C.c_uint32),
                ("chunk_order", C.c_uint32), ("operand_residency", C.c_uint32), ("hub_rows", C.c_uint32)]


class cute_plan_info(C.Structure):
    _fields_ = [("N", C.c_uint32), ("slabWidth", C.c_uint32), ("numSlabs", C.c_uint32), ("numChunks", C.c_uint32),
                ("numAtomicChunks", C.c_uint32), ("numBrickPanels", C.c_uint32), ("numRowPanelsSparse", C.c_uint32),
                ("numEmptyPanels", C.c_uint32), ("slots", C.c_uint32), ("precision", C.c_uint32),
                ("path", C.c_uint32), ("mfmaShape", C.c_uint32), ("pipeline", C.c_uint32),
                ("fusedLaunch", C.c_uint32), ("dealtChunks", C.c_uint32), ("partialTileKiB", C.c_uint32), ("hubRows", C.c_uint32)]


i32p = C.POINTER(C.c_int32)


class cute_coo(C.Structure):
    _fields_ = [("dimY", C.c_int32), ("dimX", C.c_int32), ("nnz", C.c_int32), ("rows", i32p), ("cols", i32p),
                ("values", f32p)]


class cute_csr_i32(C.Structure):
    _fields_ = [("nrows", C.c_int32), ("ncols", C.c_int32), ("nnz", C.c_int32), ("rowPtr", i32p), ("cols", i32p),
                ("values", f32p)]


class cute_bcsr(C.Structure):
    _fields_ = [("R", C.c_int32), ("C", C.c_int32), ("nrows", C.c_int32), ("ncols", C.c_int32), ("nblks", C.c_int32),
                ("rowPtr", i32p), ("cols", i32p), ("values", f32p)]


class cute_blocked_ell(C.Structure):
    _fields_ = [("blockSize", C.c_int32), ("height", C.c_int32), ("width", C.c_int32), ("numBlocks", C.c_int32),
                ("numElems", C.c_int32), ("ellColIdx", i32p), ("ellValues", f32p)]


class cute_split(C.Structure):
    _fields_ = [("totalTiles", C.c_int32), ("numHeavyTiles", C.c_int32), ("numHeavyElems", C.c_int32),
                ("numLightTiles", C.c_int32), ("numLightElems", C.c_int32), ("heavy", cute_coo), ("light", cute_coo)]


class cute_hybrid_info(C.Structure):
    _fields_ = [("tileSize", C.c_int32), ("threshold", C.c_int32), ("mode", C.c_int32), ("totalTiles", C.c_int32),
                ("heavyTiles", C.c_int32), ("heavyElems", C.c_int32), ("lightTiles", C.c_int32), ("lightElems", C.c_int32),
                ("ellHeight", C.c_int32), ("ellWidth", C.c_int32), ("stats", C.c_float * 4)]


class cute_block_class(C.Structure):
    _fields_ = [("blockRow", C.c_int32), ("blockCol", C.c_int32), ("nnz", C.c_int32), ("underloads", C.c_int32),
                ("overloads", C.c_int32), ("kind", C.c_int32)]


STATIC_SCRATCH_BYTES = 32 << 20      # CUTE_STATIC_SCRATCH_BYTES
PATH_AUTO, PATH_BRICK, PATH_ROWS = 0, 1, 2
PREC_FP32, PREC_BF16X3 = 0, 1

_lib = None


def load_library():
    """Loads libcutespmm.so; raises if it has not been built (no fallback exists)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise CuteError(-8, "libcutespmm.so is not built (run python -m cutespmm_ae_amd.build); no fallback path")
    # torch carries its own copy of the HIP runtime.  Importing it first makes the dynamic
    # loader bind this library to that same copy (matching SONAME); loaded the other way
    # round the process would hold two HIP runtimes and the second one finds no device.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(LIB_PATH)
    lib.cute_status_string.restype = C.c_char_p
    lib.cute_status_string.argtypes = [C.c_int]
    lib.cute_last_hip_error.restype = C.c_char_p
    lib.cute_free.argtypes = [C.c_void_p]
    lib.cute_mtx_read.argtypes = [C.c_char_p, C.c_int, C.POINTER(cute_csr)]
    lib.cute_csr_release.argtypes = [C.POINTER(cute_csr)]
    lib.cute_csr_sort_rows.argtypes = [C.POINTER(cute_csr)]
    lib.cute_csr_merge_duplicates.argtypes = [C.POINTER(cute_csr)]
    lib.cute_spmm_coo.argtypes = [u32p, u32p, f32p, f32p, f32p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32]
    lib.cute_offsets_fit.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64]
    lib.cute_hrpb_build.argtypes = [C.c_uint32, C.c_uint32, u32p, u32p, f32p, C.POINTER(cute_hrpb_host)]
    lib.cute_hrpb_host_release.argtypes = [C.POINTER(cute_hrpb_host)]
    lib.cute_hrpb_retile.argtypes = [C.POINTER(cute_hrpb_host), C.POINTER(cute_hrpb_tiled)]
    lib.cute_hrpb_untile.argtypes = [C.POINTER(cute_hrpb_tiled), C.POINTER(cute_hrpb_host)]
    lib.cute_hrpb_tiled_release.argtypes = [C.POINTER(cute_hrpb_tiled)]
    lib.cute_quad_build.argtypes = [C.c_uint32, C.c_uint32, u32p, u32p, f32p, C.POINTER(cute_quad_lists)]
    lib.cute_quad_build_strips.argtypes = lib.cute_quad_build.argtypes
    lib.cute_quad_census.argtypes = [C.c_uint32, u32p, u32p, f32p, u32p, u32p]
    lib.cute_quad_pack.argtypes = [C.c_uint32, u32p, u32p, f32p, C.c_uint32, u32p, u64p, u32p, f32p]
    lib.cute_hrpb_upload_layout.argtypes = [C.POINTER(cute_hrpb_host), C.c_int, C.POINTER(C.c_void_p)]
    lib.cute_quad_release.argtypes = [C.POINTER(cute_quad_lists)]
    lib.cute_quad_release.restype = None
    lib.cute_blocked_ell_upload.argtypes = [C.POINTER(cute_blocked_ell), C.POINTER(C.c_void_p)]
    lib.cute_blocked_ell_dev_free.argtypes = [C.c_void_p]
    lib.cute_blocked_ell_dev_free.restype = None
    lib.cute_blocked_ell_spmm.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_int, C.c_void_p]
    lib.cute_hrpb_save.argtypes = [C.POINTER(cute_hrpb_host), C.c_char_p]
    lib.cute_hrpb_load.argtypes = [C.c_char_p, C.POINTER(cute_csr), C.POINTER(cute_hrpb_host)]
    lib.cute_partition.restype = C.c_int64
    lib.cute_partition.argtypes = [C.c_uint32, u32p, C.c_uint32, C.c_uint32, u32p, C.c_uint64]
    lib.cute_check_gemm_correctness.restype = C.c_float
    lib.cute_check_gemm_correctness.argtypes = [f32p, f32p, C.c_uint32, C.c_uint32]
    lib.cute_backward_error.restype = C.c_float
    lib.cute_backward_error.argtypes = [u32p, u32p, f32p, f32p, f32p, f32p, C.c_uint32, C.c_uint32]
    lib.cute_gen_matrix.argtypes = [C.c_int, C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32, C.POINTER(cute_csr)]
    lib.cute_gen_dense.argtypes = [C.c_uint64, C.c_int, C.c_uint64, f32p]
    lib.cute_hrpb_upload.argtypes = [C.POINTER(cute_hrpb_host), C.POINTER(C.c_void_p)]
    lib.cute_hrpb_dev_free.argtypes = [C.c_void_p]
    lib.cute_hrpb_upload_device_csr.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                                C.POINTER(C.c_void_p)]
    lib.cute_hrpb_dev_layout_sizes.argtypes = [C.c_void_p, u32p, u64p, u64p, u64p, u32p]
    lib.cute_hrpb_dev_read_layouts.argtypes = [C.c_void_p, u32p, u32p, f32p, u32p, u32p, f32p]
    lib.cute_hrpb_dev_bytes.restype = C.c_uint64
    lib.cute_hrpb_dev_bytes.argtypes = [C.c_void_p]
    lib.cute_hrpb_dev_csr.argtypes = [C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p)]
    lib.cute_spmm_plan_create.argtypes = [C.c_void_p, C.c_uint32, C.POINTER(cute_tunables), C.POINTER(C.c_void_p)]
    lib.cute_spmm_plan_info.argtypes = [C.c_void_p, C.POINTER(cute_plan_info)]
    lib.cute_spmm_plan_free.argtypes = [C.c_void_p]
    lib.cute_spmm_run.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.cute_spmm_run_static.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.cute_spmm_run_scratch.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64]
    lib.cute_spmm_plan_scratch_bytes.restype = C.c_uint64
    lib.cute_spmm_plan_scratch_bytes.argtypes = [C.c_void_p]
    lib.cute_device_layout.argtypes = [C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_uint64), C.POINTER(C.c_int)]
    lib.cute_csr_spmm_dev.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_uint32, C.c_uint32, C.c_void_p]
    lib.cute_gpu_csr_spmm.restype = C.c_float
    lib.cute_gpu_csr_spmm.argtypes = [u32p, u32p, f32p, C.c_uint32, f32p, f32p, C.c_uint32, C.c_uint32, C.c_uint32,
                                      C.c_int, C.c_int]
    lib.cute_spmm_time.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, f32p]
    lib.cute_csr_spmm_time.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p,
                                       C.c_int, C.c_int, f32p]
    lib.cute_device_info.argtypes = [C.POINTER(C.c_int), C.POINTER(C.c_int), C.c_char_p, C.c_size_t]
    lib.cute_coo_read.argtypes = [C.c_char_p, C.POINTER(cute_coo)]
    lib.cute_coo_merge_duplicates.argtypes = [C.POINTER(cute_coo)]
    lib.cute_coo_save_mtx.argtypes = [C.POINTER(cute_coo), C.c_char_p]
    lib.cute_coo_release.argtypes = [C.POINTER(cute_coo)]
    lib.cute_coo_to_csr.argtypes = [C.POINTER(cute_coo), C.POINTER(cute_csr_i32)]
    lib.cute_csr_i32_release.argtypes = [C.POINTER(cute_csr_i32)]
    lib.cute_csr_to_dense.argtypes = [C.POINTER(cute_csr_i32), f32p]
    lib.cute_csr_count_blocks.restype = C.c_int64
    lib.cute_csr_count_blocks.argtypes = [C.POINTER(cute_csr_i32), C.c_int32, C.c_int32]
    lib.cute_csr_to_bcsr.argtypes = [C.POINTER(cute_csr_i32), C.c_int32, C.c_int32, C.POINTER(cute_bcsr)]
    lib.cute_bcsr_release.argtypes = [C.POINTER(cute_bcsr)]
    lib.cute_blocked_ell_build.argtypes = [C.POINTER(cute_csr_i32), C.c_int32, C.POINTER(cute_blocked_ell)]
    lib.cute_blocked_ell_to_dense.argtypes = [C.POINTER(cute_blocked_ell), C.c_int32, f32p]
    lib.cute_blocked_ell_release.argtypes = [C.POINTER(cute_blocked_ell)]
    lib.cute_splitter_split.argtypes = [C.POINTER(cute_csr_i32), C.c_int32, C.c_int32, C.POINTER(cute_split)]
    lib.cute_split_release.argtypes = [C.POINTER(cute_split)]
    lib.cute_classify_blocks.argtypes = [C.POINTER(cute_csr_i32), C.c_int32, C.c_float, C.c_float,
                                         C.POINTER(C.POINTER(cute_block_class)), C.POINTER(C.c_int64)]
    lib.cute_block_stats.argtypes = [C.POINTER(cute_csr_i32), C.c_int32, f32p]
    lib.cute_split_by_class.argtypes = [C.POINTER(cute_csr_i32), C.c_int32, C.c_float, C.c_float, C.POINTER(cute_split)]
    lib.cute_hybrid_create.argtypes = [C.POINTER(cute_csr_i32), C.c_int32, C.c_int32, C.c_int32, C.c_float, C.c_float,
                                       C.POINTER(C.c_void_p)]
    lib.cute_hybrid_get_info.argtypes = [C.c_void_p, C.POINTER(cute_hybrid_info)]
    lib.cute_hybrid_spmm.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p]
    lib.cute_hybrid_free.argtypes = [C.c_void_p]
    lib.cute_hybrid_free.restype = None
    lib.cute_anxs.argtypes = [C.POINTER(cute_csr_i32), C.c_int32, C.c_int32, f32p]
    lib.cute_sequential_spmm.restype = C.c_float
    lib.cute_sequential_spmm.argtypes = [C.POINTER(cute_csr_i32), C.POINTER(C.c_double), C.POINTER(C.c_double),
                                         C.POINTER(C.c_double), C.c_int32, C.c_int32, C.c_int32]
    _lib = lib
    return lib


def _status_string(s):
    try:
        return load_library().cute_status_string(int(s)).decode()
    except Exception:  # library missing: still produce a readable message
        return "status"


def _last_hip_error():
    try:
        return load_library().cute_last_hip_error().decode()
    except Exception:
        return ""


def _check(rc, where):
    if rc != 0:
        raise CuteError(rc, where)


def _as(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _ptr(a, t):
    return a.ctypes.data_as(t)


class _Owned(np.ndarray):
    """ndarray view of library-owned memory that keeps its owner object alive."""
    _owner = None


def _view(ptr, n, dtype, owner=None):
    n = int(n)
    if n == 0:
        return np.zeros(0, dtype)
    a = np.ctypeslib.as_array(ptr, shape=(n,)).view(dtype).view(_Owned)
    a._owner = owner
    return a


# --------------------------------------------------------------------------------------
# loaders / generators
# --------------------------------------------------------------------------------------
class CSR:
    """Owner of a ``cute_csr``; fields M, K, nnz, rowPtr, cols, vals (numpy views)."""

    def __init__(self, raw):
        self._raw = raw
        self.M, self.K, self.nnz = raw.M, raw.K, raw.nnz
        self._attach()

    def _attach(self):
        raw = self._raw
        self.rowPtr = _view(raw.rowPtr, raw.M + 1, np.uint32, self._keep)
        self.cols = _view(raw.cols, raw.nnz, np.uint32, self._keep)
        self.vals = _view(raw.vals, raw.nnz, np.float32, self._keep)

    @property
    def _keep(self):
        # the arrays outlive this wrapper if somebody still holds a view of them
        if not hasattr(self, "_guard"):
            self._guard = _CsrGuard(self._raw)
        return self._guard

    def sort_rows(self):
        _check(load_library().cute_csr_sort_rows(C.byref(self._raw)), "cute_csr_sort_rows")
        return self

    def merge_duplicates(self):
        """Sorts the rows and adds up entries that share a position (in file order); nnz shrinks."""
        _check(load_library().cute_csr_merge_duplicates(C.byref(self._raw)), "cute_csr_merge_duplicates")
        self.nnz = self._raw.nnz
        self._attach()
        return self


class _CsrGuard:
    def __init__(self, raw):
        self.raw = raw

    def __del__(self):
        try:
            load_library().cute_csr_release(C.byref(self.raw))
        except Exception:
            pass


class MTX_READER(CSR):
    """``MTX_READER(path)``: MatrixMarket file -> CSR with the reference's quirks
    (dims padded to 16, symmetric mirrored, all values 1.0f unless ``keep_values``)."""

    def __init__(self, file_path, keep_values=False):
        raw = cute_csr()
        _check(load_library().cute_mtx_read(os.fsencode(file_path), int(bool(keep_values)), C.byref(raw)),
               "cute_mtx_read(%s)" % file_path)
        super().__init__(raw)


# stock parameters of the five benchmark configurations
CONFIGS = {
    1: dict(kind=1, p0=4096, p1=16, p2=0, N=32, name="uniform_4096_16nnz_N32"),
    2: dict(kind=2, p0=256, p1=0, p2=0, N=128, name="stencil9_256x256_N128"),
    3: dict(kind=3, p0=8000, p1=200, p2=0, N=128, name="fem_8000x6x6_N128"),
    4: dict(kind=4, p0=17, p1=10, p2=0, N=64, name="rmat_2p17_deg10_N64"),
    5: dict(kind=5, p0=1048576, p1=32, p2=2048, N=256, name="banded_1M_32nnz_N256"),
}
SEED_BASE = 0xC07E5B00


def gen_matrix(kind, seed, p0, p1=0, p2=0):
    raw = cute_csr()
    _check(load_library().cute_gen_matrix(int(kind), C.c_uint64(seed), int(p0), int(p1), int(p2), C.byref(raw)),
           "cute_gen_matrix")
    return CSR(raw)


def gen_config(cfg, scale=1.0):
    """Matrix of benchmark configuration ``cfg`` (1..5); ``scale`` < 1 shrinks the row count."""
    c = CONFIGS[cfg]
    p0 = c["p0"]
    if scale != 1.0:
        if c["kind"] == 2:
            p0 = max(16, int(p0 * scale ** 0.5) // 16 * 16)
        elif c["kind"] == 4:
            p0 = max(8, int(round(p0 + np.log2(scale))))
        elif c["kind"] == 3:
            p0 = max(64, int(p0 * scale) // 8 * 8)
        else:
            p0 = max(256, int(p0 * scale) // 16 * 16)
    return gen_matrix(c["kind"], SEED_BASE + cfg, p0, c["p1"], c["p2"])


def gen_dense(seed, rows, cols, dist=2):
    """dist 0: U(0,1), 1: U(-1,1), 2: N(0,1).  Element i depends only on (seed, i)."""
    out = np.empty((rows, cols), np.float32)
    _check(load_library().cute_gen_dense(C.c_uint64(seed), int(dist), C.c_uint64(rows * cols), _ptr(out, f32p)),
           "cute_gen_dense")
    return out


# --------------------------------------------------------------------------------------
# format
# --------------------------------------------------------------------------------------
class HRPB:
    """``HRPB(M, K, rowPtr, cols, vals)``: canonical arrays as public fields
    (blockedRowPtr, activeCols, sizePtr, blocksData, numRowPanels) as in data.cu:56-72.
    ``upload()`` creates the device twin (data.cu:327-334); ``freeDevice()`` drops it."""

    def __init__(self, M, K, rowPtr, cols, vals):
        self.rowPtr = _as(rowPtr, np.uint32)
        self.cols = _as(cols, np.uint32)
        self.vals = _as(vals, np.float32)
        self._raw = cute_hrpb_host()
        self._dev = C.c_void_p()
        _check(load_library().cute_hrpb_build(int(M), int(K), _ptr(self.rowPtr, u32p), _ptr(self.cols, u32p),
                                              _ptr(self.vals, f32p), C.byref(self._raw)), "cute_hrpb_build")
        self._publish()

    def _publish(self):
        r = self._raw
        self.M, self.K = r.M, r.K
        self.numRowPanels, self.numBlocks, self.numWords = r.numRowPanels, r.numBlocks, r.numWords
        self.num_bricks, self.numNNZ = r.numBricks, r.nnz
        self._guard = _HrpbGuard(r, self._dev)
        self.blockedRowPtr = _view(r.blockedRowPtr, r.numRowPanels + 1, np.uint32, self._guard)
        self.activeCols = _view(r.activeCols, r.numBlocks * 16, np.uint32, self._guard)
        self.sizePtr = _view(r.sizePtr, r.numBlocks + 1, np.uint64, self._guard)
        self.blocksData = _view(r.blocksData, r.numWords, np.uint32, self._guard)

    def save(self, path):
        """Writes the CSR arrays and the canonical format to a versioned, checksummed binary file."""
        _check(load_library().cute_hrpb_save(C.byref(self._raw), os.fsencode(path)), "cute_hrpb_save")

    @classmethod
    def load(cls, path):
        """The object a previous ``save`` wrote, without reading or converting the matrix again."""
        lib = load_library()
        self = cls.__new__(cls)
        csr = cute_csr()
        self._raw = cute_hrpb_host()
        self._dev = C.c_void_p()
        _check(lib.cute_hrpb_load(os.fsencode(path), C.byref(csr), C.byref(self._raw)), "cute_hrpb_load")
        # the CSR arrays move into numpy-owned memory, which the format object then borrows
        self.rowPtr = _view(csr.rowPtr, csr.M + 1, np.uint32).copy()
        self.cols = _view(csr.cols, csr.nnz, np.uint32).copy()
        self.vals = _view(csr.vals, csr.nnz, np.float32).copy()
        lib.cute_csr_release(C.byref(csr))
        self._raw.rowPtr, self._raw.cols, self._raw.vals = _ptr(self.rowPtr, u32p), _ptr(self.cols, u32p), _ptr(self.vals, f32p)
        self._publish()
        return self

    def as_dict(self):
        return dict(M=self.M, K=self.K, numRowPanels=self.numRowPanels, numBlocks=self.numBlocks,
                    numWords=self.numWords, blockedRowPtr=self.blockedRowPtr, activeCols=self.activeCols,
                    sizePtr=self.sizePtr, blocksData=self.blocksData)

    def retile(self):
        """Host copy of the MFMA-tiled device layout: dict(hdr[nb,32], vals, blockedRowPtr)."""
        t = cute_hrpb_tiled()
        _check(load_library().cute_hrpb_retile(C.byref(self._raw), C.byref(t)), "cute_hrpb_retile")
        out = dict(numBlocks=t.numBlocks, numVals=t.numVals,
                   hdr=_view(t.hdr, t.numBlocks * 32, np.uint32).reshape(-1, 32).copy(),
                   vals=_view(t.vals, t.numVals, np.float32).copy(),
                   blockedRowPtr=_view(t.blockedRowPtr, t.numRowPanels + 1, np.uint32).copy())
        load_library().cute_hrpb_tiled_release(C.byref(t))
        return out

    def retile_roundtrip(self):
        """retile then untile; returns the canonical arrays rebuilt from the tiled form."""
        lib = load_library()
        t, back = cute_hrpb_tiled(), cute_hrpb_host()
        _check(lib.cute_hrpb_retile(C.byref(self._raw), C.byref(t)), "cute_hrpb_retile")
        rc = lib.cute_hrpb_untile(C.byref(t), C.byref(back))
        lib.cute_hrpb_tiled_release(C.byref(t))
        _check(rc, "cute_hrpb_untile")
        out = dict(numBlocks=back.numBlocks, numWords=back.numWords, nnz=back.nnz, numBricks=back.numBricks,
                   blockedRowPtr=_view(back.blockedRowPtr, back.numRowPanels + 1, np.uint32).copy(),
                   activeCols=_view(back.activeCols, back.numBlocks * 16, np.uint32).copy(),
                   sizePtr=_view(back.sizePtr, back.numBlocks + 1, np.uint64).copy(),
                   blocksData=_view(back.blocksData, back.numWords, np.uint32).copy())
        lib.cute_hrpb_host_release(C.byref(back))
        return out

    def upload(self, quad_layout=0):
        """Device twin (made once).  quad_layout: 0 library's choice, 1 lockstep lists per panel,
        2 one list per 4-row strip; only the first call's choice counts."""
        if not self._dev:
            _check(load_library().cute_hrpb_upload_layout(C.byref(self._raw), int(quad_layout), C.byref(self._dev)),
                   "cute_hrpb_upload_layout")
        return self._dev

    def device_bytes(self):
        return load_library().cute_hrpb_dev_bytes(self._dev) if self._dev else 0

    def device_layouts(self):
        """Host copies of the layouts the device twin holds (see ``_dev_layouts``)."""
        return _dev_layouts(self.upload(), self.M)

    def freeDevice(self):
        if self._dev:
            load_library().cute_hrpb_dev_free(self._dev)
            self._dev.value = None


class _HrpbGuard:
    """Releases the host arrays and the device twin once the HRPB object and every view
    of its arrays are gone (the CSR arrays it borrows are numpy-owned and kept by HRPB)."""

    def __init__(self, raw, dev):
        self.raw, self.dev = raw, dev

    def __del__(self):
        try:
            lib = load_library()
            if self.dev:
                lib.cute_hrpb_dev_free(self.dev)
            lib.cute_hrpb_host_release(C.byref(self.raw))
        except Exception:
            pass


def partition(blockedRowPtr, nbN, slots):
    """spmm.cu:776-812 arithmetic -> uint32 [n,4] {start, end, panel, atomic}."""
    brp = _as(blockedRowPtr, np.uint32)
    P = len(brp) - 1
    lib = load_library()
    n = lib.cute_partition(P, _ptr(brp, u32p), int(nbN), int(slots), None, 0)
    if n < 0:
        raise CuteError(int(n), "cute_partition")
    out = np.zeros((max(n, 1), 4), np.uint32)
    lib.cute_partition(P, _ptr(brp, u32p), int(nbN), int(slots), _ptr(out, u32p), n)
    return out[:n]


# --------------------------------------------------------------------------------------
# plan + launch
# --------------------------------------------------------------------------------------
def _dev_ptr(t):
    import torch
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
        raise TypeError("expected a contiguous float32 tensor on the GPU")
    return C.c_void_p(t.data_ptr())


def quad_lists(M, K, rowPtr, cols, vals, strips=False):
    """Host copy of the 4x4x1 MFMA kernel's layout built from a CSR matrix:
    dict(groupPtr[U+1], cols[G,16], vals[G,64], tail[U], numPairs, rowsPerList); U = 16-row panels,
    or 4-row strips with ``strips=True``."""
    rowPtr = np.ascontiguousarray(rowPtr, np.uint32)
    cols = np.ascontiguousarray(cols, np.uint32)
    vals = np.ascontiguousarray(vals, np.float32)
    q = cute_quad_lists()
    build = load_library().cute_quad_build_strips if strips else load_library().cute_quad_build
    _check(build(int(M), int(K), _ptr(rowPtr, u32p), _ptr(cols, u32p), _ptr(vals, f32p), C.byref(q)), "cute_quad_build")
    out = dict(numGroups=int(q.numGroups), numPairs=int(q.numPairs), rowsPerList=int(q.rowsPerList),
               tail=_view(q.tail, q.numRowPanels, np.uint32).copy(),
               groupPtr=_view(q.groupPtr, q.numRowPanels + 1, np.uint32).copy(),
               cols=_view(q.cols, q.numGroups * 16, np.uint32).reshape(-1, 16).copy(),
               vals=_view(q.vals, q.numGroups * 64, np.float32).reshape(-1, 64).copy())
    load_library().cute_quad_release(C.byref(q))
    return out


def quad_pack(M, rowPtr, cols, vals, strips=False):
    """The device form of the quad lists as ``cute_hrpb_upload`` builds it, straight from the CSR matrix:
    dict(groupPtr[U+1], recs[G,20] = 16 columns + slot mask (2 words) + first value + 0, packed = stored values)."""
    lib = load_library()
    rowPtr, cols, vals = _as(rowPtr, np.uint32), _as(cols, np.uint32), _as(vals, np.float32)
    S = (int(M) + 3) // 4
    pairs, stored = np.zeros(S, np.uint32), np.zeros(S, np.uint32)
    _check(lib.cute_quad_census(int(M), _ptr(rowPtr, u32p), _ptr(cols, u32p), _ptr(vals, f32p), _ptr(pairs, u32p),
                                _ptr(stored, u32p)), "cute_quad_census")
    if strips:
        groups = (pairs.astype(np.int64) + 15) // 16
        per_unit = stored.astype(np.int64)
    else:
        groups = (pairs.reshape(-1, 4).max(1).astype(np.int64) + 3) // 4
        per_unit = stored.reshape(-1, 4).sum(1).astype(np.int64)
    groupPtr = np.concatenate([[0], np.cumsum(groups)]).astype(np.uint32)
    valBase = np.concatenate([[0], np.cumsum(per_unit)]).astype(np.uint64)
    recs = np.zeros((int(groupPtr[-1]), 20), np.uint32)
    packed = np.zeros(int(valBase[-1]), np.float32)
    _check(lib.cute_quad_pack(int(M), _ptr(rowPtr, u32p), _ptr(cols, u32p), _ptr(vals, f32p), 4 if strips else 16,
                              _ptr(groupPtr, u32p), _ptr(valBase, u64p), _ptr(recs, u32p), _ptr(packed, f32p)), "cute_quad_pack")
    return dict(groupPtr=groupPtr, recs=recs, packed=packed, stripPairs=pairs, stripVals=stored)


def _dev_layouts(dev, M):
    """Host copies of the layouts a device handle holds: dict with hdr [nb,32], tileVals, blockedRowPtr (brick tiles,
    empty if not built) and recs [groups,20], quadVals, groupPtr, rowsPerList (quad lists, empty if not built)."""
    lib = load_library()
    nb, rows = C.c_uint32(), C.c_uint32()
    ntv, ng, nqv = C.c_uint64(), C.c_uint64(), C.c_uint64()
    _check(lib.cute_hrpb_dev_layout_sizes(dev, C.byref(nb), C.byref(ntv), C.byref(ng), C.byref(nqv), C.byref(rows)),
           "cute_hrpb_dev_layout_sizes")
    units = M // rows.value
    out = dict(blockedRowPtr=np.zeros(M // 16 + 1, np.uint32), hdr=np.zeros((nb.value, 32), np.uint32),
               tileVals=np.zeros(ntv.value, np.float32), groupPtr=np.zeros(units + 1, np.uint32),
               recs=np.zeros((ng.value, 20), np.uint32), quadVals=np.zeros(nqv.value, np.float32), rowsPerList=rows.value)
    _check(lib.cute_hrpb_dev_read_layouts(dev, _ptr(out["blockedRowPtr"], u32p), _ptr(out["hdr"], u32p), _ptr(out["tileVals"], f32p),
                                          _ptr(out["groupPtr"], u32p), _ptr(out["recs"], u32p), _ptr(out["quadVals"], f32p)),
           "cute_hrpb_dev_read_layouts")
    return out


class DeviceHRPB:
    """``DeviceHRPB(M, K, rowPtr, cols, vals)`` with int32 / float32 GPU tensors: the format built on the device from a
    CSR matrix that already lives there (HRPB::HRPB + DATASTRUCT, data.cu:80-335, without the host).  Takes the place
    of an ``HRPB`` in ``SPMM_TC(hrpb, N)``."""

    def __init__(self, M, K, rowPtr, cols, vals, quad_layout=0):
        import torch
        for t, dt in ((rowPtr, torch.int32), (cols, torch.int32), (vals, torch.float32)):
            if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dt and t.is_contiguous()):
                raise TypeError("rowPtr and cols must be contiguous int32 GPU tensors, vals a contiguous float32 GPU tensor")
        if rowPtr.numel() != int(M) + 1 or cols.numel() != vals.numel():
            raise ValueError("rowPtr must have M+1 entries, cols and vals one per nonzero")
        self.M, self.K, self.numNNZ = int(M), int(K), int(cols.numel())
        self._dev = C.c_void_p()
        _check(load_library().cute_hrpb_upload_device_csr(self.M, self.K, self.numNNZ, C.c_void_p(rowPtr.data_ptr()),
                                                          C.c_void_p(cols.data_ptr()), C.c_void_p(vals.data_ptr()),
                                                          int(quad_layout), C.byref(self._dev)), "cute_hrpb_upload_device_csr")

    def upload(self, quad_layout=0):
        return self._dev

    def device_bytes(self):
        return load_library().cute_hrpb_dev_bytes(self._dev)

    def layouts(self):
        return _dev_layouts(self._dev, self.M)

    def freeDevice(self):
        if self._dev:
            load_library().cute_hrpb_dev_free(self._dev)
            self._dev = C.c_void_p()

    def __del__(self):
        try:
            self.freeDevice()
        except Exception:
            pass


def _stream_ptr(stream):
    import torch
    s = stream if stream is not None else torch.cuda.current_stream()
    return C.c_void_p(s.cuda_stream)


class SPMM_TC:
    """``SPMM_TC(hrpb, N)`` plans (spmm.cu:276-822); ``run(MatB, MatC)`` launches
    (spmm.cu:823-839) on torch's current stream.  MatB [K,N], MatC [M,N] float32 GPU tensors."""

    def __init__(self, hrpb, N, path=PATH_AUTO, precision=PREC_FP32, min_reuse=0.0, slots=0, max_chunk_blocks=0,
                 brick_groups=0, pipeline=0, mfma_shape=0, max_row_nnz=0, chunk_order=0, operand_residency=0, hub_rows=0):
        self.hrpb = hrpb
        self.M, self.K, self.N = hrpb.M, hrpb.K, int(N)
        self._plan = C.c_void_p()
        t = cute_tunables(path=path, precision=precision, min_reuse=min_reuse, slots=slots,
                          max_chunk_blocks=max_chunk_blocks, brick_groups=brick_groups, pipeline=pipeline, mfma_shape=mfma_shape,
                          max_row_nnz=max_row_nnz, chunk_order=chunk_order, operand_residency=operand_residency, hub_rows=hub_rows)
        _check(load_library().cute_spmm_plan_create(hrpb.upload(), self.N, C.byref(t), C.byref(self._plan)),
               "cute_spmm_plan_create")
        info = cute_plan_info()
        _check(load_library().cute_spmm_plan_info(self._plan, C.byref(info)), "cute_spmm_plan_info")
        self.info = {k: getattr(info, k) for k, _ in cute_plan_info._fields_ if k != "reserved"}
        self.numRowPanelsSplit = info.numChunks
        self.kernel_name = ("csr_rows_batched" if info.numChunks == 0 else
                            "hrpb_quad_hub_f32" if info.hubRows else
                            ("hrpb_quad_rows_f32" if info.fusedLaunch else "hrpb_quad_f32") if info.mfmaShape == 2 else
                            "hrpb_brick_rows_f32" if info.fusedLaunch else
                            "hrpb_brick_bf16x3" if info.precision == PREC_BF16X3 else
                            "hrpb_brick_f32_rolling" if info.pipeline == 1 else "hrpb_brick_f32")

    def _check_shapes(self, MatB, MatC):
        if tuple(MatB.shape) != (self.K, self.N) or tuple(MatC.shape) != (self.M, self.N):
            raise ValueError("MatB must be [%d,%d] and MatC [%d,%d]" % (self.K, self.N, self.M, self.N))

    def run(self, MatB, MatC, stream=None):
        self._check_shapes(MatB, MatC)
        _check(load_library().cute_spmm_run(self._plan, _dev_ptr(MatB), _dev_ptr(MatC), _stream_ptr(stream)),
               "cute_spmm_run")
        return MatC

    def run_static(self, MatB, MatC, stream=None):
        """``run`` without any allocation behind it: partial tiles go to the library's static device array."""
        self._check_shapes(MatB, MatC)
        _check(load_library().cute_spmm_run_static(self._plan, _dev_ptr(MatB), _dev_ptr(MatC), _stream_ptr(stream)),
               "cute_spmm_run_static")
        return MatC

    @property
    def scratch_bytes(self):
        """Bytes of partial tiles one launch stores (0 when no panel is cut)."""
        return int(load_library().cute_spmm_plan_scratch_bytes(self._plan))

    def run_scratch(self, MatB, MatC, scratch, stream=None):
        """``run`` with the partial tiles in ``scratch`` (a GPU tensor of at least ``scratch_bytes`` bytes, or None
        when that is 0): one plan can then run on several streams at once, each call with its own buffer."""
        self._check_shapes(MatB, MatC)
        ptr = C.c_void_p(scratch.data_ptr()) if scratch is not None else C.c_void_p()
        nbytes = scratch.numel() * scratch.element_size() if scratch is not None else 0
        _check(load_library().cute_spmm_run_scratch(self._plan, _dev_ptr(MatB), _dev_ptr(MatC), _stream_ptr(stream), ptr, nbytes),
               "cute_spmm_run_scratch")
        return MatC

    def time(self, MatB, MatC, warmup=3, iters=20, stream=None):
        """Per-launch milliseconds (HIP events on the launch stream)."""
        self._check_shapes(MatB, MatC)
        ms = np.zeros(iters, np.float32)
        _check(load_library().cute_spmm_time(self._plan, _dev_ptr(MatB), _dev_ptr(MatC), _stream_ptr(stream),
                                             int(warmup), int(iters), _ptr(ms, f32p)), "cute_spmm_time")
        return ms

    def __del__(self):
        try:
            if self._plan:
                load_library().cute_spmm_plan_free(self._plan)
        except Exception:
            pass


def csr_spmm_time(alg, hrpb, MatB, MatC, warmup=3, iters=20, stream=None):
    ms = np.zeros(iters, np.float32)
    _check(load_library().cute_csr_spmm_time(int(alg), hrpb.upload(), _dev_ptr(MatB), _dev_ptr(MatC),
                                             int(MatB.shape[1]), _stream_ptr(stream), int(warmup), int(iters),
                                             _ptr(ms, f32p)), "cute_csr_spmm_time")
    return ms


def csr_spmm_dev(alg, hrpb, MatB, MatC, stream=None):
    lib = load_library()
    rp, cl, vl = C.c_void_p(), C.c_void_p(), C.c_void_p()
    _check(lib.cute_hrpb_dev_csr(hrpb.upload(), C.byref(rp), C.byref(cl), C.byref(vl)), "cute_hrpb_dev_csr")
    _check(lib.cute_csr_spmm_dev(int(alg), rp, cl, vl, _dev_ptr(MatB), _dev_ptr(MatC), hrpb.M, int(MatB.shape[1]),
                                 _stream_ptr(stream)), "cute_csr_spmm_dev")
    return MatC


def csr_spmm_tensors(alg, rowPtr, cols, vals, MatB, MatC, stream=None):
    """The plain CSR kernels on caller-owned GPU tensors: rowPtr/cols int32 (or uint32 bits), vals float32."""
    import torch
    for t in (rowPtr, cols):
        if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.int32 and t.is_contiguous()):
            raise TypeError("rowPtr and cols must be contiguous int32 tensors on the GPU")
    M = int(rowPtr.numel()) - 1
    _check(load_library().cute_csr_spmm_dev(int(alg), C.c_void_p(rowPtr.data_ptr()), C.c_void_p(cols.data_ptr()),
                                            _dev_ptr(vals), _dev_ptr(MatB), _dev_ptr(MatC), M, int(MatB.shape[1]),
                                            _stream_ptr(stream)), "cute_csr_spmm_dev")
    return MatC


def GPU_CSR_cuSPARSE_NEW(rowPtr, cols, vals, nnz, hB, hC, m, k, n, iters, alg=2):
    """Host arrays in, host C out, returns ms per launch (signature of spmm.cu:860-861)."""
    rowPtr, cols, vals = _as(rowPtr, np.uint32), _as(cols, np.uint32), _as(vals, np.float32)
    hB = _as(hB, np.float32)
    assert hC.dtype == np.float32 and hC.flags.c_contiguous
    ms = load_library().cute_gpu_csr_spmm(_ptr(rowPtr, u32p), _ptr(cols, u32p), _ptr(vals, f32p), int(nnz),
                                          _ptr(hB, f32p), _ptr(hC, f32p), int(m), int(k), int(n), int(iters), int(alg))
    if ms < 0:
        raise CuteError(int(ms), "cute_gpu_csr_spmm")
    return ms


# --------------------------------------------------------------------------------------
# metrics
# --------------------------------------------------------------------------------------
def spmm_coo(rows, cols, vals, B, M, K=None):
    """``spmm_coo`` (inc.h:71-83) on the host: C[M,N] from COO arrays in array order, fp32."""
    rows, cols, vals = _as(rows, np.uint32), _as(cols, np.uint32), _as(vals, np.float32)
    B = _as(B, np.float32)
    K = B.shape[0] if K is None else int(K)
    out = np.empty((int(M), B.shape[1]), np.float32)
    _check(load_library().cute_spmm_coo(_ptr(rows, u32p), _ptr(cols, u32p), _ptr(vals, f32p), _ptr(B, f32p),
                                        _ptr(out, f32p), int(M), K, B.shape[1], len(rows)), "cute_spmm_coo")
    return out


def offsets_fit(M, K, N, num_vals=0, partial_rows=0):
    return bool(load_library().cute_offsets_fit(int(M), int(K), int(N), int(num_vals), int(partial_rows)))


def check_gemm_correctness_coo(C_ref, C_test, M=None, N=None):
    a, b = _as(C_ref, np.float32), _as(C_test, np.float32)
    M = a.shape[0] if M is None else M
    N = a.shape[1] if N is None else N
    return float(load_library().cute_check_gemm_correctness(_ptr(a, f32p), _ptr(b, f32p), int(M), int(N)))


def backward_error(rowPtr, cols, vals, B, C_ref, C_test):
    rowPtr, cols, vals = _as(rowPtr, np.uint32), _as(cols, np.uint32), _as(vals, np.float32)
    B, a, b = _as(B, np.float32), _as(C_ref, np.float32), _as(C_test, np.float32)
    return float(load_library().cute_backward_error(_ptr(rowPtr, u32p), _ptr(cols, u32p), _ptr(vals, f32p),
                                                    _ptr(B, f32p), _ptr(a, f32p), _ptr(b, f32p),
                                                    len(rowPtr) - 1, B.shape[1]))


def device_info():
    cus, ws = C.c_int(), C.c_int()
    name = C.create_string_buffer(64)
    _check(load_library().cute_device_info(C.byref(cus), C.byref(ws), name, 64), "cute_device_info")
    xcds, per, whole, cache = C.c_int(), C.c_int(), C.c_int(), C.c_uint64()
    _check(load_library().cute_device_layout(C.byref(xcds), C.byref(per), C.byref(cache), C.byref(whole)), "cute_device_layout")
    return dict(num_cus=cus.value, wave_size=ws.value, arch=name.value.decode(), num_xcds=xcds.value, cus_per_xcd=per.value,
                cache_bytes=cache.value, whole_chip=bool(whole.value))


# --------------------------------------------------------------------------------------
# second API family (inc/SparseCoo.hpp, inc/CSR.hpp, inc/prepareBlkEll.hpp, inc/splitter.hpp)
# Arrays are copied into numpy-owned memory; the library's copies are released at once.
# --------------------------------------------------------------------------------------
def _take(ptr, n, dtype):
    n = int(n)
    return np.ctypeslib.as_array(ptr, shape=(n,)).astype(dtype, copy=True) if n else np.zeros(0, dtype)


def _coo_fields(raw):
    return (raw.dimY, raw.dimX, raw.nnz, _take(raw.rows, raw.nnz, np.int32), _take(raw.cols, raw.nnz, np.int32),
            _take(raw.values, raw.nnz, np.float32))


class SparseCoo:
    """``SparseCoo(path)`` (inc/SparseCoo.hpp:91-157) or ``SparseCoo(dimY, dimX, rows, cols, values)``."""

    def __init__(self, *args):
        if len(args) == 1:
            raw = cute_coo()
            _check(load_library().cute_coo_read(os.fsencode(args[0]), C.byref(raw)), "cute_coo_read(%s)" % args[0])
            self.dimY, self.dimX, self.nnz, self.rows, self.cols, self.values = _coo_fields(raw)
            load_library().cute_coo_release(C.byref(raw))
        else:
            self.dimY, self.dimX = int(args[0]), int(args[1])
            self.rows, self.cols, self.values = _as(args[2], np.int32), _as(args[3], np.int32), _as(args[4], np.float32)
            self.nnz = len(self.rows)

    def _raw(self):
        return cute_coo(self.dimY, self.dimX, self.nnz, _ptr(self.rows, i32p), _ptr(self.cols, i32p),
                        _ptr(self.values, f32p))

    def save_mtx(self, path):
        raw = self._raw()
        _check(load_library().cute_coo_save_mtx(C.byref(raw), os.fsencode(path)), "cute_coo_save_mtx")

    def merge_duplicates(self):
        """Adds up entries that share a position (file order); the arrays shrink."""
        self.rows, self.cols, self.values = self.rows.copy(), self.cols.copy(), self.values.copy()
        raw = self._raw()
        _check(load_library().cute_coo_merge_duplicates(C.byref(raw)), "cute_coo_merge_duplicates")
        self.nnz = raw.nnz
        self.rows, self.cols, self.values = self.rows[:self.nnz], self.cols[:self.nnz], self.values[:self.nnz]
        return self


class CSR_Matrix:
    """``CSR_Matrix(coo)`` = coo2CSR (inc/CSR.hpp:162-187); fields nrows, ncols, nnz, rowPtr, cols, values."""

    def __init__(self, coo=None, nrows=None, ncols=None, rowPtr=None, cols=None, values=None):
        if coo is not None:
            raw, src = cute_csr_i32(), coo._raw()
            _check(load_library().cute_coo_to_csr(C.byref(src), C.byref(raw)), "cute_coo_to_csr")
            self.nrows, self.ncols, self.nnz = raw.nrows, raw.ncols, raw.nnz
            self.rowPtr = _take(raw.rowPtr, raw.nrows + 1, np.int32)
            self.cols, self.values = _take(raw.cols, raw.nnz, np.int32), _take(raw.values, raw.nnz, np.float32)
            load_library().cute_csr_i32_release(C.byref(raw))
        else:
            self.nrows, self.ncols = int(nrows), int(ncols)
            self.rowPtr, self.cols, self.values = _as(rowPtr, np.int32), _as(cols, np.int32), _as(values, np.float32)
            self.nnz = len(self.cols)

    def _raw(self):
        return cute_csr_i32(self.nrows, self.ncols, self.nnz, _ptr(self.rowPtr, i32p), _ptr(self.cols, i32p),
                            _ptr(self.values, f32p))

    def ToDense(self):
        dense = np.zeros((self.nrows, self.ncols), np.float32)
        raw = self._raw()
        _check(load_library().cute_csr_to_dense(C.byref(raw), _ptr(dense, f32p)), "cute_csr_to_dense")
        return dense

    def csr_count_blocks(self, R, Cc):
        raw = self._raw()
        n = load_library().cute_csr_count_blocks(C.byref(raw), int(R), int(Cc))
        if n < 0:
            raise CuteError(int(n), "cute_csr_count_blocks")
        return int(n)

    def to_BCSR(self, R, Cc):
        raw, out = self._raw(), cute_bcsr()
        _check(load_library().cute_csr_to_bcsr(C.byref(raw), int(R), int(Cc), C.byref(out)), "cute_csr_to_bcsr")
        res = dict(R=out.R, C=out.C, BCSR_nrows=out.nrows, BCSR_ncols=out.ncols, BCSR_nblks=out.nblks,
                   BCSR_rowPtr=_take(out.rowPtr, out.nrows + 1, np.int32), BCSR_cols=_take(out.cols, out.nblks, np.int32),
                   BCSR_values=_take(out.values, out.nblks * out.R * out.C, np.float32))
        load_library().cute_bcsr_release(C.byref(out))
        return res

    def sequentioal_spmm(self, B):
        """inc/SPMM.cuh:123-187: double-precision CPU product; returns (C, ms)."""
        B = _as(B, np.float64)
        vals = _as(self.values, np.float64)
        Cm = np.zeros((self.nrows, B.shape[1]), np.float64)
        raw = self._raw()
        dp = C.POINTER(C.c_double)
        ms = load_library().cute_sequential_spmm(C.byref(raw), _ptr(vals, dp), _ptr(B, dp), _ptr(Cm, dp), self.nrows,
                                                 self.ncols, B.shape[1])
        if ms < 0:
            raise CuteError(int(ms), "cute_sequential_spmm")
        return Cm, ms


class preprocess:
    """``preprocess(csr, BlockSize)``: Blocked-ELL (inc/prepareBlkEll.hpp:185-196) with the getters of :267-290."""

    def __init__(self, A_CSR, BlockSize):
        raw, out = A_CSR._raw(), cute_blocked_ell()
        _check(load_library().cute_blocked_ell_build(C.byref(raw), int(BlockSize), C.byref(out)), "cute_blocked_ell_build")
        self.BlockSize, self._h, self._w = out.blockSize, out.height, out.width
        self._nb, self._ne, self._ncols = out.numBlocks, out.numElems, A_CSR.ncols
        self._idx = _take(out.ellColIdx, out.height * out.width, np.int32).reshape(out.height, out.width)
        self._val = _take(out.ellValues, out.height * out.blockSize * out.width * out.blockSize,
                          np.float32).reshape(out.height * out.blockSize, out.width * out.blockSize)
        load_library().cute_blocked_ell_release(C.byref(out))

    def get_ellColIdx(self): return self._idx
    def get_ellColIdx_height(self): return self._h
    def get_ellColIdx_width(self): return self._w
    def get_ellValues(self): return self._val
    def get_num_blocks(self): return self._nb
    def get_num_elems(self): return self._ne

    def _raw(self):
        return cute_blocked_ell(self.BlockSize, self._h, self._w, self._nb, self._ne, _ptr(self._idx, i32p),
                                _ptr(self._val, f32p))

    def spmm(self, MatB, MatC, accumulate=False, stream=None):
        """MatC[height*BlockSize, N] (+)= ELL . MatB[ncols, N] on the GPU (float32 tensors); the device
        copy of the format is made on first use."""
        if getattr(self, "_dev", None) is None:
            dev, raw = C.c_void_p(), self._raw()
            _check(load_library().cute_blocked_ell_upload(C.byref(raw), C.byref(dev)), "cute_blocked_ell_upload")
            self._dev = _DevGuard(dev, "cute_blocked_ell_dev_free")
        N = int(MatB.shape[1])
        if tuple(MatB.shape) != (self._ncols, N) or tuple(MatC.shape) != (self._h * self.BlockSize, N):
            raise ValueError("MatB must be [%d,N] and MatC [%d,N]" % (self._ncols, self._h * self.BlockSize))
        _check(load_library().cute_blocked_ell_spmm(self._dev.handle, _dev_ptr(MatB), _dev_ptr(MatC), N,
                                                    int(bool(accumulate)), _stream_ptr(stream)), "cute_blocked_ell_spmm")
        return MatC

    def blockedELLToDense(self):
        dense = np.zeros((self._h * self.BlockSize, self._ncols), np.float32)
        raw = self._raw()
        _check(load_library().cute_blocked_ell_to_dense(C.byref(raw), self._ncols, _ptr(dense, f32p)),
               "cute_blocked_ell_to_dense")
        return dense


class _DevGuard:
    """Frees a device handle of the library when the last owner goes."""

    def __init__(self, handle, free_name):
        self.handle, self._free = handle, free_name

    def __del__(self):
        try:
            if self.handle:
                getattr(load_library(), self._free)(self.handle)
        except Exception:
            pass


class Splitter:
    """``Splitter(csr, tile_size, NNZThreshold)`` (inc/splitter.hpp:126-142) with its seven getters."""

    def __init__(self, A_CSR, tile_size, NNZThreshold):
        raw, out = A_CSR._raw(), cute_split()
        _check(load_library().cute_splitter_split(C.byref(raw), int(tile_size), int(NNZThreshold), C.byref(out)),
               "cute_splitter_split")
        self._c = (out.totalTiles, out.numHeavyTiles, out.numHeavyElems, out.numLightTiles, out.numLightElems)
        self._heavy = SparseCoo(*_coo_fields(out.heavy)[:2], *_coo_fields(out.heavy)[3:])
        self._light = SparseCoo(*_coo_fields(out.light)[:2], *_coo_fields(out.light)[3:])
        load_library().cute_split_release(C.byref(out))

    def get_total_tiles(self): return self._c[0]
    def get_num_heavy_tiles(self): return self._c[1]
    def get_num_heavy_elems(self): return self._c[2]
    def get_num_light_tiles(self): return self._c[3]
    def get_num_light_elems(self): return self._c[4]
    def get_heavyMatrix(self): return self._heavy
    def get_lightMatrix(self): return self._light


class ClassSplitter(Splitter):
    """The split the block classifier implies (inc/preprocess.hpp:172-283): entries of dense and 2:4-sparse blocks are
    the heavy matrix, entries of very sparse blocks the light one.  Same getters as ``Splitter``; tiles count blocks."""

    def __init__(self, A_CSR, BlockSize, deviation_threshold, underload_dominance=0.5):
        raw, out = A_CSR._raw(), cute_split()
        _check(load_library().cute_split_by_class(C.byref(raw), int(BlockSize), float(deviation_threshold),
                                                  float(underload_dominance), C.byref(out)), "cute_split_by_class")
        self._c = (out.totalTiles, out.numHeavyTiles, out.numHeavyElems, out.numLightTiles, out.numLightElems)
        self._heavy = SparseCoo(*_coo_fields(out.heavy)[:2], *_coo_fields(out.heavy)[3:])
        self._light = SparseCoo(*_coo_fields(out.light)[:2], *_coo_fields(out.light)[3:])
        load_library().cute_split_release(C.byref(out))


HYBRID_SPLITTER, HYBRID_CLASSIFIER = 0, 1


class HybridSpMM:
    """The hybrid of inc/SPMM.cuh:2528-2933 as one library call: heavy tiles as Blocked-ELL through the fp32 MFMA
    kernel, the remainder as CSR through the row kernel, both into one C.  ``mode`` HYBRID_SPLITTER (tile nnz
    threshold; 0 = chosen from the block statistics) or HYBRID_CLASSIFIER (inc/preprocess.hpp:172-193)."""

    def __init__(self, A_CSR, tile_size=16, nnz_threshold=0, mode=HYBRID_SPLITTER, deviation_threshold=0.5,
                 underload_dominance=0.5):
        raw = A_CSR._raw()
        self.nrows, self.ncols = A_CSR.nrows, A_CSR.ncols
        self._h = C.c_void_p()
        _check(load_library().cute_hybrid_create(C.byref(raw), int(tile_size), int(nnz_threshold), int(mode),
                                                 float(deviation_threshold), float(underload_dominance), C.byref(self._h)),
               "cute_hybrid_create")
        info = cute_hybrid_info()
        _check(load_library().cute_hybrid_get_info(self._h, C.byref(info)), "cute_hybrid_get_info")
        self.info = {k: getattr(info, k) for k, _ in cute_hybrid_info._fields_ if k != "stats"}
        self.info["stats"] = [float(x) for x in info.stats]

    def spmm(self, MatB, MatC, stream=None):
        if tuple(MatB.shape)[0] != self.ncols or tuple(MatC.shape) != (self.nrows, MatB.shape[1]):
            raise ValueError("MatB must be [%d,N] and MatC [%d,N]" % (self.ncols, self.nrows))
        _check(load_library().cute_hybrid_spmm(self._h, _dev_ptr(MatB), _dev_ptr(MatC), int(MatB.shape[1]), _stream_ptr(stream)),
               "cute_hybrid_spmm")
        return MatC

    def __del__(self):
        try:
            if self._h:
                load_library().cute_hybrid_free(self._h)
        except Exception:
            pass


def GET_STATS(A_CSR, blocksize):
    """gpu_kernels.cu:1049-1137 -> float32[4]: mean nnz per active row and per active column of the non-empty
    blocksize^2 blocks, their number, their mean density."""
    raw = A_CSR._raw()
    stats = np.zeros(4, np.float32)
    _check(load_library().cute_block_stats(C.byref(raw), int(blocksize), _ptr(stats, f32p)), "cute_block_stats")
    return stats


def GET_ANXS(A_CSR, blocksize, axis):
    """gpu_kernels.cu:1139-1186: nonzeros per distinct column of a block row (axis true) or per distinct row of
    a block column (axis false)."""
    raw = A_CSR._raw()
    v = C.c_float()
    _check(load_library().cute_anxs(C.byref(raw), int(blocksize), 1 if axis else 0, C.byref(v)), "cute_anxs")
    return float(v.value)


def classify_blocks(A_CSR, BlockSize, deviation_threshold, underload_dominance):
    """inc/preprocess.hpp:64-193 -> int32 array [n, 6]: blockRow, blockCol, nnz, underloads, overloads, kind."""
    raw = A_CSR._raw()
    out, n = C.POINTER(cute_block_class)(), C.c_int64()
    _check(load_library().cute_classify_blocks(C.byref(raw), int(BlockSize), float(deviation_threshold),
                                               float(underload_dominance), C.byref(out), C.byref(n)),
           "cute_classify_blocks")
    arr = np.zeros((n.value, 6), np.int32)
    if n.value:
        arr[:] = np.ctypeslib.as_array(C.cast(out, i32p), shape=(n.value, 6))
    load_library().cute_free(C.cast(out, C.c_void_p))
    return arr
