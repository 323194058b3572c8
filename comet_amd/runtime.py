"""ctypes binding of libcomet_hip_rt.so (include/comet_hip_rt.h) plus thin host
objects that mirror how COMET's lowered code and its Python front end hold
tensors: dense tensors as contiguous row-major float64, sparse matrices as the
(pos, crd, val) CSR tuple (frontends/numpy-scipy/cometpy/MLIRGen/lowering.py:
298-321 in pnnl/COMET passes exactly these arrays to compiled kernels).

There is no CPU fallback: if the shared library has not been built, or no
MI355X is present, every entry point raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# COMET_HIP_LIB points at an alternative build of the same library (used when tuning kernel parameters)
LIB_PATH = os.environ.get("COMET_HIP_LIB") or os.path.join(_HERE, "libcomet_hip_rt.so")


class CometHipError(RuntimeError):
    pass


class TtgtPlan(C.Structure):
    _fields_ = [
        ("rankA", C.c_int32), ("rankB", C.c_int32), ("rankC", C.c_int32),
        ("a_idx", C.c_int32 * 8), ("b_idx", C.c_int32 * 8), ("c_idx", C.c_int32 * 8),
        ("permA", C.c_int32 * 8), ("permB", C.c_int32 * 8), ("permC", C.c_int32 * 8),
        ("transA", C.c_int32), ("transB", C.c_int32), ("transC", C.c_int32), ("swapAB", C.c_int32),
        ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64),
        ("cost", C.c_double),
        ("candidate", C.c_int32), ("ncandidates", C.c_int32),
    ]


class Memref1D(C.Structure):
    _fields_ = [("allocated", C.c_void_p), ("aligned", C.c_void_p), ("offset", C.c_int64),
                ("sizes", C.c_int64 * 1), ("strides", C.c_int64 * 1)]


class Memref2D(C.Structure):
    _fields_ = [("allocated", C.c_void_p), ("aligned", C.c_void_p), ("offset", C.c_int64),
                ("sizes", C.c_int64 * 2), ("strides", C.c_int64 * 2)]


# name -> (restype, argtypes); every symbol include/comet_hip_rt.h declares
_i64, _i32, _f64, _vp, _int = C.c_int64, C.c_int32, C.c_double, C.c_void_p, C.c_int
_pi64 = C.POINTER(C.c_int64)
_m1, _m2 = C.POINTER(Memref1D), C.POINTER(Memref2D)
SIGNATURES = {
    "comet_hip_init": (_int, [_int]),
    "comet_hip_finalize": (_int, []),
    "comet_hip_last_error": (C.c_char_p, []),
    "comet_hip_device_name": (_int, [C.c_char_p, _i64]),
    "comet_hip_malloc": (_i64, [_i64]),
    "comet_hip_free": (_int, [_i64]),
    "comet_hip_memcpy": (_int, [_i64, _vp, _i64, _i64]),
    "comet_hip_memset": (_int, [_i64, _int, _i64]),
    "comet_hip_sync": (_int, []),
    "HipMallocF64": (_i64, [_i64]),
    "HipMallocI64": (_i64, [_i64]),
    "HipMallocI32": (_i64, [_i64]),
    "HipFree": (None, [_i64]),
    "HipMemcpyF64": (None, [_i64, _vp, _vp, _i64, _i64, _i64, _i64]),
    "HipMemcpyI64": (None, [_i64, _vp, _vp, _i64, _i64, _i64, _i64]),
    "HipMemcpyI32": (None, [_i64, _vp, _vp, _i64, _i64, _i64, _i64]),
    "HipMemcpyIndex": (None, [_i64, _vp, _vp, _i64, _i64, _i64, _i64]),
    "comet_hip_csr_upload_i64": (_i64, [_i64, _i64, _vp, _vp, _vp]),
    "comet_hip_csr_upload_i32": (_i64, [_i64, _i64, _vp, _vp, _vp]),
    "comet_hip_csr_wrap": (_i64, [_i64, _i64, _i64, _i64, _i64, _i64]),
    "comet_hip_csr_dims": (_int, [_i64, _pi64, _pi64, _pi64]),
    "comet_hip_csr_arrays": (_int, [_i64, _pi64, _pi64, _pi64]),
    "comet_hip_csr_download_i64": (_int, [_i64, _vp, _vp, _vp]),
    "comet_hip_csr_download_i32": (_int, [_i64, _vp, _vp, _vp]),
    "comet_hip_csr_invalidate": (_int, [_i64]),
    "comet_hip_csr_destroy": (_int, [_i64]),
    "comet_hip_spmv_csr_f64": (_int, [_i64, _i64, _i64, _int]),
    "comet_hip_spmm_csr_f64": (_int, [_i64, _i64, _i64, _i64, _i64, _i64, _int]),
    "comet_hip_spmm_csr_f64_noalloc": (_int, [_i64, _i64, _i64, _i64, _i64, _i64, _int, _i64]),
    "comet_hip_spgemm_csr_symbolic": (_int, [_i64, _i64, _i64, _i64, _pi64]),
    "comet_hip_spgemm_csr_numeric": (_int, [_i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64]),
    "comet_hip_spgemm_csr": (_i64, [_i64, _i64, _i64]),
    "comet_hip_spgemm_csr_numeric_semiring": (_int, [_i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int]),
    "comet_hip_spgemm_csr_semiring": (_i64, [_i64, _i64, _i64, _int, _int]),
    "comet_hip_vecmat_csr_f64": (_int, [_i64, _i64, _i64, _int]),
    "comet_hip_densemat_csr_f64": (_int, [_i64, _i64, _i64, _i64, _i64, _i64, _int]),
    "comet_hip_eltwise_csr_dense_csr": (_i64, [_i64, _i64, _i64, _int]),
    "comet_hip_sddmm_csr_f64": (_i64, [_i64, _i64, _i64, _i64, _i64, _i64]),
    "comet_hip_sddmm_csr_values_f64": (_int, [_i64, _i64, _i64, _i64, _i64, _i64, _i64]),
    "comet_print_memref_f64": (None, [_i64, C.c_void_p]),
    "comet_print_memref_f32": (None, [_i64, C.c_void_p]),
    "comet_print_memref_i64": (None, [_i64, C.c_void_p]),
    "comet_print_memref_i32": (None, [_i64, C.c_void_p]),
    "comet_print_memref_index": (None, [_i64, C.c_void_p]),
    "comet_sort_index": (None, [_i64, C.c_void_p, _i64, _i64]),
    "comet_sort64": (None, [_i64, C.c_void_p, _i64, _i64]),
    "comet_sort32": (None, [_i64, C.c_void_p, _i64, _i64]),
    "getTime": (C.c_double, []),
    "printElapsedTime": (None, [C.c_double, C.c_double]),
    "comet_hip_eltwise_csr_dense_dense": (_int, [_i64, _i64, _i64, _i64, _i64, _int]),
    "comet_hip_eltwise_dense_f64": (_int, [_i64, _i64, _i64, _i64, _int]),
    "comet_hip_mtx_read_csr": (_i64, [C.c_char_p, _int]),
    "comet_hip_read_input_sizes_2D_f64": (None, [_i32, _i32, _i32, _i32, _i32, _int, _vp, _i32]),
    "comet_hip_read_input_2D_f64_i64": (None, [_i32, _i32, _i32, _i32, _i32] + [_int, _vp] * 9 + [_i32]),
    "comet_hip_read_input_2D_f64_i32": (None, [_i32, _i32, _i32, _i32, _i32] + [_int, _vp] * 9 + [_i32]),
    "comet_hip_read_input_2D_handle": (_i64, [_i32, _i32]),
    "comet_hip_csr_from_coo_i64": (_i64, [_i64, _i64, _i64, _vp, _vp, _vp, _int]),
    "comet_hip_csr_from_coo_device": (_i64, [_i64, _i64, _i64, _i64, _i64, _i64, _int]),
    "comet_hip_csr_from_dcsr_i64": (_i64, [_i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    "comet_hip_csr_to_coo_i64": (_int, [_i64, _vp, _vp, _vp]),
    "comet_hip_csr_to_dcsr_i64": (_int, [_i64, _pi64, _vp, _vp, _vp, _vp]),
    "comet_hip_csr_transpose": (_i64, [_i64]),
    "comet_hip_spgemm_masked_sum": (_int, [_i64, _i64, _i64, C.POINTER(_f64)]),
    "comet_hip_reduce_sum_f64": (_int, [_i64, _i64, C.POINTER(_f64)]),
    "comet_hip_eltwise_mult_csr": (_i64, [_i64, _i64]),
    "comet_hip_transpose_f64": (_int, [_i32, _vp, _vp, _i64, _i64]),
    "comet_hip_dgemm_f64": (_int, [_i64, _i64, _i64, _i64, _i64, _i64, _f64]),
    "comet_hip_ttgt_plan": (_int, [_i32, _vp, _i32, _vp, _i32, _vp, _vp, _i32, C.POINTER(TtgtPlan)]),
    "comet_hip_ttgt_contract": (_int, [C.POINTER(TtgtPlan), _vp, _vp, _vp, _i64, _i64, _i64, _f64]),
    "comet_hip_timer_start": (_int, []),
    "comet_hip_timer_stop": (_int, [C.POINTER(_f64)]),
    "comet_hip_profile_enable": (_int, [_int]),
    "comet_hip_profile_reset": (_int, []),
    "comet_hip_profile_query": (_int, [C.c_char_p, _pi64, C.POINTER(_f64)]),
    "comet_hip_profile_name": (_int, [_i32, C.c_char_p, _i64]),
    "comet_hip_copy_f64": (_int, [_i64, _i64, _i64]),
    "comet_hip_debug_dot_table_words": (_int, [_int]),
    "comet_hip_debug_masked_sum_registers": (_int, [C.POINTER(_int), C.POINTER(_int)]),
    "comet_hip_stream_create": (_i64, []),
    "comet_hip_stream_sync": (_int, [_i64]),
    "comet_hip_stream_destroy": (_int, [_i64]),
    "comet_hip_stream_bench": (_int, [_int, _i64, _i64, _i64, _int]),
    "comet_hip_mem_info": (_int, [C.POINTER(_i64), C.POINTER(_i64)]),
    "comet_hip_mfma_f64_peak": (_int, [_i64, C.POINTER(C.c_double)]),
    "comet_hip_gather_rows_bench": (_int, [_i64, _i64, _i64, _i64, _i64, _i64]),
    "_mlir_ciface_comet_hip_spgemm_csr_sizes_semiring_f64_i64": (None, [_i64, _i64, _m1, _m1, _m1, _m1, _m1, _m1, _m1, _m1, _m1, _i32, _i32]),
    "_mlir_ciface_comet_hip_spgemm_csr_sizes_semiring_f64_i32": (None, [_i64, _i64, _m1, _m1, _m1, _m1, _m1, _m1, _m1, _m1, _m1, _i32, _i32]),
    "_mlir_ciface_comet_hip_spgemm_csr_fill_semiring_f64_i64": (None, [_m1, _m1, _m1]),
    "_mlir_ciface_comet_hip_spgemm_csr_fill_semiring_f64_i32": (None, [_m1, _m1, _m1]),
    "_mlir_ciface_comet_hip_ttgt_contract_f64": (None, [_i64, _vp, _i64, _vp, _i64, _vp, _m1, _m1, _m1, _f64]),
    "_mlir_ciface_linalg_matmul_viewsxs_viewsxs_viewsxs": (None, [_m2, _m2, _m2, _int, _int, _f64, _f64]),
    "read_input_sizes_2D_f64": (None, [_i32, _i32, _i32, _i32, _i32, _int, _vp, _i32]),
    "read_input_2D_f64_i64": (None, [_i32, _i32, _i32, _i32, _i32] + [_int, _vp] * 9 + [_i32]),
    "read_input_2D_f64_i32": (None, [_i32, _i32, _i32, _i32, _i32] + [_int, _vp] * 9 + [_i32]),
    "_mlir_ciface_comet_hip_spmv_csr_f64_i64": (None, [_m1, _m1, _m1, _m1, _m1]),
    "_mlir_ciface_comet_hip_spmm_csr_f64_i64": (None, [_m1, _m1, _m1, _m2, _m2]),
    "_mlir_ciface_comet_hip_spgemm_csr_sizes_f64_i64": (None, [_i64, _i64, _m1, _m1, _m1, _m1, _m1, _m1, _m1, _m1, _m1]),
    "_mlir_ciface_comet_hip_spgemm_csr_fill_f64_i64": (None, [_m1, _m1, _m1]),
    "_mlir_ciface_comet_hip_tricount_f64_i64": (_f64, [_i64, _m1, _m1, _m1]),
    "_mlir_ciface_comet_hip_spmv_csr_f64_i32": (None, [_m1, _m1, _m1, _m1, _m1]),
    "_mlir_ciface_comet_hip_spmm_csr_f64_i32": (None, [_m1, _m1, _m1, _m2, _m2]),
    "_mlir_ciface_comet_hip_spgemm_csr_sizes_f64_i32": (None, [_i64, _i64, _m1, _m1, _m1, _m1, _m1, _m1, _m1, _m1, _m1]),
    "_mlir_ciface_comet_hip_spgemm_csr_fill_f64_i32": (None, [_m1, _m1, _m1]),
    "_mlir_ciface_comet_hip_tricount_f64_i32": (_f64, [_i64, _m1, _m1, _m1]),
}

_lib = None


def lib():
    """Load the shared library (never builds, never falls back)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise CometHipError(
                f"{LIB_PATH} is missing: build it first (python -m comet_amd.build or __graft_entry__.build())")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _check(rc, what=""):
    if rc != 0:
        raise CometHipError(f"{what}: [{rc}] {lib().comet_hip_last_error().decode()}")


def _handle(h, what):
    if not h:
        raise CometHipError(f"{what}: {lib().comet_hip_last_error().decode()}")
    return h


def init(device=0):
    _check(lib().comet_hip_init(device), "comet_hip_init")


def device_name():
    buf = C.create_string_buffer(256)
    _check(lib().comet_hip_device_name(buf, 256), "comet_hip_device_name")
    return buf.value.decode()


def sync():
    _check(lib().comet_hip_sync(), "comet_hip_sync")


def _vptr(a):
    return a.ctypes.data_as(C.c_void_p)


class DeviceArray:
    """A contiguous row-major array in HBM."""

    def __init__(self, shape, dtype=np.float64, zero=False):
        self.shape = tuple(int(s) for s in (shape if np.ndim(shape) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.size = int(np.prod(self.shape)) if self.shape else 1
        self.nbytes = self.size * self.dtype.itemsize
        self.ptr = _handle(lib().comet_hip_malloc(max(self.nbytes, 1)), "comet_hip_malloc")
        if zero:
            self.fill_zero()

    @classmethod
    def from_numpy(cls, a, dtype=None):
        a = np.ascontiguousarray(a, dtype=dtype or a.dtype)
        d = cls(a.shape, a.dtype)
        if a.size:
            _check(lib().comet_hip_memcpy(d.ptr, _vptr(a), a.nbytes, 0), "upload")
        return d

    def to_numpy(self, count=None):
        """Copy to the host: the whole array, or its first `count` elements (flat)."""
        if count is None:
            out = np.empty(self.shape, dtype=self.dtype)
        else:
            if count < 0 or count > self.size:
                raise ValueError("count outside the array")
            out = np.empty(count, dtype=self.dtype)
        if out.size:
            _check(lib().comet_hip_memcpy(self.ptr, _vptr(out), out.nbytes, 1), "download")
        return out

    def fill_zero(self):
        _check(lib().comet_hip_memset(self.ptr, 0, self.nbytes), "memset")

    def free(self):
        if self.ptr:
            _check(lib().comet_hip_free(self.ptr), "comet_hip_free")
            self.ptr = 0

    def __del__(self):
        try:
            if self.ptr and _lib is not None:
                _lib.comet_hip_free(self.ptr)
                self.ptr = 0
        except Exception:
            pass


class CsrMatrix:
    """Device CSR matrix: pos int64[nrows+1], crd int32[nnz], val float64[nnz]."""

    def __init__(self, handle):
        self.handle = handle

    @classmethod
    def from_arrays(cls, shape, pos, crd, val):
        nrows, ncols = shape
        pos = np.asarray(pos)
        if pos.dtype == np.int32:
            pos = np.ascontiguousarray(pos, dtype=np.int32)
            crd = np.ascontiguousarray(crd, dtype=np.int32)
            fn = lib().comet_hip_csr_upload_i32
        else:
            pos = np.ascontiguousarray(pos, dtype=np.int64)
            crd = np.ascontiguousarray(crd, dtype=np.int64)
            fn = lib().comet_hip_csr_upload_i64
        val = np.ascontiguousarray(val, dtype=np.float64)
        if len(pos) != nrows + 1 or len(crd) != len(val):
            raise ValueError("inconsistent CSR arrays")
        return cls(_handle(fn(nrows, ncols, _vptr(pos), _vptr(crd), _vptr(val)), "comet_hip_csr_upload"))

    @classmethod
    def from_scipy(cls, m):
        m = m.tocsr()
        m.sort_indices()
        return cls.from_arrays(m.shape, m.indptr.astype(np.int64), m.indices.astype(np.int64), m.data)

    @classmethod
    def from_mtx(cls, path, read_mode=1):
        """MatrixMarket file -> device CSR; read_mode as in comet_read(id, mode): 1 all, 2 strictly lower,
        3 lower, 4 strictly upper, 5 upper."""
        return cls(_handle(lib().comet_hip_mtx_read_csr(os.fsencode(path), int(read_mode)), "comet_hip_mtx_read_csr"))

    @classmethod
    def from_file_id(cls, file_id, read_mode=1):
        """comet_read(file_id, read_mode): the file named by SPARSE_FILE_NAME<file_id>."""
        return cls(_handle(lib().comet_hip_read_input_2D_handle(int(file_id), int(read_mode)),
                           "comet_hip_read_input_2D_handle"))

    @classmethod
    def from_coo(cls, shape, row, col, val, read_mode=1):
        """Tuples in any order (ordered on the GPU by (row, col), ties in input order)."""
        row = np.ascontiguousarray(row, dtype=np.int64)
        col = np.ascontiguousarray(col, dtype=np.int64)
        val = np.ascontiguousarray(val, dtype=np.float64)
        if not (len(row) == len(col) == len(val)):
            raise ValueError("row, col and val must have one entry per tuple")
        h = lib().comet_hip_csr_from_coo_i64(int(shape[0]), int(shape[1]), len(val), _vptr(row), _vptr(col),
                                             _vptr(val), int(read_mode))
        return cls(_handle(h, "comet_hip_csr_from_coo_i64"))

    @classmethod
    def from_coo_device(cls, shape, row, col, val, read_mode=1):
        """row, col: int32 DeviceArrays; val: float64 DeviceArray."""
        if row.dtype != np.int32 or col.dtype != np.int32 or val.dtype != np.float64:
            raise ValueError("device tuples must be int32 / int32 / float64")
        h = lib().comet_hip_csr_from_coo_device(int(shape[0]), int(shape[1]), val.size, row.ptr, col.ptr, val.ptr,
                                                int(read_mode))
        return cls(_handle(h, "comet_hip_csr_from_coo_device"))

    @classmethod
    def from_dcsr(cls, shape, a1crd, a2pos, a2crd, aval):
        """The reference's DCSR arrays: ids of the rows that store anything, then CSR over those rows."""
        a1crd = np.ascontiguousarray(a1crd, dtype=np.int64)
        a2pos = np.ascontiguousarray(a2pos, dtype=np.int64)
        a2crd = np.ascontiguousarray(a2crd, dtype=np.int64)
        aval = np.ascontiguousarray(aval, dtype=np.float64)
        if len(a2pos) != len(a1crd) + 1:
            raise ValueError("a2pos must hold one more entry than a1crd")
        h = lib().comet_hip_csr_from_dcsr_i64(int(shape[0]), int(shape[1]), len(a1crd), _vptr(a1crd), _vptr(a2pos),
                                              _vptr(a2crd), _vptr(aval))
        return cls(_handle(h, "comet_hip_csr_from_dcsr_i64"))

    def to_coo(self):
        nnz = self.nnz
        row, col, val = np.zeros(nnz, dtype=np.int64), np.zeros(nnz, dtype=np.int64), np.zeros(nnz)
        _check(lib().comet_hip_csr_to_coo_i64(self.handle, _vptr(row), _vptr(col), _vptr(val)),
               "comet_hip_csr_to_coo_i64")
        return row, col, val

    def to_dcsr(self):
        """(a1pos, a1crd, a2pos, a2crd, aval) as the reference's reader lays DCSR out."""
        stored = C.c_int64()
        _check(lib().comet_hip_csr_to_dcsr_i64(self.handle, C.byref(stored), None, None, None, None),
               "comet_hip_csr_to_dcsr_i64")
        nnz = self.nnz
        a1crd = np.zeros(stored.value, dtype=np.int64)
        a2pos = np.zeros(stored.value + 1, dtype=np.int64)
        a2crd, aval = np.zeros(nnz, dtype=np.int64), np.zeros(nnz)
        _check(lib().comet_hip_csr_to_dcsr_i64(self.handle, C.byref(stored), _vptr(a1crd), _vptr(a2pos),
                                               _vptr(a2crd), _vptr(aval)), "comet_hip_csr_to_dcsr_i64")
        return np.array([0, stored.value], dtype=np.int64), a1crd, a2pos, a2crd, aval

    def transpose(self):
        return CsrMatrix(_handle(lib().comet_hip_csr_transpose(self.handle), "comet_hip_csr_transpose"))

    def dims(self):
        r, c, n = C.c_int64(), C.c_int64(), C.c_int64()
        _check(lib().comet_hip_csr_dims(self.handle, C.byref(r), C.byref(c), C.byref(n)), "comet_hip_csr_dims")
        return r.value, c.value, n.value

    @property
    def shape(self):
        return self.dims()[:2]

    @property
    def nnz(self):
        return self.dims()[2]

    def device_arrays(self):
        p, c, v = C.c_int64(), C.c_int64(), C.c_int64()
        _check(lib().comet_hip_csr_arrays(self.handle, C.byref(p), C.byref(c), C.byref(v)), "comet_hip_csr_arrays")
        return p.value, c.value, v.value

    def to_arrays(self, index_dtype=np.int64):
        nrows, _, nnz = self.dims()
        idt = np.dtype(index_dtype)
        pos = np.zeros(nrows + 1, dtype=idt)
        crd = np.zeros(nnz, dtype=idt)
        val = np.zeros(nnz, dtype=np.float64)
        fn = lib().comet_hip_csr_download_i64 if idt == np.int64 else lib().comet_hip_csr_download_i32
        _check(fn(self.handle, _vptr(pos), _vptr(crd) if nnz else None, _vptr(val) if nnz else None), "csr download")
        return pos, crd, val

    def invalidate(self):
        """Drop what the kernels cached about this matrix (needed after writing into wrapped arrays)."""
        _check(lib().comet_hip_csr_invalidate(self.handle), "comet_hip_csr_invalidate")

    def free(self):
        if self.handle:
            _check(lib().comet_hip_csr_destroy(self.handle), "comet_hip_csr_destroy")
            self.handle = 0

    def __del__(self):
        try:
            if self.handle and _lib is not None:
                _lib.comet_hip_csr_destroy(self.handle)
                self.handle = 0
        except Exception:
            pass


# ----------------------------------------------------------------------------- operators
def spmv(A, x, y=None, accumulate=None):
    """y (+)= A @ x on device arrays; returns y.  accumulate defaults to True when y is given
    (the reference always adds into the output it was handed)."""
    nrows, ncols = A.shape
    if x.size != ncols:
        raise ValueError("x has the wrong length")
    if y is None:
        y = DeviceArray(nrows)
        accumulate = False if accumulate is None else accumulate
        if accumulate:
            y.fill_zero()
    elif accumulate is None:
        accumulate = True
    _check(lib().comet_hip_spmv_csr_f64(A.handle, x.ptr, y.ptr, int(accumulate)), "comet_hip_spmv_csr_f64")
    return y


def spmm(A, B, Cm=None, accumulate=None):
    nrows, ncols = A.shape
    if B.shape[0] != ncols:
        raise ValueError("B has the wrong number of rows")
    K = B.shape[1]
    if Cm is None:
        Cm = DeviceArray((nrows, K))
        accumulate = False if accumulate is None else accumulate
        if accumulate:
            Cm.fill_zero()
    elif accumulate is None:
        accumulate = True
    _check(lib().comet_hip_spmm_csr_f64(A.handle, K, B.ptr, K, Cm.ptr, K, int(accumulate)), "comet_hip_spmm_csr_f64")
    return Cm


# operator codes of the C ABI (COMET_SR_* / COMET_OP_*), by the names the .ta language uses
REDUCE_OPS = {"plus": 0, "+": 0, "min": 1, "max": 2, "any": 3}
MULT_OPS = {"times": 0, "*": 0, "first": 1, "second": 2, "pair": 3, "plus": 4, "+": 4, "minus": 5, "-": 5,
            "min": 6, "max": 7, "div": 8, "/": 8}


def _semiring_codes(semiring):
    if semiring is None:
        return 0, 0
    reduce_op, mult_op = semiring
    if reduce_op not in REDUCE_OPS or mult_op not in MULT_OPS:
        raise ValueError(f"unknown semiring {semiring!r}")
    return REDUCE_OPS[reduce_op], MULT_OPS[mult_op]


def spgemm(A, B, mask=None, semiring=None):
    """C = A @(reduce, mult) B as a new CsrMatrix; semiring=None is (plus, times)."""
    r, m = _semiring_codes(semiring)
    h = lib().comet_hip_spgemm_csr_semiring(A.handle, B.handle, mask.handle if mask is not None else 0, r, m)
    return CsrMatrix(_handle(h, "comet_hip_spgemm_csr_semiring"))


def spgemm_symbolic(A, B, mask=None):
    """Returns (device row pointer int64[nrows+1], nnz)."""
    pos = DeviceArray(A.shape[0] + 1, np.int64)
    nnz = C.c_int64()
    _check(lib().comet_hip_spgemm_csr_symbolic(A.handle, B.handle, mask.handle if mask is not None else 0,
                                               pos.ptr, C.byref(nnz)), "comet_hip_spgemm_csr_symbolic")
    return pos, nnz.value


def spgemm_numeric(A, B, pos, row_begin, row_end, crd, val, mask=None, semiring=None):
    r, m = _semiring_codes(semiring)
    _check(lib().comet_hip_spgemm_csr_numeric_semiring(A.handle, B.handle, mask.handle if mask is not None else 0,
                                                       pos.ptr, row_begin, row_end, crd.ptr, val.ptr, r, m),
           "comet_hip_spgemm_csr_numeric_semiring")


def spgemm_masked_sum(A, B, mask):
    out = C.c_double()
    _check(lib().comet_hip_spgemm_masked_sum(A.handle, B.handle, mask.handle, C.byref(out)),
           "comet_hip_spgemm_masked_sum")
    return out.value


def triangle_count(L):
    """SUM(C) for C<L> = L * L with L strictly lower triangular."""
    return spgemm_masked_sum(L, L, L)


def reduce_sum(x, n=None):
    out = C.c_double()
    _check(lib().comet_hip_reduce_sum_f64(x.ptr, x.size if n is None else n, C.byref(out)), "comet_hip_reduce_sum_f64")
    return out.value


def sum_values(A):
    """SUM over the stored values of a sparse matrix (the DSL's SUM(A[i,j]))."""
    _, _, v = A.device_arrays()
    out = C.c_double()
    _check(lib().comet_hip_reduce_sum_f64(v, A.nnz, C.byref(out)), "comet_hip_reduce_sum_f64")
    return out.value


def vecmat(x, B, y=None, accumulate=None):
    """y (+)= x @ B for a dense vector x and a sparse B."""
    nrows, ncols = B.shape
    if x.size != nrows:
        raise ValueError("x has the wrong length")
    if y is None:
        y, accumulate = DeviceArray(ncols), False
    elif accumulate is None:
        accumulate = True
    _check(lib().comet_hip_vecmat_csr_f64(B.handle, x.ptr, y.ptr, int(accumulate)), "comet_hip_vecmat_csr_f64")
    return y


def densemat(A, B, Cm=None, accumulate=None):
    """C (+)= A @ B for a dense A (M x nrows(B)) and a sparse B."""
    nrows, ncols = B.shape
    if len(A.shape) != 2 or A.shape[1] != nrows:
        raise ValueError("A has the wrong shape")
    M = A.shape[0]
    if Cm is None:
        Cm, accumulate = DeviceArray((M, ncols)), False
    elif accumulate is None:
        accumulate = True
    _check(lib().comet_hip_densemat_csr_f64(B.handle, M, A.ptr, nrows, Cm.ptr, ncols, int(accumulate)),
           "comet_hip_densemat_csr_f64")
    return Cm


def eltwise_csr_dense(A, D, out=None, op="times"):
    """A (op) D elementwise for a sparse A and a dense D of the same shape (op: a MULT_OPS name; "times" is
    the language's .*): a CsrMatrix with A's structure, or, when a dense `out` is given, written into it at
    A's stored positions."""
    if tuple(D.shape) != tuple(A.shape):
        raise ValueError("operands differ in shape")
    code = MULT_OPS[op]
    if out is None:
        return CsrMatrix(_handle(lib().comet_hip_eltwise_csr_dense_csr(A.handle, D.ptr, A.shape[1], code),
                                 "comet_hip_eltwise_csr_dense_csr"))
    _check(lib().comet_hip_eltwise_csr_dense_dense(A.handle, D.ptr, A.shape[1], out.ptr, A.shape[1], code),
           "comet_hip_eltwise_csr_dense_dense")
    return out


def sddmm(B, Cm, D, out_values=None):
    """B .* (Cm @ D) for a sparse B (nrows x ncols), dense Cm (nrows x K) and D (K x ncols): a CsrMatrix with
    B's structure, or, when a DeviceArray `out_values` of nnz(B) doubles is given, just the values written
    there; the dense product is never formed."""
    nrows, ncols = B.shape
    if len(Cm.shape) != 2 or len(D.shape) != 2 or Cm.shape[0] != nrows or D.shape[1] != ncols or \
            Cm.shape[1] != D.shape[0]:
        raise ValueError("SDDMM needs B (n x m), C (n x K) and D (K x m)")
    K = Cm.shape[1]
    if out_values is not None:
        if out_values.size < B.nnz:
            raise ValueError("out_values is shorter than the number of stored entries")
        _check(lib().comet_hip_sddmm_csr_values_f64(B.handle, K, Cm.ptr, K, D.ptr, ncols, out_values.ptr),
               "comet_hip_sddmm_csr_values_f64")
        return out_values
    return CsrMatrix(_handle(lib().comet_hip_sddmm_csr_f64(B.handle, K, Cm.ptr, K, D.ptr, ncols),
                             "comet_hip_sddmm_csr_f64"))


def eltwise_mult_dense(A, D, out=None):
    return eltwise_csr_dense(A, D, out, "times")


def eltwise_dense(A, B, out=None, op="times"):
    """out = A (op) B over dense arrays of one shape."""
    if tuple(A.shape) != tuple(B.shape):
        raise ValueError("operands differ in shape")
    if out is None:
        out = DeviceArray(A.shape)
    _check(lib().comet_hip_eltwise_dense_f64(A.size, A.ptr, B.ptr, out.ptr, MULT_OPS[op]), "comet_hip_eltwise_dense_f64")
    return out


def eltwise_mult(A, B):
    return CsrMatrix(_handle(lib().comet_hip_eltwise_mult_csr(A.handle, B.handle), "comet_hip_eltwise_mult_csr"))


def transpose(x, perm, out=None):
    perm = np.ascontiguousarray(perm, dtype=np.int32)
    shape = np.array(x.shape, dtype=np.int64)
    if out is None:
        out = DeviceArray([x.shape[p] for p in perm])
    _check(lib().comet_hip_transpose_f64(len(perm), _vptr(shape), _vptr(perm), x.ptr, out.ptr),
           "comet_hip_transpose_f64")
    return out


def dgemm(A, B, Cm=None, beta=0.0):
    M, K = A.shape
    K2, N = B.shape
    if K != K2:
        raise ValueError("inner dimensions differ")
    if Cm is None:
        Cm = DeviceArray((M, N))
        beta = 0.0
    _check(lib().comet_hip_dgemm_f64(M, N, K, A.ptr, B.ptr, Cm.ptr, beta), "comet_hip_dgemm_f64")
    return Cm


def label_ids(a, b, c):
    """Label numbering by first appearance in A, B, C (frontends/comet_dsl/mlir/MLIRGen.cpp:2236-2276)."""
    ids = {}
    for s in (a, b, c):
        for ch in s:
            ids.setdefault(ch, len(ids))
    conv = lambda s: np.array([ids[ch] for ch in s], dtype=np.int32)
    return ids, conv(a), conv(b), conv(c)


def ttgt_plan(a, b, c, extent, which=-1):
    ids, al, bl, cl = label_ids(a, b, c)
    ext = np.zeros(len(ids), dtype=np.int64)
    for ch, i in ids.items():
        ext[i] = extent[ch]
    plan = TtgtPlan()
    _check(lib().comet_hip_ttgt_plan(len(al), _vptr(al), len(bl), _vptr(bl), len(cl), _vptr(cl), _vptr(ext), which,
                                     C.byref(plan)), "comet_hip_ttgt_plan")
    return plan


def ttgt_contract(a, b, c, A, B, Cm=None, beta=0.0, which=-1, plan=None):
    """Cm[c] = beta*Cm + sum A[a]*B[b] through transposes + GEMM.  Returns (Cm, plan)."""
    extent = {}
    for s, t in ((a, A), (b, B)):
        for ch, n in zip(s, t.shape):
            if extent.setdefault(ch, n) != n:
                raise ValueError(f"label {ch} has two extents")
    if plan is None:
        plan = ttgt_plan(a, b, c, extent, which)
    cshape = [extent[ch] for ch in c]
    if Cm is None:
        Cm = DeviceArray(cshape, zero=True)
    ash, bsh, csh = (np.array(s, dtype=np.int64) for s in (A.shape, B.shape, cshape))
    _check(lib().comet_hip_ttgt_contract(C.byref(plan), _vptr(ash), _vptr(bsh), _vptr(csh), A.ptr, B.ptr, Cm.ptr, beta),
           "comet_hip_ttgt_contract")
    return Cm, plan


# ----------------------------------------------------------------------------- timing
def timer_start():
    _check(lib().comet_hip_timer_start(), "comet_hip_timer_start")


def timer_stop():
    ms = C.c_double()
    _check(lib().comet_hip_timer_stop(C.byref(ms)), "comet_hip_timer_stop")
    return ms.value


def profile_enable(on=True):
    _check(lib().comet_hip_profile_enable(int(on)), "comet_hip_profile_enable")


def profile_reset():
    _check(lib().comet_hip_profile_reset(), "comet_hip_profile_reset")


def profile_report():
    """{kernel name: (launches, total ms)} measured with HIP events on the library's stream."""
    n = C.c_int64()
    _check(lib().comet_hip_profile_query(None, C.byref(n), None), "comet_hip_profile_query")
    out = {}
    buf = C.create_string_buffer(256)
    for i in range(n.value):
        _check(lib().comet_hip_profile_name(i, buf, 256), "comet_hip_profile_name")
        cnt, ms = C.c_int64(), C.c_double()
        _check(lib().comet_hip_profile_query(buf.value, C.byref(cnt), C.byref(ms)), "comet_hip_profile_query")
        out[buf.value.decode()] = (cnt.value, ms.value)
    return out


def memref1d(a):
    m = Memref1D()
    m.allocated = m.aligned = a.ctypes.data
    m.offset = 0
    m.sizes[0] = a.shape[0]
    m.strides[0] = 1
    return m


def memref2d(a):
    m = Memref2D()
    m.allocated = m.aligned = a.ctypes.data
    m.offset = 0
    m.sizes[0], m.sizes[1] = a.shape
    m.strides[0], m.strides[1] = a.shape[1], 1
    return m


def memref_nd(a):
    """An unranked-memref descriptor of a contiguous array: (struct, void pointer to it); keep the struct alive
    while the pointer is in use.  StridedMemRefType<T, N> = {T *allocated; T *aligned; int64 offset;
    int64 sizes[N]; int64 strides[N]}."""
    n = a.ndim

    class _M(C.Structure):
        _fields_ = [("allocated", C.c_void_p), ("aligned", C.c_void_p), ("offset", C.c_int64),
                    ("sizes", C.c_int64 * n), ("strides", C.c_int64 * n)]

    m = _M()
    m.allocated = m.aligned = a.ctypes.data
    m.offset = 0
    for d in range(n):
        m.sizes[d] = a.shape[d]
        m.strides[d] = a.strides[d] // a.itemsize
    return m, C.cast(C.pointer(m), C.c_void_p)

