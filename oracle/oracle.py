"""ctypes loader for the CPU checker in comet_oracle.c.

Test infrastructure only: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg, never by the comet_amd package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcomet_oracle.so")
TT_MAXRANK = 8

i64p = np.ctypeslib.ndpointer(dtype=np.int64, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
f64p = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")


class TtgtPlan(C.Structure):
    _fields_ = [
        ("rankA", C.c_int32), ("rankB", C.c_int32), ("rankC", C.c_int32),
        ("a_idx", C.c_int32 * TT_MAXRANK), ("b_idx", C.c_int32 * TT_MAXRANK), ("c_idx", C.c_int32 * TT_MAXRANK),
        ("permA", C.c_int32 * TT_MAXRANK), ("permB", C.c_int32 * TT_MAXRANK), ("permC", C.c_int32 * TT_MAXRANK),
        ("transA", C.c_int32), ("transB", C.c_int32), ("transC", C.c_int32), ("swapAB", C.c_int32),
        ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64),
        ("cost", C.c_double),
    ]


def build(force=False):
    """Compile libcomet_oracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH) or (
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "comet_oracle.c"))):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libcomet_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    L = C.CDLL(_LIB_PATH)
    vp = C.c_void_p
    L.oracle_spmv_csr.argtypes = [C.c_int64, i64p, i64p, f64p, f64p, f64p]
    L.oracle_spmv_csr.restype = None
    L.oracle_spmm_csr.argtypes = [C.c_int64, C.c_int64, i64p, i64p, f64p, f64p, f64p]
    L.oracle_spmm_csr.restype = None
    L.oracle_vecmat_csr.argtypes = [C.c_int64, i64p, i64p, f64p, f64p, f64p]
    L.oracle_vecmat_csr.restype = None
    L.oracle_densemat_csr.argtypes = [C.c_int64, C.c_int64, C.c_int64, f64p, i64p, i64p, f64p, f64p]
    L.oracle_densemat_csr.restype = None
    L.oracle_eltwise_csr_dense.argtypes = [C.c_int64, C.c_int64, i64p, i64p, f64p, f64p, C.c_int, f64p]
    L.oracle_eltwise_csr_dense.restype = None
    L.oracle_sddmm_csr.argtypes = [C.c_int64, C.c_int64, i64p, i64p, f64p, C.c_int64, f64p, f64p, f64p]
    L.oracle_sddmm_csr.restype = None
    L.oracle_eltwise_dense.argtypes = [C.c_int64, f64p, f64p, C.c_int, f64p]
    L.oracle_eltwise_dense.restype = None
    L.oracle_spgemm_symbolic.argtypes = [C.c_int64, C.c_int64, C.c_int64, i64p, i64p, i64p, i64p, vp, vp, i64p]
    L.oracle_spgemm_symbolic.restype = C.c_int64
    L.oracle_spgemm_symbolic_omp.argtypes = L.oracle_spgemm_symbolic.argtypes
    L.oracle_spgemm_symbolic_omp.restype = C.c_int64
    L.oracle_spgemm_numeric.argtypes = [C.c_int64, C.c_int64, C.c_int64, i64p, i64p, f64p, i64p, i64p, f64p,
                                        vp, vp, i64p, f64p]
    L.oracle_spgemm_numeric.restype = C.c_int64
    L.oracle_spgemm_numeric_semiring.argtypes = [C.c_int64, C.c_int64, C.c_int64, i64p, i64p, f64p, i64p, i64p, f64p,
                                                 vp, vp, C.c_int, C.c_int, i64p, f64p]
    L.oracle_spgemm_numeric_semiring.restype = C.c_int64
    L.oracle_reduce_sum.argtypes = [f64p, C.c_int64]
    L.oracle_reduce_sum.restype = C.c_double
    L.oracle_eltwise_mult_csr.argtypes = [C.c_int64, i64p, i64p, f64p, i64p, i64p, f64p, i64p, i64p, f64p]
    L.oracle_eltwise_mult_csr.restype = C.c_int64
    L.oracle_tricount_masked.argtypes = [C.c_int64, C.c_int64, i64p, i64p, f64p]
    L.oracle_tricount_masked.restype = C.c_double
    L.oracle_sort_idx.argtypes = [i64p, C.c_int64]
    L.oracle_sort_idx.restype = None
    L.oracle_tricount_masked_omp.argtypes = [C.c_int64, C.c_int64, i64p, i64p, f64p]
    L.oracle_tricount_masked_omp.restype = C.c_double
    L.oracle_spgemm_numeric_omp.argtypes = [C.c_int64, C.c_int64, C.c_int64, i64p, i64p, f64p, i64p, i64p, f64p,
                                            vp, vp, i64p, i64p, f64p]
    L.oracle_spgemm_numeric_omp.restype = C.c_int64
    L.oracle_coo_to_csr.argtypes = [C.c_int64, C.c_int64, i64p, i64p, f64p, C.c_int, vp, vp, vp]
    L.oracle_coo_to_csr.restype = C.c_int64
    L.oracle_read_mtx_csr.argtypes = [C.c_char_p, C.c_int, i64p, vp, vp, vp]
    L.oracle_read_mtx_csr.restype = C.c_int
    L.oracle_format_f64.argtypes = [f64p, C.c_int64, C.c_char_p, C.c_int64]
    L.oracle_format_f64.restype = C.c_int64
    L.oracle_format_i64.argtypes = [i64p, C.c_int64, C.c_char_p, C.c_int64]
    L.oracle_format_i64.restype = C.c_int64
    L.oracle_ttgt_plan.argtypes = [C.c_int32, i32p, C.c_int32, i32p, C.c_int32, i32p, i64p, C.c_int32,
                                   C.POINTER(TtgtPlan), C.POINTER(C.c_int32)]
    L.oracle_ttgt_plan.restype = C.c_int32
    L.oracle_transpose.argtypes = [C.c_int32, i64p, i32p, f64p, f64p]
    L.oracle_transpose.restype = None
    L.oracle_gemm_ijk.argtypes = [C.c_int64, C.c_int64, C.c_int64, f64p, f64p, f64p]
    L.oracle_gemm_ijk.restype = None
    L.oracle_ttgt_contract.argtypes = [C.POINTER(TtgtPlan), i64p, i64p, i64p, f64p, f64p, f64p, C.c_double]
    L.oracle_ttgt_contract.restype = C.c_int
    L.oracle_contract_direct.argtypes = [C.c_int32, i64p, C.c_int32, i32p, C.c_int32, i32p, C.c_int32, i32p,
                                         f64p, f64p, f64p]
    L.oracle_contract_direct.restype = None
    _lib = L
    return L


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def _f64(a):
    return np.ascontiguousarray(a, dtype=np.float64)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


# --------------------------------------------------------------------------- wrappers
def spmv(pos, crd, val, x, y0=None):
    pos, crd, val, x = _i64(pos), _i64(crd), _f64(val), _f64(x)
    n = len(pos) - 1
    y = np.zeros(n) if y0 is None else _f64(y0).copy()
    lib().oracle_spmv_csr(n, pos, crd, val, x, y)
    return y


def spmm(pos, crd, val, B, C0=None):
    pos, crd, val, B = _i64(pos), _i64(crd), _f64(val), _f64(B)
    n, K = len(pos) - 1, B.shape[1]
    Cm = np.zeros((n, K)) if C0 is None else _f64(C0).copy()
    lib().oracle_spmm_csr(n, K, pos, crd, val, B, Cm)
    return Cm


def vecmat(x, pos, crd, val, ncols, y0=None):
    pos, crd, val, x = _i64(pos), _i64(crd), _f64(val), _f64(x)
    y = np.zeros(ncols) if y0 is None else _f64(y0).copy()
    lib().oracle_vecmat_csr(len(pos) - 1, pos, crd, val, x, y)
    return y


def densemat(A, pos, crd, val, ncols, C0=None):
    pos, crd, val, A = _i64(pos), _i64(crd), _f64(val), _f64(A)
    Cm = np.zeros((A.shape[0], ncols)) if C0 is None else _f64(C0).copy()
    lib().oracle_densemat_csr(A.shape[0], len(pos) - 1, ncols, A, pos, crd, val, Cm)
    return Cm


def eltwise_csr_dense(pos, crd, val, D, op="times"):
    """Values of A (op) D at A's stored positions, in storage order."""
    pos, crd, val, D = _i64(pos), _i64(crd), _f64(val), _f64(D)
    out = np.zeros(max(len(val), 1))
    lib().oracle_eltwise_csr_dense(len(pos) - 1, D.shape[1], pos, crd, val, D, MULT_OPS[op], out)
    return out[:len(val)]


def sddmm(pos, crd, val, C, D):
    """Values of B .* (C @ D) at B's stored positions; C is nrows x K, D is K x ncols."""
    pos, crd, val, C, D = _i64(pos), _i64(crd), _f64(val), _f64(C), _f64(D)
    out = np.zeros(max(len(val), 1))
    lib().oracle_sddmm_csr(len(pos) - 1, D.shape[1], pos, crd, val, C.shape[1], C, D, out)
    return out[:len(val)]


def eltwise_mult_dense(pos, crd, val, D):
    return eltwise_csr_dense(pos, crd, val, D, "times")


def eltwise_dense(a, b, op="times"):
    a, b = _f64(a), _f64(b)
    out = np.zeros(a.shape)
    lib().oracle_eltwise_dense(a.size, a, b, MULT_OPS[op], out)
    return out


def spgemm_symbolic(Apos, Acrd, Bpos, Bcrd, ncolsB, mask=None, rows=None, threads=False):
    """Per-row output counts for rows [r0,r1) (default: all rows)."""
    Apos, Acrd, Bpos, Bcrd = _i64(Apos), _i64(Acrd), _i64(Bpos), _i64(Bcrd)
    r0, r1 = (0, len(Apos) - 1) if rows is None else rows
    mpos = mcrd = None
    if mask is not None:
        mpos, mcrd = _i64(mask[0]), _i64(mask[1])
    cnt = np.zeros(max(r1 - r0, 1), dtype=np.int64)
    fn = lib().oracle_spgemm_symbolic_omp if threads else lib().oracle_spgemm_symbolic
    total = fn(r0, r1, ncolsB, Apos, Acrd, Bpos, Bcrd, _ptr(mpos), _ptr(mcrd), cnt)
    return cnt[: r1 - r0], int(total)


REDUCE_OPS = {"plus": 0, "min": 1, "max": 2, "any": 3}
MULT_OPS = {"times": 0, "first": 1, "second": 2, "pair": 3, "plus": 4, "minus": 5, "min": 6, "max": 7, "div": 8}


def spgemm(Apos, Acrd, Aval, Bpos, Bcrd, Bval, ncolsB, mask=None, rows=None, semiring=None, threads=False):
    """Symbolic + numeric; returns (pos, crd, val) for rows [r0,r1) with pos starting at 0.
    semiring = (reduce, mult) names from REDUCE_OPS / MULT_OPS; None is the plain plus-times routine.
    threads=True: the numeric phase row-parallel over the host's cores (plus-times only; same output)."""
    Apos, Acrd, Aval = _i64(Apos), _i64(Acrd), _f64(Aval)
    Bpos, Bcrd, Bval = _i64(Bpos), _i64(Bcrd), _f64(Bval)
    r0, r1 = (0, len(Apos) - 1) if rows is None else rows
    cnt, total = spgemm_symbolic(Apos, Acrd, Bpos, Bcrd, ncolsB, mask, (r0, r1), threads and semiring is None)
    pos = np.zeros(r1 - r0 + 1, dtype=np.int64)
    np.cumsum(cnt, out=pos[1:])
    crd = np.zeros(max(total, 1), dtype=np.int64)
    val = np.zeros(max(total, 1), dtype=np.float64)
    mpos = mcrd = None
    if mask is not None:
        mpos, mcrd = _i64(mask[0]), _i64(mask[1])
    if semiring is None and threads:
        wrote = lib().oracle_spgemm_numeric_omp(r0, r1, ncolsB, Apos, Acrd, Aval, Bpos, Bcrd, Bval,
                                                _ptr(mpos), _ptr(mcrd), pos, crd, val)
    elif semiring is None:
        wrote = lib().oracle_spgemm_numeric(r0, r1, ncolsB, Apos, Acrd, Aval, Bpos, Bcrd, Bval,
                                            _ptr(mpos), _ptr(mcrd), crd, val)
    else:
        wrote = lib().oracle_spgemm_numeric_semiring(r0, r1, ncolsB, Apos, Acrd, Aval, Bpos, Bcrd, Bval,
                                                     _ptr(mpos), _ptr(mcrd), REDUCE_OPS[semiring[0]],
                                                     MULT_OPS[semiring[1]], crd, val)
    assert wrote == total, (wrote, total)
    return pos, crd[:total], val[:total]


def reduce_sum(val):
    val = _f64(val)
    return float(lib().oracle_reduce_sum(val if len(val) else np.zeros(1), len(val)))


def eltwise_mult(Apos, Acrd, Aval, Bpos, Bcrd, Bval):
    Apos, Acrd, Aval = _i64(Apos), _i64(Acrd), _f64(Aval)
    Bpos, Bcrd, Bval = _i64(Bpos), _i64(Bcrd), _f64(Bval)
    n = len(Apos) - 1
    cap = max(1, min(len(Acrd), len(Bcrd)))
    Cpos = np.zeros(n + 1, dtype=np.int64)
    Ccrd = np.zeros(cap, dtype=np.int64)
    Cval = np.zeros(cap)
    nnz = lib().oracle_eltwise_mult_csr(n, Apos, Acrd, Aval, Bpos, Bcrd, Bval, Cpos, Ccrd, Cval)
    return Cpos, Ccrd[:nnz], Cval[:nnz]


def tricount_masked(pos, crd, val, ncols=None, threads=False):
    pos, crd, val = _i64(pos), _i64(crd), _f64(val)
    n = len(pos) - 1
    fn = lib().oracle_tricount_masked_omp if threads else lib().oracle_tricount_masked
    return float(fn(n, n if ncols is None else ncols, pos, crd, val))


def coo_layout(pos, crd, val):
    """The reader's COO arrays for a matrix given as CSR of the kept tuples: A1pos = [0, nnz], A1crd = row
    of every tuple, A2pos unused (-1), A2crd = columns (lib/ExecutionEngine/SparseUtils.cpp:1855-1896; the
    tuples are the same stable (row, col) order the CSR arrays hold)."""
    pos = _i64(pos)
    rows = np.repeat(np.arange(len(pos) - 1, dtype=np.int64), np.diff(pos))
    return np.array([0, len(rows)], dtype=np.int64), rows, np.array([-1], dtype=np.int64), _i64(crd), _f64(val)


def dcsr_layout(pos, crd, val):
    """The reader's DCSR arrays (DcsrMatrix::Init, lib/ExecutionEngine/SparseUtils.cpp:686-735): one A1crd
    entry and one A2pos entry per row that stores anything, a closing A2pos entry, A1pos = [0, stored rows]."""
    pos = _i64(pos)
    a1crd, a2pos = [], []
    for r in range(len(pos) - 1):          # walk the ordered tuples row by row, as the reference does
        if pos[r + 1] != pos[r]:
            a1crd.append(r)
            a2pos.append(int(pos[r]))
    a2pos.append(int(pos[-1]))
    return (np.array([0, len(a1crd)], dtype=np.int64), np.array(a1crd, dtype=np.int64),
            np.array(a2pos, dtype=np.int64), _i64(crd), _f64(val))


def coo_to_csr(nrows, row, col, val, mode=1):
    """Tuples in any order -> (pos, crd, val) the way the reader orders and filters them."""
    row, col, val = _i64(row), _i64(col), _f64(val)
    n = len(row)
    pos = np.zeros(nrows + 1, dtype=np.int64)
    crd = np.zeros(max(n, 1), dtype=np.int64)
    out = np.zeros(max(n, 1))
    kept = lib().oracle_coo_to_csr(nrows, n, row, col, val, mode, _ptr(pos), _ptr(crd), _ptr(out))
    return pos, crd[:kept], out[:kept]


def read_mtx_csr(path, mode=1):
    dims = np.zeros(3, dtype=np.int64)
    rc = lib().oracle_read_mtx_csr(path.encode(), mode, dims, None, None, None)
    if rc:
        raise RuntimeError(f"oracle_read_mtx_csr({path}) failed with code {rc}")
    nrows, ncols, nnz = (int(v) for v in dims)
    pos = np.zeros(nrows + 1, dtype=np.int64)
    crd = np.zeros(max(nnz, 1), dtype=np.int64)
    val = np.zeros(max(nnz, 1))
    rc = lib().oracle_read_mtx_csr(path.encode(), mode, dims, _ptr(pos), _ptr(crd), _ptr(val))
    if rc:
        raise RuntimeError(f"oracle_read_mtx_csr({path}) failed with code {rc}")
    return (nrows, ncols), pos, crd[:nnz], val[:nnz]


def format_f64(v):
    v = _f64(np.ravel(v))
    cap = 32 * len(v) + 64
    buf = C.create_string_buffer(cap)
    lib().oracle_format_f64(v if len(v) else np.zeros(1), len(v), buf, cap)
    return buf.value.decode()


def format_i64(v):
    v = _i64(np.ravel(v))
    cap = 24 * len(v) + 64
    buf = C.create_string_buffer(cap)
    lib().oracle_format_i64(v if len(v) else np.zeros(1, dtype=np.int64), len(v), buf, cap)
    return buf.value.decode()


def labels_to_ids(a, b, c):
    """Label ids in order of first appearance in A, then B, then C
    (frontends/comet_dsl/mlir/MLIRGen.cpp:2236-2276)."""
    ids = {}
    for s in (a, b, c):
        for ch in s:
            ids.setdefault(ch, len(ids))
    conv = lambda s: np.array([ids[ch] for ch in s], dtype=np.int32)
    return ids, conv(a), conv(b), conv(c)


def ttgt_plan(a, b, c, extent, which=-1):
    """a,b,c: label strings (storage order); extent: dict label->size."""
    ids, al, bl, cl = labels_to_ids(a, b, c)
    ext = np.zeros(len(ids), dtype=np.int64)
    for ch, i in ids.items():
        ext[i] = extent[ch]
    plan = TtgtPlan()
    ncand = C.c_int32(0)
    chosen = lib().oracle_ttgt_plan(len(al), al, len(bl), bl, len(cl), cl, ext, which,
                                    C.byref(plan), C.byref(ncand))
    if chosen < 0:
        raise ValueError("not a TTGT-expressible contraction or bad candidate number")
    return plan, int(chosen), int(ncand.value), ids


def transpose(x, perm):
    x = _f64(x)
    perm = np.ascontiguousarray(perm, dtype=np.int32)
    out = np.empty([x.shape[p] for p in perm])
    lib().oracle_transpose(x.ndim, np.array(x.shape, dtype=np.int64), perm, x, out)
    return out


def gemm_ijk(A, B, C0=None):
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    Cm = np.zeros((M, N)) if C0 is None else _f64(C0).copy()
    lib().oracle_gemm_ijk(M, N, K, A, B, Cm)
    return Cm


def ttgt_contract(a, b, c, A, B, C0=None, beta=0.0, which=-1):
    A, B = _f64(A), _f64(B)
    extent = {}
    for s, t in ((a, A), (b, B)):
        for ch, n in zip(s, t.shape):
            extent[ch] = n
    plan, chosen, ncand, ids = ttgt_plan(a, b, c, extent, which)
    cshape = [extent[ch] for ch in c]
    Ct = np.zeros(cshape) if C0 is None else _f64(C0).copy()
    rc = lib().oracle_ttgt_contract(C.byref(plan), np.array(A.shape, dtype=np.int64),
                                    np.array(B.shape, dtype=np.int64), np.array(cshape, dtype=np.int64),
                                    A, B, Ct, beta)
    if rc:
        raise MemoryError("oracle_ttgt_contract")
    return Ct, plan, chosen


def contract_direct(a, b, c, A, B, C0=None):
    A, B = _f64(A), _f64(B)
    ids, al, bl, cl = labels_to_ids(a, b, c)
    extent = {}
    for s, t in ((a, A), (b, B)):
        for ch, n in zip(s, t.shape):
            extent[ch] = n
    ext = np.zeros(len(ids), dtype=np.int64)
    for ch, i in ids.items():
        ext[i] = extent[ch]
    cshape = [extent[ch] for ch in c]
    Ct = np.zeros(cshape) if C0 is None else _f64(C0).copy()
    lib().oracle_contract_direct(len(ids), ext, len(al), al, len(bl), bl, len(cl), cl, A, B, Ct)
    return Ct
