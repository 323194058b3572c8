"""CPU-side checks of the C-ABI library: it loads, exports what the header declares,
reports errors instead of crashing, and its host-only logic (the TTGT plan) agrees with
the checker.  No kernel is launched here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from comet_amd import runtime as rt
from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "comet_hip_rt.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b((?:comet_hip_|_mlir_ciface_comet_hip_|_mlir_ciface_linalg_|read_input_|Hip|"
                       r"comet_print_memref_|comet_sort)[A-Za-z0-9_]+|getTime|printElapsedTime)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    lib = rt.lib()
    names = _declared_symbols()
    assert len(names) >= 45
    for n in names:
        assert hasattr(lib, n), f"{n} declared in comet_hip_rt.h but not exported"
    assert set(names) == set(rt.SIGNATURES), set(names) ^ set(rt.SIGNATURES)


def test_plan_struct_layout_matches_header():
    # 3 ranks + 6*8 index slots + 4 flags = 55 int32 -> padded to 224 bytes, 3 int64, 1 double, 2 int32
    assert C.sizeof(rt.TtgtPlan) == 224 + 24 + 8 + 8


def _no_gpu():
    try:
        rt.init(0)
        return False
    except rt.CometHipError:
        return True


def test_errors_are_reported_not_fatal():
    if not _no_gpu():
        pytest.skip("GPU present: covered by the gpu tests")
    with pytest.raises(rt.CometHipError) as e:
        rt.init(0)
    assert "no HIP device" in str(e.value) or "failed" in str(e.value)
    # every compute entry point refuses to run instead of falling back to the CPU
    assert rt.lib().comet_hip_malloc(16) == 0
    assert rt.lib().comet_hip_spmv_csr_f64(1, 0, 0, 0) != 0
    assert rt.lib().comet_hip_spmm_csr_f64(1, 4, 0, 4, 0, 4, 0) != 0
    assert rt.lib().comet_hip_dgemm_f64(4, 4, 4, 0, 0, 0, 0.0) != 0
    pos = np.array([0, 1], dtype=np.int64)
    crd = np.array([0], dtype=np.int64)
    val = np.array([1.0])
    assert rt.lib().comet_hip_csr_upload_i64(1, 1, pos.ctypes.data, crd.ctypes.data, val.ctypes.data) == 0
    assert rt.lib().comet_hip_last_error()


CASES = [("aebf", "dfce", "abcd"), ("cima", "mc", "ia"), ("icmn", "mnca", "ia"), ("ca", "ic", "ia"),
         ("aedf", "bfce", "abcd"), ("ab", "bc", "ac"), ("ba", "cb", "ca")]


@pytest.mark.parametrize("a,b,c", CASES)
def test_ttgt_plan_matches_checker(a, b, c):
    sizes = dict(zip("abcdefimn", [2, 3, 4, 5, 3, 2, 3, 4, 2]))
    ref, chosen, ncand, _ = orc.ttgt_plan(a, b, c, sizes)
    for which in [-1] + list(range(ncand)):
        ref, chosen, _, _ = orc.ttgt_plan(a, b, c, sizes, which)
        got = rt.ttgt_plan(a, b, c, sizes, which)
        assert got.candidate == chosen and got.ncandidates == ncand
        for f in ("rankA", "rankB", "rankC", "transA", "transB", "transC", "swapAB", "M", "N", "K"):
            assert getattr(got, f) == getattr(ref, f), (which, f)
        assert got.cost == ref.cost
        for f in ("a_idx", "b_idx", "c_idx", "permA", "permB", "permC"):
            assert list(getattr(got, f)) == list(getattr(ref, f)), (which, f)


def test_ttgt_plan_for_the_benchmark_contraction():
    p = rt.ttgt_plan("aebf", "dfce", "abcd", {ch: 64 for ch in "abcdef"})
    assert (p.candidate, p.ncandidates) == (4, 16)
    assert (p.transA, p.transB, p.transC, p.swapAB) == (1, 1, 0, 0)
    assert (p.M, p.N, p.K) == (4096, 4096, 4096)


def test_ttgt_plan_rejects_non_gemm_expressions():
    with pytest.raises(rt.CometHipError):
        rt.ttgt_plan("ab", "ab", "ab", {"a": 2, "b": 2})        # element-wise: label in A, B and C
    with pytest.raises(rt.CometHipError):
        rt.ttgt_plan("ab", "bc", "ac", {"a": 2, "b": 2, "c": 2}, which=99)


def test_host_utilities_print_sort_and_time(tmp_path):
    """comet_print_memref_*, comet_sort_* and the timers keep the reference's argument lists and text form
    (include/comet/ExecutionEngine/RunnerUtils.h:232-266, lib/ExecutionEngine/StatUtils.cpp:42-59); they need
    no GPU.  Run in a child process so that the C library's stdout can be captured."""
    import subprocess, sys, textwrap
    code = textwrap.dedent("""
        import ctypes as C, numpy as np
        from comet_amd import runtime as rt
        L = rt.lib()
        def desc(a, shape=None, strides=None, offset=0):
            shape = list(a.shape if shape is None else shape)
            strides = list((np.array(a.strides) // a.itemsize) if strides is None else strides)
            n = len(shape)
            class D(C.Structure):
                _fields_ = [("alloc", C.c_void_p), ("aligned", C.c_void_p), ("offset", C.c_int64),
                            ("sizes", C.c_int64 * n), ("strides", C.c_int64 * n)]
            d = D(a.ctypes.data, a.ctypes.data, offset, (C.c_int64 * n)(*shape), (C.c_int64 * n)(*strides))
            return n, d
        keep = []
        def call(fn, a, *extra, **kw):
            n, d = desc(a, **kw); keep.append((a, d))
            fn(n, C.byref(d), *extra)
        call(L.comet_print_memref_f64, np.array([[4.08, 7.65], [0.1 + 0.2, 1e-7], [123456789.0, -0.0]]))
        call(L.comet_print_memref_i64, np.array([0, 2, 4, 5], dtype=np.int64))
        call(L.comet_print_memref_index, np.array([7], dtype=np.int64))
        call(L.comet_print_memref_i32, np.array([[1, -2], [3, 4]], dtype=np.int32))
        call(L.comet_print_memref_f32, np.array([1.5, 2.25], dtype=np.float32))
        call(L.comet_print_memref_f64, np.zeros((0, 3)))                      # empty: prints nothing
        base = np.arange(12, dtype=np.float64)
        call(L.comet_print_memref_f64, base, shape=[2, 3], strides=[1, 4], offset=1)      # a strided view
        v = np.array([9, 3, 7, 1, 8, 2], dtype=np.int64)
        call(L.comet_sort_index, v, 1, 5)
        call(L.comet_print_memref_i64, v)
        w = np.array([5, 4, 3, 2, 1], dtype=np.int32)
        call(L.comet_sort32, w, 0, 5)
        call(L.comet_print_memref_i32, w)
        t0 = L.getTime(); t1 = L.getTime()
        assert 0.0 <= t1 - t0 < 5.0 and t0 > 1.0e9
        L.printElapsedTime(1.0, 3.5)
    """)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert r.returncode == 0, r.stderr
    assert r.stdout == ("data = \n4.08,7.65,0.3,1e-07,1.23457e+08,-0,\n"
                        "data = \n0,2,4,5,\n"
                        "data = \n7,\n"
                        "data = \n1,-2,3,4,\n"
                        "data = \n1.5,2.25,\n"
                        "data = \n1,5,9,2,6,10,\n"
                        "data = \n9,1,3,7,8,2,\n"
                        "data = \n1,2,3,4,5,\n"
                        "ELAPSED_TIME = 2.500000\n")


def test_corrupt_size_lines_and_plans_are_refused_without_a_gpu(tmp_path):
    """Sizes taken from a file or a caller are bounded before anything is reserved or indexed with them."""
    L = rt.lib()
    path = str(tmp_path / "big.mtx")
    with open(path, "w") as f:
        f.write("%%MatrixMarket matrix coordinate real general\n3 3 4000000000000\n1 1 1.0\n")
    assert L.comet_hip_mtx_read_csr(path.encode(), 1) == 0
    assert b"declares" in L.comet_hip_last_error() or b"HIP device" in L.comet_hip_last_error()


def test_lds_fp64_regions_start_on_eight_bytes():
    """The masked-product kernel puts per-wavefront fp64 sums behind a table whose size depends on the column
    count; an odd number of 32-bit words in front of them would misalign its 64-bit LDS atomics.  Every size the
    host can ask for (2^20 columns = 32768 words at most) must give an even offset."""
    L = rt.lib()
    for words in list(range(1, 4097)) + list(range(4097, 32769, 7)) + [32768]:
        off = L.comet_hip_debug_dot_table_words(words)
        assert off > 0 and off % 2 == 0, (words, off)

