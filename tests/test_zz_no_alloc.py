"""The allocation-free SpMM entry point (comet_hip_spmm_csr_f64_noalloc) against the ordinary one, through
the C ABI: two calls in a row, the second on a smaller matrix, so that what the first call left in the
library's static scratch is still there when the second runs.  Both entry points run the same kernels on
matrices of this size, so the results are compared bit for bit; the ordinary one is itself checked against
the CPU checker here."""
import numpy as np
import pytest

from comet_amd import gen
from comet_amd import runtime as rt
from oracle import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    rt.init(0)
    yield
    rt.sync()


def _free_bytes():
    import ctypes
    free, total = ctypes.c_int64(0), ctypes.c_int64(0)
    assert rt.lib().comet_hip_mem_info(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def _product(n, mean, K, seed, accumulate, ld_pad=0, stream=0):
    pos, crd, val = gen.zipf_csr(n=n, mean=mean, cap=512, seed=seed)
    B = gen.dense((n, K + ld_pad), seed=seed + 1)
    C0 = gen.dense((n, K + ld_pad), seed=seed + 2)
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    dB = rt.DeviceArray.from_numpy(B)
    ld = K + ld_pad
    out = []
    for name in ("comet_hip_spmm_csr_f64", "comet_hip_spmm_csr_f64_noalloc"):
        dC = rt.DeviceArray.from_numpy(C0)
        if name.endswith("noalloc"):
            rt.sync()
            before = _free_bytes()
            rc = rt.lib().comet_hip_spmm_csr_f64_noalloc(A.handle, K, dB.ptr, ld, dC.ptr, ld, int(accumulate), stream)
            if stream:
                assert rt.lib().comet_hip_stream_sync(stream) == 0
            rt.sync()
            assert _free_bytes() == before, "the allocation-free entry point changed the free device memory"
        else:
            rc = rt.lib().comet_hip_spmm_csr_f64(A.handle, K, dB.ptr, ld, dC.ptr, ld, int(accumulate))
        assert rc == 0, rt.lib().comet_hip_last_error().decode()
        out.append(dC.to_numpy())
    # the ordinary entry point against the checker (tolerance of rows cut by a chunk boundary)
    Bk = np.ascontiguousarray(B[:, :K])
    want = orc.spmm(pos, crd, val, Bk) + (C0[:, :K] if accumulate else 0.0)
    bound = orc.spmm(pos, crd, np.abs(val), np.abs(Bk)) + (np.abs(C0[:, :K]) if accumulate else 0.0)
    assert np.all(np.abs(out[0][:, :K] - want) <= 1e-12 * bound)
    return out, len(crd)


def test_noalloc_spmm_matches_ordinary_entry_point_twice_in_a_row():
    # first call: 24,000 rows, about 290,000 nonzeros (1,100 chunks), K = 64
    (ref1, got1), nnz1 = _product(24_000, 12.0, 64, seed=11, accumulate=False)
    assert np.array_equal(ref1, got1)
    # second call, smaller, K = 40 with padded leading dimensions, accumulating: the scratch still holds the
    # first call's table and carry slots
    (ref2, got2), nnz2 = _product(3_000, 6.0, 40, seed=12, accumulate=True, ld_pad=2)
    assert nnz2 < nnz1
    assert np.array_equal(ref2, got2)
    # and once more on the first size: nothing the smaller call left behind matters either
    (ref3, got3), _ = _product(24_000, 12.0, 64, seed=11, accumulate=False)
    assert np.array_equal(ref3, got3) and np.array_equal(got3, got1)


def test_noalloc_spmm_runs_on_the_callers_stream():
    # a stream of the caller's own: the kernels go there (and the result is there once that stream is through)
    s = rt.lib().comet_hip_stream_create()
    assert s != 0
    try:
        (ref, got), _ = _product(6_000, 8.0, 64, seed=21, accumulate=False, stream=s)
        assert np.array_equal(ref, got)
    finally:
        assert rt.lib().comet_hip_stream_destroy(s) == 0


def test_noalloc_spmm_refuses_what_the_scratch_cannot_hold():
    n = 4096
    pos = np.arange(n + 1, dtype=np.int64)
    crd = np.zeros(n, dtype=np.int64)
    A = rt.CsrMatrix.from_arrays((n, 1), pos, crd, np.ones(n))
    K = 64 * 600                        # 600 tiles x 16 chunks = 9,600 slots > 8,192
    rc = rt.lib().comet_hip_spmm_csr_f64_noalloc(A.handle, K, 8, K, 8, K, 0, 0)     # pointers are never touched
    assert rc == 4                      # COMET_HIP_ERR_SIZE
    assert "static scratch" in rt.lib().comet_hip_last_error().decode()


def test_noalloc_spmm_empty_matrix_clears_or_keeps_c():
    A = rt.CsrMatrix.from_arrays((5, 7), np.zeros(6, dtype=np.int64), np.zeros(0, dtype=np.int64), np.zeros(0))
    C0 = gen.dense((5, 4), seed=3)
    B = rt.DeviceArray.from_numpy(gen.dense((7, 4), seed=4))
    for acc in (0, 1):
        dC = rt.DeviceArray.from_numpy(C0)
        assert rt.lib().comet_hip_spmm_csr_f64_noalloc(A.handle, 4, B.ptr, 4, dC.ptr, 4, acc, 0) == 0
        assert np.array_equal(dC.to_numpy(), C0 if acc else np.zeros_like(C0))
