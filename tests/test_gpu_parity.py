"""Parity of the HIP path (called through the C ABI) against the CPU checker on identical
seeded inputs, the reference's golden vectors, and size-independent properties.

Bars: row pointers, column indices and triangle counts bit-exact; fp64 values within
1e-12 relative.  Where a value is a sum of signed products the tolerance is taken
relative to sum(|a||b|) of that entry (the bound summation-order changes obey):
|got - want| <= 1e-12 * sum|a*b|."""
import ctypes as C
import os

import numpy as np
import pytest
import scipy.sparse as sp

from comet_amd import gen
from comet_amd import runtime as rt
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
RTOL = 1e-12


@pytest.fixture(scope="module", autouse=True)
def _device():
    rt.init(0)
    print("device:", rt.device_name(), flush=True)
    yield
    rt.sync()


def _mtx(golden_dir, name, mode=1):
    return orc.read_mtx_csr(os.path.join(golden_dir, name), mode)


def _rand_csr(rng, n, m, density, signed=True):
    A = sp.random(n, m, density=density, random_state=rng, format="csr",
                  data_rvs=lambda k: rng.uniform(-1, 1, k) if signed else rng.uniform(0.1, 1, k))
    A.sort_indices()
    return A.indptr.astype(np.int64), A.indices.astype(np.int64), A.data.copy()


def _abs_csr(pos, crd, val):
    return pos, crd, np.abs(val)


# ----------------------------------------------------------------- runtime plumbing
def test_upload_download_roundtrip_both_index_widths():
    rng = np.random.default_rng(0)
    pos, crd, val = _rand_csr(rng, 300, 200, 0.05)
    A = rt.CsrMatrix.from_arrays((300, 200), pos, crd, val)
    assert A.dims() == (300, 200, len(crd))
    for idt in (np.int64, np.int32):
        p, c, v = A.to_arrays(idt)
        assert np.array_equal(p, pos) and np.array_equal(c, crd) and np.array_equal(v, val)
    B = rt.CsrMatrix.from_arrays((300, 200), pos.astype(np.int32), crd.astype(np.int32), val)
    p, c, v = B.to_arrays()
    assert np.array_equal(p, pos) and np.array_equal(c, crd) and np.array_equal(v, val)


def test_bad_inputs_are_rejected():
    pos = np.array([0, 2, 1], dtype=np.int64)
    with pytest.raises(rt.CometHipError):
        rt.CsrMatrix.from_arrays((2, 2), pos, np.zeros(1, dtype=np.int64), np.zeros(1))
    with pytest.raises(rt.CometHipError):      # column out of range
        rt.CsrMatrix.from_arrays((1, 2), np.array([0, 1]), np.array([5]), np.ones(1))
    with pytest.raises(rt.CometHipError) as e:   # columns of a row must not decrease (duplicates may stay)
        rt.CsrMatrix.from_arrays((2, 4), np.array([0, 3, 4]), np.array([0, 2, 1, 3]), np.ones(4))
    assert "must not decrease" in str(e.value)
    rt.CsrMatrix.from_arrays((2, 4), np.array([0, 3, 4]), np.array([1, 1, 2, 0]), np.ones(4))
    with pytest.raises(rt.CometHipError):
        rt.CsrMatrix.from_arrays((2, 4), np.array([0, 3, 4], dtype=np.int32), np.array([3, 2, 2, 0], dtype=np.int32),
                                 np.ones(4))
    assert rt.lib().comet_hip_spmv_csr_f64(12345, 0, 0, 0) != 0      # unknown handle
    A = rt.CsrMatrix.from_arrays((1, 2), np.array([0, 1]), np.array([1]), np.ones(1))
    B = rt.CsrMatrix.from_arrays((3, 2), np.array([0, 0, 0, 0]), np.zeros(0, dtype=np.int64), np.zeros(0))
    with pytest.raises(rt.CometHipError):      # inner dimensions differ
        rt.spgemm(A, B)


def test_scan_and_reduce():
    rng = np.random.default_rng(1)
    v = rng.integers(0, 1000, 100_003).astype(np.float64)
    d = rt.DeviceArray.from_numpy(v)
    assert rt.reduce_sum(d) == v.sum()            # integers: exact whatever the order
    w = rng.uniform(-1, 1, 1_000_003)
    got = rt.reduce_sum(rt.DeviceArray.from_numpy(w))
    assert abs(got - orc.reduce_sum(w)) <= RTOL * np.abs(w).sum()
    assert rt.reduce_sum(rt.DeviceArray(0), 0) == 0.0


# ----------------------------------------------------------------- SpMV
def test_spmv_golden(golden, golden_dir):
    g = golden["spmv_csr"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"])
    A = rt.CsrMatrix.from_arrays((nr, nc), pos, crd, val)
    y = rt.DeviceArray.from_numpy(np.full(nr, g["y_fill"]))
    rt.spmv(A, rt.DeviceArray.from_numpy(np.full(nc, g["x_fill"])), y)
    assert orc.format_f64(y.to_numpy()) == g["printed"]


@pytest.mark.parametrize("n,m,density,seed", [(1000, 777, 0.01, 0), (4097, 5000, 0.002, 1), (300, 300, 0.2, 2)])
def test_spmv_bit_exact_vs_checker(n, m, density, seed):
    rng = np.random.default_rng(seed)
    pos, crd, val = _rand_csr(rng, n, m, density)
    x = rng.uniform(-1, 1, m)
    y0 = rng.uniform(-1, 1, n)
    A = rt.CsrMatrix.from_arrays((n, m), pos, crd, val)
    dx = rt.DeviceArray.from_numpy(x)
    got_acc = rt.spmv(A, dx, rt.DeviceArray.from_numpy(y0)).to_numpy()
    assert np.array_equal(got_acc, orc.spmv(pos, crd, val, x, y0))
    got = rt.spmv(A, dx).to_numpy()
    assert np.array_equal(got, orc.spmv(pos, crd, val, x))


def test_spmv_poisson_shape_scaled_down():
    pos, crd, val = gen.poisson_csr(n=200_000, mean=10.0, seed=1)
    x = gen.dense(200_000, seed=11)
    A = rt.CsrMatrix.from_arrays((200_000, 200_000), pos, crd, val)
    got = rt.spmv(A, rt.DeviceArray.from_numpy(x)).to_numpy()
    assert np.array_equal(got, orc.spmv(pos, crd, val, x))


@pytest.mark.parametrize("per_block", [False, True])
def test_spmv_column_blocked_plan_is_bit_exact(per_block, monkeypatch):
    # x larger than an L2: the library re-stores A in column blocks and goes through them in order - in one launch
    # with the row sums on chip, or (the switch; also what it does when one grid has no lanes for all rows) one
    # launch per block with the sums going through y; the additions must still happen in the checker's order
    if per_block:
        monkeypatch.setenv("COMET_HIP_SPMV_LAUNCH_PER_BLOCK", "1")
    n = 600_000
    pos, crd, val = gen.poisson_csr(n=n, mean=4.0, seed=5)
    assert len(crd) > (1 << 20)
    x, y0 = gen.dense(n, seed=15), gen.dense(n, seed=16)
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    dx = rt.DeviceArray.from_numpy(x)
    assert np.array_equal(rt.spmv(A, dx).to_numpy(), orc.spmv(pos, crd, val, x))
    assert np.array_equal(rt.spmv(A, dx, rt.DeviceArray.from_numpy(y0)).to_numpy(), orc.spmv(pos, crd, val, x, y0))
    assert np.array_equal(rt.spmv(A, dx).to_numpy(), orc.spmv(pos, crd, val, x))      # plan reused


@pytest.mark.parametrize("n,m,mean", [(3000, 2_000_000, 400.0), (40_000, 700_000, 30.0), (1_300_000, 450_000, 1.0)])
def test_spmv_column_blocked_plan_shapes(n, m, mean):
    """The one-launch form deals the rows evenly to the workgroups the GPU holds at once: few rows (a part of the
    lanes own one), rows of many nonzeros cut by the column blocks, more rows than lanes (several per lane)."""
    rng = np.random.default_rng(n)
    lens = rng.poisson(mean, n)
    pos = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    crd = np.sort((rng.random(int(pos[-1])) * m).astype(np.int64) + np.repeat(np.arange(n, dtype=np.int64) * m, lens)) \
        - np.repeat(np.arange(n, dtype=np.int64) * m, lens)       # sorted inside each row, repeats allowed
    assert len(crd) > (1 << 20)
    val, x, y0 = rng.uniform(-1, 1, len(crd)), rng.uniform(-1, 1, m), rng.uniform(-1, 1, n)
    A = rt.CsrMatrix.from_arrays((n, m), pos, crd, val)
    dx = rt.DeviceArray.from_numpy(x)
    want = orc.spmv(pos, crd, val, x, y0)
    got = rt.spmv(A, dx, rt.DeviceArray.from_numpy(y0)).to_numpy()
    # a row's share of one column block has fewer than 128 products here, so every row is summed in its own order
    assert np.array_equal(got, want)
    assert np.array_equal(rt.spmv(A, dx).to_numpy(), orc.spmv(pos, crd, val, x))


def test_spmv_column_blocked_plan_long_rows():
    """Rows whose share of a column block is long (added by the whole workgroup, to rounding) next to short ones
    (bit-exact) in a matrix that runs as column blocks, several rows per lane."""
    rng = np.random.default_rng(23)
    n, m = 700_000, 600_000
    lens = rng.poisson(2.0, n)
    for at, l in ((0, 5000), (1, 3), (2, 40_000), (255, 700), (256, 513), (300_000, 130_000), (n - 1, 2500)):
        lens[at] = l
    pos = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    off = np.repeat(np.arange(n, dtype=np.int64) * m, lens)
    crd = np.sort((rng.random(int(pos[-1])) * m).astype(np.int64) + off) - off
    val, x, y0 = rng.uniform(-1, 1, len(crd)), rng.uniform(-1, 1, m), rng.uniform(-1, 1, n)
    A = rt.CsrMatrix.from_arrays((n, m), pos, crd, val)
    got = rt.spmv(A, rt.DeviceArray.from_numpy(x), rt.DeviceArray.from_numpy(y0)).to_numpy()
    want = orc.spmv(pos, crd, val, x, y0)
    short = lens < 128
    assert np.array_equal(got[short], want[short])
    bound = orc.spmv(pos, crd, np.abs(val), np.abs(x), np.abs(y0))
    assert np.all(np.abs(got - want) <= RTOL * bound)


@pytest.mark.parametrize("acc", [False, True])
def test_spmv_long_rows(acc):
    """Rows of 127 nonzeros and fewer are summed by one lane in the checker's order (bit-exact); longer ones,
    here up to 60,000 nonzeros and crossing many LDS passes, by the whole workgroup (fixed order, to rounding)."""
    rng = np.random.default_rng(17)
    m = 70_000
    lens = rng.integers(0, 12, 3000)
    for at, l in ((3, 127), (4, 128), (5, 129), (700, 2048), (701, 2049), (1500, 5000), (2999, 60_000), (2000, 300)):
        lens[at] = l
    pos = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    crd = np.concatenate([np.sort(rng.choice(m, l, replace=False)) for l in lens if l]).astype(np.int64)
    val, x, y0 = rng.uniform(-1, 1, len(crd)), rng.uniform(-1, 1, m), rng.uniform(-1, 1, len(lens))
    A = rt.CsrMatrix.from_arrays((len(lens), m), pos, crd, val)
    y = rt.DeviceArray.from_numpy(y0) if acc else None
    got = rt.spmv(A, rt.DeviceArray.from_numpy(x), y).to_numpy()
    want = orc.spmv(pos, crd, val, x, y0 if acc else None)
    short = lens < 128
    assert np.array_equal(got[short], want[short])
    bound = orc.spmv(pos, crd, np.abs(val), np.abs(x), np.abs(y0) if acc else None)
    assert np.all(np.abs(got - want) <= RTOL * bound)
    assert np.array_equal(rt.spmv(A, rt.DeviceArray.from_numpy(x), rt.DeviceArray.from_numpy(y0) if acc else None)
                          .to_numpy(), got)                          # the same bits every time


def test_spmv_edge_cases():
    # empty matrix rows, one very long row (longer than an LDS pass), trailing empty rows
    n, m = 600, 9000
    pos = np.zeros(n + 1, dtype=np.int64)
    pos[5:] = 7000
    pos[300:] = 7003
    crd = np.concatenate([np.arange(7000), np.array([1, 5, 8999])]).astype(np.int64)
    rng = np.random.default_rng(3)
    val = rng.uniform(-1, 1, len(crd))
    x = rng.uniform(-1, 1, m)
    A = rt.CsrMatrix.from_arrays((n, m), pos, crd, val)
    got = rt.spmv(A, rt.DeviceArray.from_numpy(x)).to_numpy()
    want = orc.spmv(pos, crd, val, x)
    short = np.diff(pos) < 128           # longer rows are added by the whole workgroup, in another fixed order
    assert np.array_equal(got[short], want[short])
    assert np.all(np.abs(got - want) <= RTOL * orc.spmv(pos, crd, np.abs(val), np.abs(x)))
    Z = rt.CsrMatrix.from_arrays((3, 3), np.zeros(4, dtype=np.int64), np.zeros(0, dtype=np.int64), np.zeros(0))
    y = rt.spmv(Z, rt.DeviceArray.from_numpy(np.ones(3)), rt.DeviceArray.from_numpy(np.array([1.0, 2.0, 3.0])))
    assert y.to_numpy().tolist() == [1.0, 2.0, 3.0]
    assert rt.spmv(Z, rt.DeviceArray.from_numpy(np.ones(3))).to_numpy().tolist() == [0.0, 0.0, 0.0]


# ----------------------------------------------------------------- SpMM
def test_spmm_golden(golden, golden_dir):
    g = golden["spmm_csr"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"])
    A = rt.CsrMatrix.from_arrays((nr, nc), pos, crd, val)
    Cm = rt.DeviceArray.from_numpy(np.full((nr, g["K"]), g["C_fill"]))
    rt.spmm(A, rt.DeviceArray.from_numpy(np.full((nc, g["K"]), g["B_fill"])), Cm)
    assert orc.format_f64(Cm.to_numpy()) == g["printed"]


def _swept_rows(pos, K):
    """The rows the library hands to the column sweep (its rule restated), as (long, middling).  Middling: the rows
    of 32 to 127 nonzeros and the long rows the sweep has no register for, longest first, at most 288 x g; their
    sums are kept in LDS.  Long: at least 128 nonzeros, at most the
    120 x g longest (ties: lower row first) with g = 32 workgroups of the sweep per XCD - or 24, leaving CUs to
    the chunk kernel beside it, when the rows that are neither long (at g = 32) nor single hold a sixteenth of
    the matrix; COMET_HIP_SPMM_GROUPS overrides g - and only if they hold a quarter of a matrix of >= 2^19
    nonzeros."""
    lens = np.diff(pos)
    rows = np.flatnonzero(lens >= 128)
    rows = rows[np.argsort(-lens[rows], kind="stable")]
    groups = 32
    if (pos[-1] - lens[rows[:3840]].sum() - (lens == 1).sum()) * 16 >= pos[-1]:
        groups = 24
    groups = int(os.environ.get("COMET_HIP_SPMM_GROUPS", groups))
    medium = np.concatenate([rows[120 * groups:], _by_length(lens, np.flatnonzero((lens >= 32) & (lens < 128)))])
    if "COMET_HIP_SPMM_MEDIUM" not in os.environ:        # the library keeps such rows in LDS only when asked to
        medium = medium[:0]
    rows = rows[:120 * groups]
    if not (16 <= K <= 2048) or pos[-1] < (1 << 19) or 4 * lens[rows].sum() < pos[-1]:
        return rows[:0], rows[:0]
    return rows, medium[:288 * groups]


def _by_length(lens, rows):
    return rows[np.argsort(-lens[rows], kind="stable")]


def _bit_exact_rows(pos, K):
    """Rows summed in the checker's order: those that lie inside one 256-nonzero chunk of the matrix the
    chunk kernel sees (with long rows: the rows of two and more nonzeros that are not long, packed), and the
    rows of at most one nonzero."""
    lens = np.diff(pos)
    light = lens.copy()
    long_rows, medium_rows = _swept_rows(pos, K)
    if len(long_rows):
        light[long_rows] = 0
        light[medium_rows] = 0      # summed per XCD, then across: not the checker's order
        light[lens == 1] = 0        # these ride on the sweep: one product each
    lpos = np.concatenate([[0], np.cumsum(light)])
    return (lens <= 1) | ((light > 0) & (lpos[:-1] // 256 == (lpos[1:] - 1) // 256))


def _spmm_check(pos, crd, val, B, C0=None):
    n = len(pos) - 1
    A = rt.CsrMatrix.from_arrays((n, B.shape[0]), pos, crd, val)
    dB = rt.DeviceArray.from_numpy(B)
    if C0 is None:
        got = rt.spmm(A, dB).to_numpy()
    else:
        got = rt.spmm(A, dB, rt.DeviceArray.from_numpy(C0)).to_numpy()
    want = orc.spmm(pos, crd, val, B, C0)
    inside = _bit_exact_rows(pos, B.shape[1])
    assert np.array_equal(got[inside], want[inside])
    bound = orc.spmm(pos, crd, np.abs(val), np.abs(B), None if C0 is None else np.abs(C0))
    assert np.all(np.abs(got - want) <= RTOL * bound + 0.0)
    return got, want


@pytest.mark.parametrize("n,m,K,density,seed", [(500, 400, 64, 0.02, 0), (1000, 1000, 64, 0.3, 1),
                                                (257, 129, 7, 0.1, 2), (64, 64, 130, 0.2, 3)])
def test_spmm_vs_checker(n, m, K, density, seed):
    rng = np.random.default_rng(seed)
    pos, crd, val = _rand_csr(rng, n, m, density)
    B = rng.uniform(-1, 1, (m, K))
    _spmm_check(pos, crd, val, B)
    _spmm_check(pos, crd, val, B, rng.uniform(-1, 1, (n, K)))


def test_spmm_zipf_shape_scaled_down():
    pos, crd, val = gen.zipf_csr(n=50_000, mean=16.0, cap=4096, seed=2)
    B = gen.dense((50_000, 64), seed=12)
    got, want = _spmm_check(pos, crd, val, B)
    assert np.diff(pos).max() > 1024     # really has rows that span several chunks


def test_spmm_edge_cases():
    rng = np.random.default_rng(5)
    # leading, interior and trailing empty rows; a row ending exactly on a chunk boundary; one huge row
    lens = np.array([0, 0, 256, 0, 1, 255, 0, 1000, 0, 0, 3, 0], dtype=np.int64)
    m = 2000
    pos = np.zeros(len(lens) + 1, dtype=np.int64)
    np.cumsum(lens, out=pos[1:])
    crd = np.concatenate([np.sort(rng.choice(m, l, replace=False)) for l in lens]).astype(np.int64)
    val = rng.uniform(-1, 1, len(crd))
    B = rng.uniform(-1, 1, (m, 64))
    got, want = _spmm_check(pos, crd, val, B)
    assert np.all(got[lens == 0] == 0.0)
    C0 = rng.uniform(-1, 1, (len(lens), 64))
    got, want = _spmm_check(pos, crd, val, B, C0)
    assert np.array_equal(got[lens == 0], C0[lens == 0])
    # no nonzeros at all
    Z = rt.CsrMatrix.from_arrays((4, 5), np.zeros(5, dtype=np.int64), np.zeros(0, dtype=np.int64), np.zeros(0))
    out = rt.spmm(Z, rt.DeviceArray.from_numpy(np.ones((5, 3))), rt.DeviceArray.from_numpy(np.ones((4, 3))),
                  accumulate=False)
    assert np.all(out.to_numpy() == 0.0)


def test_spmm_linearity_at_full_width():
    # size-independent property: A(B1 + B2) == AB1 + AB2 up to rounding, on a bigger power-law matrix
    pos, crd, val = gen.zipf_csr(n=100_000, mean=16.0, cap=4096, seed=7)
    A = rt.CsrMatrix.from_arrays((100_000, 100_000), pos, crd, val)
    B1, B2 = gen.dense((100_000, 64), seed=21), gen.dense((100_000, 64), seed=22)
    c1 = rt.spmm(A, rt.DeviceArray.from_numpy(B1)).to_numpy()
    c2 = rt.spmm(A, rt.DeviceArray.from_numpy(B2)).to_numpy()
    c12 = rt.spmm(A, rt.DeviceArray.from_numpy(B1 + B2)).to_numpy()
    scale = np.abs(c1) + np.abs(c2) + 1.0
    assert np.all(np.abs(c12 - (c1 + c2)) <= 1e-9 * scale)


# ----------------------------------------------------------------- SpGEMM
def test_spgemm_golden(golden, golden_dir):
    for key, masked in (("spgemm_csr", False), ("spgemm_csr_masked", True)):
        g = golden[key]
        (nr, nc), pos, crd, val = _mtx(golden_dir, g["A"])
        A = rt.CsrMatrix.from_arrays((nr, nc), pos, crd, val)
        Cm = rt.spgemm(A, A, A if masked else None)
        p, c, v = Cm.to_arrays()
        assert p.tolist() == g["pos"] and c.tolist() == g["crd"]
        assert orc.format_f64(v) == g["printed_val"]


SEMIRING_CASES = ["any_pair", "min_first", "min_plus", "min_second", "plus_first", "plus_pair", "plus_second",
                  "plus_times"]


@pytest.mark.parametrize("name", SEMIRING_CASES)
def test_spgemm_semiring_golden(golden, golden_dir, name):
    g = golden["spgemm_csr_semiring"]
    c = g["cases"][name]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["A"])
    A = rt.CsrMatrix.from_arrays((nr, nc), pos, crd, val)
    p, cc, v = rt.spgemm(A, A, semiring=(c["reduce"], c["mult"])).to_arrays()
    assert p.tolist() == g["pos"] and cc.tolist() == g["crd"]
    assert orc.format_f64(v) == c["printed_val"]


@pytest.mark.parametrize("reduce", ["plus", "min", "max", "any"])
@pytest.mark.parametrize("mult", ["times", "first", "second", "pair", "plus", "minus", "min", "max", "div"])
def test_spgemm_semiring_vs_checker(reduce, mult):
    rng = np.random.default_rng(sum(map(ord, reduce + mult)))
    n, k, m = 300, 257, 2000
    apos, acrd, aval = _rand_csr(rng, n, k, 0.05)
    bpos, bcrd, bval = _rand_csr(rng, k, m, 0.04)
    bval = np.abs(bval) + 0.5          # keeps div finite
    A = rt.CsrMatrix.from_arrays((n, k), apos, acrd, aval)
    B = rt.CsrMatrix.from_arrays((k, m), bpos, bcrd, bval)
    p, c, v = rt.spgemm(A, B, semiring=(reduce, mult)).to_arrays()
    wp, wc, wv = orc.spgemm(apos, acrd, aval, bpos, bcrd, bval, m, semiring=(reduce, mult))
    assert np.array_equal(p, wp) and np.array_equal(c, wc)
    if reduce == "plus":    # sums arrive in any order
        _, _, count = orc.spgemm(apos, acrd, aval, bpos, bcrd, bval, m, semiring=("plus", "pair"))
        amax, bmax, bmin = np.abs(aval).max(), bval.max(), bval.min()
        biggest = max(amax * bmax, amax + bmax, amax / bmin, 1.0)       # no product exceeds this
        assert np.all(np.abs(v - wv) <= RTOL * count * biggest)
    else:                   # min, max and any do not depend on the order: bit-exact
        assert np.array_equal(v, wv)


def test_spgemm_semiring_masked_rowblocks_and_reuse():
    """A masked min-plus product in two row blocks, then plain plus-times on the same handles: the
    accumulators a semiring leaves behind must not leak into the next call."""
    rng = np.random.default_rng(12)
    n = 500
    pos, crd, val = _rand_csr(rng, n, n, 0.03, signed=False)
    mpos, mcrd, _ = _rand_csr(rng, n, n, 0.05)
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    Mk = rt.CsrMatrix.from_arrays((n, n), mpos, mcrd, np.ones(len(mcrd)))
    cpos, nnz = rt.spgemm_symbolic(A, A, Mk)
    hp = cpos.to_numpy()
    wp, wc, wv = orc.spgemm(pos, crd, val, pos, crd, val, n, mask=(mpos, mcrd), semiring=("min", "plus"))
    assert np.array_equal(hp, wp)
    for r0, r1 in ((0, 211), (211, n)):
        cnt = int(hp[r1] - hp[r0])
        dcrd = rt.DeviceArray(max(cnt, 1), np.int32)
        dval = rt.DeviceArray(max(cnt, 1))
        rt.spgemm_numeric(A, A, cpos, r0, r1, dcrd, dval, mask=Mk, semiring=("min", "plus"))
        assert np.array_equal(dcrd.to_numpy()[:cnt], wc[hp[r0]:hp[r1]])
        assert np.array_equal(dval.to_numpy()[:cnt], wv[hp[r0]:hp[r1]])
    for sr in (("max", "times"), ("any", "second"), None):
        p, c, v = rt.spgemm(A, A, semiring=sr).to_arrays()
        wp, wc, wv = orc.spgemm(pos, crd, val, pos, crd, val, n, semiring=sr)
        assert np.array_equal(p, wp) and np.array_equal(c, wc)
        if sr is None:
            assert np.allclose(v, wv, rtol=1e-12, atol=0)
        else:
            assert np.array_equal(v, wv)


def test_spgemm_semiring_rejects_unknown_operator():
    pos = np.array([0, 1], dtype=np.int64)
    A = rt.CsrMatrix.from_arrays((1, 1), pos, np.array([0], dtype=np.int64), np.array([1.0]))
    h = rt.lib().comet_hip_spgemm_csr_semiring(A.handle, A.handle, 0, 9, 0)
    assert h == 0 and b"semiring" in rt.lib().comet_hip_last_error()


def _spgemm_check(a, b, ncolsB, mask=None):
    (apos, acrd, aval), (bpos, bcrd, bval) = a, b
    n, kdim = len(apos) - 1, len(bpos) - 1
    A = rt.CsrMatrix.from_arrays((n, kdim), apos, acrd, aval)
    B = rt.CsrMatrix.from_arrays((kdim, ncolsB), bpos, bcrd, bval)
    Mk = None if mask is None else rt.CsrMatrix.from_arrays((n, ncolsB), mask[0], mask[1], np.ones(len(mask[1])))
    Cm = rt.spgemm(A, B, Mk)
    p, c, v = Cm.to_arrays()
    wp, wc, wv = orc.spgemm(apos, acrd, aval, bpos, bcrd, bval, ncolsB, mask=mask)
    assert np.array_equal(p, wp), "row pointers differ"
    assert np.array_equal(c, wc), "column indices differ"
    _, _, bound = orc.spgemm(apos, acrd, np.abs(aval), bpos, bcrd, np.abs(bval), ncolsB, mask=mask)
    assert np.all(np.abs(v - wv) <= RTOL * bound)
    return p, c, v


@pytest.mark.parametrize("n,k,m,density,seed,signed", [(300, 200, 250, 0.05, 0, True), (1000, 1000, 1000, 0.01, 1, False),
                                                       (64, 64, 40_000, 0.05, 2, True), (2000, 50, 33, 0.3, 3, True)])
def test_spgemm_vs_checker(n, k, m, density, seed, signed):
    rng = np.random.default_rng(seed)
    a = _rand_csr(rng, n, k, density, signed)
    b = _rand_csr(rng, k, m, density, signed)
    _spgemm_check(a, b, m)


@pytest.mark.parametrize("dot", [True, False])
@pytest.mark.parametrize("seed", [0, 1])
def test_spgemm_masked_vs_checker(seed, dot, monkeypatch):
    # a masked product is taken pair by pair of the mask (dot products) or, with the switch, row by row of A
    if not dot:
        monkeypatch.setenv("COMET_HIP_SPGEMM_NO_DOT", "1")
    rng = np.random.default_rng(seed)
    a = _rand_csr(rng, 400, 400, 0.04, signed=False)
    mk = _rand_csr(rng, 400, 400, 0.1, signed=False)
    _spgemm_check(a, a, 400, mask=(mk[0], mk[1]))


@pytest.mark.parametrize("n,k,m,da,db,dm,seed", [(500, 300, 700, 0.05, 0.04, 0.08, 0), (64, 5000, 64, 0.3, 0.3, 0.9, 1),
                                                 (3000, 33, 2000, 0.2, 0.1, 0.01, 2), (200, 40_000, 300, 0.01, 0.002, 0.5, 3),
                                                 (50, 70, (1 << 20) + 999, 0.3, 0.00001, 0.00002, 4)])
def test_spgemm_masked_dot_products(n, k, m, da, db, dm, seed):
    """C<M> = A*B with three different rectangular matrices: rows of A against columns of B pair by pair of the mask,
    the shorter list of a pair streamed against a table of the longer; whole and in row blocks; empty rows and
    columns; an inner dimension that is no multiple of 32; more than 2^20 columns of B."""
    rng = np.random.default_rng(100 + seed)
    a = _rand_csr(rng, n, k, da, signed=True)
    b = _rand_csr(rng, k, m, db, signed=True)
    mk = _rand_csr(rng, n, m, dm, signed=False)
    _spgemm_check(a, b, m, mask=(mk[0], mk[1]))
    A = rt.CsrMatrix.from_arrays((n, k), *a)
    B = rt.CsrMatrix.from_arrays((k, m), *b)
    Mk = rt.CsrMatrix.from_arrays((n, m), mk[0], mk[1], np.ones(len(mk[1])))
    dpos, nnz = rt.spgemm_symbolic(A, B, mask=Mk)
    hp = dpos.to_numpy()
    wp, wc, wv = orc.spgemm(*a, *b, m, mask=(mk[0], mk[1]))
    _, _, bound = orc.spgemm(a[0], a[1], np.abs(a[2]), b[0], b[1], np.abs(b[2]), m, mask=(mk[0], mk[1]))
    assert np.array_equal(hp, wp) and nnz == wp[-1]
    for rb, re in ((0, n // 3), (n // 3, n // 3 + 1), (n // 3 + 1, n)):
        cnt = int(hp[re] - hp[rb])
        dc, dv = rt.DeviceArray(max(cnt, 1), np.int32), rt.DeviceArray(max(cnt, 1))
        rt.spgemm_numeric(A, B, dpos, rb, re, dc, dv, mask=Mk)
        assert np.array_equal(dc.to_numpy(cnt), wc[hp[rb]:hp[re]])
        assert np.all(np.abs(dv.to_numpy(cnt) - wv[hp[rb]:hp[re]]) <= RTOL * bound[hp[rb]:hp[re]])


@pytest.mark.parametrize("semiring", [("min", "plus"), ("max", "times"), ("plus", "first"), ("min", "div"), ("max", "minus"),
                                      ("plus", "pair"), ("any", "second")])
def test_spgemm_masked_dot_products_semirings(semiring):
    """The dot-product form under other semirings: the order of the two operands of `mult` is A's entry first in
    both halves; min and max are exact, sums to rounding; `any` takes the walk by rows."""
    rng = np.random.default_rng(77)
    n, k, m = 700, 900, 800
    a = _rand_csr(rng, n, k, 0.05, signed=True)
    b = _rand_csr(rng, k, m, 0.04, signed=True)
    b = (b[0], b[1], np.where(b[2] < 0, b[2] - 0.25, b[2] + 0.25))          # keeps div finite
    la = np.diff(a[0])
    mk = _rand_csr(rng, n, m, 0.2, signed=False)
    A = rt.CsrMatrix.from_arrays((n, k), *a)
    B = rt.CsrMatrix.from_arrays((k, m), *b)
    Mk = rt.CsrMatrix.from_arrays((n, m), mk[0], mk[1], np.ones(len(mk[1])))
    wp, wc, wv = orc.spgemm(*a, *b, m, mask=(mk[0], mk[1]), semiring=semiring)
    for _ in range(2):
        p, c, v = rt.spgemm(A, B, Mk, semiring=semiring).to_arrays()
        assert np.array_equal(p, wp) and np.array_equal(c, wc)
        if semiring[0] == "plus":
            _, _, bound = orc.spgemm(a[0], a[1], np.abs(a[2]), b[0], b[1], np.abs(b[2]), m, mask=(mk[0], mk[1]),
                                     semiring=semiring)
            assert np.all(np.abs(v - wv) <= RTOL * np.maximum(bound, 1.0))
        else:
            assert np.array_equal(v, wv)
    _spgemm_check(a, b, m, mask=(mk[0], mk[1]))        # plus-times afterwards finds nothing left behind


def test_spgemm_masked_inner_dimension_beyond_the_table():
    """More than 2^20 columns of A (= rows of B): the table over k of the dot-product form does not fit LDS, and the
    masked product is walked by rows."""
    rng = np.random.default_rng(5)
    n, k, m = 40, (1 << 20) + 77, 300
    cols = np.sort(rng.choice(k, 2000, replace=False))            # the inner indices that are used at all
    a = _rows_of_lengths(rng, rng.integers(0, 60, n), k, pick=cols)
    lb = np.zeros(k, dtype=np.int64); lb[cols] = rng.integers(0, 8, len(cols))
    b = _rows_of_lengths(rng, lb, m)
    mk = _rand_csr(rng, n, m, 0.5, signed=False)
    rt.profile_reset(); rt.profile_enable(True)
    _spgemm_check(a, b, m, mask=(mk[0], mk[1]))
    rt.sync()
    fired = rt.profile_report()
    rt.profile_enable(False)
    assert not any("dot" in name for name in fired), sorted(fired)


def test_spgemm_masked_dot_products_hubs_and_repeats():
    """Lists of very different lengths (a few rows of A and columns of B with thousands of entries among short ones:
    each half of the pairs has work), and a matrix that holds a column twice in a row, which the tables cannot
    take: that product is walked row by row as before."""
    rng = np.random.default_rng(41)
    n = k = m = 6000
    la = rng.integers(0, 12, n); la[rng.choice(n, 8, replace=False)] = 4000
    lb = rng.integers(0, 12, k); lb[rng.choice(k, 8, replace=False)] = 3000
    a = _rows_of_lengths(rng, la, k)
    bt = _rows_of_lengths(rng, lb, k)                    # rows here = columns of B: transpose on the host
    rows_b = np.repeat(np.arange(m), lb)
    order = np.lexsort((rows_b, bt[1]))
    bpos = np.concatenate([[0], np.cumsum(np.bincount(bt[1], minlength=k))]).astype(np.int64)
    b = (bpos, rows_b[order].astype(np.int64), bt[2][order])
    lm = rng.integers(0, 40, n); lm[rng.choice(n, 5, replace=False)] = 5000
    mk = _rows_of_lengths(rng, lm, m)
    _spgemm_check(a, b, m, mask=(mk[0], mk[1]))
    # the same product with an entry of A stored twice
    apos, acrd, aval = a
    r = int(np.argmax(la))
    at = int(apos[r]) + 5
    acrd2 = np.insert(acrd, at, acrd[at]); aval2 = np.insert(aval, at, 0.5)
    apos2 = apos.copy(); apos2[r + 1:] += 1
    _spgemm_check((apos2, acrd2, aval2), b, m, mask=(mk[0], mk[1]))


def test_spgemm_wide_matrix_uses_global_bitmap():
    # more than 2^20 columns: the row bitmap no longer fits LDS
    rng = np.random.default_rng(4)
    ncols = (1 << 20) + 4097
    a = _rand_csr(rng, 50, 60, 0.2, signed=False)
    bpos = np.arange(0, 61 * 40, 40, dtype=np.int64)
    bcrd = np.concatenate([np.sort(rng.choice(ncols, 40, replace=False)) for _ in range(60)]).astype(np.int64)
    bval = rng.uniform(0.1, 1, len(bcrd))
    _spgemm_check(a, (bpos, bcrd, bval), ncols)
    rows = [np.unique(rng.choice(bcrd, 30)) for _ in range(50)]     # mask rows drawn from reachable columns
    mk_pos = np.zeros(51, dtype=np.int64)
    np.cumsum([len(r) for r in rows], out=mk_pos[1:])
    _spgemm_check(a, (bpos, bcrd, bval), ncols, mask=(mk_pos, np.concatenate(rows)))


def test_spgemm_row_blocks_equal_whole():
    pos, crd, val = gen.rmat_symmetric_csr(scale=11, edge_factor=8, seed=5)
    n = 1 << 11
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    dpos, nnz = rt.spgemm_symbolic(A, A)
    wp, wc, wv = orc.spgemm(pos, crd, val, pos, crd, val, n)
    hp = dpos.to_numpy()
    assert np.array_equal(hp, wp) and nnz == wp[-1]
    for rb, re in ((0, 7), (7, 1024), (1024, n)):
        cnt = int(hp[re] - hp[rb])
        dc, dv = rt.DeviceArray(max(cnt, 1), np.int32), rt.DeviceArray(max(cnt, 1))
        rt.spgemm_numeric(A, A, dpos, rb, re, dc, dv)
        c, v = dc.to_numpy()[:cnt], dv.to_numpy()[:cnt]
        assert np.array_equal(c, wc[hp[rb]:hp[re]])
        assert np.all(np.abs(v - wv[hp[rb]:hp[re]]) <= RTOL * np.abs(wv[hp[rb]:hp[re]]))


def _rows_of_lengths(rng, lengths, ncols, pick=None, signed=True):
    """CSR with the given row lengths; columns drawn without repetition from `pick` (default: all columns)."""
    pos = np.zeros(len(lengths) + 1, dtype=np.int64)
    np.cumsum(lengths, out=pos[1:])
    pool = np.arange(ncols) if pick is None else np.asarray(pick)
    crd = np.concatenate([np.sort(rng.choice(pool, l, replace=False)) for l in lengths] + [np.zeros(0, dtype=np.int64)])
    val = rng.uniform(-1, 1, len(crd)) if signed else rng.uniform(0.1, 1, len(crd))
    return pos, crd.astype(np.int64), val


@pytest.mark.parametrize("row_major", [False, True])
@pytest.mark.parametrize("m,long_len,wide,cols32", [(200_000, 2000, None, False), (40_000, 1200, None, False),
                                                    (40_000, 1200, 1 << 40, False), (200_000, 2000, 1 << 40, False),
                                                    (200_000, 2000, 0, False), (200_000, 2000, 0, True),
                                                    (1_000_000, 3000, None, False), (1_000_000, 3000, None, True)])
def test_spgemm_rows_of_every_class(m, long_len, wide, cols32, row_major, monkeypatch):
    # Rows of B: 200 long ones and 200 of 10 entries.  Rows of A pick among them so that the product has rows
    # for each numeric kernel: no products, a few (values kept in a slab), thousands spread thinly over the
    # column blocks (several blocks per visit, values compact) and many per block (one block per visit).
    # `wide` moves the border between the last two: with 1 << 40 every heavy row takes the several-block
    # kernel, and with 40,000 columns the thick rows then exceed the compact array, so their visits are cut
    # short at a block boundary; with 0 every heavy row takes one block per visit.
    # The one-block kernel reads B's columns as 16-bit numbers inside their block (a copy the library keeps with the
    # block pointers), or with cols32 the 32-bit ones.  It takes its rows block by block, all rows through block 0
    # first (a row's place in C is handed from block to block), or with row_major each row through all its blocks.
    if row_major:
        monkeypatch.setenv("COMET_HIP_SPGEMM_ROW_MAJOR", "1")
    if wide is not None:
        monkeypatch.setenv("COMET_HIP_SPGEMM_WIDE", str(wide))
    if cols32:
        monkeypatch.setenv("COMET_HIP_SPGEMM_WIDE_COLUMNS", "1")
    rng = np.random.default_rng(17)
    k = 400
    b = _rows_of_lengths(rng, [long_len] * 200 + [10] * 200, m)
    long_rows, short_rows = np.arange(200), np.arange(200, 400)
    lengths, picks = [], []
    for n_long, n_short in [(0, 0), (0, 5), (1, 0), (3, 2), (10, 0), (25, 40), (40, 0), (120, 3), (200, 200), (0, 200),
                            (2, 0), (60, 0), (0, 1), (7, 7)] * 3:
        lengths.append(n_long + n_short)
        picks.append(np.sort(np.concatenate([rng.choice(long_rows, n_long, replace=False),
                                             rng.choice(short_rows, n_short, replace=False)])))
    apos = np.zeros(len(lengths) + 1, dtype=np.int64)
    np.cumsum(lengths, out=apos[1:])
    acrd = np.concatenate(picks).astype(np.int64)
    a = (apos, acrd, rng.uniform(-1, 1, len(acrd)))
    first = _spgemm_check(a, b, m)
    second = _spgemm_check(a, b, m)          # the kernels leave their LDS and slabs clean
    assert np.array_equal(first[1], second[1])


@pytest.mark.parametrize("semiring", [("min", "plus"), ("max", "times"), ("any", "second"), ("any", "pair"),
                                      ("plus", "first"), ("min", "div")])
@pytest.mark.parametrize("m,long_len,wide", [(200_000, 2000, None), (40_000, 1200, 1 << 40), (200_000, 2000, 0)])
def test_spgemm_semiring_rows_of_every_class(semiring, m, long_len, wide, monkeypatch):
    # the rows of test_spgemm_rows_of_every_class under other semirings: the kernels that keep a row's values in
    # LDS hold keys there instead of sums (min, max: order-preserving keys; any: the place of the product)
    if wide is not None:
        monkeypatch.setenv("COMET_HIP_SPGEMM_WIDE", str(wide))
    rng = np.random.default_rng(29)
    k = 400
    bpos, bcrd, bval = _rows_of_lengths(rng, [long_len] * 200 + [10] * 200, m)
    bval = np.where(bval < 0, bval - 0.25, bval + 0.25)          # keeps div finite
    long_rows, short_rows = np.arange(200), np.arange(200, 400)
    lengths, picks = [], []
    for n_long, n_short in [(0, 0), (0, 5), (1, 0), (3, 2), (10, 0), (25, 40), (40, 0), (120, 3), (200, 200), (0, 200),
                            (2, 0), (60, 0), (0, 1), (7, 7)] * 2:
        lengths.append(n_long + n_short)
        picks.append(np.sort(np.concatenate([rng.choice(long_rows, n_long, replace=False),
                                             rng.choice(short_rows, n_short, replace=False)])))
    apos = np.zeros(len(lengths) + 1, dtype=np.int64)
    np.cumsum(lengths, out=apos[1:])
    acrd = np.concatenate(picks).astype(np.int64)
    aval = rng.uniform(-1, 1, len(acrd))
    A = rt.CsrMatrix.from_arrays((len(lengths), k), apos, acrd, aval)
    B = rt.CsrMatrix.from_arrays((k, m), bpos, bcrd, bval)
    wp, wc, wv = orc.spgemm(apos, acrd, aval, bpos, bcrd, bval, m, semiring=semiring)
    for _ in range(2):          # twice: the accumulators are left clean
        p, c, v = rt.spgemm(A, B, semiring=semiring).to_arrays()
        assert np.array_equal(p, wp) and np.array_equal(c, wc)
        if semiring[0] == "plus":
            _, _, bound = orc.spgemm(apos, acrd, np.abs(aval), bpos, bcrd, np.abs(bval), m, semiring=semiring)
            assert np.all(np.abs(v - wv) <= RTOL * bound)
        else:
            assert np.array_equal(v, wv)
    p, c, v = rt.spgemm(A, B).to_arrays()          # and a plus-times product after them finds nothing left behind
    _, _, pv = orc.spgemm(apos, acrd, aval, bpos, bcrd, bval, m)
    _, _, bound = orc.spgemm(apos, acrd, np.abs(aval), bpos, bcrd, np.abs(bval), m)
    assert np.array_equal(c, wc) and np.all(np.abs(v - pv) <= RTOL * bound)


@pytest.mark.parametrize("semiring", [None, "rows", ("min", "plus"), ("any", "first")])
def test_spgemm_masked_long_mask_rows(semiring, monkeypatch):
    # mask rows of 0, 5, 6144 (the longest the hash table of the slab kernel takes), 6145, 20,000 and 70,000
    # entries: the long ones take the one-block kernel, which adds every product and drops the columns outside
    # the mask when a block is written out; the row pointers come from the masked symbolic phase
    # (plus-times goes pair by pair of the mask unless told otherwise: "rows" is that product walked row by row)
    if semiring == "rows":
        monkeypatch.setenv("COMET_HIP_SPGEMM_NO_DOT", "1")
        semiring = None
    rng = np.random.default_rng(31)
    k, m = 300, 100_000
    bpos, bcrd, bval = _rows_of_lengths(rng, [3000] * 200 + [10] * 100, m, signed=False)
    lengths = [50, 0, 7, 120, 300, 1, 64, 200] * 3
    apos, acrd, aval = _rows_of_lengths(rng, lengths, k, signed=False)
    mlens = [20_000, 70_000, 6145, 0, 6144, 5, 70_000, 30_000] * 3
    mpos, mcrd, _ = _rows_of_lengths(rng, mlens, m)
    A = rt.CsrMatrix.from_arrays((len(lengths), k), apos, acrd, aval)
    B = rt.CsrMatrix.from_arrays((k, m), bpos, bcrd, bval)
    Mk = rt.CsrMatrix.from_arrays((len(lengths), m), mpos, mcrd, np.ones(len(mcrd)))
    wp, wc, wv = orc.spgemm(apos, acrd, aval, bpos, bcrd, bval, m, mask=(mpos, mcrd), semiring=semiring)
    for _ in range(2):
        p, c, v = rt.spgemm(A, B, Mk, semiring=semiring).to_arrays()
        assert np.array_equal(p, wp) and np.array_equal(c, wc)
        if semiring is None:
            assert np.all(np.abs(v - wv) <= RTOL * np.abs(wv))       # positive values: no cancellation
        else:
            assert np.array_equal(v, wv)
    _spgemm_check((apos, acrd, aval), (bpos, bcrd, bval), m)        # and nothing is left behind for a plain product


@pytest.mark.parametrize("wide,row_major", [(1 << 40, False), (0, False), (0, True)])
def test_spgemm_rows_with_more_entries_than_lanes(wide, row_major, monkeypatch):
    # more than 1024 entries in a row of A: the LDS kernels then fetch the row's entries again at every visit
    # instead of holding one per lane; `wide` sends the rows through either kernel, row_major the one-block
    # kernel's rows one after the other instead of block by block
    monkeypatch.setenv("COMET_HIP_SPGEMM_WIDE", str(wide))
    if row_major:
        monkeypatch.setenv("COMET_HIP_SPGEMM_ROW_MAJOR", "1")
    rng = np.random.default_rng(23)
    k, m = 3000, 40_000
    b = _rows_of_lengths(rng, rng.integers(0, 17, k), m)
    a = _rows_of_lengths(rng, [2500, 1100, 30, 0, 1025, 3000, 2049], k)
    _spgemm_check(a, b, m)


def test_spgemm_block_by_block_wait_is_bounded(monkeypatch):
    # Block by block, the workgroup that writes a row's entries of one column block waits for the count of the
    # block before, which another workgroup publishes.  The wait gives up after a number of polls (here: one, so
    # that it may well do so), the kernel then still ends and the call fails with an error instead of returning a
    # wrong product; the next call, with the usual patience, is right.
    rng = np.random.default_rng(41)
    k, m = 64, 100_000
    b = _rows_of_lengths(rng, [3000] * k, m)
    a = _rows_of_lengths(rng, [40] * 300, k)
    monkeypatch.setenv("COMET_HIP_SPGEMM_WIDE", "0")
    monkeypatch.setenv("COMET_HIP_SPGEMM_PATIENCE", "1")
    try:
        _spgemm_check(a, b, m)
    except RuntimeError as e:
        assert "never arrived" in str(e)
    monkeypatch.delenv("COMET_HIP_SPGEMM_PATIENCE")
    _spgemm_check(a, b, m)


@pytest.mark.parametrize("scale", [16, 20])
def test_spgemm_rmat_row_blocks_vs_checker(scale):
    """C = A*A on the benchmark's own generator at edge factor 16 - at scale 16 (65,536 vertices, 1.8 M entries,
    1.24e9 products) and at the benchmark's scale 20 (31 M entries, 7.0e10 products): the symbolic phase over all
    rows, the numeric phase on sampled blocks of 64 rows against the checker.  At scale 16 the block with the
    heaviest row, the hub rows at the low ids, the tail, and random ones; at scale 20, where the hub rows alone
    would keep the checker busy for minutes, the heaviest block of at most 1.5e8 products, the tail, the middle
    and random ones of at most 5e7.  Real R-MAT rows of every class (values in a slab, several column blocks per
    visit, one block per visit) go through the kernel that serves their class."""
    n = 1 << scale
    pos, crd, val = gen.rmat_symmetric_csr(scale=scale, edge_factor=16, seed=20)
    deg = np.diff(pos)
    rowprod = np.zeros(n, dtype=np.int64)
    nz = deg > 0
    rowprod[nz] = np.add.reduceat(deg[crd], pos[:-1][nz])
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    dpos, nnzC = rt.spgemm_symbolic(A, A)
    hpos = dpos.to_numpy()
    assert hpos[0] == 0 and hpos[-1] == nnzC and np.all(np.diff(hpos) >= 0)
    rng = np.random.default_rng(5)
    if scale == 16:
        starts = {int(np.argmax(rowprod)) // 64 * 64, 0, 64, n - 64, n // 2}
        starts |= {int(b) * 64 for b in rng.choice(n // 64, 10, replace=False)}
    else:
        blockprod = rowprod.reshape(-1, 64).sum(axis=1)
        fits = np.flatnonzero(blockprod <= 150_000_000)
        starts = {int(fits[np.argmax(blockprod[fits])]) * 64, n - 64, n // 2}
        starts |= {int(b) * 64 for b in rng.choice(np.flatnonzero(blockprod <= 50_000_000), 8, replace=False)}
    rt.profile_reset()
    rt.profile_enable(True)
    checked = 0
    for r0 in sorted(starts):
        r1 = r0 + 64
        cp, cc, cv = orc.spgemm(pos, crd, val, pos, crd, val, n, rows=(r0, r1))
        assert np.array_equal(cp, hpos[r0:r1 + 1] - hpos[r0]), f"row pointer of rows [{r0},{r1})"
        cnt = int(hpos[r1] - hpos[r0])
        dcrd, dval = rt.DeviceArray(max(cnt, 1), np.int32), rt.DeviceArray(max(cnt, 1))
        rt.spgemm_numeric(A, A, dpos, r0, r1, dcrd, dval)
        gc, gv = dcrd.to_numpy(cnt), dval.to_numpy(cnt)
        assert np.array_equal(gc, cc), f"columns of rows [{r0},{r1})"
        assert np.all(np.abs(gv - cv) <= RTOL * np.abs(cv)), f"values of rows [{r0},{r1})"      # all products positive
        checked += int(rowprod[r0:r1].sum())
    rt.sync()
    fired = rt.profile_report()
    rt.profile_enable(False)
    for k in ("spgemm_numeric", "spgemm_numeric_span", "spgemm_numeric_dense_blocks"):
        assert k in fired and fired[k][0] > 0, f"{k} never ran on these rows"
    assert checked > 50_000_000
    # the masked product C<A> = A*A on the same blocks (structure = mask entries that receive a product)
    mpos, mnnz = rt.spgemm_symbolic(A, A, mask=A)
    hm = mpos.to_numpy()
    for r0 in sorted(starts)[:6 if scale == 16 else 3]:
        r1 = r0 + 64
        cp, cc, cv = orc.spgemm(pos, crd, val, pos, crd, val, n, mask=(pos, crd), rows=(r0, r1))
        assert np.array_equal(cp, hm[r0:r1 + 1] - hm[r0])
        cnt = int(hm[r1] - hm[r0])
        dcrd, dval = rt.DeviceArray(max(cnt, 1), np.int32), rt.DeviceArray(max(cnt, 1))
        rt.spgemm_numeric(A, A, mpos, r0, r1, dcrd, dval, mask=A)
        assert np.array_equal(dcrd.to_numpy(cnt), cc)
        assert np.all(np.abs(dval.to_numpy(cnt) - cv) <= RTOL * np.abs(cv))
    if scale > 16:          # (test_headline_workloads_at_full_size counts the triangles of that graph)
        return
    # and the triangle count of the same graph
    lpos, lcrd, lval = gen.strictly_lower(pos, crd, np.ones_like(val))
    L = rt.CsrMatrix.from_arrays((n, n), lpos, lcrd, lval)
    assert rt.triangle_count(L) == orc.tricount_masked(lpos, lcrd, lval)


def test_spgemm_empty_and_repeatable():
    Z = rt.CsrMatrix.from_arrays((3, 3), np.zeros(4, dtype=np.int64), np.zeros(0, dtype=np.int64), np.zeros(0))
    p, c, v = rt.spgemm(Z, Z).to_arrays()
    assert p.tolist() == [0, 0, 0, 0] and len(c) == 0
    # the dense slabs and bitmaps must be left clean: a second product gives the same answer
    rng = np.random.default_rng(9)
    a = _rand_csr(rng, 500, 500, 0.03, signed=False)
    first = _spgemm_check(a, a, 500)
    second = _spgemm_check(a, a, 500)
    assert np.array_equal(first[1], second[1])


# ----------------------------------------------------------------- triangle counting / SUM / eltwise
def test_triangle_count_golden(golden, golden_dir):
    g = golden["triangle_count"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"], g["read_mode"])
    L = rt.CsrMatrix.from_arrays((nr, nc), pos, crd, val)
    assert rt.triangle_count(L) == g["count"]
    # the two-statement program: C<L> = L*L ; SUM(C)
    assert rt.sum_values(rt.spgemm(L, L, L)) == g["count"]
    # the unmasked program: SUM((L*L) .* L)
    E = rt.eltwise_mult(rt.spgemm(L, L), L)
    assert E.to_arrays()[2].sum() == g["count"]


@pytest.mark.parametrize("scale,ef,seed", [(10, 8, 1), (13, 16, 2)])
def test_triangle_count_rmat_vs_checker_and_trace(scale, ef, seed):
    pos, crd, val = gen.rmat_symmetric_csr(scale=scale, edge_factor=ef, seed=seed, values="ones")
    lpos, lcrd, lval = gen.strictly_lower(pos, crd, val)
    n = 1 << scale
    L = rt.CsrMatrix.from_arrays((n, n), lpos, lcrd, lval)
    got = rt.triangle_count(L)
    assert got == orc.tricount_masked(lpos, lcrd, lval)
    if scale <= 10:
        Adj = sp.csr_matrix((val, crd, pos), shape=(n, n))
        assert got == (Adj @ Adj @ Adj).diagonal().sum() / 6
    # invariant: the upper-triangular formulation counts the same triangles
    U = sp.csr_matrix((lval, lcrd, lpos), shape=(n, n)).T.tocsr()
    U.sort_indices()
    Ud = rt.CsrMatrix.from_scipy(U)
    assert rt.triangle_count(Ud) == got


def test_headline_workloads_at_full_size(monkeypatch):
    """The benchmark's own SpMM, SpMV, triangle-count and TTGT inputs at their full sizes, every entry of the
    results against the checker (the SpGEMM of that size writes 285 GB: test_spgemm_rmat_row_blocks_vs_checker
    samples it, and so does bench.py): the products without a plan (a matrix's first) and with it (its second)."""
    monkeypatch.delenv("COMET_HIP_PLAN_AT_ONCE")
    n, K = 500_000, 64
    pos, crd, val = gen.zipf_csr(n=n, mean=16.0, cap=4096, seed=2)
    B = gen.dense((n, K), seed=3)
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    dB, dC = rt.DeviceArray.from_numpy(B), rt.DeviceArray((n, K))
    want = orc.spmm(pos, crd, val, B)
    bound = orc.spmm(pos, crd, np.abs(val), np.abs(B))
    for call in range(2):
        rep = _kernels_of(lambda: rt.spmm(A, dB, dC, accumulate=False))
        assert ("spmm_heavy_sweep" in rep) == (call == 1)
        assert np.all(np.abs(dC.to_numpy() - want) <= RTOL * bound), f"spmm, call {call}"
    del A, dB, dC, B, want, bound
    n = 1_000_000
    pos, crd, val = gen.poisson_csr(n=n, mean=10.0, seed=1)
    x = gen.dense(n, seed=4)
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    dx, dy = rt.DeviceArray.from_numpy(x), rt.DeviceArray(n)
    want = orc.spmv(pos, crd, val, x)
    for call in range(2):
        rt.spmv(A, dx, dy, accumulate=False)
        assert np.array_equal(dy.to_numpy(), want), f"spmv, call {call}"
    del A, dx, dy
    pos, crd, val = gen.rmat_symmetric_csr(scale=20, edge_factor=16, seed=20, values="ones")
    lpos, lcrd, lval = gen.strictly_lower(pos, crd, val)
    L = rt.CsrMatrix.from_arrays((1 << 20, 1 << 20), lpos, lcrd, lval)
    assert rt.triangle_count(L) == orc.tricount_masked(lpos, lcrd, lval)
    del L, lpos, lcrd, lval
    # the contraction of the TTGT workload, every extent 64 (a 4096^3 GEMM), against the same GEMM by the host's BLAS
    # (the checker's triple loop would take minutes): |difference| <= 1e-12 * sum |a||b| for every entry
    A, B = gen.dense((64,) * 4, seed=5), gen.dense((64,) * 4, seed=6)
    Cm, _ = rt.ttgt_contract("aebf", "dfce", "abcd", rt.DeviceArray.from_numpy(A), rt.DeviceArray.from_numpy(B))
    A2 = np.ascontiguousarray(A.transpose(0, 2, 1, 3)).reshape(4096, 4096)          # [a b | e f]
    B2 = np.ascontiguousarray(B.transpose(3, 1, 2, 0)).reshape(4096, 4096)          # [e f | c d]
    assert np.all(np.abs(Cm.to_numpy().reshape(4096, 4096) - A2 @ B2) <= RTOL * (np.abs(A2) @ np.abs(B2)))


def test_masked_sum_general_values():
    rng = np.random.default_rng(3)
    a = _rand_csr(rng, 300, 300, 0.05)
    mk = _rand_csr(rng, 300, 300, 0.2)
    A = rt.CsrMatrix.from_arrays((300, 300), *a)
    Mk = rt.CsrMatrix.from_arrays((300, 300), *mk)
    got = rt.spgemm_masked_sum(A, A, Mk)
    wp, wc, wv = orc.spgemm(*a, *a, 300, mask=(mk[0], mk[1]))
    _, _, bound = orc.spgemm(a[0], a[1], np.abs(a[2]), a[0], a[1], np.abs(a[2]), 300, mask=(mk[0], mk[1]))
    assert abs(got - orc.reduce_sum(wv)) <= RTOL * bound.sum()


def _pattern_case(rng, ncols, entries, blen, mlen, nrows, bvalue):
    """`nrows` output rows with `entries` stored entries each (random values), every one naming a row of B with
    `blen` columns and the one value `bvalue`; a mask row of `mlen` columns, half of them taken from the columns B
    uses so that products do meet the mask."""
    rows = [np.sort(rng.choice(ncols, blen, replace=False)) for _ in range(entries)]
    bpos = np.zeros(ncols + 1, np.int64)
    bpos[1:entries + 1] = np.cumsum([blen] * entries)
    bpos[entries + 1:] = bpos[entries]
    bcrd = np.concatenate(rows).astype(np.int32)
    b = (bpos, bcrd, np.full(len(bcrd), bvalue))
    apos = np.zeros(ncols + 1, np.int64)
    apos[ncols - nrows + 1:] = np.arange(1, nrows + 1) * entries
    a = (apos, np.tile(np.arange(entries, dtype=np.int32), nrows), rng.uniform(0.5, 1.5, entries * nrows))
    used = np.unique(bcrd)
    masks = [np.unique(np.concatenate([rng.choice(used, min(mlen // 2, len(used)), replace=False),
                                       rng.choice(ncols, mlen - mlen // 2, replace=False)])) for _ in range(nrows)]
    mpos = np.zeros(ncols + 1, np.int64)
    mpos[ncols - nrows + 1:] = np.cumsum([len(m) for m in masks])
    mcrd = np.concatenate(masks).astype(np.int32)
    return a, b, (mpos, mcrd, np.ones(len(mcrd)))


@pytest.mark.parametrize("only", [None, "workgroup", "wavefront"])
def test_masked_sum_pattern_matrix(only, monkeypatch):
    """B with one value for all its entries takes kernels of its own that count the hits of a row of B instead of
    fetching values.  Every class of rows - few and many entries in A's row (more than a wavefront's 64 and a
    workgroup's 1024 lanes), rows of B below and above the lengths at which four, two and one of them share a
    wavefront and longer than one turn, mask rows that fit the wavefront's table (up to 48 columns), that do not,
    and empty ones - through both kernels together and through each alone."""
    if only:
        monkeypatch.setenv("COMET_HIP_MASKED_SUM_ONLY", only)
    rng = np.random.default_rng(11)
    ncols = 1 << 13
    cases = [(e, bl, ml, nr) for e in (1, 17, 70, 257, 1100) for bl in (3, 63, 64, 255, 256, 511, 512, 1027, 2500)
             for ml in (0, 4, 48, 49, 300) for nr in (1, 7)]
    for k, (e, bl, ml, nr) in enumerate(cases):
        if k % 3 != (0 if only is None else 1 if only == "workgroup" else 2) and (e, bl) != (257, 63):
            continue            # a third of the grid per mode, and the round with one row left over in all of them
        a, b, m = _pattern_case(rng, ncols, e, bl, ml, nr, 0.75)
        A, B, M = (rt.CsrMatrix.from_arrays((ncols, ncols), *x) for x in (a, b, m))
        got = rt.spgemm_masked_sum(A, B, M)
        wp, wc, wv = orc.spgemm(*a, *b, ncols, mask=(m[0], m[1]))
        want = orc.reduce_sum(wv)
        assert abs(got - want) <= RTOL * abs(want), (e, bl, ml, nr)
    # the same kernels on a graph, whole numbers: exact
    pos, crd, val = gen.rmat_symmetric_csr(scale=13, edge_factor=16, seed=5, values="ones")
    lpos, lcrd, lval = gen.strictly_lower(pos, crd, val)
    L = rt.CsrMatrix.from_arrays((1 << 13, 1 << 13), lpos, lcrd, lval)
    rep = _kernels_of(lambda: rt.triangle_count(L))
    assert ("spgemm_masked_sum" in rep) == (only != "wavefront")
    assert ("spgemm_masked_sum_small" in rep) == (only != "workgroup")
    assert rt.triangle_count(L) == orc.tricount_masked(lpos, lcrd, lval)
    # an infinite value in a row of A whose products all miss the mask adds nothing
    a, b, m = _pattern_case(rng, ncols, 5, 100, 10, 1, 1.0)
    mpos = np.zeros(ncols + 1, np.int64)
    mpos[ncols] = 10
    m = (mpos, np.setdiff1d(np.arange(ncols, dtype=np.int32), b[1])[:10].astype(np.int32), np.ones(10))
    a[2][:] = np.inf
    A, B, M = (rt.CsrMatrix.from_arrays((ncols, ncols), *x) for x in (a, b, m))
    assert rt.spgemm_masked_sum(A, B, M) == 0.0


def test_masked_sum_kernels_share_a_simd():
    """The two kernels of the pattern-matrix masked sum run side by side on the same CUs only while four wavefronts
    of the workgroup kernel and one of the wavefront kernel fit the 512 vector registers of a SIMD (allotted in
    eights): one register more in the first and the triangle count takes 40 % longer."""
    import ctypes as C
    wg, wave = C.c_int(), C.c_int()
    rt._check(rt.lib().comet_hip_debug_masked_sum_registers(C.byref(wg), C.byref(wave)), "registers")
    up8 = lambda r: (r + 7) // 8 * 8
    assert 4 * up8(wg.value) + up8(wave.value) <= 512, (wg.value, wave.value)


def test_eltwise_golden_and_random(golden, golden_dir):
    g = golden["eltwise_mult_csr"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["A"])
    A = rt.CsrMatrix.from_arrays((nr, nc), pos, crd, val)
    p, c, v = rt.eltwise_mult(A, A).to_arrays()
    assert p.tolist() == g["pos"] and c.tolist() == g["crd"] and orc.format_f64(v) == g["printed_val"]
    rng = np.random.default_rng(2)
    a, b = _rand_csr(rng, 500, 300, 0.1), _rand_csr(rng, 500, 300, 0.1)
    p, c, v = rt.eltwise_mult(rt.CsrMatrix.from_arrays((500, 300), *a), rt.CsrMatrix.from_arrays((500, 300), *b)).to_arrays()
    wp, wc, wv = orc.eltwise_mult(*a, *b)
    assert np.array_equal(p, wp) and np.array_equal(c, wc) and np.array_equal(v, wv)


# ----------------------------------------------------------------- transposes, GEMM, TTGT
@pytest.mark.parametrize("shape,perm", [((3, 4, 5, 2), (0, 2, 1, 3)), ((3, 4, 5, 2), (3, 1, 2, 0)),
                                        ((7, 9), (1, 0)), ((16, 33, 65), (2, 0, 1)), ((4, 1, 6, 1, 5), (4, 3, 2, 1, 0)),
                                        ((5, 6, 7), (0, 1, 2)), ((64, 3, 64), (2, 1, 0))])
def test_transpose_matches_checker(shape, perm):
    rng = np.random.default_rng(0)
    x = rng.uniform(-1, 1, shape)
    got = rt.transpose(rt.DeviceArray.from_numpy(x), perm).to_numpy()
    assert np.array_equal(got, orc.transpose(x, perm))
    assert np.array_equal(got, np.transpose(x, perm))


@pytest.mark.parametrize("M,N,K", [(128, 128, 16), (256, 384, 128), (100, 70, 33), (1, 5, 9), (130, 129, 1), (16, 16, 4)])
def test_dgemm_vs_checker(M, N, K):
    rng = np.random.default_rng(M + N + K)
    A, B, C0 = rng.uniform(-1, 1, (M, K)), rng.uniform(-1, 1, (K, N)), rng.uniform(-1, 1, (M, N))
    dA, dB = rt.DeviceArray.from_numpy(A), rt.DeviceArray.from_numpy(B)
    bound = np.abs(A) @ np.abs(B)
    got = rt.dgemm(dA, dB).to_numpy()
    assert np.all(np.abs(got - orc.gemm_ijk(A, B)) <= RTOL * bound)
    got1 = rt.dgemm(dA, dB, rt.DeviceArray.from_numpy(C0), beta=1.0).to_numpy()
    assert np.all(np.abs(got1 - orc.gemm_ijk(A, B, C0)) <= RTOL * (bound + np.abs(C0)))


def test_ttgt_goldens(golden):
    for g in golden["ttgt"]:
        A = np.full([g["extent"][ch] for ch in g["A"]], g["A_fill"])
        B = np.full([g["extent"][ch] for ch in g["B"]], g["B_fill"])
        Cm, plan = rt.ttgt_contract(g["A"], g["B"], g["C"], rt.DeviceArray.from_numpy(A), rt.DeviceArray.from_numpy(B))
        assert orc.format_f64(Cm.to_numpy()) == g["printed"], g["source"]


@pytest.mark.parametrize("a,b,c", [("aebf", "dfce", "abcd"), ("cima", "mc", "ia"), ("icmn", "mnca", "ia")])
def test_ttgt_every_candidate_vs_checker(a, b, c):
    rng = np.random.default_rng(4)
    sizes = dict(zip("abcdefimn", [4, 3, 8, 5, 6, 7, 3, 4, 2]))
    A = rng.uniform(-1, 1, [sizes[ch] for ch in a])
    B = rng.uniform(-1, 1, [sizes[ch] for ch in b])
    dA, dB = rt.DeviceArray.from_numpy(A), rt.DeviceArray.from_numpy(B)
    bound = np.einsum(f"{a},{b}->{c}", np.abs(A), np.abs(B))
    ncand = rt.ttgt_plan(a, b, c, sizes).ncandidates
    C0 = rng.uniform(-1, 1, bound.shape)
    for which in [-1] + list(range(ncand)):
        want, _, chosen = orc.ttgt_contract(a, b, c, A, B, which=which)
        Cm, plan = rt.ttgt_contract(a, b, c, dA, dB, which=which)
        assert plan.candidate == chosen
        assert np.all(np.abs(Cm.to_numpy() - want) <= RTOL * bound), which
        want1, _, _ = orc.ttgt_contract(a, b, c, A, B, C0=C0, beta=1.0, which=which)
        Cm1, _ = rt.ttgt_contract(a, b, c, dA, dB, Cm=rt.DeviceArray.from_numpy(C0), beta=1.0, which=which)
        assert np.all(np.abs(Cm1.to_numpy() - want1) <= RTOL * (bound + np.abs(C0))), which


def test_ttgt_benchmark_contraction_scaled_down():
    # same index pattern as the 64^4 contraction at extent 16: GEMM 256 x 256 x 256
    rng = np.random.default_rng(6)
    A, B = rng.uniform(-1, 1, (16,) * 4), rng.uniform(-1, 1, (16,) * 4)
    Cm, plan = rt.ttgt_contract("aebf", "dfce", "abcd", rt.DeviceArray.from_numpy(A), rt.DeviceArray.from_numpy(B))
    assert plan.candidate == 4
    want, _, _ = orc.ttgt_contract("aebf", "dfce", "abcd", A, B)
    bound = np.einsum("aebf,dfce->abcd", np.abs(A), np.abs(B))
    assert np.all(np.abs(Cm.to_numpy() - want) <= RTOL * bound)
    assert np.allclose(Cm.to_numpy(), np.einsum("aebf,dfce->abcd", A, B), rtol=0, atol=1e-11)


# ----------------------------------------------------------------- memref entry points
@pytest.mark.parametrize("idt", [np.int64, np.int32])
def test_mlir_ciface_entry_points(golden, golden_dir, idt):
    """The memref-descriptor forms for both index widths: i64 (CPU lowering) and i32 (what --target=GPU makes
    the lowered code pass, frontends/comet_dsl/comet.cpp:817-823)."""
    sfx = "i64" if idt == np.int64 else "i32"
    fn = lambda name: getattr(rt.lib(), f"_mlir_ciface_comet_hip_{name}_f64_{sfx}")
    (nr, nc), pos, crd, val = _mtx(golden_dir, "test_rank2.mtx")
    pos, crd = pos.astype(idt), crd.astype(idt)
    x, y = np.full(nc, 1.7), np.zeros(nr)
    fn("spmv_csr")(rt.memref1d(pos), rt.memref1d(crd), rt.memref1d(val), rt.memref1d(x), rt.memref1d(y))
    assert orc.format_f64(y) == golden["spmv_csr"]["printed"]
    B, Cm = np.full((nc, 4), 1.7), np.zeros((nr, 4))
    fn("spmm_csr")(rt.memref1d(pos), rt.memref1d(crd), rt.memref1d(val), rt.memref2d(B), rt.memref2d(Cm))
    assert orc.format_f64(Cm) == golden["spmm_csr"]["printed"]
    sizes = np.zeros(1, dtype=np.int64)          # sizes are `index` values for either width
    empty = np.zeros(0, dtype=idt)
    fn("spgemm_csr_sizes")(nr, nc, rt.memref1d(pos), rt.memref1d(crd), rt.memref1d(val),
                           rt.memref1d(pos), rt.memref1d(crd), rt.memref1d(val),
                           rt.memref1d(empty), rt.memref1d(empty), rt.memref1d(sizes))
    assert sizes[0] == 9
    cp, cc, cv = np.zeros(nr + 1, dtype=idt), np.zeros(9, dtype=idt), np.zeros(9)
    fn("spgemm_csr_fill")(rt.memref1d(cp), rt.memref1d(cc), rt.memref1d(cv))
    g = golden["spgemm_csr"]
    assert cp.tolist() == g["pos"] and cc.tolist() == g["crd"] and orc.format_f64(cv) == g["printed_val"]
    # the masked product through the same pair of calls (mask = B, the reference's masked golden)
    fn("spgemm_csr_sizes")(nr, nc, rt.memref1d(pos), rt.memref1d(crd), rt.memref1d(val),
                           rt.memref1d(pos), rt.memref1d(crd), rt.memref1d(val),
                           rt.memref1d(pos), rt.memref1d(crd), rt.memref1d(sizes))
    gm = golden["spgemm_csr_masked"]
    assert sizes[0] == len(gm["crd"])
    cp, cc, cv = np.zeros(nr + 1, dtype=idt), np.zeros(int(sizes[0]), dtype=idt), np.zeros(int(sizes[0]))
    fn("spgemm_csr_fill")(rt.memref1d(cp), rt.memref1d(cc), rt.memref1d(cv))
    assert cp.tolist() == gm["pos"] and cc.tolist() == gm["crd"] and orc.format_f64(cv) == gm["printed_val"]
    (tr, tc), tpos, tcrd, tval = _mtx(golden_dir, "tc.mtx", 2)
    assert fn("tricount")(tc, rt.memref1d(tpos.astype(idt)), rt.memref1d(tcrd.astype(idt)), rt.memref1d(tval)) == 5.0
    # two of the reference's semiring goldens through the semiring pair of calls
    gs = golden["spgemm_csr_semiring"]
    for name in ("min_plus", "any_pair"):
        case = gs["cases"][name]
        r, m = rt.REDUCE_OPS[case["reduce"]], rt.MULT_OPS[case["mult"]]
        fn("spgemm_csr_sizes_semiring")(nr, nc, rt.memref1d(pos), rt.memref1d(crd), rt.memref1d(val),
                                        rt.memref1d(pos), rt.memref1d(crd), rt.memref1d(val),
                                        rt.memref1d(empty), rt.memref1d(empty), rt.memref1d(sizes), r, m)
        assert sizes[0] == len(gs["crd"])
        cp, cc, cv = np.zeros(nr + 1, dtype=idt), np.zeros(int(sizes[0]), dtype=idt), np.zeros(int(sizes[0]))
        fn("spgemm_csr_fill_semiring")(rt.memref1d(cp), rt.memref1d(cc), rt.memref1d(cv))
        assert cp.tolist() == gs["pos"] and cc.tolist() == gs["crd"] and orc.format_f64(cv) == case["printed_val"]


def test_mlir_ciface_dense_contraction(golden):
    """The contraction on host memrefs in one call: the reference's four constant-fill results, a random rank-4
    case against the checker (overwriting and accumulating), and the reference's matmul entry point by name."""
    L = rt.lib()

    def contract(a, b, c, A, B, Cm, beta):
        ids, al, bl, cl = rt.label_ids(a, b, c)
        labs = [np.array(x, dtype=np.int64) + 10 for x in (al, bl, cl)]       # any integers will do as labels
        (ma, pa), (mb, pb), (mc, pc) = rt.memref_nd(A), rt.memref_nd(B), rt.memref_nd(Cm)
        L._mlir_ciface_comet_hip_ttgt_contract_f64(A.ndim, pa, B.ndim, pb, Cm.ndim, pc, rt.memref1d(labs[0]),
                                                   rt.memref1d(labs[1]), rt.memref1d(labs[2]), beta)

    for g in golden["ttgt"]:
        A = np.full([g["extent"][ch] for ch in g["A"]], g["A_fill"])
        B = np.full([g["extent"][ch] for ch in g["B"]], g["B_fill"])
        Cm = np.full([g["extent"][ch] for ch in g["C"]], 99.0)        # beta = 0 overwrites
        contract(g["A"], g["B"], g["C"], A, B, Cm, 0.0)
        assert orc.format_f64(Cm) == g["printed"], g["source"]
    sizes = {"a": 5, "b": 3, "c": 4, "d": 6, "e": 7, "f": 2}
    a, b, c = "aebf", "dfce", "abcd"
    A = gen.dense([sizes[ch] for ch in a], seed=61)
    B = gen.dense([sizes[ch] for ch in b], seed=62)
    C0 = gen.dense([sizes[ch] for ch in c], seed=63)
    bound = np.einsum("aebf,dfce->abcd", np.abs(A), np.abs(B))
    want0, _, _ = orc.ttgt_contract(a, b, c, A, B)
    got0 = np.zeros_like(C0)
    contract(a, b, c, A, B, got0, 0.0)
    assert np.all(np.abs(got0 - want0) <= RTOL * bound)
    want1, _, _ = orc.ttgt_contract(a, b, c, A, B, C0=C0, beta=1.0)
    got1 = C0.copy()
    contract(a, b, c, A, B, got1, 1.0)
    assert np.all(np.abs(got1 - want1) <= RTOL * (bound + np.abs(C0)))
    # _mlir_ciface_linalg_matmul_viewsxs_viewsxs_viewsxs: strided views, alpha and beta as given
    Am, Bm = gen.dense((37, 29), seed=64), gen.dense((29, 41), seed=65)
    big = gen.dense((37, 50), seed=66)
    Cv = big[:, 3:44]                        # a view with row stride 50
    want = 1.5 * (Am @ Bm) + 0.5 * Cv
    mc = rt.memref2d(Cv)
    mc.aligned = mc.allocated = big.ctypes.data
    mc.offset = 3
    mc.strides[0], mc.strides[1] = 50, 1
    L._mlir_ciface_linalg_matmul_viewsxs_viewsxs_viewsxs(rt.memref2d(Am), rt.memref2d(Bm), mc, 6, 8, 1.5, 0.5)
    assert np.all(np.abs(Cv - want) <= RTOL * (1.5 * (np.abs(Am) @ np.abs(Bm)) + np.abs(want)))
    assert np.array_equal(big[:, :3], gen.dense((37, 50), seed=66)[:, :3])      # nothing outside the view is touched


# ----------------------------------------------------------------- input side and other layouts
def test_mtx_reader_goldens(golden, golden_dir):
    for g in golden["read_csr"]:
        A = rt.CsrMatrix.from_mtx(os.path.join(golden_dir, g["matrix"]), g["mode"])
        p, c, v = A.to_arrays()
        assert p.tolist() == g["pos"] and c.tolist() == g["crd"], g["source"]
        assert orc.format_f64(v) == g["printed_val"], g["source"]
    for g in golden["read_coo"]:
        A = rt.CsrMatrix.from_mtx(os.path.join(golden_dir, g["matrix"]), g["mode"])
        r, c, v = A.to_coo()
        assert r.tolist() == g["a1crd"] and c.tolist() == g["a2crd"], g["source"]
        assert orc.format_f64(v) == g["printed_val"], g["source"]


def _desc(a):
    """(descriptor struct, void pointer to it); the struct must stay alive while the pointer is used"""
    m = rt.memref1d(a)
    return m, C.cast(C.pointer(m), C.c_void_p)


def _memref_idx(n, idt=np.int64):
    a = np.full(max(n, 1), 7, dtype=idt)
    return (a,) + _desc(a)


@pytest.mark.parametrize("idt", [np.int64, np.int32])
@pytest.mark.parametrize("layout", ["CSR", "COO", "DCSR"])
def test_reader_file_id_protocol(golden, golden_dir, monkeypatch, layout, idt):
    """The two reader calls with the reference's argument lists, for the three layouts its matrix tests use and
    both index widths (read_input_2D_f64_i64 / _i32, lib/ExecutionEngine/SparseUtils.cpp:2403-2447)."""
    L = rt.lib()
    # the i64 case goes through the names lowered code calls (read_input_*), the i32 case through the prefixed ones
    read = L.read_input_2D_f64_i64 if idt == np.int64 else L.comet_hip_read_input_2D_f64_i32
    read_sizes = L.read_input_sizes_2D_f64 if idt == np.int64 else L.comet_hip_read_input_sizes_2D_f64
    monkeypatch.setenv("SPARSE_FILE_NAME3", os.path.join(golden_dir, "test_rank2.mtx"))
    fmt = {"CSR": (0, 0, 1, 0), "COO": (2, 0, 3, 0), "DCSR": (1, 0, 1, 0)}[layout]
    for mode in (1, 3):
        (nr, nc), pos, crd, val = _mtx(golden_dir, "test_rank2.mtx", mode)
        sizes = np.zeros(13, dtype=np.int64)
        sizes_m, sizes_p = _desc(sizes)
        read_sizes(3, *fmt, 1, sizes_p, mode)
        want = {"CSR": (None, pos[:0], pos, crd, val), "COO": orc.coo_layout(pos, crd, val),
                "DCSR": orc.dcsr_layout(pos, crd, val)}[layout]
        if layout == "CSR":
            assert sizes[:11].tolist() == [1, 1, 0, 0, nr + 1, len(crd), 0, 0, len(crd), nr, nc]
        elif layout == "COO":
            assert sizes[:11].tolist() == [2, len(crd), 0, 0, 1, len(crd), 0, 0, len(crd), nr, nc]
        else:
            stored = len(want[1])
            assert sizes[:11].tolist() == [2, stored, 0, 0, stored + 1, len(crd), 0, 0, len(crd), nr, nc]
        arrs = [_memref_idx(int(sizes[i]), idt) for i in range(8)]
        aval = np.zeros(max(int(sizes[8]), 1))
        args = []
        for i in (0, 1, 2, 3, 4, 5, 6, 7):
            args += [1, arrs[i][2]]
        aval_m, aval_p = _desc(aval)
        read(3, *fmt, *args, 1, aval_p, mode)
        a1pos, a1crd, a2pos, a2crd = (arrs[i][0] for i in (0, 1, 4, 5))
        assert arrs[2][0][0] == -1 and arrs[3][0][0] == -1 and arrs[6][0][0] == -1 and arrs[7][0][0] == -1
        assert np.array_equal(aval[:len(val)], val)
        if layout == "CSR":
            assert a1pos[0] == nr and a1crd[0] == -1
            assert np.array_equal(a2pos, pos) and np.array_equal(a2crd[:len(crd)], crd)
        elif layout == "COO":
            assert a1pos.tolist() == [0, len(crd)] and a2pos[0] == -1
            assert np.array_equal(a1crd[:len(crd)], want[1]) and np.array_equal(a2crd[:len(crd)], crd)
        else:
            assert a1pos.tolist() == want[0].tolist()
            assert np.array_equal(a1crd, want[1]) and np.array_equal(a2pos, want[2])
            assert np.array_equal(a2crd[:len(crd)], crd)
    # the device-handle form of the same read, and its failure without the variable
    A = rt.CsrMatrix.from_file_id(3, 5)
    (nr, nc), pos, crd, val = _mtx(golden_dir, "test_rank2.mtx", 5)
    p, c, v = A.to_arrays()
    assert np.array_equal(p, pos) and np.array_equal(c, crd) and np.array_equal(v, val)
    monkeypatch.delenv("SPARSE_FILE_NAME4", raising=False)
    assert L.comet_hip_read_input_2D_handle(4, 1) == 0
    assert b"SPARSE_FILE_NAME4" in L.comet_hip_last_error()


def _write_mtx(path, header, size_line, lines):
    with open(path, "w") as f:
        f.write(header + "\n% a comment\n" + size_line + "\n" + "\n".join(lines) + "\n")


@pytest.mark.parametrize("flavour", ["general", "symmetric", "skew-symmetric", "pattern", "array", "duplicates"])
@pytest.mark.parametrize("mode", [1, 2, 3, 4, 5])
def test_mtx_reader_flavours_vs_checker(tmp_path, flavour, mode):
    rng = np.random.default_rng(len(flavour) * 7 + mode)
    n, m = 61, 61
    path = str(tmp_path / "m.mtx")
    if flavour == "array":
        m = 17
        D = rng.uniform(-1, 1, (n, m))
        _write_mtx(path, "%%MatrixMarket matrix array real general", f"{n} {m}", [repr(float(v)) for v in D.T.ravel()])
    else:
        ent = [(i, j) for i in range(n) for j in range(m) if rng.random() < 0.1]
        if flavour in ("symmetric", "skew-symmetric"):
            ent = [(i, j) for i, j in ent if (i >= j if flavour == "symmetric" else i > j)]
        if flavour == "duplicates":
            ent = ent + ent[::3] + ent[::5]
        rng.shuffle(ent)
        vals = rng.uniform(-1, 1, len(ent))
        if flavour == "pattern":
            lines = [f"{i + 1} {j + 1}" for i, j in ent]
        else:
            lines = [f"{i + 1} {j + 1} {float(v)!r}" for (i, j), v in zip(ent, vals)]
        lines.insert(len(lines) // 2, "")          # a blank line in the middle is skipped
        kind = {"pattern": "pattern general", "duplicates": "real general"}.get(flavour, "real " + flavour)
        _write_mtx(path, "%%MatrixMarket matrix coordinate " + kind, f"{n} {m} {len(ent)}", lines)
    (nr, nc), pos, crd, val = orc.read_mtx_csr(path, mode)
    A = rt.CsrMatrix.from_mtx(path, mode)
    assert A.shape == (nr, nc)
    p, c, v = A.to_arrays()
    assert np.array_equal(p, pos) and np.array_equal(c, crd) and np.array_equal(v, val)


def test_coo_dcsr_transpose_conversions():
    rng = np.random.default_rng(21)
    n, m, nnz = 3000, 1777, 200_000
    row = rng.integers(0, n, nnz)
    row[row % 7 == 3] = 5                    # many duplicates of one row, and rows that stay empty
    col = rng.integers(0, m, nnz)
    val = rng.uniform(-1, 1, nnz)
    order = np.lexsort((col, row))           # stable: ties keep input order
    srow, scol, sval = row[order], col[order], val[order]
    pos = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(np.bincount(srow, minlength=n), out=pos[1:])
    A = rt.CsrMatrix.from_coo((n, m), row, col, val)
    p, c, v = A.to_arrays()
    assert np.array_equal(p, pos) and np.array_equal(c, scol) and np.array_equal(v, sval)
    r2, c2, v2 = A.to_coo()
    assert np.array_equal(r2, srow) and np.array_equal(c2, scol) and np.array_equal(v2, sval)
    # read modes filter the ordered tuples
    keep = srow >= scol
    L3 = rt.CsrMatrix.from_coo((n, m), row, col, val, read_mode=3)
    r3, c3, v3 = L3.to_coo()
    assert np.array_equal(r3, srow[keep]) and np.array_equal(c3, scol[keep]) and np.array_equal(v3, sval[keep])
    # DCSR out and back
    a1pos, a1crd, a2pos, a2crd, aval = A.to_dcsr()
    w = orc.dcsr_layout(pos, scol, sval)
    for got, want in zip((a1pos, a1crd, a2pos, a2crd, aval), w):
        assert np.array_equal(got, want)
    Bm = rt.CsrMatrix.from_dcsr((n, m), a1crd, a2pos, a2crd, aval)
    for got, want in zip(Bm.to_arrays(), (pos, scol, sval)):
        assert np.array_equal(got, want)
    # transpose: ordered by (column, row), ties in the order of the source; twice gives the source back
    T = A.transpose()
    assert T.shape == (m, n)
    torder = np.lexsort((srow, scol))
    tp, tc, tv = T.to_arrays()
    tpos = np.zeros(m + 1, dtype=np.int64)
    np.cumsum(np.bincount(scol, minlength=m), out=tpos[1:])
    assert np.array_equal(tp, tpos) and np.array_equal(tc, srow[torder]) and np.array_equal(tv, sval[torder])
    for got, want in zip(T.transpose().to_arrays(), (pos, scol, sval)):
        assert np.array_equal(got, want)
    # empty matrix
    E = rt.CsrMatrix.from_coo((4, 5), [], [], [])
    assert E.to_arrays()[0].tolist() == [0, 0, 0, 0, 0] and E.transpose().shape == (5, 4)
    assert E.to_dcsr()[0].tolist() == [0, 0]


def test_spmv_spmm_other_layouts_golden(golden, golden_dir):
    """mult_spmv/spmm_{COO,DCSR}xDense: the file read into the layout's arrays, handed back, same kernels."""
    path = os.path.join(golden_dir, "test_rank2.mtx")
    A = rt.CsrMatrix.from_mtx(path)
    nr, nc = A.shape
    r, c, v = A.to_coo()
    a1pos, a1crd, a2pos, a2crd, aval = A.to_dcsr()
    for M in (rt.CsrMatrix.from_coo((nr, nc), r, c, v), rt.CsrMatrix.from_dcsr((nr, nc), a1crd, a2pos, a2crd, aval)):
        y = rt.spmv(M, rt.DeviceArray.from_numpy(np.full(nc, 1.7)), rt.DeviceArray(nr, zero=True))
        assert orc.format_f64(y.to_numpy()) == golden["spmv_other_layouts"]["printed"]
        Cm = rt.spmm(M, rt.DeviceArray.from_numpy(np.full((nc, 4), 1.7)), rt.DeviceArray((nr, 4), zero=True))
        assert orc.format_f64(Cm.to_numpy()) == golden["spmm_other_layouts"]["printed"]


def test_reader_rejects_bad_input(tmp_path):
    L = rt.lib()
    assert L.comet_hip_mtx_read_csr(str(tmp_path / "missing.mtx").encode(), 1) == 0
    assert b"cannot open" in L.comet_hip_last_error()
    bad = tmp_path / "bad.mtx"
    bad.write_text("%%MatrixMarket matrix coordinate real general\n3 3 1\n4 1 2.0\n")
    assert L.comet_hip_mtx_read_csr(str(bad).encode(), 1) == 0 and b"outside" in L.comet_hip_last_error()
    assert L.comet_hip_mtx_read_csr(str(bad).encode(), 9) == 0 and b"read mode" in L.comet_hip_last_error()
    row = np.array([0, 5], dtype=np.int64)
    h = L.comet_hip_csr_from_coo_i64(3, 3, 2, row.ctypes.data, row.ctypes.data, np.zeros(2).ctypes.data, 1)
    assert h == 0 and b"outside" in L.comet_hip_last_error()
    # tuples that are already on the device are checked there
    drow = rt.DeviceArray.from_numpy(np.array([0, 2, 1], dtype=np.int32))
    dcol = rt.DeviceArray.from_numpy(np.array([1, 3, 0], dtype=np.int32))
    dval = rt.DeviceArray.from_numpy(np.ones(3))
    h = L.comet_hip_csr_from_coo_device(3, 3, 3, drow.ptr, dcol.ptr, dval.ptr, 1)
    assert h == 0 and b"outside" in L.comet_hip_last_error()
    dcol = rt.DeviceArray.from_numpy(np.array([1, 2, 0], dtype=np.int32))
    M = rt.CsrMatrix.from_coo_device((3, 3), drow, dcol, dval)
    assert M.to_arrays()[0].tolist() == [0, 1, 2, 3] and M.to_arrays()[1].tolist() == [1, 0, 2]


# ----------------------------------------------------------------- SpMM: long rows through the column sweep
def _kernels_of(fn):
    rt.profile_reset()
    rt.profile_enable(True)
    fn()
    rt.sync()
    rep = rt.profile_report()
    rt.profile_enable(False)
    return rep


def _sweep_check(pos, crd, val, B, C0=None, ld_pad=0):
    """SpMM on a matrix whose long rows take the sweep: every row within the summation-order bound, and the
    rows that lie inside one 256-nonzero chunk of the matrix without its long rows bit-exact."""
    n, m = len(pos) - 1, B.shape[0]
    K = B.shape[1]
    A = rt.CsrMatrix.from_arrays((n, m), pos, crd, val)
    Bp = np.zeros((m, K + ld_pad)); Bp[:, :K] = B
    Cp = np.full((n, K + ld_pad), 123.0)
    if C0 is not None:
        Cp[:, :K] = C0
    dB, dC = rt.DeviceArray.from_numpy(Bp), rt.DeviceArray.from_numpy(Cp)
    L = rt.lib()
    run = lambda: rt._check(L.comet_hip_spmm_csr_f64(A.handle, K, dB.ptr, K + ld_pad, dC.ptr, K + ld_pad,
                                                     int(C0 is not None)), "spmm")
    rep = _kernels_of(run)
    swept = K % 2 == 0 and ld_pad % 2 == 0       # the sweep loads pairs of columns: even K and leading dimensions
    assert ("spmm_heavy_sweep" in rep) == swept, sorted(rep)
    out = dC.to_numpy()
    assert np.all(out[:, K:] == 123.0)             # the padding of C is not touched
    got = out[:, :K]
    want = orc.spmm(pos, crd, val, B, C0)
    bound = orc.spmm(pos, crd, np.abs(val), np.abs(B), None if C0 is None else np.abs(C0))
    assert np.all(np.abs(got - want) <= RTOL * bound)
    long_rows, _ = _swept_rows(pos, K if swept else 0)
    inside = _bit_exact_rows(pos, K if swept else 0)
    assert inside.sum() > 0 and np.array_equal(got[inside], want[inside])
    # a second call on the same handle reuses the plan and gives the same bits
    if C0 is None:
        run(); assert np.array_equal(dC.to_numpy()[:, :K], got)
    return len(long_rows)


@pytest.mark.parametrize("medium", [False, True])
@pytest.mark.parametrize("K,acc,pad", [(64, False, 0), (64, True, 0), (20, False, 4), (100, True, 6), (64, False, 3),
                                        (33, True, 0)])
def test_spmm_long_rows_sweep(K, acc, pad, medium, monkeypatch):
    if medium:      # rows of 32..127 nonzeros ride on the sweep too, their sums in LDS
        monkeypatch.setenv("COMET_HIP_SPMM_MEDIUM", "1")
    pos, crd, val = gen.zipf_csr(n=40_000, mean=16.0, cap=4096, seed=7)
    assert len(crd) >= 1 << 19
    B = gen.dense((40_000, K), seed=8)
    C0 = gen.dense((40_000, K), seed=9) if acc else None
    nlong = _sweep_check(pos, crd, val, B, C0, pad)
    assert nlong > 100 if (K % 2 == 0 and pad % 2 == 0) else nlong == 0


def test_spmm_plan_waits_for_the_second_product(monkeypatch):
    # The plan of a matrix costs some forty products, so a matrix multiplied once (what a .ta program does) goes
    # through the chunk kernel whole; the plan is made when the same handle is multiplied again, and kept.
    monkeypatch.delenv("COMET_HIP_PLAN_AT_ONCE")
    pos, crd, val = gen.zipf_csr(n=40_000, mean=16.0, cap=4096, seed=7)
    assert len(crd) >= 1 << 19
    B = gen.dense((40_000, 64), seed=8)
    A = rt.CsrMatrix.from_arrays((40_000, 40_000), pos, crd, val)
    dB, dC = rt.DeviceArray.from_numpy(B), rt.DeviceArray((40_000, 64))
    want = orc.spmm(pos, crd, val, B)
    bound = orc.spmm(pos, crd, np.abs(val), np.abs(B))
    seen = []
    for _ in range(3):
        rep = _kernels_of(lambda: rt.spmm(A, dB, dC, accumulate=False))
        seen.append("spmm_heavy_sweep" in rep)
        assert np.all(np.abs(dC.to_numpy() - want) <= RTOL * bound)
    assert seen == [False, True, True]


def test_spmv_plan_waits_for_the_second_product(monkeypatch):
    # the same rule for the column-blocked copy an SpMV keeps of a matrix whose x outgrows an L2; with or
    # without it the additions happen in the checker's order
    monkeypatch.delenv("COMET_HIP_PLAN_AT_ONCE")
    n = 600_000
    pos, crd, val = gen.poisson_csr(n=n, mean=4.0, seed=5)
    x = gen.dense(n, seed=15)
    A = rt.CsrMatrix.from_arrays((n, n), pos, crd, val)
    dx, dy = rt.DeviceArray.from_numpy(x), rt.DeviceArray(n)
    want = orc.spmv(pos, crd, val, x)
    seen = []
    for _ in range(3):
        rep = _kernels_of(lambda: rt.spmv(A, dx, dy, accumulate=False))
        seen.append("spmv_csr_blocks" in rep)
        assert np.array_equal(dy.to_numpy(), want)
    assert seen == [False, True, True]


@pytest.mark.parametrize("groups,held", [(None, 2880), (32, 3840), (16, 1920)])
def test_spmm_more_long_rows_than_the_sweep_holds(groups, held, monkeypatch):
    """5000 rows of 300 nonzeros: the longest the sweep has room for (ties: lowest row ids) sweep, the others
    stay on the chunk kernel, which here holds enough of the matrix to run beside the sweep on CUs that it
    leaves free (24 workgroups per XCD; 32 and 16 forced); an empty row and a short row sit between them."""
    if groups is not None:
        monkeypatch.setenv("COMET_HIP_SPMM_GROUPS", str(groups))
        monkeypatch.setenv("COMET_HIP_SPMM_MEDIUM", "1")       # and the rows without a register keep their sums in LDS
    rng = np.random.default_rng(31)
    n, m = 5002, 3000
    lens = np.full(n, 300); lens[17] = 0; lens[4000] = 3
    pos = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    crd = np.concatenate([np.sort(rng.choice(m, l, replace=False)) for l in lens]).astype(np.int64)
    val = rng.uniform(-1, 1, len(crd))
    assert _sweep_check(pos, crd, val, gen.dense((m, 64), seed=2)) == held


@pytest.mark.parametrize("acc", [False, True])
def test_spmm_sweep_with_only_single_and_empty_rows_besides(acc):
    """2100 rows of 260 nonzeros, and around them rows of one nonzero and empty rows only: nothing is left
    for the chunk kernel; the single products are stored (or added to C) by the sweep, bit-exact."""
    rng = np.random.default_rng(41)
    n, m, K = 9000, 5000, 32
    lens = np.where(np.arange(n) % 3 == 0, 1, 0); lens[rng.choice(n, 2100, replace=False)] = 260
    pos = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    assert pos[-1] >= 1 << 19
    crd = np.concatenate([np.sort(rng.choice(m, l, replace=False)) for l in lens if l]).astype(np.int64)
    val = rng.uniform(-1, 1, len(crd))
    C0 = gen.dense((n, K), seed=5) if acc else None
    assert _sweep_check(pos, crd, val, gen.dense((m, K), seed=4), C0) == 2100
    A = rt.CsrMatrix.from_arrays((n, m), pos, crd, val)
    rep = _kernels_of(lambda: rt.spmm(A, rt.DeviceArray.from_numpy(gen.dense((m, K), seed=4))))
    assert "spmm_csr_nnzsplit" not in rep and "spmm_heavy_sweep" in rep, sorted(rep)


# ----------------------------------------------------------------- dense operand on the left, CSR .* Dense
def test_vecmat_densemat_eltwise_dense_golden(golden, golden_dir):
    A = rt.CsrMatrix.from_mtx(os.path.join(golden_dir, "test_rank2.mtx"))
    nr, nc = A.shape
    g = golden["vecmat_csr"]
    y = rt.vecmat(rt.DeviceArray.from_numpy(np.full(nr, g["x_fill"])), A, rt.DeviceArray(nc, zero=True))
    assert orc.format_f64(y.to_numpy()) == g["printed"]
    g = golden["densemat_csr"]
    Cm = rt.densemat(rt.DeviceArray.from_numpy(np.full((g["M"], nr), g["a_fill"])), A,
                     rt.DeviceArray((g["M"], nc), zero=True))
    assert orc.format_f64(Cm.to_numpy()) == g["printed"]
    g = golden["eltwise_mult_csr_dense"]
    D = rt.DeviceArray.from_numpy(np.full((nr, nc), g["d_fill"]))
    p, c, v = rt.eltwise_mult_dense(A, D).to_arrays()
    assert p.tolist() == g["pos"] and c.tolist() == g["crd"] and orc.format_f64(v) == g["printed_val"]
    out = rt.eltwise_mult_dense(A, D, rt.DeviceArray((nr, nc), zero=True))
    assert orc.format_f64(out.to_numpy()) == g["printed_dense"]


@pytest.mark.parametrize("n,m,M,density,seed", [(300, 200, 7, 0.05, 0), (1000, 1500, 64, 0.02, 1), (50, 3000, 33, 0.2, 2)])
def test_vecmat_densemat_vs_checker(n, m, M, density, seed):
    rng = np.random.default_rng(seed)
    pos, crd, val = _rand_csr(rng, n, m, density)
    B = rt.CsrMatrix.from_arrays((n, m), pos, crd, val)
    x, y0 = rng.uniform(-1, 1, n), rng.uniform(-1, 1, m)
    y = rt.vecmat(rt.DeviceArray.from_numpy(x), B, rt.DeviceArray.from_numpy(y0)).to_numpy()
    assert np.array_equal(y, orc.vecmat(x, pos, crd, val, m, y0))             # same order of additions: bit-exact
    assert np.array_equal(rt.vecmat(rt.DeviceArray.from_numpy(x), B).to_numpy(), orc.vecmat(x, pos, crd, val, m))
    A, C0 = rng.uniform(-1, 1, (M, n)), rng.uniform(-1, 1, (M, m))
    want = orc.densemat(A, pos, crd, val, m, C0)
    got = rt.densemat(rt.DeviceArray.from_numpy(A), B, rt.DeviceArray.from_numpy(C0)).to_numpy()
    bound = orc.densemat(np.abs(A), pos, crd, np.abs(val), m, np.abs(C0))
    assert np.all(np.abs(got - want) <= RTOL * bound)
    tpos = np.concatenate([[0], np.cumsum(np.bincount(crd, minlength=m))])
    inside = tpos[:-1] // 256 == (np.maximum(tpos[1:], tpos[:-1] + 1) - 1) // 256   # columns summed by one wavefront
    assert np.array_equal(got[:, inside], want[:, inside])
    got0 = rt.densemat(rt.DeviceArray.from_numpy(A), B).to_numpy()
    assert np.all(np.abs(got0 - orc.densemat(A, pos, crd, val, m)) <= RTOL * bound)
    # CSR .* Dense
    D = rng.uniform(-1, 1, (n, m))
    dD = rt.DeviceArray.from_numpy(D)
    p, c, v = rt.eltwise_mult_dense(B, dD).to_arrays()
    assert np.array_equal(p, pos) and np.array_equal(c, crd) and np.array_equal(v, orc.eltwise_mult_dense(pos, crd, val, D))
    keep = rng.uniform(-1, 1, (n, m))
    out = rt.eltwise_mult_dense(B, dD, rt.DeviceArray.from_numpy(keep)).to_numpy()
    keep[np.repeat(np.arange(n), np.diff(pos)), crd] = v
    assert np.array_equal(out, keep)


def test_ttgt_refuses_a_plan_that_is_not_one():
    """A plan handed in by the caller is checked before its ranks and permutations index anything."""
    import copy
    A = rt.DeviceArray.from_numpy(gen.dense((4, 5, 6), seed=1))
    B = rt.DeviceArray.from_numpy(gen.dense((6, 5, 3), seed=2))
    plan = rt.ttgt_plan("abc", "cbd", "ad", {"a": 4, "b": 5, "c": 6, "d": 3}, 1)
    good, _ = rt.ttgt_contract("abc", "cbd", "ad", A, B, plan=plan)
    assert good.to_numpy().shape == (4, 3)
    for field, value in (("rankC", 9), ("rankA", 0), ("permA", (0, 0, 2)), ("permB", (0, 1, 7))):
        bad = copy.copy(plan)
        if field.startswith("perm"):
            setattr(bad, "trans" + field[-1], 1)
            arr = getattr(bad, field)
            for i, v in enumerate(value):
                arr[i] = v
        else:
            setattr(bad, field, value)
        with pytest.raises(rt.CometHipError):
            rt.ttgt_contract("abc", "cbd", "ad", A, B, plan=bad)


def test_wrapped_device_arrays_are_checked():
    """comet_hip_csr_wrap and comet_hip_csr_invalidate look at caller-filled device arrays once and refuse what
    would send a kernel outside its buffers; nothing here launches a product on bad data."""
    L = rt.lib()
    good = (np.array([0, 2, 2, 5], dtype=np.int64), np.array([0, 3, 1, 1, 2], dtype=np.int32), np.ones(5))

    def wrap(pos, crd, nnz=5, ncols=4):
        dpos, dcrd, dval = rt.DeviceArray.from_numpy(pos), rt.DeviceArray.from_numpy(crd), rt.DeviceArray.from_numpy(good[2])
        return L.comet_hip_csr_wrap(3, ncols, nnz, dpos.ptr, dcrd.ptr, dval.ptr), (dpos, dcrd, dval)

    h, keep = wrap(good[0], good[1])
    assert h != 0
    for pos, crd, kw in [
        (good[0], np.array([0, 4, 1, 1, 2], dtype=np.int32), {}),                    # column == ncols
        (good[0], np.array([0, -1, 1, 1, 2], dtype=np.int32), {}),                   # negative column
        (good[0], np.array([3, 0, 1, 1, 2], dtype=np.int32), {}),                    # columns go down inside row 0
        (np.array([0, 3, 2, 5], dtype=np.int64), good[1], {}),                       # pos decreases
        (np.array([1, 2, 2, 5], dtype=np.int64), good[1], {}),                       # pos[0] != 0
        (good[0], good[1], {"nnz": 4}),                                              # pos[nrows] != nnz
        (np.array([0, 2, 9, 5], dtype=np.int64), good[1], {}),                       # a row pointer past nnz
    ]:
        bad, _keep = wrap(pos, crd, **kw)
        assert bad == 0
        assert b"not a valid matrix" in L.comet_hip_last_error()
    # arrays rewritten in place: invalidate looks again
    keep[1].free()
    assert L.comet_hip_csr_destroy(h) == 0
    dpos, dcrd, dval = (rt.DeviceArray.from_numpy(a) for a in good)
    h = L.comet_hip_csr_wrap(3, 4, 5, dpos.ptr, dcrd.ptr, dval.ptr)
    assert h != 0
    worse = np.array([0, 3, 1, 7, 2], dtype=np.int32)
    assert L.comet_hip_memcpy(dcrd.ptr, worse.ctypes.data, worse.nbytes, 0) == 0
    assert L.comet_hip_csr_invalidate(h) == 1           # COMET_HIP_ERR_ARG
    # the handle now refuses every product (nothing is launched on the arrays the check turned down) ...
    dx, dy = rt.DeviceArray.from_numpy(np.ones(4)), rt.DeviceArray(3)
    assert L.comet_hip_spmv_csr_f64(h, dx.ptr, dy.ptr, 0) == 3          # COMET_HIP_ERR_HANDLE
    assert b"failed the check" in L.comet_hip_last_error()
    assert L.comet_hip_spmm_csr_f64(h, 1, dx.ptr, 1, dy.ptr, 1, 0) == 3
    assert L.comet_hip_spgemm_csr(h, h, 0) == 0 and b"failed the check" in L.comet_hip_last_error()
    # ... until the arrays are put right and looked at again
    assert L.comet_hip_memcpy(dcrd.ptr, good[1].ctypes.data, good[1].nbytes, 0) == 0
    assert L.comet_hip_csr_invalidate(h) == 0
    assert L.comet_hip_spmv_csr_f64(h, dx.ptr, dy.ptr, 0) == 0
    assert np.array_equal(dy.to_numpy(), np.array([2.0, 0.0, 3.0]))
    assert L.comet_hip_csr_destroy(h) == 0


def test_wrapped_arrays_changed_in_place_need_invalidate():
    """A handle over caller-owned device arrays caches re-ordered copies; after the caller rewrites the values
    comet_hip_csr_invalidate makes every kernel see them."""
    pos, crd, val = gen.zipf_csr(n=40_000, mean=16.0, cap=4096, seed=11)      # large enough for every plan
    n, nnz = 40_000, len(crd)
    dpos = rt.DeviceArray.from_numpy(pos.astype(np.int64))
    dcrd = rt.DeviceArray.from_numpy(crd.astype(np.int32))
    dval = rt.DeviceArray.from_numpy(val)
    L = rt.lib()
    A = rt.CsrMatrix(rt._handle(L.comet_hip_csr_wrap(n, n, nnz, dpos.ptr, dcrd.ptr, dval.ptr), "wrap"))
    B = gen.dense((n, 32), seed=12)
    x = gen.dense(n, seed=13)
    dB, dx = rt.DeviceArray.from_numpy(B), rt.DeviceArray.from_numpy(x)
    first = rt.spmm(A, dB).to_numpy()
    y1 = rt.spmv(A, dx).to_numpy()
    z1 = rt.vecmat(dx, A).to_numpy()
    val2 = -2.0 * val
    rt._check(L.comet_hip_memcpy(dval.ptr, val2.ctypes.data, val2.nbytes, 0), "upload")
    A.invalidate()
    assert np.array_equal(rt.spmm(A, dB).to_numpy(), -2.0 * first)       # scaling by -2 is exact
    assert np.array_equal(rt.spmv(A, dx).to_numpy(), -2.0 * y1)
    assert np.array_equal(rt.vecmat(dx, A).to_numpy(), -2.0 * z1)


def test_eltwise_monoid_golden_and_checker(golden, golden_dir):
    for g in golden["eltwise_monoid"]["dense"]:
        a, b = np.full(g["shape"], g["a"]), np.full(g["shape"], g["b"])
        out = rt.eltwise_dense(rt.DeviceArray.from_numpy(a), rt.DeviceArray.from_numpy(b), op=g["op"])
        assert orc.format_f64(out.to_numpy()) == g["printed"], g["source"]
    for g in golden["eltwise_monoid"]["coo_dense"]:
        A = rt.CsrMatrix.from_mtx(os.path.join(golden_dir, g["matrix"]))
        D = rt.DeviceArray.from_numpy(np.full(A.shape, g["d_fill"]))
        r, c, v = rt.eltwise_csr_dense(A, D, op=g["op"]).to_coo()
        assert r.tolist() == g["a1crd"] and c.tolist() == g["a2crd"] and orc.format_f64(v) == g["printed_val"]
    rng = np.random.default_rng(5)
    pos, crd, val = _rand_csr(rng, 400, 300, 0.05)
    A = rt.CsrMatrix.from_arrays((400, 300), pos, crd, val)
    D = rng.uniform(0.5, 2.0, (400, 300))
    x, y = rng.uniform(-1, 1, 100_003), rng.uniform(0.5, 2, 100_003)
    for op in rt.MULT_OPS:
        if op in ("*", "+", "-", "/"):
            continue
        got = rt.eltwise_csr_dense(A, rt.DeviceArray.from_numpy(D), op=op).to_arrays()[2]
        assert np.array_equal(got, orc.eltwise_csr_dense(pos, crd, val, D, op)), op
        got = rt.eltwise_dense(rt.DeviceArray.from_numpy(x), rt.DeviceArray.from_numpy(y), op=op).to_numpy()
        assert np.array_equal(got, orc.eltwise_dense(x, y, op)), op


# ----------------------------------------------------------------- SDDMM
def test_sddmm_golden(golden, golden_dir):
    g = golden["kernels_and_compound"]["sddmm"]
    B = rt.CsrMatrix.from_mtx(os.path.join(golden_dir, g["matrix"]))
    nr, nc = B.shape
    A = rt.sddmm(B, rt.DeviceArray.from_numpy(np.full((nr, g["K"]), g["c_fill"])),
                 rt.DeviceArray.from_numpy(np.full((g["K"], nc), g["d_fill"])))
    p, c, v = A.to_arrays()
    printed = orc.format_i64([nr]) + orc.format_i64([-1]) + orc.format_i64(p) + orc.format_i64(c) + orc.format_f64(v)
    assert printed == g["printed"]


@pytest.mark.parametrize("n,m,K,density,seed", [(300, 200, 7, 0.05, 0), (2000, 1500, 64, 0.02, 1), (50, 3000, 33, 0.2, 2),
                                                (100, 100, 0, 0.1, 3), (513, 257, 1, 0.3, 4)])
def test_sddmm_vs_checker(n, m, K, density, seed):
    """Same additions in the same order as the checker: bit-exact; rows without entries in between."""
    rng = np.random.default_rng(seed)
    pos, crd, val = _rand_csr(rng, n, m, density)
    B = rt.CsrMatrix.from_arrays((n, m), pos, crd, val)
    Cm, D = rng.uniform(-1, 1, (n, K)), rng.uniform(-1, 1, (K, m))
    A = rt.sddmm(B, rt.DeviceArray.from_numpy(Cm), rt.DeviceArray.from_numpy(D))
    p, c, v = A.to_arrays()
    assert np.array_equal(p, pos) and np.array_equal(c, crd)
    assert np.array_equal(v, orc.sddmm(pos, crd, val, Cm, D))


def test_sddmm_empty_and_errors():
    B = rt.CsrMatrix.from_arrays((4, 5), np.zeros(5, dtype=np.int64), np.zeros(0, dtype=np.int64), np.zeros(0))
    A = rt.sddmm(B, rt.DeviceArray((4, 3), zero=True), rt.DeviceArray((3, 5), zero=True))
    assert A.to_arrays()[0].tolist() == [0] * 5 and A.nnz == 0
    with pytest.raises(ValueError):
        rt.sddmm(B, rt.DeviceArray((4, 3), zero=True), rt.DeviceArray((2, 5), zero=True))
    L = rt.lib()
    assert L.comet_hip_sddmm_csr_f64(B.handle, 3, 0, 2, 0, 5) == 0          # ldc < K
    assert b"sddmm" in L.comet_hip_last_error()


def test_sddmm_values_into_a_caller_array():
    rng = np.random.default_rng(9)
    pos, crd, val = _rand_csr(rng, 700, 400, 0.03)
    B = rt.CsrMatrix.from_arrays((700, 400), pos, crd, val)
    Cm, D = rng.uniform(-1, 1, (700, 20)), rng.uniform(-1, 1, (20, 400))
    out = rt.DeviceArray.from_numpy(np.full(len(val) + 3, 7.0))
    rt.sddmm(B, rt.DeviceArray.from_numpy(Cm), rt.DeviceArray.from_numpy(D), out_values=out)
    got = out.to_numpy()
    assert np.array_equal(got[:len(val)], orc.sddmm(pos, crd, val, Cm, D)) and np.all(got[len(val):] == 7.0)
    assert rt.lib().comet_hip_sddmm_csr_values_f64(B.handle, 20, 0, 20, 0, 400, out.ptr) != 0      # null operands
