"""The seeded input generators: determinism and the properties the benchmark shapes state."""
import numpy as np

from comet_amd import gen


def _check_csr(pos, crd, val, n):
    assert pos[0] == 0 and pos[-1] == len(crd) == len(val) and np.all(np.diff(pos) >= 0)
    rows = np.repeat(np.arange(len(pos) - 1), np.diff(pos))
    key = rows * n + crd
    assert np.all(np.diff(key) > 0)          # sorted by (row, col), no duplicates
    assert crd.min() >= 0 and crd.max() < n


def test_poisson_csr_small():
    pos, crd, val = gen.poisson_csr(n=5000, mean=10.0, seed=1)
    _check_csr(pos, crd, val, 5000)
    assert abs(np.diff(pos).mean() - 10.0) < 0.3
    assert val.min() >= -1 and val.max() <= 1
    pos2, crd2, val2 = gen.poisson_csr(n=5000, mean=10.0, seed=1)
    assert np.array_equal(pos, pos2) and np.array_equal(crd, crd2) and np.array_equal(val, val2)


def test_zipf_csr_small():
    pos, crd, val = gen.zipf_csr(n=20000, mean=16.0, cap=512, seed=2)
    _check_csr(pos, crd, val, 20000)
    lens = np.diff(pos)
    assert lens.min() >= 1 and lens.max() <= 512
    assert 13.0 < lens.mean() <= 16.5      # duplicates may shrink rows slightly
    assert np.median(lens) == 1            # power law: most rows are short


def test_rmat_small():
    pos, crd, val = gen.rmat_symmetric_csr(scale=10, edge_factor=8, seed=3)
    n = 1 << 10
    _check_csr(pos, crd, val, n)
    rows = np.repeat(np.arange(n), np.diff(pos))
    assert not np.any(rows == crd)                                  # no self loops
    fwd = set(zip(rows.tolist(), crd.tolist()))
    assert all((c, r) in fwd for r, c in fwd)                       # symmetric pattern
    assert val.min() > 0 and val.max() <= 1
    assert np.diff(pos)[:16].mean() > 4 * np.diff(pos).mean()       # low ids are the hubs
    lpos, lcrd, lval = gen.strictly_lower(pos, crd, val)
    lrows = np.repeat(np.arange(n), np.diff(lpos))
    assert np.all(lcrd < lrows) and len(lcrd) * 2 == len(crd)
