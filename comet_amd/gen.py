"""Seeded synthetic inputs for the five benchmark shapes.

Everything is generated once on the host with numpy's PCG64 and handed to both
the HIP path and the CPU checker, so the two sides always see identical bytes.
CSR arrays come back as (pos int64[n+1], crd int64[nnz], val float64[nnz]) with
columns sorted ascending and unique inside each row, which is the layout the
reference's reader produces (lib/ExecutionEngine/SparseUtils.cpp:404-533).
"""
import numpy as np


def _rows_from_lengths(rng, lens, ncols):
    """Draw lens[i] uniform columns per row, sort, drop duplicates (a row may shrink)."""
    lens = np.asarray(lens, dtype=np.int64)
    n = len(lens)
    total = int(lens.sum())
    rows = np.repeat(np.arange(n, dtype=np.int64), lens)
    cols = rng.integers(0, ncols, size=total, dtype=np.int64)
    key = rows * np.int64(ncols) + cols
    key = np.unique(key)  # sorts by (row, col) and removes duplicates
    rows = key // ncols
    crd = key - rows * ncols
    pos = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(np.bincount(rows, minlength=n), out=pos[1:])
    return pos, crd


def poisson_csr(n=1_000_000, mean=10.0, seed=1):
    """SpMV shape: n x n, Poisson(mean) row lengths, uniform columns, values U[-1,1]."""
    rng = np.random.Generator(np.random.PCG64(seed))
    lens = rng.poisson(mean, n)
    pos, crd = _rows_from_lengths(rng, lens, n)
    val = rng.uniform(-1.0, 1.0, len(crd))
    return pos, crd, val


def zipf_lengths(rng, n, s=1.5, mean=16.0, cap=4096):
    """Power-law row lengths: z ~ Zipf(s) untruncated, len = clip(ceil(alpha*z), 1, cap)
    with alpha found by bisection so that the mean is `mean`."""
    z = rng.zipf(s, n).astype(np.float64)

    def lens_for(alpha):
        return np.clip(np.ceil(alpha * z), 1, cap)

    lo, hi = 0.0, 64.0
    for _ in range(80):
        mid = 0.5 * (lo + hi)
        if lens_for(mid).mean() < mean:
            lo = mid
        else:
            hi = mid
    return lens_for(hi).astype(np.int64), hi


def zipf_csr(n=500_000, s=1.5, mean=16.0, cap=4096, seed=2):
    """SpMM shape: n x n, Zipf(s) row lengths rescaled to `mean` and capped, uniform
    columns, values U[-1,1]."""
    rng = np.random.Generator(np.random.PCG64(seed))
    lens, alpha = zipf_lengths(rng, n, s, mean, cap)
    pos, crd = _rows_from_lengths(rng, lens, n)
    val = rng.uniform(-1.0, 1.0, len(crd))
    return pos, crd, val


def dense(shape, seed, lo=-1.0, hi=1.0):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.uniform(lo, hi, shape)


def rmat_edges(scale=20, edge_factor=16, abcd=(0.57, 0.19, 0.19, 0.05), seed=20, chunk=1 << 22):
    """R-MAT edge list: per edge `scale` levels, most significant bit first, one uniform
    draw per level choosing a quadrant; no noise, no vertex relabelling."""
    rng = np.random.Generator(np.random.PCG64(seed))
    a, b, c, _ = abcd
    ne = edge_factor << scale
    src = np.empty(ne, dtype=np.int64)
    dst = np.empty(ne, dtype=np.int64)
    for s0 in range(0, ne, chunk):
        m = min(chunk, ne - s0)
        u = np.zeros(m, dtype=np.int64)
        v = np.zeros(m, dtype=np.int64)
        for _ in range(scale):
            r = rng.random(m)
            ubit = (r >= a + b)                       # quadrants (1,0) and (1,1)
            vbit = ((r >= a) & (r < a + b)) | (r >= a + b + c)   # (0,1) and (1,1)
            u = (u << 1) | ubit
            v = (v << 1) | vbit
        src[s0:s0 + m] = u
        dst[s0:s0 + m] = v
    return src, dst


def rmat_symmetric_csr(scale=20, edge_factor=16, seed=20, values="uniform"):
    """Adjacency matrix of the symmetrised R-MAT graph: self-loops dropped, reverse
    edges added, duplicates removed, CSR sorted.  values: "uniform" -> U(0,1] drawn per
    stored entry, "ones" -> 1.0."""
    n = 1 << scale
    src, dst = rmat_edges(scale, edge_factor, seed=seed)
    keep = src != dst
    src, dst = src[keep], dst[keep]
    key = np.concatenate([src * np.int64(n) + dst, dst * np.int64(n) + src])
    del src, dst
    key = np.unique(key)
    rows = key // n
    crd = key - rows * n
    del key
    pos = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(np.bincount(rows, minlength=n), out=pos[1:])
    del rows
    if values == "ones":
        val = np.ones(len(crd))
    else:
        rng = np.random.Generator(np.random.PCG64(seed + 1))
        val = 1.0 - rng.random(len(crd))             # (0, 1]
    return pos, crd, val


def strictly_lower(pos, crd, val):
    """Strictly lower-triangular part (the LOWER_TRI_STRICT read mode,
    lib/ExecutionEngine/SparseUtils.cpp:40-47,461-475)."""
    n = len(pos) - 1
    rows = np.repeat(np.arange(n, dtype=np.int64), np.diff(pos))
    keep = crd < rows
    lpos = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(np.bincount(rows[keep], minlength=n), out=lpos[1:])
    return lpos, crd[keep], val[keep]
