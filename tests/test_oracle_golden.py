"""Pins the CPU checker (oracle/) against evidence that does not come from the
checker itself: the expected outputs held by the reference's integration tests,
scipy/numpy library routines, dense brute force and algebraic invariants."""
import itertools
import os

import numpy as np
import pytest
import scipy.sparse as sp

from oracle import oracle as orc


def _mtx(golden_dir, name, mode=1):
    return orc.read_mtx_csr(os.path.join(golden_dir, name), mode)


def _rand_csr(rng, n, m, density, signed=True):
    A = sp.random(n, m, density=density, random_state=rng, format="csr",
                  data_rvs=lambda k: rng.uniform(-1, 1, k) if signed else rng.uniform(0.1, 1, k))
    A.sort_indices()
    return A


# ----------------------------------------------------------------- reader / print format
def test_reader_goldens(golden, golden_dir):
    for g in golden["read_csr"]:
        (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"], g["mode"])
        assert nr == 5
        assert pos.tolist() == g["pos"], g["source"]
        assert crd.tolist() == g["crd"], g["source"]
        assert orc.format_f64(val) == g["printed_val"], g["source"]


def test_format():
    assert orc.format_f64([4.08, 7.65, 5.1, 13.77, 17.34]) == "data = \n4.08,7.65,5.1,13.77,17.34,\n"
    assert orc.format_i64([5]) == "data = \n5,\n"
    assert orc.format_i64([-1]) == "data = \n-1,\n"
    assert orc.format_f64([]) == ""
    assert orc.format_f64([128123.2, 32030.72]) == "data = \n128123,32030.7,\n"


# ----------------------------------------------------------------- SpMV / SpMM
def test_spmv_golden(golden, golden_dir):
    g = golden["spmv_csr"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"])
    y = orc.spmv(pos, crd, val, np.full(nc, g["x_fill"]), np.full(nr, g["y_fill"]))
    assert orc.format_f64(y) == g["printed"]


def test_spmm_golden(golden, golden_dir):
    g = golden["spmm_csr"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"])
    Cm = orc.spmm(pos, crd, val, np.full((nc, g["K"]), g["B_fill"]), np.full((nr, g["K"]), g["C_fill"]))
    assert orc.format_f64(Cm) == g["printed"]


@pytest.mark.parametrize("seed", [0, 1])
def test_spmv_spmm_vs_scipy_and_bruteforce(seed):
    rng = np.random.default_rng(seed)
    A = _rand_csr(rng, 57, 43, 0.15)
    x = rng.uniform(-1, 1, 43)
    B = rng.uniform(-1, 1, (43, 7))
    y0 = rng.uniform(-1, 1, 57)
    y = orc.spmv(A.indptr, A.indices, A.data, x, y0)
    np.testing.assert_allclose(y, y0 + A @ x, rtol=0, atol=1e-13)
    # sequential order, unfused: bit-exact against a python loop
    ref = y0.copy()
    for i in range(57):
        for p in range(A.indptr[i], A.indptr[i + 1]):
            ref[i] = ref[i] + A.data[p] * x[A.indices[p]]
    assert np.array_equal(y, ref)
    Cm = orc.spmm(A.indptr, A.indices, A.data, B)
    np.testing.assert_allclose(Cm, A.toarray() @ B, rtol=0, atol=1e-13)
    ref = np.zeros((57, 7))
    for i in range(57):
        for p in range(A.indptr[i], A.indptr[i + 1]):
            ref[i] = ref[i] + A.data[p] * B[A.indices[p]]
    assert np.array_equal(Cm, ref)


def test_spmv_empty_rows_and_accumulate():
    pos = np.array([0, 0, 2, 2], dtype=np.int64)
    crd = np.array([0, 2], dtype=np.int64)
    val = np.array([2.0, 3.0])
    y = orc.spmv(pos, crd, val, np.array([1.0, 5.0, 7.0]), np.array([10.0, 20.0, 30.0]))
    assert y.tolist() == [10.0, 43.0, 30.0]


# ----------------------------------------------------------------- SpGEMM
def test_spgemm_golden(golden, golden_dir):
    g = golden["spgemm_csr"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["A"])
    Cpos, Ccrd, Cval = orc.spgemm(pos, crd, val, pos, crd, val, nc)
    assert Cpos.tolist() == g["pos"]
    assert Ccrd.tolist() == g["crd"]
    assert orc.format_f64(Cval) == g["printed_val"]


SEMIRING_CASES = ["any_pair", "min_first", "min_plus", "min_second", "plus_first", "plus_pair", "plus_second",
                  "plus_times"]


@pytest.mark.parametrize("name", SEMIRING_CASES)
def test_spgemm_semiring_golden(golden, golden_dir, name):
    g = golden["spgemm_csr_semiring"]
    c = g["cases"][name]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["A"])
    Cpos, Ccrd, Cval = orc.spgemm(pos, crd, val, pos, crd, val, nc, semiring=(c["reduce"], c["mult"]))
    assert Cpos.tolist() == g["pos"]
    assert Ccrd.tolist() == g["crd"]
    assert orc.format_f64(Cval) == c["printed_val"]


def _semiring_bruteforce(A, B, reduce, mult, mask=None):
    """Independent statement: gather the products of every (i, j) in traversal order, then fold."""
    mul = {"times": lambda a, b: a * b, "first": lambda a, b: a, "second": lambda a, b: b,
           "pair": lambda a, b: 1.0, "plus": lambda a, b: a + b, "minus": lambda a, b: a - b,
           "min": min, "max": max, "div": lambda a, b: a / b}[mult]
    out = []
    for i in range(A.shape[0]):
        cols = {}
        for p in range(A.indptr[i], A.indptr[i + 1]):
            k = A.indices[p]
            for q in range(B.indptr[k], B.indptr[k + 1]):
                cols.setdefault(int(B.indices[q]), []).append(mul(float(A.data[p]), float(B.data[q])))
        row = {}
        for j, es in cols.items():
            if mask is not None and not mask[i, j]:
                continue
            if reduce == "plus":
                acc = 0.0
                for e in es:
                    acc = acc + e
            elif reduce == "min":
                acc = min(es)
            elif reduce == "max":
                acc = max([0.0] + es)      # the reference starts max from 0, not from -inf
            else:
                acc = es[-1]
            row[j] = acc
        out.append(row)
    return out


@pytest.mark.parametrize("reduce", ["plus", "min", "max", "any"])
@pytest.mark.parametrize("mult", ["times", "first", "second", "pair", "plus", "minus", "min", "max", "div"])
def test_spgemm_semiring_bruteforce(reduce, mult):
    rng = np.random.default_rng(sum(map(ord, reduce + mult)))
    A = sp.random(23, 31, density=0.2, format="csr", random_state=rng, data_rvs=lambda n: rng.uniform(-2, 2, n))
    B = sp.random(31, 19, density=0.25, format="csr", random_state=rng, data_rvs=lambda n: rng.uniform(0.5, 3, n))
    A.sort_indices(); B.sort_indices()
    Cpos, Ccrd, Cval = orc.spgemm(A.indptr, A.indices, A.data, B.indptr, B.indices, B.data, 19,
                                  semiring=(reduce, mult))
    want = _semiring_bruteforce(A, B, reduce, mult)
    for i, row in enumerate(want):
        got = dict(zip(Ccrd[Cpos[i]:Cpos[i + 1]].tolist(), Cval[Cpos[i]:Cpos[i + 1]].tolist()))
        assert sorted(got) == sorted(row)
        assert list(got) == sorted(got)
        for j in row:
            assert got[j] == row[j], (i, j, got[j], row[j])


def test_spgemm_semiring_masked_bruteforce():
    rng = np.random.default_rng(77)
    A = sp.random(20, 20, density=0.3, format="csr", random_state=rng, data_rvs=lambda n: rng.uniform(0.5, 2, n))
    M = sp.random(20, 20, density=0.3, format="csr", random_state=rng)
    A.sort_indices(); M.sort_indices()
    Md = M.toarray() != 0
    Cpos, Ccrd, Cval = orc.spgemm(A.indptr, A.indices, A.data, A.indptr, A.indices, A.data, 20,
                                  mask=(M.indptr, M.indices), semiring=("min", "plus"))
    want = _semiring_bruteforce(A, A, "min", "plus", mask=Md)
    for i, row in enumerate(want):
        got = dict(zip(Ccrd[Cpos[i]:Cpos[i + 1]].tolist(), Cval[Cpos[i]:Cpos[i + 1]].tolist()))
        assert got == row


def test_spgemm_semiring_plus_times_is_the_plain_routine():
    rng = np.random.default_rng(3)
    A = sp.random(40, 40, density=0.2, format="csr", random_state=rng, data_rvs=lambda n: rng.uniform(-1, 1, n))
    A.sort_indices()
    plain = orc.spgemm(A.indptr, A.indices, A.data, A.indptr, A.indices, A.data, 40)
    semi = orc.spgemm(A.indptr, A.indices, A.data, A.indptr, A.indices, A.data, 40, semiring=("plus", "times"))
    for x, y in zip(plain, semi):
        assert np.array_equal(x, y)


def test_spgemm_masked_golden(golden, golden_dir):
    g = golden["spgemm_csr_masked"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["A"])
    Cpos, Ccrd, Cval = orc.spgemm(pos, crd, val, pos, crd, val, nc, mask=(pos, crd))
    assert Cpos.tolist() == g["pos"]
    assert Ccrd.tolist() == g["crd"]
    assert orc.format_f64(Cval) == g["printed_val"]


@pytest.mark.parametrize("seed,signed", [(0, False), (1, True), (2, True)])
def test_spgemm_vs_scipy(seed, signed):
    rng = np.random.default_rng(seed)
    A = _rand_csr(rng, 61, 47, 0.12, signed)
    B = _rand_csr(rng, 47, 53, 0.12, signed)
    Cpos, Ccrd, Cval = orc.spgemm(A.indptr, A.indices, A.data, B.indptr, B.indices, B.data, 53)
    # structure = pattern product (scipy drops exact zeros from a value product, the reference keeps them)
    P = (sp.csr_matrix((np.ones_like(A.data), A.indices, A.indptr), A.shape)
         @ sp.csr_matrix((np.ones_like(B.data), B.indices, B.indptr), B.shape)).tocsr()
    P.sort_indices()
    assert np.array_equal(Cpos, P.indptr)
    assert np.array_equal(Ccrd, P.indices)
    dense = A.toarray() @ B.toarray()
    rows = np.repeat(np.arange(61), np.diff(Cpos))
    np.testing.assert_allclose(Cval, dense[rows, Ccrd], rtol=0, atol=1e-13)
    # invariants
    assert Cpos[0] == 0 and Cpos[-1] == len(Ccrd) and np.all(np.diff(Cpos) >= 0)
    for i in range(61):
        assert np.all(np.diff(Ccrd[Cpos[i]:Cpos[i + 1]]) > 0)


def test_spgemm_summation_order_bit_exact():
    rng = np.random.default_rng(5)
    A = _rand_csr(rng, 30, 30, 0.3)
    Cpos, Ccrd, Cval = orc.spgemm(A.indptr, A.indices, A.data, A.indptr, A.indices, A.data, 30)
    for i in range(30):
        acc = {}
        for p in range(A.indptr[i], A.indptr[i + 1]):
            k = A.indices[p]
            for q in range(A.indptr[k], A.indptr[k + 1]):
                j = A.indices[q]
                v = A.data[p] * A.data[q]
                acc[j] = acc[j] + v if j in acc else v
        cols = sorted(acc)
        assert Ccrd[Cpos[i]:Cpos[i + 1]].tolist() == cols
        assert Cval[Cpos[i]:Cpos[i + 1]].tolist() == [acc[j] for j in cols]


def test_spgemm_row_range_matches_full():
    rng = np.random.default_rng(6)
    A = _rand_csr(rng, 40, 40, 0.2, signed=False)
    full = orc.spgemm(A.indptr, A.indices, A.data, A.indptr, A.indices, A.data, 40)
    part = orc.spgemm(A.indptr, A.indices, A.data, A.indptr, A.indices, A.data, 40, rows=(10, 25))
    lo, hi = full[0][10], full[0][25]
    assert np.array_equal(part[0], full[0][10:26] - lo)
    assert np.array_equal(part[1], full[1][lo:hi])
    assert np.array_equal(part[2], full[2][lo:hi])


@pytest.mark.parametrize("seed", [0, 3])
def test_spgemm_masked_bruteforce(seed):
    rng = np.random.default_rng(seed)
    A = _rand_csr(rng, 35, 35, 0.2, signed=False)
    Mk = _rand_csr(rng, 35, 35, 0.3, signed=False)
    Cpos, Ccrd, Cval = orc.spgemm(A.indptr, A.indices, A.data, A.indptr, A.indices, A.data, 35,
                                  mask=(Mk.indptr, Mk.indices))
    dense = A.toarray() @ A.toarray()
    pat = ((A.toarray() != 0).astype(int) @ (A.toarray() != 0).astype(int) > 0) & (Mk.toarray() != 0)
    ri, ci = np.nonzero(pat)
    assert np.array_equal(np.repeat(np.arange(35), np.diff(Cpos)), ri)
    assert np.array_equal(Ccrd, ci)
    np.testing.assert_allclose(Cval, dense[ri, ci], rtol=0, atol=1e-13)


def test_spgemm_empty():
    pos = np.zeros(4, dtype=np.int64)
    e = np.zeros(0, dtype=np.int64)
    Cpos, Ccrd, Cval = orc.spgemm(pos, e, np.zeros(0), pos, e, np.zeros(0), 3)
    assert Cpos.tolist() == [0, 0, 0, 0] and len(Ccrd) == 0 and len(Cval) == 0


# ----------------------------------------------------------------- SUM / eltwise / triangles
def test_sum_golden(golden, golden_dir):
    (nr, nc), pos, crd, val = _mtx(golden_dir, golden["sum_csr"]["matrix"])
    assert "%g" % orc.reduce_sum(val) == golden["sum_csr"]["printed"]


def test_eltwise_golden(golden, golden_dir):
    g = golden["eltwise_mult_csr"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["A"])
    Cpos, Ccrd, Cval = orc.eltwise_mult(pos, crd, val, pos, crd, val)
    assert Cpos.tolist() == g["pos"] and Ccrd.tolist() == g["crd"]
    assert orc.format_f64(Cval) == g["printed_val"]


def test_eltwise_vs_scipy():
    rng = np.random.default_rng(9)
    A = _rand_csr(rng, 40, 31, 0.3, signed=False)
    B = _rand_csr(rng, 40, 31, 0.3, signed=False)
    Cpos, Ccrd, Cval = orc.eltwise_mult(A.indptr, A.indices, A.data, B.indptr, B.indices, B.data)
    R = A.multiply(B).tocsr()
    R.sort_indices()
    assert np.array_equal(Cpos, R.indptr) and np.array_equal(Ccrd, R.indices)
    assert np.array_equal(Cval, R.data)


def test_triangle_count_golden(golden, golden_dir):
    g = golden["triangle_count"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"], g["read_mode"])
    # masked two-step program: C<L> = L*L ; SUM(C)
    Cpos, Ccrd, Cval = orc.spgemm(pos, crd, val, pos, crd, val, nc, mask=(pos, crd))
    assert orc.reduce_sum(Cval) == g["count"]
    # fused streaming form
    assert orc.tricount_masked(pos, crd, val) == g["count"]
    # unmasked program: SUM((L*L) .* L)
    Fpos, Fcrd, Fval = orc.spgemm(pos, crd, val, pos, crd, val, nc)
    Epos, Ecrd, Eval = orc.eltwise_mult(Fpos, Fcrd, Fval, pos, crd, val)
    assert orc.reduce_sum(Eval) == g["count"]


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_triangle_count_trace_identity(seed):
    rng = np.random.default_rng(seed)
    n = 60
    U = np.triu(rng.random((n, n)) < 0.15, 1)
    Adj = (U | U.T).astype(np.int64)
    expected = int(np.trace(Adj @ Adj @ Adj)) // 6
    brute = sum(1 for a, b, c in itertools.combinations(range(n), 3) if Adj[a, b] and Adj[b, c] and Adj[a, c])
    assert brute == expected
    L = sp.csr_matrix(np.tril(Adj, -1).astype(float))
    L.sort_indices()
    assert orc.tricount_masked(L.indptr, L.indices, L.data) == expected


# ----------------------------------------------------------------- TTGT
def test_ttgt_goldens(golden):
    for g in golden["ttgt"]:
        A = np.full([g["extent"][ch] for ch in g["A"]], g["A_fill"])
        B = np.full([g["extent"][ch] for ch in g["B"]], g["B_fill"])
        Cd = orc.contract_direct(g["A"], g["B"], g["C"], A, B)
        assert orc.format_f64(Cd) == g["printed"], g["source"]
        Ct, plan, chosen = orc.ttgt_contract(g["A"], g["B"], g["C"], A, B)
        assert orc.format_f64(Ct) == g["printed"], g["source"]
        # closed form: every output = (product of contracted extents) * a * b
        kprod = np.prod([g["extent"][ch] for ch in set(g["A"]) - set(g["C"])])
        np.testing.assert_allclose(Ct, kprod * g["A_fill"] * g["B_fill"], rtol=1e-14)


def test_ttgt_doc_example_candidate0(golden):
    g = golden["ttgt_doc_example"]
    ext = {ch: 3 for ch in "abcdef"}
    plan, chosen, ncand, ids = orc.ttgt_plan(g["A"], g["B"], g["C"], ext, which=0)
    inv = {v: k for k, v in ids.items()}
    assert ncand == 16 and chosen == 0
    assert "".join(inv[i] for i in plan.a_idx[:4]) == g["candidate0"]["A_target"]
    assert "".join(inv[i] for i in plan.b_idx[:4]) == g["candidate0"]["B_target"]
    assert "".join(inv[i] for i in plan.c_idx[:4]) == g["candidate0"]["C_target"]
    assert (plan.transA, plan.transB, plan.transC, plan.swapAB) == (1, 1, 1, 0)
    # permutation convention: output dim i = input dim perm[i]
    assert list(plan.permA[:4]) == [0, 2, 1, 3]      # aebf -> abef
    assert list(plan.permB[:4]) == [3, 1, 0, 2]      # dfce -> efdc
    assert list(plan.permC[:4]) == [0, 1, 3, 2]      # abcd -> abdc


def test_ttgt_selection_for_the_64_4_contraction():
    ext = {ch: 64 for ch in "abcdef"}
    plan, chosen, ncand, ids = orc.ttgt_plan("aebf", "dfce", "abcd", ext)
    inv = {v: k for k, v in ids.items()}
    # cheapest by the cost rule: A->abef (leading index kept: 1 unit), B->efcd (1/0.71), C in place
    assert chosen == 4
    assert "".join(inv[i] for i in plan.b_idx[:4]) == "efcd"
    assert (plan.transA, plan.transB, plan.transC, plan.swapAB) == (1, 1, 0, 0)
    assert (plan.M, plan.N, plan.K) == (4096, 4096, 4096)
    assert plan.cost == pytest.approx(4096 * 4096 * (1 + 1 / 0.71))


def test_transpose_matches_numpy():
    rng = np.random.default_rng(0)
    x = rng.random((3, 4, 5, 2))
    for perm in itertools.permutations(range(4)):
        assert np.array_equal(orc.transpose(x, perm), np.transpose(x, perm))


def test_gemm_ijk():
    rng = np.random.default_rng(1)
    A, B, C0 = rng.uniform(-1, 1, (9, 13)), rng.uniform(-1, 1, (13, 7)), rng.uniform(-1, 1, (9, 7))
    out = orc.gemm_ijk(A, B, C0)
    np.testing.assert_allclose(out, C0 + A @ B, rtol=0, atol=1e-14)
    ref = C0.copy()
    for i in range(9):
        for j in range(7):
            for k in range(13):
                ref[i, j] = ref[i, j] + A[i, k] * B[k, j]
    assert np.array_equal(out, ref)


@pytest.mark.parametrize("a,b,c", [("aebf", "dfce", "abcd"), ("cima", "mc", "ia"), ("icmn", "mnca", "ia"),
                                   ("ca", "ic", "ia"), ("aedf", "bfce", "abcd")])
def test_ttgt_every_candidate_matches_einsum(a, b, c):
    rng = np.random.default_rng(4)
    sizes = dict(zip("abcdefimn", [2, 3, 4, 5, 3, 2, 3, 4, 2]))
    A = rng.uniform(-1, 1, [sizes[ch] for ch in a])
    B = rng.uniform(-1, 1, [sizes[ch] for ch in b])
    ref = np.einsum(f"{a},{b}->{c}", A, B)
    plan, chosen, ncand, _ = orc.ttgt_plan(a, b, c, sizes)
    for which in [-1] + list(range(ncand)):
        Ct, _, _ = orc.ttgt_contract(a, b, c, A, B, which=which)
        np.testing.assert_allclose(Ct, ref, rtol=0, atol=1e-13, err_msg=f"candidate {which}")
    np.testing.assert_allclose(orc.contract_direct(a, b, c, A, B), ref, rtol=0, atol=1e-13)
    # beta = 1 accumulates into C
    C0 = rng.uniform(-1, 1, ref.shape)
    for which in (0, ncand - 1):
        Ct, _, _ = orc.ttgt_contract(a, b, c, A, B, C0=C0, beta=1.0, which=which)
        np.testing.assert_allclose(Ct, C0 + ref, rtol=0, atol=1e-13)


# ----------------------------------------------------------------- reader: other layouts and file flavours
def test_read_coo_golden(golden, golden_dir):
    for g in golden["read_coo"]:
        _, pos, crd, val = _mtx(golden_dir, g["matrix"], g["mode"])
        a1pos, a1crd, a2pos, a2crd, aval = orc.coo_layout(pos, crd, val)
        assert a1pos.tolist() == g["a1pos"], g["source"]
        assert a1crd.tolist() == g["a1crd"], g["source"]
        assert a2pos.tolist() == g["a2pos"] and a2crd.tolist() == g["a2crd"], g["source"]
        assert orc.format_f64(aval) == g["printed_val"], g["source"]


def test_dcsr_layout_invariants():
    """No test of the reference prints a DCSR tensor; what fixes the layout is that expanding it gives the
    CSR arrays back and that only rows with entries are listed, in ascending order."""
    rng = np.random.default_rng(4)
    A = sp.random(40, 30, density=0.05, format="csr", random_state=rng)
    A.sort_indices()
    a1pos, a1crd, a2pos, a2crd, aval = orc.dcsr_layout(A.indptr, A.indices, A.data)
    lens = np.diff(A.indptr)
    assert a1pos.tolist() == [0, int((lens > 0).sum())]
    assert a1crd.tolist() == np.flatnonzero(lens > 0).tolist()
    assert np.array_equal(np.diff(a2pos), lens[lens > 0]) and a2pos[0] == 0
    assert np.array_equal(a2crd, A.indices) and np.array_equal(aval, A.data)


def _write_mtx(path, header, size_line, lines):
    with open(path, "w") as f:
        f.write(header + "\n% a comment\n" + size_line + "\n" + "\n".join(lines) + "\n")


@pytest.mark.parametrize("flavour", ["general", "symmetric", "skew-symmetric", "pattern", "array"])
def test_reader_flavours_vs_scipy(tmp_path, flavour):
    import scipy.io
    rng = np.random.default_rng(len(flavour))
    n = 9
    path = str(tmp_path / "m.mtx")
    if flavour == "array":
        D = rng.uniform(-1, 1, (n, 6)).round(3)
        _write_mtx(path, "%%MatrixMarket matrix array real general", f"{n} 6", [repr(float(v)) for v in D.T.ravel()])
    else:
        D = np.where(rng.random((n, n)) < 0.3, rng.uniform(-1, 1, (n, n)).round(3), 0.0)
        if flavour == "symmetric":
            D = np.tril(D) + np.tril(D, -1).T
            ent = [(i, j) for i in range(n) for j in range(i + 1) if D[i, j] != 0]
        elif flavour == "skew-symmetric":
            D = np.tril(D, -1) - np.tril(D, -1).T
            ent = [(i, j) for i in range(n) for j in range(i) if D[i, j] != 0]
        else:
            ent = [(i, j) for i in range(n) for j in range(n) if D[i, j] != 0]
        rng.shuffle(ent)
        if flavour == "pattern":
            D = (D != 0).astype(float)
            lines = [f"{i + 1} {j + 1}" for i, j in ent]
            head = "%%MatrixMarket matrix coordinate pattern general"
        else:
            lines = [f"{i + 1} {j + 1} {float(D[i, j])!r}" for i, j in ent]
            head = "%%MatrixMarket matrix coordinate real " + (flavour if flavour != "general" else "general")
        _write_mtx(path, head, f"{n} {n} {len(ent)}", lines)
    (nr, nc), pos, crd, val = orc.read_mtx_csr(path, 1)
    got = sp.csr_matrix((val, crd, pos), shape=(nr, nc)).toarray()
    assert np.array_equal(got, D)
    assert np.array_equal(got, scipy.io.mmread(path).toarray() if flavour != "array" else scipy.io.mmread(path))
    for r in range(nr):                        # columns ascending inside every row
        assert np.all(np.diff(crd[pos[r]:pos[r + 1]]) > 0)


# ----------------------------------------------------------------- dense operand on the left, CSR .* Dense
def test_vecmat_densemat_golden(golden, golden_dir):
    g = golden["vecmat_csr"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"])
    y = orc.vecmat(np.full(nr, g["x_fill"]), pos, crd, val, nc, np.full(nc, g["y_fill"]))
    assert orc.format_f64(y) == g["printed"]
    g = golden["densemat_csr"]
    Cm = orc.densemat(np.full((g["M"], nr), g["a_fill"]), pos, crd, val, nc, np.full((g["M"], nc), g["c_fill"]))
    assert orc.format_f64(Cm) == g["printed"]


def test_vecmat_densemat_order_and_scipy():
    rng = np.random.default_rng(8)
    B = sp.random(37, 23, density=0.3, format="csr", random_state=rng, data_rvs=lambda n: rng.uniform(-1, 1, n))
    B.sort_indices()
    x, A = rng.uniform(-1, 1, 37), rng.uniform(-1, 1, (5, 37))
    y0, C0 = rng.uniform(-1, 1, 23), rng.uniform(-1, 1, (5, 23))
    y = orc.vecmat(x, B.indptr, B.indices, B.data, 23, y0)
    Cm = orc.densemat(A, B.indptr, B.indices, B.data, 23, C0)
    assert np.allclose(y, y0 + x @ B.toarray(), rtol=1e-13) and np.allclose(Cm, C0 + A @ B.toarray(), rtol=1e-13)
    Bd = B.toarray()
    for j in range(23):                  # ascending contracted index, multiply then add, starting from the output
        acc = y0[j]
        for i in range(37):
            if Bd[i, j] != 0:
                acc = acc + x[i] * Bd[i, j]
        assert y[j] == acc
    acc = C0[3, 7]
    for i in range(37):
        if Bd[i, 7] != 0:
            acc = acc + A[3, i] * Bd[i, 7]
    assert Cm[3, 7] == acc


def test_eltwise_mult_csr_dense_golden(golden, golden_dir):
    g = golden["eltwise_mult_csr_dense"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"])
    v = orc.eltwise_mult_dense(pos, crd, val, np.full((nr, nc), g["d_fill"]))
    assert pos.tolist() == g["pos"] and crd.tolist() == g["crd"]
    assert orc.format_f64(v) == g["printed_val"]
    dense = np.zeros((nr, nc))
    dense[np.repeat(np.arange(nr), np.diff(pos)), crd] = v
    assert orc.format_f64(dense) == g["printed_dense"]


def test_eltwise_monoid_golden(golden, golden_dir):
    for g in golden["eltwise_monoid"]["dense"]:
        out = orc.eltwise_dense(np.full(g["shape"], g["a"]), np.full(g["shape"], g["b"]), g["op"])
        assert orc.format_f64(out) == g["printed"], g["source"]
    for g in golden["eltwise_monoid"]["coo_dense"]:
        (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"])
        v = orc.eltwise_csr_dense(pos, crd, val, np.full((nr, nc), g["d_fill"]), g["op"])
        a1pos, a1crd, _, a2crd, _ = orc.coo_layout(pos, crd, val)
        assert a1pos.tolist() == g["a1pos"] and a1crd.tolist() == g["a1crd"] and a2crd.tolist() == g["a2crd"]
        assert orc.format_f64(v) == g["printed_val"], g["source"]


def test_sddmm_golden_and_brute_force(golden, golden_dir):
    """kernels/sddmm.ta: B .* (C x D) at B's entries; then an independent restatement on random data (T formed
    as a sum of outer products in ascending k, which adds in the same order) and scipy within rounding."""
    g = golden["kernels_and_compound"]["sddmm"]
    (nr, nc), pos, crd, val = _mtx(golden_dir, g["matrix"])
    v = orc.sddmm(pos, crd, val, np.full((nr, g["K"]), g["c_fill"]), np.full((g["K"], nc), g["d_fill"]))
    printed = orc.format_i64([nr]) + orc.format_i64([-1]) + orc.format_i64(pos) + orc.format_i64(crd) + orc.format_f64(v)
    assert printed == g["printed"]
    rng = np.random.default_rng(5)
    A = sp.random(40, 30, 0.15, random_state=3, format="csr"); A.sort_indices()
    Cm, D = rng.uniform(-1, 1, (40, 9)), rng.uniform(-1, 1, (9, 30))
    got = orc.sddmm(A.indptr, A.indices, A.data, Cm, D)
    T = np.zeros((40, 30))
    for k in range(9):
        T = T + np.outer(Cm[:, k], D[k, :])
    rows = np.repeat(np.arange(40), np.diff(A.indptr))
    assert np.array_equal(got, A.data * T[rows, A.indices])
    assert np.allclose(got, A.data * (Cm @ D)[rows, A.indices], rtol=1e-13, atol=1e-15)
    # a dropped term, a transposed operand or B's value left out would all show here
    assert np.array_equal(orc.sddmm(A.indptr, A.indices, A.data, Cm[:, :0], D[:0, :]), A.data * 0.0)


def test_checker_sort_is_a_sort():
    """The checker sorts a row's touched columns with its own introsort (what std::sort is, inlined on the element
    type); against numpy on the inputs that break a careless quicksort, including ones long enough for the
    depth limit to send it to heapsort."""
    rng = np.random.default_rng(7)
    cases = [np.zeros(0, dtype=np.int64), np.array([5], dtype=np.int64)]
    for n in (2, 3, 15, 16, 17, 31, 33, 100, 1000, 4097, 70_000):
        base = rng.permutation(n * 3)[:n].astype(np.int64)          # distinct, as a row's columns are
        organ = np.concatenate([np.arange(0, n, 2), np.arange(n - 1 - (n % 2 == 0), 0, -2)]).astype(np.int64)
        cases += [base, np.sort(base), np.sort(base)[::-1].copy(), organ,
                  np.concatenate([np.sort(base[: n // 2]), np.sort(base[n // 2:])]),
                  rng.integers(0, 4, n).astype(np.int64)]                # heavy duplicates (never produced by a row, still sorted)
    # a median-of-three killer for the (first+1, middle, last) sample
    n = 4096
    killer = np.arange(n, dtype=np.int64)
    killer[1::2] = np.arange(n // 2, n)
    killer[0::2] = np.arange(0, n // 2)
    cases.append(killer)
    for a in cases:
        got = a.copy()
        orc.lib().oracle_sort_idx(got, len(got))
        assert np.array_equal(got, np.sort(a)), len(a)


def test_row_parallel_checker_equals_sequential():
    from comet_amd import gen
    """The OpenMP forms (the stronger CPU baseline of the benchmark) produce what the sequential forms produce."""
    n = 3000
    pos, crd, val = gen.zipf_csr(n=n, mean=12.0, cap=1500, seed=41)
    val = np.abs(val) + 0.1
    for mask in (None, (pos, crd)):
        p0, c0, v0 = orc.spgemm(pos, crd, val, pos, crd, val, n, mask=mask)
        p1, c1, v1 = orc.spgemm(pos, crd, val, pos, crd, val, n, mask=mask, threads=True)
        assert np.array_equal(p0, p1) and np.array_equal(c0, c1) and np.array_equal(v0, v1)
        p2, c2, v2 = orc.spgemm(pos, crd, val, pos, crd, val, n, mask=mask, rows=(100, 900), threads=True)
        assert np.array_equal(c2, c0[p0[100]:p0[900]]) and np.array_equal(v2, v0[p0[100]:p0[900]])
    apos, acrd, aval = gen.rmat_symmetric_csr(scale=11, edge_factor=8, seed=5, values="ones")
    lpos, lcrd, _ = gen.strictly_lower(apos, acrd, aval)
    ones = np.ones(len(lcrd))
    assert orc.tricount_masked(lpos, lcrd, ones, threads=True) == orc.tricount_masked(lpos, lcrd, ones)

