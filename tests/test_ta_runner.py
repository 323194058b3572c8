"""The .ta runner against the reference's printed expectations.  The programs are written here from the
operation each golden entry names (tests/golden/reference_goldens.json cites the reference test it comes
from); the expectations are turned into CHECK / CHECK-NEXT lines and verified with LLVM's FileCheck when the
image has it, by exact text comparison otherwise."""
import io
import os
import shutil
import subprocess

import numpy as np
import pytest

from comet_amd import ta_run

pytestmark = pytest.mark.gpu

FILECHECK = shutil.which("FileCheck") or "/opt/rocm/lib/llvm/bin/FileCheck"


def _run(program, files, tmp_path, monkeypatch, golden_dir):
    for i, name in enumerate(files):
        monkeypatch.setenv(f"SPARSE_FILE_NAME{i}", os.path.join(golden_dir, name))
    out = io.StringIO()
    ta_run.run_text(program, out)
    return out.getvalue()


def _check(output, expected_text, tmp_path):
    """expected_text: the printed form, "data = \\n...\\n" blocks in order."""
    lines = [l for l in expected_text.split("\n") if l != ""]
    if os.path.exists(FILECHECK):
        check = tmp_path / "expect.check"
        check.write_text("\n".join(("# CHECK: " if i == 0 else "# CHECK-NEXT: ") + l for i, l in enumerate(lines)) + "\n")
        r = subprocess.run([FILECHECK, str(check)], input=output, text=True, capture_output=True)
        assert r.returncode == 0, r.stderr + "\n--- output ---\n" + output
    assert [l.rstrip() for l in output.split("\n") if l.strip()] == [l.rstrip() for l in lines]


def _decl(fmt_a="CSR"):
    return f"""
def main() {{
    IndexLabel [a] = [?];
    IndexLabel [b] = [?];
    IndexLabel [c] = [?];
    IndexLabel [k4] = [4];
    Tensor<double> A([a, b], {{{fmt_a}}});
"""


def _ints(v):
    return "data = \n" + "".join(f"{int(x)}," for x in v) + "\n"


@pytest.mark.parametrize("fmt", ["CSR", "COO", "DCSR"])
def test_spmv_spmm_programs(golden, golden_dir, tmp_path, monkeypatch, fmt):
    prog = _decl(fmt) + """
    Tensor<double> x([b], {Dense});
    Tensor<double> y([a], {Dense});
    Tensor<double> B([b, k4], {Dense});
    Tensor<double> C([a, k4], {Dense});
    A[a, b] = comet_read(0);
    x[b] = 1.7;   y[a] = 0.0;
    B[b, k4] = 1.7;   C[a, k4] = 0.0;
    y[a] = A[a, b] * x[b];
    C[a, k4] = A[a, b] * B[b, k4];
    print(y);
    print(C);
}
"""
    out = _run(prog, ["test_rank2.mtx"], tmp_path, monkeypatch, golden_dir)
    _check(out, golden["spmv_csr"]["printed"] + golden["spmm_csr"]["printed"], tmp_path)


@pytest.mark.parametrize("name", ["plus_times", "min_plus", "any_pair", "plus_second", "min_first"])
def test_spgemm_semiring_programs(golden, golden_dir, tmp_path, monkeypatch, name):
    g = golden["spgemm_csr_semiring"]
    c = g["cases"][name]
    tok = {"plus": "+", "times": "*"}
    op = "*" if name == "plus_times" else f"@({tok.get(c['reduce'], c['reduce'])},{tok.get(c['mult'], c['mult'])})"
    prog = _decl() + f"""
    Tensor<double> B([b, c], {{CSR}});
    Tensor<double> C([a, c], {{CSR}});
    A[a, b] = comet_read(0);
    B[b, c] = comet_read(1);
    C[a, c] = A[a, b] {op} B[b, c];
    print(C);
}}
"""
    out = _run(prog, [g["A"], g["B"]], tmp_path, monkeypatch, golden_dir)
    want = _ints([len(g["pos"]) - 1]) + _ints([-1]) + _ints(g["pos"]) + _ints(g["crd"]) + c["printed_val"]
    _check(out, want, tmp_path)


def test_triangle_count_program(golden, golden_dir, tmp_path, monkeypatch):
    prog = """
def main() {
    IndexLabel [i] = [?];   IndexLabel [j] = [?];   IndexLabel [k] = [?];
    Tensor<double> L([i, j], {CSR});
    Tensor<double> C([i, j], {CSR});
    L[i, j] = comet_read(0, 2);           # strictly lower triangle
    C[i, k]<L, push> = L[i, j] * L[j, k];
    var ntri = SUM(C[i, j]);
    print(ntri);
}
"""
    out = _run(prog, ["tc.mtx"], tmp_path, monkeypatch, golden_dir)
    _check(out, "data = \n5,\n", tmp_path)


def test_read_modes_and_layout_printing(golden, golden_dir, tmp_path, monkeypatch):
    for g in golden["read_csr"][2:4]:
        prog = _decl("CSR") + f"    A[a, b] = comet_read(0, {g['mode']});\n    print(A);\n}}\n"
        out = _run(prog, [g["matrix"]], tmp_path, monkeypatch, golden_dir)
        _check(out, _ints([len(g["pos"]) - 1]) + _ints([-1]) + _ints(g["pos"]) + _ints(g["crd"]) + g["printed_val"],
               tmp_path)
    for g in golden["read_coo"]:
        prog = _decl("COO") + f"    A[a, b] = comet_read(0, {g['mode']});\n    print(A);\n}}\n"
        out = _run(prog, [g["matrix"]], tmp_path, monkeypatch, golden_dir)
        _check(out, _ints(g["a1pos"]) + _ints(g["a1crd"]) + _ints(g["a2pos"]) + _ints(g["a2crd"]) + g["printed_val"],
               tmp_path)


def test_dense_contraction_sum_transpose_and_elementwise(golden, golden_dir, tmp_path, monkeypatch):
    prog = """
def main() {
    IndexLabel [i] = [3];  IndexLabel [j] = [5];  IndexLabel [k] = [2];  IndexLabel [l] = [4];
    IndexLabel [r] = [?];  IndexLabel [s] = [?];
    Tensor<double> A([i, k, j], {Dense});
    Tensor<double> B([l, k], {Dense});
    Tensor<double> C([i, j, l], {Dense});
    Tensor<double> T([j, i, l], {Dense});
    Tensor<double> S([r, s], {CSR});
    Tensor<double> P([r, s], {CSR});
    A[i, k, j] = 2.0;   B[l, k] = 0.25;   C[i, j, l] = 1.5;
    C[i, j, l] = A[i, k, j] * B[l, k];
    T[j, i, l] = transpose(C[i, j, l], {j, i, l});
    var total = SUM(T[j, i, l]);
    print(total);
    S[r, s] = comet_read(0);
    P[r, s] = S[r, s] .* S[r, s];
    var sq = SUM(P[r, s]);
    print(sq);
    var t0 = getTime();
    var t1 = getTime();
    printElapsedTime(t0, t1);
}
"""
    out = _run(prog, ["test_rank2.mtx"], tmp_path, monkeypatch, golden_dir)
    lines = out.strip().split("\n")
    # every C element: 1.5 + 2 terms of 2.0*0.25 = 2.5; 60 elements
    assert lines[0].strip() == "data =" and lines[1] == "150,"
    vals = np.array([1, 1.4, 2, 2.5, 3, 4.1, 4, 5.2, 5])
    assert lines[3] == f"{(vals * vals).sum():g},"
    assert lines[4].startswith("ELAPSED_TIME = ")


def test_unsupported_statement_is_named():
    with pytest.raises(ta_run.TaError, match="not supported"):
        ta_run.Program().run("def main() { IndexLabel [a] = [4]; for (x in a) {} }")


def test_dense_left_and_csr_times_dense_programs(golden, golden_dir, tmp_path, monkeypatch):
    prog = """
def main() {
    IndexLabel [m] = [4];  IndexLabel [a] = [?];  IndexLabel [b] = [?];
    Tensor<double> S([a, b], {CSR});
    Tensor<double> x([a], {Dense});      Tensor<double> y([b], {Dense});
    Tensor<double> A([m, a], {Dense});   Tensor<double> C([m, b], {Dense});
    Tensor<double> D([a, b], {Dense});   Tensor<double> E([a, b], {CSR});   Tensor<double> F([a, b], {Dense});
    S[a, b] = comet_read(0);
    x[a] = 1.7;  y[b] = 0.0;  A[m, a] = 1.7;  C[m, b] = 0.0;  D[a, b] = 2.7;  F[a, b] = 0.0;
    y[b] = x[a] * S[a, b];
    C[m, b] = A[m, a] * S[a, b];
    E[a, b] = S[a, b] .* D[a, b];
    F[a, b] = D[a, b] .* S[a, b];
    print(y);  print(C);  print(E);  print(F);
}
"""
    out = _run(prog, ["test_rank2.mtx"], tmp_path, monkeypatch, golden_dir)
    g = golden["eltwise_mult_csr_dense"]
    want = (golden["vecmat_csr"]["printed"] + golden["densemat_csr"]["printed"] + _ints([5]) + _ints([-1]) +
            _ints(g["pos"]) + _ints(g["crd"]) + g["printed_val"] + g["printed_dense"])
    _check(out, want, tmp_path)


def test_elementwise_monoid_programs(golden, golden_dir, tmp_path, monkeypatch):
    tok = {"plus": "+", "minus": "-", "times": "*", "min": "min"}
    for g in golden["eltwise_monoid"]["dense"]:
        labels = "abcd"[:len(g["shape"])]
        idx = ", ".join(labels)
        decl = "".join(f"    IndexLabel [{l}] = [{n}];\n" for l, n in zip(labels, g["shape"]))
        prog = ("def main() {\n" + decl +
                "".join(f"    Tensor<double> {t}([{idx}], {{Dense}});\n" for t in "ABC") +
                f"    A[{idx}] = {g['a']};\n    B[{idx}] = {g['b']};\n    C[{idx}] = 0.0;\n" +
                f"    C[{idx}] = A[{idx}] @({tok[g['op']]}) B[{idx}];\n    print(C);\n}}\n")
        _check(_run(prog, [], tmp_path, monkeypatch, golden_dir), g["printed"], tmp_path)
    for g in golden["eltwise_monoid"]["coo_dense"]:
        prog = _decl("COO") + f"""
    Tensor<double> D([a, b], {{Dense}});
    Tensor<double> E([a, b], {{COO}});
    A[a, b] = comet_read(0);
    D[a, b] = {g['d_fill']};
    E[a, b] = A[a, b] @({tok[g['op']]}) D[a, b];
    print(E);
}}
"""
        out = _run(prog, [g["matrix"]], tmp_path, monkeypatch, golden_dir)
        _check(out, _ints(g["a1pos"]) + _ints(g["a1crd"]) + _ints([-1]) + _ints(g["a2crd"]) + g["printed_val"], tmp_path)


# ------------------------------------------------------ kernels/ and compound_exps/ of the reference's tests
def _kc_programs(g):
    """name -> (program, input files); sizes and fills come from the golden entry."""
    lab = lambda **kw: "".join(f"    IndexLabel [{k}] = [{v}];\n" for k, v in kw.items())
    ten = lambda *decls: "".join(f"    Tensor<double> {n}([{', '.join(ls)}], {{{f}}});\n" for n, ls, f in decls)
    body = lambda text: "def main() {\n" + text + "}\n"
    P = {}
    e = g["sddmm"]
    P["sddmm"] = (body(lab(i="?", j="?", k=e["K"]) +
                       ten(("B", "ij", "CSR"), ("C", "ik", "Dense"), ("D", "kj", "Dense"), ("A", "ij", "CSR"),
                           ("T", "ij", "Dense")) +
                       f"    B[i, j] = comet_read(0);\n    C[i, k] = {e['c_fill']};\n    D[k, j] = {e['d_fill']};\n"
                       "    T[i, j] = 0.0;\n    T[i, j] = C[i, k] * D[k, j];\n    A[i, j] = B[i, j] .* T[i, j];\n"
                       "    print(A);\n"), [e["matrix"]])
    e = g["gnn"]
    P["gnn"] = (body(lab(i="?", k="?", j=e["J"], h=e["H"]) +
                     ten(("B", "ik", "CSR"), ("C", "kh", "Dense"), ("D", "hj", "Dense"), ("A", "ij", "Dense"),
                         ("T", "ih", "Dense")) +
                     f"    B[i, k] = comet_read(0);\n    C[k, h] = {e['c_fill']};\n    D[h, j] = {e['d_fill']};\n"
                     "    A[i, j] = 0.0;\n    T[i, h] = 0.0;\n    T[i, h] = B[i, k] * C[k, h];\n"
                     "    A[i, j] = T[i, h] * D[h, j];\n    print(A);\n"), [e["matrix"]])
    e = g["gram_matrix"]
    P["gram_matrix"] = (body(f"    IndexLabel [i, k] = [{e['I']}];\n" + lab(j=e["J"]) +
                             ten(("A", "ij", "Dense"), ("B", "ii", "Dense")) +
                             f"    A[i, j] = {e['a_fill']};\n    B[i, k] = 0.0;\n"
                             "    B[i, k] = A[i, j] * transpose(A[k, j], {j, k});\n    print(B);\n"), [])
    e = g["csr_dense_chain"]
    P["csr_dense_chain"] = (body(lab(i="?", j="?", k=e["K"], l=e["L"]) +
                                 ten(("B", "ij", "CSR"), ("A", "il", "Dense"), ("C", "jk", "Dense"),
                                     ("D", "kl", "Dense")) +
                                 f"    B[i, j] = comet_read(0);\n    A[i, l] = 0.0;\n    C[j, k] = {e['c_fill']};\n"
                                 f"    D[k, l] = {e['d_fill']};\n    A[i, l] = B[i, j] * C[j, k] * D[k, l];\n"
                                 "    print(A);\n"), [e["matrix"]])
    e = g["csr_mult_dtranspose"]
    P["csr_mult_dtranspose"] = (body(lab(i=e["I"], j="?", k="?") +
                                     "    Tensor<double> A([k, j], CSR);\n    Tensor<double> B([i, j], Dense);\n"
                                     "    Tensor<double> C([k, i], Dense);\n"
                                     f"    A[k, j] = comet_read(0);\n    B[i, j] = {e['b_fill']};\n    C[k, i] = 0.0;\n"
                                     "    C[k, i] = A[k, j] * transpose(B[i, j], {j, i});\n    print(C);\n"),
                                [e["matrix"]])
    e = g["dtranspose_eltwise_csr"]
    P["dtranspose_eltwise_csr"] = (body(lab(i="?", j="?") +
                                        ten(("B", "ji", "CSR"), ("C", "ji", "CSR"), ("A", "ij", "Dense")) +
                                        f"    B[j, i] = comet_read(0);\n    A[i, j] = {e['a_fill']};\n"
                                        "    C[j, i] = transpose(A[i, j], {j, i}) .* B[j, i];\n    print(C);\n"),
                                   [e["matrix"]])
    e = g["dtranspose_mult_csr"]
    P["dtranspose_mult_csr"] = (body(lab(i="?", j=e["J"], k="?") +
                                     ten(("B", "ik", "CSR"), ("A", "ij", "Dense"), ("C", "jk", "Dense")) +
                                     f"    B[i, k] = comet_read(0);\n    A[i, j] = {e['a_fill']};\n    C[j, k] = 0.0;\n"
                                     "    C[j, k] = transpose(A[i, j], {j, i}) * B[i, k];\n    print(C);\n"),
                                [e["matrix"]])
    e = g["dense_chain"]
    si, sj, sk, sl = e["sizes"]
    P["dense_chain"] = (body(lab(i=si, j=sj, k=sk, l=sl) +
                             ten(("A", "ij", "Dense"), ("B", "jk", "Dense"), ("C", "kl", "Dense"), ("D", "il", "Dense")) +
                             f"    A[i, j] = {e['fills'][0]};\n    B[j, k] = {e['fills'][1]};\n"
                             f"    C[k, l] = {e['fills'][2]};\n    D[i, l] = 0.0;\n"
                             "    D[i, l] = A[i, j] * B[j, k] * C[k, l];\n    print(D);\n"), [])
    e = g["dense_eltwise_dtranspose"]
    for name, expr in (("dense_eltwise_dtranspose", "B[j, i] .* transpose(A[i, j], {j, i})"),
                       ("dtranspose_eltwise_dense", "transpose(A[i, j], {j, i}) .* B[j, i]")):
        P[name] = (body(lab(i=e["N"], j=e["N"]) + ten(("A", "ij", "Dense"), ("B", "ji", "Dense"), ("C", "ji", "Dense")) +
                        f"    A[i, j] = {e['a_fill']};\n    B[j, i] = {e['b_fill']};\n    C[j, i] = 0.0;\n"
                        f"    C[j, i] = {expr};\n    print(C);\n"), [])
    e = g["dense_mult_dtranspose"]
    P["dense_mult_dtranspose"] = (body(lab(i=e["N"], j=e["N"], k=e["N"]) +
                                       ten(("B", "ij", "Dense"), ("A", "kj", "Dense"), ("C", "ki", "Dense")) +
                                       f"    B[i, j] = {e['b_fill']};\n    A[k, j] = {e['a_fill']};\n    C[k, i] = 0.0;\n"
                                       "    C[k, i] = A[k, j] * transpose(B[i, j], {j, i});\n    print(C);\n"), [])
    e = g["dtranspose_mult_dense"]
    P["dtranspose_mult_dense"] = (body(lab(i=e["N"], j=e["N"], k=e["N"]) +
                                       ten(("A", "ij", "Dense"), ("B", "ik", "Dense"), ("C", "jk", "Dense")) +
                                       f"    A[i, j] = {e['a_fill']};\n    B[i, k] = {e['b_fill']};\n    C[j, k] = 0.0;\n"
                                       "    C[j, k] = transpose(A[i, j], {j, i}) * B[i, k];\n    print(C);\n"), [])
    e = g["dense_transpose_4d"]
    si, sj, sk, sl = e["sizes"]
    P["dense_transpose_4d"] = (body(lab(i=si, j=sj, k=sk, l=sl) +
                                    ten(("A", "ijkl", "Dense"), ("B", "ikjl", "Dense")) +
                                    f"    A[i, j, k, l] = {e['fill']};\n"
                                    "    B[i, k, j, l] = transpose(A[i, j, k, l], {i, k, j, l});\n    print(B);\n"), [])
    return P


_KC_NAMES = ["sddmm", "gnn", "gram_matrix", "csr_dense_chain", "csr_mult_dtranspose", "dtranspose_eltwise_csr",
             "dtranspose_mult_csr", "dense_chain", "dense_eltwise_dtranspose", "dtranspose_eltwise_dense",
             "dense_mult_dtranspose", "dtranspose_mult_dense", "dense_transpose_4d"]


@pytest.mark.parametrize("name", _KC_NAMES)
def test_kernel_and_compound_expression_programs(golden, golden_dir, tmp_path, monkeypatch, name):
    g = golden["kernels_and_compound"]
    prog, files = _kc_programs(g)[name]
    out = _run(prog, files, tmp_path, monkeypatch, golden_dir)
    _check(out, g["dense_eltwise_dtranspose" if name == "dtranspose_eltwise_dense" else name]["printed"], tmp_path)


def test_sddmm_program_never_forms_the_dense_product(golden, golden_dir, tmp_path, monkeypatch):
    """T = C x D followed by B .* T runs as one SDDMM launch; no GEMM and no dense elementwise kernel."""
    from comet_amd import runtime as rt
    g = golden["kernels_and_compound"]
    prog, files = _kc_programs(g)["sddmm"]
    rt.init(0)
    rt.profile_reset(); rt.profile_enable(True)
    _run(prog, files, tmp_path, monkeypatch, golden_dir)
    rep = rt.profile_report()
    rt.profile_enable(False)
    assert "sddmm_kernel" in rep and not any("gemm" in k or "eltwise" in k for k in rep), sorted(rep)


# ------------------------------------------------------ further dense and SUM programs of the reference's tests
def _ds_programs(g):
    lab = lambda **kw: "".join(f"    IndexLabel [{k}] = [{v}];\n" for k, v in kw.items())
    ten = lambda *decls: "".join(f"    Tensor<double> {n}([{', '.join(ls)}], {{{f}}});\n" for n, ls, f in decls)
    body = lambda text: "def main() {\n" + text + "}\n"
    P = {}
    for name, op in (("eltwise_add_dense", "+"), ("eltwise_subtract_dense", "-")):
        e = g[name]
        P[name] = (body(lab(i=e["N"], j=e["N"]) + ten(("A", "ij", "Dense"), ("B", "ij", "Dense"), ("C", "ij", "Dense")) +
                        f"    A[i, j] = {e['a']};\n    B[i, j] = {e['b']};\n    C[i, j] = 0.0;\n"
                        f"    C[i, j] = A[i, j] {op} B[i, j];\n    print(C);\n"), [])
    e = g["eltwise_mult_dense_4d"]
    P["eltwise_mult_dense_4d"] = (body(lab(a=e["N"], b=e["N"], c=e["N"], d=e["N"]) +
                                       ten(("A", "abcd", "Dense"), ("B", "abcd", "Dense"), ("C", "abcd", "Dense")) +
                                       f"    A[a, b, c, d] = {e['a']};\n    B[a, b, c, d] = {e['b']};\n"
                                       "    C[a, b, c, d] = 0.0;\n    C[a, b, c, d] = A[a, b, c, d] .* B[a, b, c, d];\n"
                                       "    print(C);\n"), [])
    e = g["dense_matvec"]
    P["dense_matvec"] = (body(lab(i=e["I"], j=e["J"]) + ten(("A", "ij", "Dense"), ("B", "j", "Dense"), ("C", "i", "Dense")) +
                              f"    A[i, j] = {e['a']};\n    B[j] = {e['b']};\n    C[i] = 0.0;\n"
                              "    C[i] = A[i, j] * B[j];\n    print(C);\n"), [])
    e = g["dense_matmul"]
    P["dense_matmul"] = (body(lab(i=e["I"], j=e["J"], k=e["K"]) +
                              ten(("A", "ij", "Dense"), ("B", "jk", "Dense"), ("C", "ik", "Dense")) +
                              f"    A[i, j] = {e['a']};\n    B[j, k] = {e['b']};\n    C[i, k] = 0.0;\n"
                              "    C[i, k] = A[i, j] * B[j, k];\n    print(C);\n"), [])
    e = g["ccsd_t1_3"]
    P["ccsd_t1_3"] = (body(f"    IndexLabel [i, c] = [{e['IC']}];\n" + lab(a=e["A"]) +
                           ten(("f", "ca", "Dense"), ("t1", "ic", "Dense"), ("i0", "ia", "Dense")) +
                           f"    f[c, a] = {e['f']};\n    t1[i, c] = {e['t1']};\n    i0[i, a] = 0.0;\n"
                           "    i0[i, a] = f[c, a] * t1[i, c];\n    print(i0);\n"), [])
    e = g["ccsd_t1_11"]
    P["ccsd_t1_11"] = (body(f"    IndexLabel [i, j, m, n] = [{e['N']}];\n    IndexLabel [a, b, c, d] = [{e['N']}];\n" +
                            ten(("i0", "ia", "Dense"), ("t1", "ia", "Dense"), ("t2", "ijab", "Dense"),
                                ("v", "abij", "Dense")) +
                            f"    i0[i, a] = 0.0;\n    t1[i, a] = {e['t1']};\n    t2[i, j, a, b] = {e['t2']};\n"
                            f"    v[i, a, j, b] = {e['v']};\n"
                            "    i0[i, a] = v[c, d, m, n] * t2[i, n, a, d] * t1[m, c];\n    print(i0[i, a]);\n"), [])
    e = g["tricount_unmasked"]
    P["tricount_unmasked"] = (body(lab(i="?", j="?", k="?") + ten(("L1", "ij", "CSR")) +
                                   f"    L1[i, j] = comet_read(0, {e['read_mode']});\n"
                                   "    var ntri = SUM(L1[i, k] * L1[k, j] .* L1[i, j]);\n    print(ntri);\n"),
                              [e["matrix"]])
    for name, idx in (("sum_dense_matrix", "ij"), ("sum_dense_tensor", "ijk")):
        e = g[name]
        ls = ", ".join(idx)
        P[name] = (body(lab(**{l: n for l, n in zip(idx, e["shape"])}) + ten(("A", idx, "Dense")) +
                        f"    A[{ls}] = {e['fill']};\n    var a = SUM(A[{ls}]);\n    print(a);\n"), [])
    e = g["sum_coo"]
    P["sum_coo"] = (body(lab(i="?", j="?") + ten(("A", "ij", "COO")) +
                         "    A[i, j] = comet_read(0);\n    var a = SUM(A[i, j]);\n    print(a);\n"), [e["matrix"]])
    e = g["transpose_dense_tensor"]
    P["transpose_dense_tensor"] = (body(lab(i=e["N"], j=e["N"], k=e["N"]) +
                                        ten(("A", "ijk", "Dense"), ("B", "kij", "Dense")) +
                                        f"    A[i, j, k] = {e['fill']};\n"
                                        "    B[k, i, j] = transpose(A[i, j, k], {k, i, j});\n    print(B);\n"), [])
    return P


_DS_NAMES = ["eltwise_add_dense", "eltwise_subtract_dense", "eltwise_mult_dense_4d", "dense_matvec", "dense_matmul",
             "ccsd_t1_3", "ccsd_t1_11", "tricount_unmasked", "sum_dense_matrix", "sum_dense_tensor", "sum_coo",
             "transpose_dense_tensor"]


@pytest.mark.parametrize("name", _DS_NAMES)
def test_dense_and_sum_programs(golden, golden_dir, tmp_path, monkeypatch, name):
    g = golden["dense_and_sum_programs"]
    prog, files = _ds_programs(g)[name]
    out = _run(prog, files, tmp_path, monkeypatch, golden_dir)
    _check(out, g[name]["printed"], tmp_path)
