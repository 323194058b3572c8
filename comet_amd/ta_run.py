"""Runs the hot-path subset of COMET's tensor-algebra language (.ta) on the MI355X library and prints
results in the text form the reference's runtime prints, so that the CHECK lines of the reference's
integration tests (test/integration/{ops,semiring,kernels}/*.ta in pnnl/COMET) can be verified with
FileCheck against this backend:

    SPARSE_FILE_NAME0=a.mtx python -m comet_amd.ta_run program.ta | FileCheck program.ta

It stands where `comet-opt ... | mlir-cpu-runner ...` stands in those tests' RUN lines.  It is an
interpreter over library calls, not a compiler: every statement maps to one entry point of
include/comet_hip_rt.h.  Statements it understands (frontends/comet_dsl/include/Parser.h for the grammar):

    IndexLabel [a] = [?];            IndexLabel [c] = [4];
    Tensor<double> A([a, b], {CSR}); formats Dense, CSR, COO, DCSR
    A[a, b] = comet_read(0);         A[a, b] = comet_read(0, 3);      (file id, read mode)
    B[b, c] = 1.7;                   (fill)
    C[a, c] = A[a, b] * B[b, c];     SpMV, SpMM, dense x sparse, SpGEMM, dense contraction (TTGT)
    C[a, c] = A[a, b] @(min,+) B[b, c];                               (SpGEMM over a semiring)
    C[i, k]<M, push> = A[i, j] * B[j, k];                             (masked SpGEMM)
    C[i, j] = A[i, j] .* B[i, j];    (CSR .* CSR, CSR .* Dense, Dense .* CSR)
    C[i, j] = A[i, j] @(+) B[i, j];  (elementwise monoids +, -, *, min, max: Dense x Dense, sparse x Dense)
    C[i, j] = A[i, j] + B[i, j];     C[i, j] = A[i, j] - B[i, j];     (dense)
    var n = SUM(L[i, k] * L[k, j] .* L[i, j]);                        (SUM of an expression)
    B[j, i] = transpose(A[i, j], {j, i});                             (dense)
    A[i, l] = B[i, j] * C[j, k] * D[k, l];                            (chains, evaluated left to right)
    C[k, i] = A[k, j] * transpose(B[i, j], {j, i});                   (transposed dense operands)
    T[i, j] = C[i, k] * D[k, j];  A[i, j] = B[i, j] .* T[i, j];       (SDDMM: T is never formed, as with --opt-fusion)
    var s = SUM(C[i, j]);  var t = getTime();  printElapsedTime(t0, t1);  print(C);  print(s);

Anything else raises TaError naming the statement.  Like the generated code, `C = A * B` adds into what C
holds (the reference's tests fill C with 0.0 first).
"""
import re
import sys
import time

import numpy as np

from . import runtime as rt


class TaError(RuntimeError):
    pass


def format_values(v):
    """include/comet/ExecutionEngine/RunnerUtils.h:232-266: "data = \\n", every element through an ostream
    (six significant digits) followed by a comma, then a newline; nothing at all for an empty tensor."""
    v = np.ravel(v)
    if v.size == 0:
        return ""
    if v.dtype.kind in "iu":
        body = "".join(f"{int(x)}," for x in v)
    else:
        body = "".join(f"{float(x):g}," for x in v)
    return "data = \n" + body + "\n"


_SEMIRING_TOKENS = {"+": "plus", "*": "times", "min": "min", "max": "max", "any": "any", "first": "first",
                    "second": "second", "pair": "pair", "-": "minus", "plus": "plus", "times": "times",
                    "minus": "minus", "/": "div"}
_FORMATS = {"Dense", "CSR", "COO", "DCSR"}


class _Tensor:
    def __init__(self, name, labels, fmt):
        self.name, self.labels, self.fmt = name, labels, fmt
        self.value = None        # DeviceArray (Dense) or CsrMatrix (every sparse format)
        self.zero = True         # Dense: holds zeros only (never written, or filled with 0.0)
        self.pending = None      # Dense: (C, D) of a product C x D that has not been formed yet


class Program:
    def __init__(self, out=sys.stdout):
        self.extent = {}         # index label -> size or None (the '?' of the language)
        self.order = []          # index labels in declaration order
        self.tensors = {}
        self.scalars = {}
        self.out = out

    # ------------------------------------------------------------------ helpers
    def _labels(self, text):
        labs = [t.strip() for t in text.split(",") if t.strip()]
        for l in labs:
            if l not in self.extent:
                raise TaError(f"index label {l} is not declared")
        return labs

    def _tensor(self, name):
        if name not in self.tensors:
            raise TaError(f"tensor {name} is not declared")
        return self.tensors[name]

    def _shape(self, labels):
        shape = []
        for l in labels:
            if self.extent[l] is None:
                raise TaError(f"the size of index {l} is not known yet (it is set by reading a sparse tensor)")
            shape.append(self.extent[l])
        return shape

    def _bind(self, labels, shape):
        for l, n in zip(labels, shape):
            if self.extent[l] is None:
                self.extent[l] = int(n)
            elif self.extent[l] != n:
                raise TaError(f"index {l} has size {self.extent[l]} but the tensor has {n}")

    def _dense(self, t):
        if t.pending is not None:           # someone needs all of it after all
            cm, d = t.pending
            t.pending = None
            t.value = rt.dgemm(self._dense(cm), self._dense(d))
            t.zero = False
        if t.value is None:       # declared, never filled: the reference allocates without initialising
            t.value = rt.DeviceArray(self._shape(t.labels), zero=True)
        return t.value

    def _written(self, t):
        t.zero = False
        t.pending = None

    def _sparse(self, t):
        if t.value is None:
            raise TaError(f"sparse tensor {t.name} is used before it is read or computed")
        return t.value

    # ------------------------------------------------------------------ statements
    def run(self, text):
        body = re.sub(r"#[^\n]*", "", text)
        m = re.search(r"def\s+main\s*\(\s*\)\s*\{(.*)\}", body, re.S)
        if not m:
            raise TaError("no `def main() { ... }`")
        for stmt in m.group(1).split(";"):
            stmt = " ".join(stmt.split())
            if stmt:
                self._statement(stmt)

    def _statement(self, s):
        for pattern, handler in self._RULES:
            m = re.fullmatch(pattern, s)
            if m:
                return handler(self, *m.groups())
        raise TaError(f"statement not supported by this runner: {s}")

    def _index_label(self, names, size):
        for name in (n.strip() for n in names.split(",")):
            self.extent[name] = None if size == "?" else int(size)
            if name not in self.order:
                self.order.append(name)

    def _declare(self, name, labels, fmt):
        if fmt not in _FORMATS:
            raise TaError(f"tensor format {fmt} is not supported by this runner")
        self.tensors[name] = _Tensor(name, self._labels(labels), fmt)

    def _read(self, name, labels, file_id, mode):
        t = self._tensor(name)
        if t.fmt == "Dense" or len(t.labels) != 2:
            raise TaError("comet_read is supported for sparse matrices")
        t.value = rt.CsrMatrix.from_file_id(int(file_id), int(mode) if mode else 1)
        self._bind(t.labels, t.value.shape)

    def _fill(self, name, labels, value):
        t = self._tensor(name)
        if t.fmt != "Dense":
            raise TaError("only dense tensors can be filled with a constant")
        t.value = rt.DeviceArray.from_numpy(np.full(self._shape(t.labels), float(value)))
        t.zero = float(value) == 0.0
        t.pending = None

    _OPERAND = re.compile(r"\s*(?:transpose\(\s*(\w+)\s*\[([^\]]*)\]\s*,\s*\{([^}]*)\}\s*\)|(\w+)\s*\[([^\]]*)\])\s*")
    _OPERATOR = re.compile(r"(\.\*|\*|\+|-|@\(\s*([^,()]+?)\s*(?:,\s*([^,()]+?)\s*)?\))")

    def _temp(self, labels, fmt):
        t = _Tensor(f"%t{len(self.tensors)}", labels, fmt)
        self.tensors[t.name] = t
        return t

    def _assign(self, cname, clabels, mask, mode, rhs):
        """C[...] = operand (operator operand)*: transposed operands become dense temporaries, a chain is
        evaluated left to right through temporaries (frontends/comet_dsl/mlir/MLIRGen.cpp builds the same
        left-leaning tree), and the last operation writes C."""
        operands, operators, at = [], [], 0
        while True:
            m = self._OPERAND.match(rhs, at)
            if not m:
                raise TaError(f"cannot read the expression: {rhs}")
            if m.group(1):          # transpose(A[..], {..})
                a = self._tensor(m.group(1))
                al, order = self._labels(m.group(2)), self._labels(m.group(3))
                if a.fmt != "Dense" or sorted(al) != sorted(order):
                    raise TaError("transpose inside an expression is supported for dense tensors")
                t = self._temp(order, "Dense")
                t.value = rt.transpose(self._dense(a), [al.index(l) for l in order])
                t.zero = False
                operands.append((t.name, ", ".join(order)))
            else:
                operands.append((m.group(4), m.group(5)))
            at = m.end()
            if at == len(rhs):
                break
            m = self._OPERATOR.match(rhs, at)
            if not m:
                raise TaError(f"cannot read the expression: {rhs}")
            operators.append(m.groups())
            at = m.end()
        if len(operands) < 2:
            raise TaError(f"statement not supported by this runner: {cname}[{clabels}] = {rhs}")
        cl = self._labels(clabels)
        while len(operands) > 2:
            (an, als), (bn, bls) = operands[0], operands[1]
            a, b = self._tensor(an), self._tensor(bn)
            al, bl = self._labels(als), self._labels(bls)
            later = set(cl)
            for _, ls in operands[2:]:
                later.update(self._labels(ls))
            op = operators[0]
            if op[0] == "*" or (op[1] is not None and op[2] is not None):
                tl = [l for l in al if l not in bl or l in later] + [l for l in bl if l not in al]
            else:
                tl = al
            fmt = "Dense" if "Dense" in (a.fmt, b.fmt) else "CSR"
            t = self._temp(tl, fmt)
            self._product(t.name, ", ".join(tl), None, None, an, als, *op, bn, bls)
            operands[:2] = [(t.name, ", ".join(tl))]
            operators.pop(0)
        (an, als), (bn, bls) = operands
        self._product(cname, clabels, mask, mode, an, als, *operators[0], bn, bls)

    def _product(self, cname, clabels, mask, _mode, aname, alabels, op, red, mul, bname, blabels):
        c, a, b = self._tensor(cname), self._tensor(aname), self._tensor(bname)
        al, bl, cl = self._labels(alabels), self._labels(blabels), self._labels(clabels)
        semiring = None
        if red is not None and mul is not None:
            try:
                semiring = (_SEMIRING_TOKENS[red.strip()], _SEMIRING_TOKENS[mul.strip()])
            except KeyError:
                raise TaError(f"semiring @({red},{mul}) is not supported") from None
        if op in (".*", "+", "-") or (red is not None and mul is None):
            # `.*`, `+`, `-`, or the monoid form A @(op) B with a single operator
            if op in (".*", "+", "-"):
                ew = {".*": "times", "+": "plus", "-": "minus"}[op]
            else:
                if red.strip() not in _SEMIRING_TOKENS:
                    raise TaError(f"elementwise operator @({red}) is not supported")
                ew = _SEMIRING_TOKENS[red.strip()]
            if not (al == bl == cl):
                raise TaError("elementwise operations need the same indices on every tensor")
            if a.fmt == b.fmt == c.fmt == "Dense":
                c.value = rt.eltwise_dense(self._dense(a), self._dense(b), op=ew)
                self._written(c)
                return
            if len(al) != 2:
                raise TaError("sparse elementwise operations are supported for matrices")
            if a.fmt == b.fmt == c.fmt == "CSR" and ew == "times":
                c.value = rt.eltwise_mult(self._sparse(a), self._sparse(b))
                return
            sp_, de_ = (a, b) if a.fmt != "Dense" else (b, a)
            commutes = ew in ("times", "plus", "min", "max")
            if sp_.fmt != "Dense" and de_.fmt == "Dense" and (sp_ is a or commutes) and c.fmt in (sp_.fmt, "Dense"):
                S = self._sparse(sp_)
                self._bind(al, S.shape)
                if de_.pending is not None and ew == "times" and c.fmt != "Dense":
                    cm, d = de_.pending          # B .* (C x D): only the sampled entries are computed
                    c.value = rt.sddmm(S, self._dense(cm), self._dense(d))
                    return
                if c.fmt == "Dense":
                    self._written(c)
                if c.fmt != "Dense":
                    c.value = rt.eltwise_csr_dense(S, self._dense(de_), op=ew)
                else:
                    rt.eltwise_csr_dense(S, self._dense(de_), self._dense(c), op=ew)
                return
            raise TaError("elementwise operations are supported for Dense x Dense, CSR .* CSR -> CSR and "
                          "sparse x Dense -> the sparse format or Dense")
        if a.fmt == "Dense" and b.fmt != "Dense" and c.fmt == "Dense":
            if semiring not in (None, ("plus", "times")) or mask:
                raise TaError("semirings and masks are supported for sparse x sparse products")
            Bm = self._sparse(b)
            self._bind(bl, Bm.shape)
            self._written(c)
            if len(bl) == 2 and al == [bl[0]] and cl == [bl[1]]:
                rt.vecmat(self._dense(a), Bm, self._dense(c), accumulate=True)
            elif len(bl) == 2 and len(al) == 2 and al[1] == bl[0] and cl == [al[0], bl[1]]:
                rt.densemat(self._dense(a), Bm, self._dense(c), accumulate=True)
            else:
                raise TaError("dense x sparse is supported as C[b] = A[a]*B[a,b] and C[a,c] = A[a,b]*B[b,c]")
            return
        if a.fmt != "Dense" and b.fmt == "Dense" and c.fmt == "Dense":
            if semiring not in (None, ("plus", "times")) or mask:
                raise TaError("semirings and masks are supported for sparse x sparse products")
            A = self._sparse(a)
            self._bind(al, A.shape)
            self._written(c)
            if len(al) == 2 and bl == [al[1]] and cl == [al[0]]:
                rt.spmv(A, self._dense(b), self._dense(c), accumulate=True)
            elif len(al) == 2 and len(bl) == 2 and bl[0] == al[1] and cl == [al[0], bl[1]]:
                rt.spmm(A, self._dense(b), self._dense(c), accumulate=True)
            else:
                raise TaError("sparse x dense is supported as C[a] = A[a,b]*B[b] and C[a,c] = A[a,b]*B[b,c]")
            return
        if a.fmt != "Dense" and b.fmt != "Dense" and c.fmt != "Dense":
            if not (len(al) == 2 and len(bl) == 2 and bl[0] == al[1] and cl == [al[0], bl[1]]):
                raise TaError("sparse x sparse is supported as C[a,c] = A[a,b]*B[b,c]")
            m = self._sparse(self._tensor(mask)) if mask else None
            c.value = rt.spgemm(self._sparse(a), self._sparse(b), mask=m, semiring=semiring)
            self._bind(cl, c.value.shape)
            return
        if a.fmt == b.fmt == c.fmt == "Dense":
            if semiring not in (None, ("plus", "times")) or mask:
                raise TaError("dense contractions are plus-times and unmasked")
            if (len(al) == len(bl) == 2 and al[1] == bl[0] and cl == [al[0], bl[1]] and c.zero
                    and c.pending is None and a is not c and b is not c):
                # a matrix product into zeros: left unformed until something reads it; `S .* T` with a sparse S
                # then computes the sampled entries only (the reference's --opt-fusion does this to SDDMM)
                c.pending = (a, b)
                c.value = None
                return
            self._dense(c)
            self._written(c)
            # one character per label, numbered as the front end does: by first appearance in A, B, C
            names = {}
            for l in al + bl + cl:
                names.setdefault(l, chr(ord("a") + len(names)))
            sa, sb, sc = ("".join(names[l] for l in ls) for ls in (al, bl, cl))
            rt.ttgt_contract(sa, sb, sc, self._dense(a), self._dense(b), self._dense(c), beta=1.0)
            return
        raise TaError(f"this combination of formats is not supported: {a.fmt} x {b.fmt} -> {c.fmt}")

    def _transpose(self, bname, blabels, aname, alabels, order):
        a, b = self._tensor(aname), self._tensor(bname)
        if a.fmt != "Dense" or b.fmt != "Dense":
            raise TaError("transpose is supported for dense tensors")
        al, bl = self._labels(alabels), self._labels(blabels)
        if self._labels(order) != bl or sorted(al) != sorted(bl):
            raise TaError("the index list of transpose must be the output's")
        b.value = rt.transpose(self._dense(a), [al.index(l) for l in bl])
        self._written(b)

    def _sum(self, var, name, _labels):
        t = self._tensor(name)
        self.scalars[var] = rt.reduce_sum(self._dense(t)) if t.fmt == "Dense" else rt.sum_values(self._sparse(t))

    def _sum_of(self, var, expr):
        """var s = SUM(A[i,k] * B[k,j] .* C[i,j]): the expression goes into a temporary that takes the indices
        and the format of its last operand (kernels/triangleCount_SandiaLL.ta:32), then its values are added."""
        last = None
        for m in self._OPERAND.finditer(expr):
            last = m
        if last is None or last.group(4) is None:
            raise TaError(f"cannot read the expression: {expr}")
        labels = self._labels(last.group(5))
        t = self._temp(labels, self._tensor(last.group(4)).fmt)
        self._assign(t.name, ", ".join(labels), None, None, expr)
        self._sum(var, t.name, None)

    def _get_time(self, var):
        rt.sync()
        self.scalars[var] = time.perf_counter()

    def _elapsed(self, t0, t1):
        self.out.write("ELAPSED_TIME = %f\n" % (self.scalars[t1] - self.scalars[t0]))

    def _print(self, name):
        if name in self.scalars:
            self.out.write(format_values(np.array([self.scalars[name]])))
            return
        t = self._tensor(name)
        if t.fmt == "Dense":
            self.out.write(format_values(self._dense(t).to_numpy()))
            return
        A = self._sparse(t)
        unused = np.array([-1], dtype=np.int64)
        if t.fmt == "CSR":      # A1pos holds the row count, A1crd is unused (SparseUtils.cpp:1898-1936)
            pos, crd, val = A.to_arrays()
            parts = [np.array([A.shape[0]], dtype=np.int64), unused, pos, crd, val]
        elif t.fmt == "COO":
            row, col, val = A.to_coo()
            parts = [np.array([0, len(val)], dtype=np.int64), row, unused, col, val]
        else:
            parts = list(A.to_dcsr())
        for p in parts:
            self.out.write(format_values(p))

    _IDX = r"\[([^\]]*)\]"
    _RULES = [
        (r"IndexLabel\s*\[\s*(\w+(?:\s*,\s*\w+)*)\s*\]\s*=\s*\[\s*(\?|\d+)\s*\]", _index_label),
        (r"Tensor\s*<\s*double\s*>\s*(\w+)\s*\(\s*\[([^\]]*)\]\s*,\s*\{?\s*(\w+)\s*\}?\s*\)", _declare),
        (r"(\w+)\s*" + _IDX + r"\s*=\s*comet_read\(\s*(\d+)\s*(?:,\s*(\d+)\s*)?\)", _read),
        (r"(\w+)\s*" + _IDX + r"\s*=\s*([-+]?[0-9.]+(?:[eE][-+]?\d+)?)", _fill),
        (r"(\w+)\s*" + _IDX + r"\s*=\s*transpose\(\s*(\w+)\s*" + _IDX + r"\s*,\s*\{([^}]*)\}\s*\)", _transpose),
        (r"(\w+)\s*" + _IDX + r"\s*(?:<\s*(\w+)\s*,\s*(\w+)\s*>)?\s*=\s*(.+)", _assign),
        (r"var\s+(\w+)\s*=\s*SUM\(\s*(\w+)\s*" + _IDX + r"\s*\)", _sum),
        (r"var\s+(\w+)\s*=\s*SUM\(\s*(.+)\)", _sum_of),
        (r"var\s+(\w+)\s*=\s*getTime\(\s*\)", _get_time),
        (r"printElapsedTime\(\s*(\w+)\s*,\s*(\w+)\s*\)", _elapsed),
        (r"print\(\s*(\w+)\s*(?:\[[^\]]*\]\s*)?\)", _print),
    ]


def run_text(text, out=sys.stdout):
    rt.init(0)
    prog = Program(out)
    prog.run(text)
    rt.sync()
    return prog


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if len(argv) != 1:
        sys.exit("usage: python -m comet_amd.ta_run program.ta   (inputs through SPARSE_FILE_NAME<id>)")
    with open(argv[0]) as f:
        run_text(f.read())


if __name__ == "__main__":
    main()
