// Memref-descriptor entry points: what `func.call` sites in lowered COMET host
// code bind to.  Operands are HOST memrefs, as for the reference's other runtime
// calls (lib/ExecutionEngine/StatUtils.cpp:89-113,
// lib/ExecutionEngine/blis_interface.cpp:143-146 in pnnl/COMET); each call
// uploads, runs the device kernels and copies the result back.  These return
// void like their counterparts, so a failure prints the message and exits, the
// reference's own error behaviour (lib/ExecutionEngine/HipGpuUtils.cpp:10-19).
#include <stdio.h>
#include <stdlib.h>

#include "common.h"

using namespace comet;

namespace {

[[noreturn]] void die(const char *where)
{
    fprintf(stderr, "comet_hip error in %s: %s\n", where, comet_hip_last_error());
    exit(1);
}

template <typename T>
const T *data1(const comet_memref_1d *m, const char *who)
{
    if (!m || (m->sizes[0] > 0 && !m->aligned)) {
        set_error(COMET_HIP_ERR_ARG, "null memref");
        die(who);
    }
    if (m->sizes[0] > 1 && m->strides[0] != 1) {
        set_error(COMET_HIP_ERR_ARG, "non-contiguous 1-D memref (stride %lld)", (long long)m->strides[0]);
        die(who);
    }
    return (const T *)m->aligned + m->offset;
}

struct DeviceBuf {
    int64_t p = 0;
    explicit DeviceBuf(int64_t bytes) : p(comet_hip_malloc(bytes)) {}
    ~DeviceBuf() { (void)comet_hip_free(p); }
};

// result of the "sizes" call, waiting for the "fill" call
int64_t g_pending_c = 0;

}  // namespace

void comet::forget_pending_product() { g_pending_c = 0; }

// Every entry point exists for both index widths: i64 is what the CPU lowering passes, i32 what lowered code
// built with --target=GPU passes (frontends/comet_dsl/comet.cpp:817-823 switches the index memrefs to i32).
namespace {

template <typename I>
int64_t upload(int64_t nrows, int64_t ncols, const I *pos, const I *crd, const double *val)
{
    if constexpr (sizeof(I) == 8)
        return comet_hip_csr_upload_i64(nrows, ncols, (const int64_t *)pos, (const int64_t *)crd, val);
    else
        return comet_hip_csr_upload_i32(nrows, ncols, (const int32_t *)pos, (const int32_t *)crd, val);
}

template <typename I>
void spmv_ciface(const char *who, comet_memref_1d *pos, comet_memref_1d *crd, comet_memref_1d *val,
                 comet_memref_1d *x, comet_memref_1d *y)
{
    const int64_t nrows = pos->sizes[0] - 1, ncols = x->sizes[0];
    if (nrows < 0 || y->sizes[0] != nrows) {
        set_error(COMET_HIP_ERR_ARG, "y has %lld entries, A has %lld rows", (long long)y->sizes[0], (long long)nrows);
        die(who);
    }
    int64_t a = upload<I>(nrows, ncols, data1<I>(pos, who), data1<I>(crd, who), data1<double>(val, who));
    if (!a)
        die(who);
    DeviceBuf dx(ncols * 8), dy(nrows * 8);
    if ((ncols && !dx.p) || (nrows && !dy.p))
        die(who);
    double *hy = (double *)data1<double>(y, who);
    if (comet_hip_memcpy(dx.p, (void *)data1<double>(x, who), ncols * 8, 0) ||
        comet_hip_memcpy(dy.p, hy, nrows * 8, 0) || comet_hip_spmv_csr_f64(a, dx.p, dy.p, 1) ||
        comet_hip_memcpy(dy.p, hy, nrows * 8, 1))
        die(who);
    (void)comet_hip_csr_destroy(a);
}

template <typename I>
void spmm_ciface(const char *who, comet_memref_1d *pos, comet_memref_1d *crd, comet_memref_1d *val,
                 comet_memref_2d *B, comet_memref_2d *C)
{
    if (!B || !C || !B->aligned || !C->aligned) {
        set_error(COMET_HIP_ERR_ARG, "null memref");
        die(who);
    }
    const int64_t nrows = pos->sizes[0] - 1, ncols = B->sizes[0], K = B->sizes[1];
    if (nrows < 0 || C->sizes[0] != nrows || C->sizes[1] != K || (K > 1 && (B->strides[1] != 1 || C->strides[1] != 1)) ||
        (ncols > 1 && B->strides[0] != K) || (nrows > 1 && C->strides[0] != K)) {
        set_error(COMET_HIP_ERR_ARG, "B/C must be contiguous row-major with matching shapes");
        die(who);
    }
    int64_t a = upload<I>(nrows, ncols, data1<I>(pos, who), data1<I>(crd, who), data1<double>(val, who));
    if (!a)
        die(who);
    DeviceBuf db(ncols * K * 8), dc(nrows * K * 8);
    if ((ncols * K && !db.p) || (nrows * K && !dc.p))
        die(who);
    double *hb = (double *)B->aligned + B->offset, *hc = (double *)C->aligned + C->offset;
    if (comet_hip_memcpy(db.p, hb, ncols * K * 8, 0) || comet_hip_memcpy(dc.p, hc, nrows * K * 8, 0) ||
        comet_hip_spmm_csr_f64(a, K, db.p, K, dc.p, K, 1) || comet_hip_memcpy(dc.p, hc, nrows * K * 8, 1))
        die(who);
    (void)comet_hip_csr_destroy(a);
}

template <typename I>
void spgemm_sizes_ciface(const char *who, int64_t nrowsA, int64_t ncolsB, comet_memref_1d *Apos, comet_memref_1d *Acrd,
                         comet_memref_1d *Aval, comet_memref_1d *Bpos, comet_memref_1d *Bcrd, comet_memref_1d *Bval,
                         comet_memref_1d *Mpos, comet_memref_1d *Mcrd, comet_memref_1d *sizes,
                         int reduce_op = COMET_SR_PLUS, int mult_op = COMET_OP_TIMES)
{
    const int64_t nrowsB = Bpos->sizes[0] - 1;
    if (Apos->sizes[0] - 1 != nrowsA || !sizes || sizes->sizes[0] < 1) {
        set_error(COMET_HIP_ERR_ARG, "inconsistent row counts or missing sizes memref");
        die(who);
    }
    if (g_pending_c) {
        (void)comet_hip_csr_destroy(g_pending_c);
        g_pending_c = 0;
    }
    int64_t a = upload<I>(nrowsA, nrowsB, data1<I>(Apos, who), data1<I>(Acrd, who), data1<double>(Aval, who));
    int64_t b = a ? upload<I>(nrowsB, ncolsB, data1<I>(Bpos, who), data1<I>(Bcrd, who), data1<double>(Bval, who)) : 0;
    int64_t m = 0;
    if (a && b && Mpos && Mpos->sizes[0] > 0) {
        // a mask carries structure only; its device value array is all zeros
        const int64_t mnnz = Mcrd->sizes[0];
        double *zeros = (double *)calloc((size_t)(mnnz > 0 ? mnnz : 1), sizeof(double));
        m = zeros ? upload<I>(nrowsA, ncolsB, data1<I>(Mpos, who), data1<I>(Mcrd, who), zeros) : 0;
        free(zeros);
        if (!m)
            die(who);
    }
    if (!a || !b)
        die(who);
    g_pending_c = comet_hip_spgemm_csr_semiring(a, b, m, reduce_op, mult_op);
    if (!g_pending_c)
        die(who);
    int64_t nnz = 0;
    (void)comet_hip_csr_dims(g_pending_c, nullptr, nullptr, &nnz);
    ((int64_t *)sizes->aligned + sizes->offset)[0] = nnz;       // sizes are `index` values for either width
    (void)comet_hip_csr_destroy(a);
    (void)comet_hip_csr_destroy(b);
    if (m)
        (void)comet_hip_csr_destroy(m);
}

template <typename I>
void spgemm_fill_ciface(const char *who, comet_memref_1d *Cpos, comet_memref_1d *Ccrd, comet_memref_1d *Cval)
{
    if (!g_pending_c) {
        set_error(COMET_HIP_ERR_ARG, "fill called without a preceding sizes call");
        die(who);
    }
    int64_t nrows = 0, nnz = 0;
    (void)comet_hip_csr_dims(g_pending_c, &nrows, nullptr, &nnz);
    if (Cpos->sizes[0] < nrows + 1 || Ccrd->sizes[0] < nnz || Cval->sizes[0] < nnz) {
        set_error(COMET_HIP_ERR_ARG, "output memrefs too small for %lld rows / %lld entries", (long long)nrows,
                  (long long)nnz);
        die(who);
    }
    int rc;
    if constexpr (sizeof(I) == 8)
        rc = comet_hip_csr_download_i64(g_pending_c, (int64_t *)data1<I>(Cpos, who), (int64_t *)data1<I>(Ccrd, who),
                                        (double *)data1<double>(Cval, who));
    else
        rc = comet_hip_csr_download_i32(g_pending_c, (int32_t *)data1<I>(Cpos, who), (int32_t *)data1<I>(Ccrd, who),
                                        (double *)data1<double>(Cval, who));
    if (rc)
        die(who);
    (void)comet_hip_csr_destroy(g_pending_c);
    g_pending_c = 0;
}

template <typename I>
double tricount_ciface(const char *who, int64_t ncols, comet_memref_1d *pos, comet_memref_1d *crd, comet_memref_1d *val)
{
    const int64_t nrows = pos->sizes[0] - 1;
    int64_t l = upload<I>(nrows, ncols, data1<I>(pos, who), data1<I>(crd, who), data1<double>(val, who));
    if (!l)
        die(who);
    double out = 0.0;
    if (comet_hip_spgemm_masked_sum(l, l, l, &out))
        die(who);
    (void)comet_hip_csr_destroy(l);
    return out;
}

}  // namespace

extern "C" void _mlir_ciface_comet_hip_spmv_csr_f64_i64(comet_memref_1d *pos, comet_memref_1d *crd,
                                                         comet_memref_1d *val, comet_memref_1d *x, comet_memref_1d *y)
{
    spmv_ciface<int64_t>("comet_hip_spmv_csr_f64_i64", pos, crd, val, x, y);
}
extern "C" void _mlir_ciface_comet_hip_spmv_csr_f64_i32(comet_memref_1d *pos, comet_memref_1d *crd,
                                                         comet_memref_1d *val, comet_memref_1d *x, comet_memref_1d *y)
{
    spmv_ciface<int32_t>("comet_hip_spmv_csr_f64_i32", pos, crd, val, x, y);
}

extern "C" void _mlir_ciface_comet_hip_spmm_csr_f64_i64(comet_memref_1d *pos, comet_memref_1d *crd,
                                                         comet_memref_1d *val, comet_memref_2d *B, comet_memref_2d *C)
{
    spmm_ciface<int64_t>("comet_hip_spmm_csr_f64_i64", pos, crd, val, B, C);
}
extern "C" void _mlir_ciface_comet_hip_spmm_csr_f64_i32(comet_memref_1d *pos, comet_memref_1d *crd,
                                                         comet_memref_1d *val, comet_memref_2d *B, comet_memref_2d *C)
{
    spmm_ciface<int32_t>("comet_hip_spmm_csr_f64_i32", pos, crd, val, B, C);
}

extern "C" void _mlir_ciface_comet_hip_spgemm_csr_sizes_f64_i64(
    int64_t nrowsA, int64_t ncolsB, comet_memref_1d *Apos, comet_memref_1d *Acrd, comet_memref_1d *Aval,
    comet_memref_1d *Bpos, comet_memref_1d *Bcrd, comet_memref_1d *Bval, comet_memref_1d *Mpos,
    comet_memref_1d *Mcrd, comet_memref_1d *sizes)
{
    spgemm_sizes_ciface<int64_t>("comet_hip_spgemm_csr_sizes_f64_i64", nrowsA, ncolsB, Apos, Acrd, Aval, Bpos, Bcrd,
                                 Bval, Mpos, Mcrd, sizes);
}
extern "C" void _mlir_ciface_comet_hip_spgemm_csr_sizes_f64_i32(
    int64_t nrowsA, int64_t ncolsB, comet_memref_1d *Apos, comet_memref_1d *Acrd, comet_memref_1d *Aval,
    comet_memref_1d *Bpos, comet_memref_1d *Bcrd, comet_memref_1d *Bval, comet_memref_1d *Mpos,
    comet_memref_1d *Mcrd, comet_memref_1d *sizes)
{
    spgemm_sizes_ciface<int32_t>("comet_hip_spgemm_csr_sizes_f64_i32", nrowsA, ncolsB, Apos, Acrd, Aval, Bpos, Bcrd,
                                 Bval, Mpos, Mcrd, sizes);
}

extern "C" void _mlir_ciface_comet_hip_spgemm_csr_fill_f64_i64(comet_memref_1d *Cpos, comet_memref_1d *Ccrd,
                                                                comet_memref_1d *Cval)
{
    spgemm_fill_ciface<int64_t>("comet_hip_spgemm_csr_fill_f64_i64", Cpos, Ccrd, Cval);
}
extern "C" void _mlir_ciface_comet_hip_spgemm_csr_fill_f64_i32(comet_memref_1d *Cpos, comet_memref_1d *Ccrd,
                                                                comet_memref_1d *Cval)
{
    spgemm_fill_ciface<int32_t>("comet_hip_spgemm_csr_fill_f64_i32", Cpos, Ccrd, Cval);
}

extern "C" double _mlir_ciface_comet_hip_tricount_f64_i64(int64_t ncols, comet_memref_1d *pos, comet_memref_1d *crd,
                                                           comet_memref_1d *val)
{
    return tricount_ciface<int64_t>("comet_hip_tricount_f64_i64", ncols, pos, crd, val);
}
extern "C" double _mlir_ciface_comet_hip_tricount_f64_i32(int64_t ncols, comet_memref_1d *pos, comet_memref_1d *crd,
                                                           comet_memref_1d *val)
{
    return tricount_ciface<int32_t>("comet_hip_tricount_f64_i32", ncols, pos, crd, val);
}

// The semiring forms of the SpGEMM pair of calls: C[a,c] = A[a,b] @(reduce, mult) B[b,c] with the operator codes of
// comet_hip_spgemm_csr_semiring (the DSL's names: frontends/comet_dsl/mlir/MLIRGen.cpp:101-147; the nests:
// lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:198-360).  The fill call is the plain one under a second name.
extern "C" void _mlir_ciface_comet_hip_spgemm_csr_sizes_semiring_f64_i64(
    int64_t nrowsA, int64_t ncolsB, comet_memref_1d *Apos, comet_memref_1d *Acrd, comet_memref_1d *Aval,
    comet_memref_1d *Bpos, comet_memref_1d *Bcrd, comet_memref_1d *Bval, comet_memref_1d *Mpos,
    comet_memref_1d *Mcrd, comet_memref_1d *sizes, int32_t reduce_op, int32_t mult_op)
{
    spgemm_sizes_ciface<int64_t>("comet_hip_spgemm_csr_sizes_semiring_f64_i64", nrowsA, ncolsB, Apos, Acrd, Aval,
                                 Bpos, Bcrd, Bval, Mpos, Mcrd, sizes, reduce_op, mult_op);
}
extern "C" void _mlir_ciface_comet_hip_spgemm_csr_sizes_semiring_f64_i32(
    int64_t nrowsA, int64_t ncolsB, comet_memref_1d *Apos, comet_memref_1d *Acrd, comet_memref_1d *Aval,
    comet_memref_1d *Bpos, comet_memref_1d *Bcrd, comet_memref_1d *Bval, comet_memref_1d *Mpos,
    comet_memref_1d *Mcrd, comet_memref_1d *sizes, int32_t reduce_op, int32_t mult_op)
{
    spgemm_sizes_ciface<int32_t>("comet_hip_spgemm_csr_sizes_semiring_f64_i32", nrowsA, ncolsB, Apos, Acrd, Aval,
                                 Bpos, Bcrd, Bval, Mpos, Mcrd, sizes, reduce_op, mult_op);
}
extern "C" void _mlir_ciface_comet_hip_spgemm_csr_fill_semiring_f64_i64(comet_memref_1d *Cpos, comet_memref_1d *Ccrd,
                                                                         comet_memref_1d *Cval)
{
    spgemm_fill_ciface<int64_t>("comet_hip_spgemm_csr_fill_semiring_f64_i64", Cpos, Ccrd, Cval);
}
extern "C" void _mlir_ciface_comet_hip_spgemm_csr_fill_semiring_f64_i32(comet_memref_1d *Cpos, comet_memref_1d *Ccrd,
                                                                         comet_memref_1d *Cval)
{
    spgemm_fill_ciface<int32_t>("comet_hip_spgemm_csr_fill_semiring_f64_i32", Cpos, Ccrd, Cval);
}

// ---------------------------------------------------------------------------
// Dense contraction, memref level.  The reference rewrites a contraction into
// transpose -> collapse -> matmul -> expand -> transpose on host memrefs
// (lib/Dialect/TensorAlgebra/Transforms/TCtoTTGTDyn.cpp:288-672) and, with
// -opt-matmul-mkernel, calls _mlir_ciface_linalg_matmul_viewsxs_viewsxs_viewsxs
// per tile (lib/ExecutionEngine/blis_interface.cpp:143-181).  Here one call
// takes the three tensors as they are declared and does upload -> plan ->
// transposes -> GEMM -> download.
// ---------------------------------------------------------------------------
namespace {

struct DenseView {
    double *data;
    int64_t offset, rank, elems;
    int64_t shape[8];
};

// an unranked memref (rank, pointer to StridedMemRefType<double, rank>) that must be contiguous row-major
DenseView dense_view(int64_t rank, void *desc, const char *who)
{
    DenseView v{};
    if (!desc || rank < 1 || rank > 8) {
        set_error(COMET_HIP_ERR_ARG, "tensor memref missing or of rank %lld (1..8)", (long long)rank);
        die(who);
    }
    char *p = static_cast<char *>(desc);
    v.data = *reinterpret_cast<double **>(p + sizeof(double *));
    v.offset = *reinterpret_cast<int64_t *>(p + 2 * sizeof(double *));
    const int64_t *sizes = reinterpret_cast<const int64_t *>(p + 2 * sizeof(double *) + sizeof(int64_t));
    const int64_t *strides = sizes + rank;
    v.rank = rank;
    v.elems = 1;
    for (int64_t d = rank - 1; d >= 0; --d) {
        if (sizes[d] < 0 || (sizes[d] > 1 && strides[d] != v.elems)) {
            set_error(COMET_HIP_ERR_ARG, "tensor memref is not contiguous row-major (dimension %lld: size %lld, stride %lld)",
                      (long long)d, (long long)sizes[d], (long long)strides[d]);
            die(who);
        }
        v.shape[d] = sizes[d];
        v.elems *= sizes[d];
    }
    if (v.elems > 0 && !v.data) {
        set_error(COMET_HIP_ERR_ARG, "null tensor memref");
        die(who);
    }
    return v;
}

}  // namespace

// a_lab / b_lab / c_lab: one `index` per dimension, the same number for the same index label
// (C[a,b,c,d] = A[a,e,b,f] * B[d,f,c,e]: a_lab = 0,4,1,5  b_lab = 3,5,2,4  c_lab = 0,1,2,3); beta 0 or 1.
extern "C" void _mlir_ciface_comet_hip_ttgt_contract_f64(int64_t rankA, void *A, int64_t rankB, void *B, int64_t rankC,
                                                          void *C, comet_memref_1d *a_lab, comet_memref_1d *b_lab,
                                                          comet_memref_1d *c_lab, double beta)
{
    const char *who = "comet_hip_ttgt_contract_f64";
    const DenseView a = dense_view(rankA, A, who), b = dense_view(rankB, B, who), c = dense_view(rankC, C, who);
    const int64_t *lab[3] = {data1<int64_t>(a_lab, who), data1<int64_t>(b_lab, who), data1<int64_t>(c_lab, who)};
    const DenseView *view[3] = {&a, &b, &c};
    const comet_memref_1d *lm[3] = {a_lab, b_lab, c_lab};
    // labels may be any integers: number them 0, 1, ... in order of first appearance and collect the extents
    int64_t seen[24], extent[24];
    int nlab = 0;
    int32_t ids[3][8];
    for (int t = 0; t < 3; ++t) {
        if (lm[t]->sizes[0] != view[t]->rank) {
            set_error(COMET_HIP_ERR_ARG, "operand %d has rank %lld and %lld labels", t, (long long)view[t]->rank,
                      (long long)lm[t]->sizes[0]);
            die(who);
        }
        for (int64_t d = 0; d < view[t]->rank; ++d) {
            int k = 0;
            while (k < nlab && seen[k] != lab[t][d])
                ++k;
            if (k == nlab) {
                seen[nlab] = lab[t][d];
                extent[nlab++] = view[t]->shape[d];
            } else if (extent[k] != view[t]->shape[d]) {
                set_error(COMET_HIP_ERR_ARG, "index label %lld has extents %lld and %lld", (long long)lab[t][d],
                          (long long)extent[k], (long long)view[t]->shape[d]);
                die(who);
            }
            ids[t][d] = k;
        }
    }
    comet_ttgt_plan plan;
    if (comet_hip_ttgt_plan((int32_t)a.rank, ids[0], (int32_t)b.rank, ids[1], (int32_t)c.rank, ids[2], extent, -1, &plan))
        die(who);
    DeviceBuf da(a.elems * 8), db(b.elems * 8), dc(c.elems * 8);
    if ((a.elems && !da.p) || (b.elems && !db.p) || (c.elems && !dc.p))
        die(who);
    double *hc = c.data + c.offset;
    if (comet_hip_memcpy(da.p, a.data + a.offset, a.elems * 8, 0) || comet_hip_memcpy(db.p, b.data + b.offset, b.elems * 8, 0) ||
        (beta != 0.0 && comet_hip_memcpy(dc.p, hc, c.elems * 8, 0)) ||
        comet_hip_ttgt_contract(&plan, a.shape, b.shape, c.shape, da.p, db.p, dc.p, beta) ||
        comet_hip_memcpy(dc.p, hc, c.elems * 8, 1))
        die(who);
}

// The reference's own name for the matrix product its TTGT lowering ends in (blis_interface.cpp:143-146):
// C = alpha * A * B + beta * C on strided 2-D views of host memory.  mr and nr (the micro-kernel's tile) mean
// nothing here: the whole product runs on the device, so a lowering that calls this once per contraction instead
// of once per tile is what makes sense with this library.
extern "C" void _mlir_ciface_linalg_matmul_viewsxs_viewsxs_viewsxs(comet_memref_2d *A, comet_memref_2d *B,
                                                                    comet_memref_2d *C, int mr, int nr, double alpha,
                                                                    double beta)
{
    const char *who = "linalg_matmul_viewsxs_viewsxs_viewsxs";
    (void)mr;
    (void)nr;
    if (!A || !B || !C || !A->aligned || !B->aligned || !C->aligned) {
        set_error(COMET_HIP_ERR_ARG, "null memref");
        die(who);
    }
    const int64_t M = A->sizes[0], K = A->sizes[1], N = B->sizes[1];
    if (B->sizes[0] != K || C->sizes[0] != M || C->sizes[1] != N || M < 0 || N < 0 || K < 0) {
        set_error(COMET_HIP_ERR_ARG, "matmul shapes do not agree");
        die(who);
    }
    if (M == 0 || N == 0)
        return;
    // strided views are packed on the host; alpha goes into A, a beta other than 0 or 1 into C
    auto pack = [](const comet_memref_2d *m, double scale) {
        const int64_t r = m->sizes[0], c = m->sizes[1];
        double *out = (double *)malloc(sizeof(double) * (size_t)(r * c > 0 ? r * c : 1));
        const double *in = (const double *)m->aligned + m->offset;
        if (out)
            for (int64_t i = 0; i < r; ++i)
                for (int64_t j = 0; j < c; ++j)
                    out[i * c + j] = scale * in[i * m->strides[0] + j * m->strides[1]];
        return out;
    };
    const bool plain_beta = beta == 0.0 || beta == 1.0;
    double *ha = pack(A, alpha), *hb = pack(B, 1.0), *hc = pack(C, plain_beta ? 1.0 : beta);
    DeviceBuf da(M * K * 8), db(K * N * 8), dc(M * N * 8);
    bool bad = !ha || !hb || !hc || (M * K && !da.p) || (K * N && !db.p) || !dc.p;
    bad = bad || comet_hip_memcpy(da.p, ha, M * K * 8, 0) || comet_hip_memcpy(db.p, hb, K * N * 8, 0) ||
          (beta != 0.0 && comet_hip_memcpy(dc.p, hc, M * N * 8, 0)) ||
          comet_hip_dgemm_f64(M, N, K, da.p, db.p, dc.p, beta == 0.0 ? 0.0 : 1.0) ||
          comet_hip_memcpy(dc.p, hc, M * N * 8, 1);
    if (!bad) {
        double *out = (double *)C->aligned + C->offset;
        for (int64_t i = 0; i < M; ++i)
            for (int64_t j = 0; j < N; ++j)
                out[i * C->strides[0] + j * C->strides[1]] = hc[i * N + j];
    }
    free(ha);
    free(hb);
    free(hc);
    if (bad)
        die(who);
}

// ---------------------------------------------------------------------------
// The small host utilities every lowered program calls besides the kernels, so
// that this library can be the only -shared-libs entry of a run: printing of
// memrefs in the runtime's text form, the index sort, wall-clock time.
// An unranked memref arrives as (rank, pointer to StridedMemRefType<T, rank>):
// {T *allocated; T *aligned; int64 offset; int64 sizes[rank]; int64 strides[rank]}.
// ---------------------------------------------------------------------------
#include <sys/time.h>

#include <algorithm>

namespace {

template <typename T>
struct Unranked {
    T *data;
    int64_t offset;
    const int64_t *sizes, *strides;
    int64_t rank;
    Unranked(int64_t r, void *desc) : rank(r)
    {
        char *p = static_cast<char *>(desc);
        data = *reinterpret_cast<T **>(p + sizeof(T *));                 // the aligned pointer
        offset = *reinterpret_cast<int64_t *>(p + 2 * sizeof(T *));
        sizes = reinterpret_cast<const int64_t *>(p + 2 * sizeof(T *) + sizeof(int64_t));
        strides = sizes + r;
    }
};

void print_one(double v) { printf("%g,", v); }      // an ostream's default form: six significant digits
void print_one(float v) { printf("%g,", (double)v); }
void print_one(int64_t v) { printf("%lld,", (long long)v); }
void print_one(int32_t v) { printf("%d,", v); }

template <typename T>
void print_dims(const T *base, int64_t dims_left, int64_t offset, const int64_t *sizes, const int64_t *strides)
{
    if (dims_left == 0) {
        print_one(base[offset]);
        return;
    }
    for (int64_t i = 0; i < sizes[0]; ++i)
        print_dims(base, dims_left - 1, offset + i * strides[0], sizes + 1, strides + 1);
}

// include/comet/ExecutionEngine/RunnerUtils.h:232-266: nothing for an empty first dimension, else "data = ",
// a line break, every element followed by a comma in row-major order of the strided view, a line break
template <typename T>
void print_memref(int64_t rank, void *desc)
{
    if (!desc || rank < 0)
        return;
    Unranked<T> m(rank, desc);
    if (rank > 0 && m.sizes[0] <= 0)
        return;
    printf("data = \n");
    print_dims(m.data, rank, m.offset, m.sizes, m.strides);
    printf("\n");
    fflush(stdout);
}

template <typename T>
void sort_range(int64_t rank, void *desc, int64_t first, int64_t last)
{
    if (!desc || last <= first)
        return;
    Unranked<T> m(rank, desc);
    std::sort(m.data + m.offset + first, m.data + m.offset + last);
}

}  // namespace

// lib/ExecutionEngine/StatUtils.cpp:109-137
extern "C" void comet_print_memref_f64(int64_t rank, void *ptr) { print_memref<double>(rank, ptr); }
extern "C" void comet_print_memref_f32(int64_t rank, void *ptr) { print_memref<float>(rank, ptr); }
extern "C" void comet_print_memref_i64(int64_t rank, void *ptr) { print_memref<int64_t>(rank, ptr); }
extern "C" void comet_print_memref_i32(int64_t rank, void *ptr) { print_memref<int32_t>(rank, ptr); }
extern "C" void comet_print_memref_index(int64_t rank, void *ptr) { print_memref<int64_t>(rank, ptr); }

// lib/ExecutionEngine/SparseUtils.cpp:2610-2626: ascending sort of elements [first, last) of a 1-D memref
extern "C" void comet_sort_index(int64_t rank, void *ptr, int64_t first, int64_t last)
{
    sort_range<int64_t>(rank, ptr, first, last);
}
extern "C" void comet_sort64(int64_t rank, void *ptr, int64_t first, int64_t last)
{
    sort_range<int64_t>(rank, ptr, first, last);
}
extern "C" void comet_sort32(int64_t rank, void *ptr, int64_t first, int64_t last)
{
    sort_range<int32_t>(rank, ptr, first, last);
}

// lib/ExecutionEngine/StatUtils.cpp:42-59.  Kernels here are asynchronous: the device is drained first, so that
// the interval between two calls covers the work launched between them.
extern "C" double getTime()
{
    if (is_initialised())
        (void)comet_hip_sync();
    struct timeval tp;
    if (gettimeofday(&tp, nullptr) != 0)
        fprintf(stderr, "Error returning time from gettimeofday\n");
    return (double)tp.tv_sec + (double)tp.tv_usec * 1.0e-6;
}

extern "C" void printElapsedTime(double stime, double etime)
{
    fprintf(stdout, "ELAPSED_TIME = %lf\n", etime - stime);
}
