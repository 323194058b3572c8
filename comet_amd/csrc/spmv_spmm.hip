// CSR SpMV and CSR SpMM for gfx950.
//
// Both kernels add products in ascending nonzero order with an unfused
// multiply then add, the order and arithmetic of the loop nests the reference
// generates (lib/Conversion/IndexTreeToSCF/IndexTreeToSCF.cpp:529-621 row
// loop, :667-700 nonzero loop, :476-489 dense inner loop, :1247-1284
// lhs = lhs + a*b), so a row handled by one wavefront reproduces the CPU
// result bit for bit.  This file is compiled with -ffp-contract=off.
#include <stdlib.h>

#include <algorithm>

#include "common.h"

namespace comet {

__device__ inline double readlane_f64(double v, int lane)
{
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __builtin_amdgcn_readlane(lo, lane);
    hi = __builtin_amdgcn_readlane(hi, lane);
    return __hiloint2double(hi, lo);
}

// ============================================================================
// SpMV: 256 rows per workgroup, one lane per row.  The workgroup streams the
// contiguous nonzero range of its rows through LDS in passes of SPMV_PASS
// products: all lanes compute val*x[crd] with coalesced loads of crd/val,
// then each lane adds the slice of the pass that belongs to its row, in
// order.  HBM traffic is the compulsory one (crd, val, pos once; x gathered).
// ============================================================================
#ifndef COMET_SPMV_T
#define COMET_SPMV_T 256
#endif
#ifndef COMET_SPMV_PASS
#define COMET_SPMV_PASS 2048
#endif
constexpr int SPMV_T = COMET_SPMV_T;         // rows (= lanes) per workgroup
constexpr int SPMV_PASS = COMET_SPMV_PASS;   // products staged in LDS per pass

template <bool ACC>
__global__ __launch_bounds__(SPMV_T) void spmv_csr_stream(const int64_t *__restrict__ pos,
                                                          const int32_t *__restrict__ crd,
                                                          const double *__restrict__ val,
                                                          const double *__restrict__ x,
                                                          double *__restrict__ y, int64_t nrows)
{
    __shared__ double prod[SPMV_PASS];
    const int tid = threadIdx.x;
    const int64_t r0 = (int64_t)blockIdx.x * SPMV_T;
    const int64_t r = r0 + tid;
    const int64_t rlast = r0 + SPMV_T < nrows ? r0 + SPMV_T : nrows;
    const int64_t ps = pos[r < nrows ? r : nrows];
    const int64_t pe = pos[r + 1 < nrows ? r + 1 : nrows];
    const int64_t bs = pos[r0], be = pos[rlast];
    double acc = 0.0;
    if (ACC && r < nrows)
        acc = y[r];
    for (int64_t cs = bs; cs < be; cs += SPMV_PASS) {
        const int64_t ce = cs + SPMV_PASS < be ? cs + SPMV_PASS : be;
        for (int64_t i = cs + tid; i < ce; i += SPMV_T)
            prod[i - cs] = val[i] * x[crd[i]];
        __syncthreads();
        const int64_t lo = ps > cs ? ps : cs, hi = pe < ce ? pe : ce;
        for (int64_t p = lo; p < hi; ++p)
            acc = acc + prod[p - cs];
        __syncthreads();
    }
    if (r < nrows)
        y[r] = acc;
}

// ----------------------------------------------------------------------------
// Column-blocked plan for SpMV.  The gather of x has no locality: with x larger
// than an L2 (4 MiB per XCD) every nonzero moves a cache line across the
// fabric.  The plan re-stores A as NB column blocks whose slice of x (<= 2 MiB)
// stays in L2, and SpMV runs one pass per block.  Pass b starts each row's
// accumulator from the y that pass b-1 left, and columns ascend inside a row,
// so the additions happen in exactly the original nonzero order: the result is
// still bit-identical to the sequential loop nest.
// ----------------------------------------------------------------------------
constexpr int SPMV_MAX_BLOCKS = 16;
// Measured on the 10^6 x 10^6 Poisson(10) matrix (x = 8 MB), ms per SpMV: one pass 0.115, slices of
// 4 MiB (2 passes) 0.075, 2 MiB (4 passes) 0.077, 1 MiB (8) 0.099, 512 KiB (16) 0.140.
constexpr int64_t SPMV_SLICE_BYTES = 2 << 20;

__device__ inline int64_t lower_bound_col(const int32_t *__restrict__ crd, int64_t lo, int64_t hi, int64_t col)
{
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (crd[mid] < col)
            lo = mid + 1;
        else
            hi = mid;
    }
    return lo;
}

// cnt[b * nrows + r] = nonzeros of row r with column in block b
__global__ void spmv_split_count(const int64_t *__restrict__ pos, const int32_t *__restrict__ crd, int64_t nrows,
                                 int nb, int64_t block_cols, int64_t *__restrict__ cnt)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= nrows)
        return;
    const int64_t s = pos[r], e = pos[r + 1];
    int64_t prev = s;
    for (int b = 0; b < nb; ++b) {
        const int64_t next = b + 1 < nb ? lower_bound_col(crd, prev, e, (int64_t)(b + 1) * block_cols) : e;
        cnt[(int64_t)b * nrows + r] = next - prev;
        prev = next;
    }
}

struct SpmvBases { int64_t v[SPMV_MAX_BLOCKS]; };

__global__ void spmv_split_scatter(const int64_t *__restrict__ pos, const int32_t *__restrict__ crd,
                                   const double *__restrict__ val, int64_t nrows, int nb, int64_t block_cols,
                                   const int64_t *__restrict__ bpos, SpmvBases base, int32_t *__restrict__ bcrd,
                                   double *__restrict__ bval)
{
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= nrows)
        return;
    int64_t p = pos[r];
    for (int b = 0; b < nb; ++b) {
        const int64_t *bp = bpos + (int64_t)b * (nrows + 1);
        const int64_t o = base.v[b] + bp[r], n = bp[r + 1] - bp[r];
        for (int64_t t = 0; t < n; ++t) {
            bcrd[o + t] = crd[p + t];
            bval[o + t] = val[p + t];
        }
        p += n;
    }
}

static Workspace g_spmv_cnt;

static int spmv_plan(Csr *a)
{
    if (a->spmv_nb > 0)
        return COMET_HIP_OK;
    int nb = 1;
    const int64_t slice_bytes = SPMV_SLICE_BYTES;
    if (a->ncols * 8 > slice_bytes + slice_bytes / 2 && a->nnz >= (1 << 20)) {
        nb = (int)std::min<int64_t>(SPMV_MAX_BLOCKS, ceil_div(a->ncols * 8, slice_bytes));
    }
    if (nb <= 1) {
        a->spmv_nb = 1;
        return COMET_HIP_OK;
    }
    const int64_t n = a->nrows, block_cols = ceil_div(a->ncols, nb);
    COMET_CHK(g_spmv_cnt.ensure(sizeof(int64_t) * (size_t)nb * (size_t)n, false));
    int64_t *cnt = (int64_t *)g_spmv_cnt.ptr;
    int64_t *bpos = nullptr;
    int32_t *bcrd = nullptr;
    double *bval = nullptr;
    COMET_HIPCHK(hipMalloc((void **)&bpos, sizeof(int64_t) * (size_t)nb * (size_t)(n + 1)));
    auto cleanup = [&]() {
        (void)hipFree(bpos);
        (void)hipFree(bcrd);
        (void)hipFree(bval);
    };
    const dim3 grid((unsigned)ceil_div(n, 256)), block(256);
    {
        KernelTimer t("spmv_split_count");
        spmv_split_count<<<grid, block, 0, stream()>>>(a->pos, a->crd, n, nb, block_cols, cnt);
    }
    SpmvBases base;
    std::vector<int64_t> totals(nb);
    for (int b = 0; b < nb; ++b) {
        int rc = exclusive_scan_i64(cnt + (int64_t)b * n, n, bpos + (int64_t)b * (n + 1));
        if (rc != COMET_HIP_OK) {
            cleanup();
            return rc;
        }
    }
    for (int b = 0; b < nb; ++b) {
        if (hipMemcpyAsync(&totals[b], bpos + (int64_t)b * (n + 1) + n, sizeof(int64_t), hipMemcpyDeviceToHost,
                           stream()) != hipSuccess) {
            cleanup();
            return set_error(COMET_HIP_ERR_HIP, "reading block sizes failed");
        }
    }
    if (hipStreamSynchronize(stream()) != hipSuccess) {
        cleanup();
        return set_error(COMET_HIP_ERR_HIP, "SpMV plan synchronisation failed");
    }
    int64_t run = 0;
    a->spmv_base.assign(nb, 0);
    for (int b = 0; b < nb; ++b) {
        base.v[b] = run;
        a->spmv_base[b] = run;
        run += totals[b];
    }
    // the blocks cut every row into consecutive segments, so they always hold all nonzeros, in order
    if (hipMalloc((void **)&bcrd, sizeof(int32_t) * (size_t)a->nnz) != hipSuccess ||
        hipMalloc((void **)&bval, sizeof(double) * (size_t)a->nnz) != hipSuccess) {
        cleanup();
        return set_error(COMET_HIP_ERR_HIP, "allocating the column-blocked copy failed");
    }
    {
        KernelTimer t("spmv_split_scatter");
        spmv_split_scatter<<<grid, block, 0, stream()>>>(a->pos, a->crd, a->val, n, nb, block_cols, bpos, base, bcrd,
                                                         bval);
    }
    if (hipGetLastError() != hipSuccess) {
        cleanup();
        return set_error(COMET_HIP_ERR_HIP, "SpMV plan kernel launch failed");
    }
    a->spmv_bpos = bpos;
    a->spmv_bcrd = bcrd;
    a->spmv_bval = bval;
    a->spmv_nb = nb;
    return COMET_HIP_OK;
}

// ============================================================================
// SpMM, nonzero-split: the nonzeros of A are cut into chunks of SPMM_CH and one
// wavefront owns each chunk, whatever rows it covers, so Zipf-distributed row
// lengths cost nothing in balance.  Lane l owns dense column (tile*64 + l): a
// gather of one B row is a single coalesced 512-byte load, issued SPMM_U deep
// before the dependent adds.  Rows that lie inside one chunk are finished by
// that wavefront in nonzero order.  A row cut by a chunk boundary leaves its
// pieces in `carry` (two 64-wide slots per chunk: [0] a piece whose row began
// in an earlier chunk, [1] a piece whose row goes on into the next) and the
// fix-up kernel adds the pieces in chunk order.
// ============================================================================
#ifndef COMET_SPMM_CH
#define COMET_SPMM_CH 256
#endif
#ifndef COMET_SPMM_U
#define COMET_SPMM_U 16
#endif
#ifndef COMET_SPMM_WAVES
#define COMET_SPMM_WAVES 4
#endif
constexpr int SPMM_CH = COMET_SPMM_CH;        // nonzeros per wavefront
constexpr int SPMM_U = COMET_SPMM_U;          // B-row loads in flight per wavefront
constexpr int SPMM_WAVES = COMET_SPMM_WAVES;  // wavefronts per workgroup

// chunk_row[c] = the row r with pos[r] <= c*SPMM_CH < pos[r+1]
__global__ void spmm_chunk_rows(const int64_t *__restrict__ pos, int64_t nrows, int64_t nchunks,
                                int32_t *__restrict__ chunk_row)
{
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= nchunks)
        return;
    const int64_t target = c * SPMM_CH;
    int64_t lo = 0, hi = nrows;   // first index in pos[0..nrows] with pos > target lies in [1, nrows]
    while (lo < hi) {
        int64_t mid = (lo + hi) >> 1;
        if (pos[mid + 1] > target)
            hi = mid;
        else
            lo = mid + 1;
    }
    chunk_row[c] = (int32_t)lo;
}

template <bool ACC>
__global__ __launch_bounds__(SPMM_WAVES * 64) void spmm_csr_nnzsplit(
    const int64_t *__restrict__ pos, const int32_t *__restrict__ crd, const double *__restrict__ val,
    int64_t nnz, int64_t nrows, const int32_t *__restrict__ chunk_row, int64_t nchunks,
    const double *__restrict__ B, int64_t ldb, double *__restrict__ C, int64_t ldc, int64_t K,
    double *__restrict__ carry)
{
    const int lane = threadIdx.x & 63;
    const int64_t chunk =
        (int64_t)blockIdx.x * SPMM_WAVES + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (chunk >= nchunks)
        return;
    const int64_t col = (int64_t)blockIdx.y * 64 + lane;
    const bool active = col < K;
    const int64_t s = chunk * SPMM_CH;
    const int64_t e = s + SPMM_CH < nnz ? s + SPMM_CH : nnz;
    int64_t r = __builtin_amdgcn_readfirstlane(chunk_row[chunk]);
    int64_t rend = pos[r + 1];
    const bool head = pos[r] < s;      // the first row of this chunk began earlier
    bool first_piece = true;
    bool open = false;                 // the current row has consumed nonzeros of this chunk
    double *carry0 = carry + (((int64_t)blockIdx.y * nchunks + chunk) * 2) * 64;

    // rows in front of the first stored nonzero are empty: chunk 0 clears them
    if (!ACC && chunk == 0 && active)
        for (int64_t z = 0; z < r; ++z)
            C[z * ldc + col] = 0.0;

    double acc = 0.0;
    // a row that goes on past this chunk leaves its C value to the fix-up kernel
    if (ACC && !head && rend <= e && active)
        acc = C[r * ldc + col];

    for (int64_t base = s; base < e; base += 64) {
        const int cnt = (int)(e - base < 64 ? e - base : 64);
        int my_crd = 0;
        double my_val = 0.0;
        if (lane < cnt) {      // A is streamed once: keep it from displacing B in the caches
            my_crd = __builtin_nontemporal_load(crd + base + lane);
            my_val = __builtin_nontemporal_load(val + base + lane);
        }
        for (int t0 = 0; t0 < cnt; t0 += SPMM_U) {
            double b[SPMM_U];
#pragma unroll
            for (int u = 0; u < SPMM_U; ++u) {
                b[u] = 0.0;
                if (t0 + u < cnt) {
                    const int64_t j = __builtin_amdgcn_readlane(my_crd, t0 + u);
                    if (active)
                        b[u] = B[j * ldb + col];
                }
            }
#pragma unroll
            for (int u = 0; u < SPMM_U; ++u) {
                if (t0 + u < cnt) {
                    const double a = readlane_f64(my_val, t0 + u);
                    const double prod = a * b[u];
                    acc = acc + prod;
                    open = true;
                    const int64_t p = base + t0 + u + 1;
                    bool holds = true;           // the first turn closes a row that holds nonzeros
                    while (p == rend) {          // row r is complete; also walks over empty rows that follow
                        if (active && (holds || !ACC)) {     // accumulating leaves empty rows untouched
                            if (first_piece && head)
                                carry0[lane] = acc;
                            else     // C is written once and not read again by this kernel
                                __builtin_nontemporal_store(acc, C + r * ldc + col);
                        }
                        first_piece = false;
                        open = false;
                        holds = false;
                        ++r;
                        if (r >= nrows)
                            break;
                        rend = pos[r + 1];
                        acc = 0.0;
                        // a row that starts here and ends later keeps its C value for the fix-up instead
                        if (ACC && active && rend > p && rend <= e)
                            acc = C[r * ldc + col];
                    }
                }
            }
        }
    }
    if (open && active) {                // the last row goes on into the next chunk
        if (first_piece && head)
            carry0[lane] = acc;
        else
            carry0[64 + lane] = acc;
    }
}

// One wavefront per chunk: if a row that began in an earlier chunk ends in this
// one, add its pieces in chunk order and write the row.
template <bool ACC>
__global__ __launch_bounds__(SPMM_WAVES * 64) void spmm_csr_fixup(
    const int64_t *__restrict__ pos, int64_t nnz, const int32_t *__restrict__ chunk_row, int64_t nchunks,
    double *__restrict__ C, int64_t ldc, int64_t K, const double *__restrict__ carry)
{
    const int lane = threadIdx.x & 63;
    const int64_t chunk =
        (int64_t)blockIdx.x * SPMM_WAVES + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (chunk >= nchunks)
        return;
    const int64_t col = (int64_t)blockIdx.y * 64 + lane;
    if (col >= K)
        return;
    const int64_t s = chunk * SPMM_CH;
    const int64_t e = s + SPMM_CH < nnz ? s + SPMM_CH : nnz;
    const int64_t r = __builtin_amdgcn_readfirstlane(chunk_row[chunk]);
    const int64_t rs = pos[r], re = pos[r + 1];
    if (rs >= s || re > e)
        return;
    const int64_t c0 = rs / SPMM_CH;
    const double *cb = carry + ((int64_t)blockIdx.y * nchunks * 2) * 64;
    double acc = cb[(c0 * 2 + 1) * 64 + lane];
    if (ACC)
        acc = C[r * ldc + col] + acc;
    for (int64_t c = c0 + 1; c <= chunk; ++c)
        acc = acc + cb[(c * 2) * 64 + lane];
    C[r * ldc + col] = acc;
}

__global__ void fill_rows_f64(double *__restrict__ C, int64_t nrows, int64_t K, int64_t ldc, double v)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t total = nrows * K;
    int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < total; i += step)
        C[(i / K) * ldc + (i % K)] = v;
}

static Workspace g_spmm_carry;

static int spmm_plan(Csr *a)
{
    const int64_t nchunks = ceil_div(a->nnz, SPMM_CH);
    if (a->spmm_chunk_row && a->spmm_nchunks == nchunks)
        return COMET_HIP_OK;
    if (a->spmm_chunk_row) {
        COMET_HIPCHK(hipFree(a->spmm_chunk_row));
        a->spmm_chunk_row = nullptr;
    }
    COMET_HIPCHK(hipMalloc((void **)&a->spmm_chunk_row, sizeof(int32_t) * (size_t)(nchunks > 0 ? nchunks : 1)));
    a->spmm_nchunks = nchunks;
    if (nchunks > 0) {
        KernelTimer t("spmm_chunk_rows");
        spmm_chunk_rows<<<dim3((unsigned)ceil_div(nchunks, 256)), dim3(256), 0, stream()>>>(
            a->pos, a->nrows, nchunks, a->spmm_chunk_row);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

}  // namespace comet

using namespace comet;

extern "C" int comet_hip_spmv_csr_f64(int64_t csr, int64_t x_dptr, int64_t y_dptr, int accumulate)
{
    COMET_CHK(ensure_init());
    Csr *a = csr_from_handle(csr);
    if (!a)
        return COMET_HIP_ERR_HANDLE;
    if ((a->ncols > 0 && !x_dptr) || (a->nrows > 0 && !y_dptr))
        return set_error(COMET_HIP_ERR_ARG, "null vector passed to comet_hip_spmv_csr_f64");
    if (a->nrows == 0)
        return COMET_HIP_OK;
    COMET_CHK(spmv_plan(a));
    const unsigned blocks = (unsigned)ceil_div(a->nrows, SPMV_T);
    const double *x = (const double *)x_dptr;
    double *y = (double *)y_dptr;
    for (int b = 0; b < a->spmv_nb; ++b) {
        const int64_t *pos = a->spmv_nb == 1 ? a->pos : a->spmv_bpos + (int64_t)b * (a->nrows + 1);
        const int32_t *crd = a->spmv_nb == 1 ? a->crd : a->spmv_bcrd + a->spmv_base[b];
        const double *val = a->spmv_nb == 1 ? a->val : a->spmv_bval + a->spmv_base[b];
        const bool acc = accumulate || b > 0;   // later passes continue the row sums the earlier ones left in y
        KernelTimer t("spmv_csr_stream");
        if (acc)
            spmv_csr_stream<true><<<dim3(blocks), dim3(SPMV_T), 0, stream()>>>(pos, crd, val, x, y, a->nrows);
        else
            spmv_csr_stream<false><<<dim3(blocks), dim3(SPMV_T), 0, stream()>>>(pos, crd, val, x, y, a->nrows);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}

extern "C" int comet_hip_spmm_csr_f64(int64_t csr, int64_t K, int64_t b_dptr, int64_t ldb, int64_t c_dptr,
                                      int64_t ldc, int accumulate)
{
    COMET_CHK(ensure_init());
    Csr *a = csr_from_handle(csr);
    if (!a)
        return COMET_HIP_ERR_HANDLE;
    if (K < 0 || ldb < K || ldc < K)
        return set_error(COMET_HIP_ERR_ARG, "bad K/ldb/ldc (%lld, %lld, %lld)", (long long)K, (long long)ldb,
                         (long long)ldc);
    if (K == 0 || a->nrows == 0)
        return COMET_HIP_OK;
    if (!c_dptr || (a->nnz > 0 && !b_dptr))
        return set_error(COMET_HIP_ERR_ARG, "null matrix passed to comet_hip_spmm_csr_f64");
    double *C = (double *)c_dptr;
    if (a->nnz == 0) {
        if (!accumulate) {
            KernelTimer t("fill_rows_f64");
            unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(a->nrows * K, 256), 65536);
            fill_rows_f64<<<dim3(blocks), dim3(256), 0, stream()>>>(C, a->nrows, K, ldc, 0.0);
            COMET_HIPCHK(hipGetLastError());
        }
        return COMET_HIP_OK;
    }
    COMET_CHK(spmm_plan(a));
    const int64_t nchunks = a->spmm_nchunks;
    const int64_t tiles = ceil_div(K, 64);
    if (tiles > 65535)
        return set_error(COMET_HIP_ERR_SIZE, "K = %lld needs more than 65535 column tiles", (long long)K);
    COMET_CHK(g_spmm_carry.ensure(sizeof(double) * (size_t)(tiles * nchunks * 2 * 64), false));
    double *carry = (double *)g_spmm_carry.ptr;
    const dim3 grid((unsigned)ceil_div(nchunks, SPMM_WAVES), (unsigned)tiles);
    const dim3 block(SPMM_WAVES * 64);
    {
        KernelTimer t("spmm_csr_nnzsplit");
        if (accumulate)
            spmm_csr_nnzsplit<true><<<grid, block, 0, stream()>>>(a->pos, a->crd, a->val, a->nnz, a->nrows,
                                                                  a->spmm_chunk_row, nchunks, (const double *)b_dptr,
                                                                  ldb, C, ldc, K, carry);
        else
            spmm_csr_nnzsplit<false><<<grid, block, 0, stream()>>>(a->pos, a->crd, a->val, a->nnz, a->nrows,
                                                                   a->spmm_chunk_row, nchunks, (const double *)b_dptr,
                                                                   ldb, C, ldc, K, carry);
    }
    {
        KernelTimer t("spmm_csr_fixup");
        if (accumulate)
            spmm_csr_fixup<true><<<grid, block, 0, stream()>>>(a->pos, a->nnz, a->spmm_chunk_row, nchunks, C, ldc, K,
                                                               carry);
        else
            spmm_csr_fixup<false><<<grid, block, 0, stream()>>>(a->pos, a->nnz, a->spmm_chunk_row, nchunks, C, ldc, K,
                                                                carry);
    }
    COMET_HIPCHK(hipGetLastError());
    return COMET_HIP_OK;
}
